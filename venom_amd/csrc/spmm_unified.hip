// Dense-staged kernel with unified waves: every wave is consumer and producer, A operands go from L2 to registers.

#include "spmm_device.h"

namespace spatha {

// ---------------------------------------------------------------------------
// Dense-staged kernel with unified waves and the A operands in registers (m <= 16, rows % 512 == 0): tile 512 x 128.
//
// The producer/consumer kernels above move 150 KB per k-step through LDS for a 256 x 128 tile (50 KB of DMA writes,
// 36.8 KB of A operand reads, 64 KB of transposing B reads) and fetch 50 KB from L2; both rates are at their limit.
// Here each of the eight waves owns 64 rows x 128 columns (128 accumulator registers), so the packed A operands of a
// row block are used by exactly one wave and go straight from L2 into its registers, two k-steps ahead; only the dense
// B stage (32 KB for m <= 8) lives in LDS, four stages deep, shared by eight 64-row blocks.  Per 256 x 128 of output and step
// that is 34.4 KB from L2 and 80 KB through LDS.  Every wave issues an eighth of each stage's DMA itself.
// Vector-memory bookkeeping: register loads and LDS-DMA loads share one counter; a step issues the gather-table entry
// and the A operands two steps ahead (7 register loads), then its share of the stage three steps ahead (4 DMA loads),
// and ends on a wait that leaves at most 7 operations in flight (see there).
// ---------------------------------------------------------------------------

// Loads into registers that complete asynchronously: the destination is the caller's variable itself ("+v"), so that no
// copy of a not-yet-arrived value can be placed behind the instruction; the caller's wait names the same variables.
__device__ __forceinline__ void bload_b128(u32x4& r, uint32_t voff, i32x4 rsrc, uint32_t soff) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "+v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void bload_b32(uint32_t& r, uint32_t voff, i32x4 rsrc, uint32_t soff) {
    asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "+v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void bload_b64(u32x2& r, uint32_t voff, i32x4 rsrc, uint32_t soff) {
    asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "+v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}

// FUSE: the instantiation that can apply bias / activation ahead of the write-out (kept apart: its temporaries would
// otherwise push the plain kernel over the register budget)
template <int OUT_LAYOUT, bool FUSE, int M_>
__global__ __launch_bounds__(512) void spmm_du_kernel(SpmmParams p) {
    using Cfg = DuCfg<M_>;
    constexpr int NB = Cfg::NB;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, PA = Cfg::PA, STAGE_BYTES = Cfg::STAGE_BYTES;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    const int S = p.S, N = p.N;
    const int Q = walk.my_tiles * S;
    const i32x4 rsrc_b = make_buffer(p.B, p.b_bytes);
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const i32x4 rsrc_g = make_buffer(p.gtab, p.gtab_bytes);

    // ---- this wave's share of the B stages (as a producer) ----
    const uint32_t row_bytes_b = (uint32_t)N * 2u;
    const int dense_rows = 16 * p.m;
    const uint32_t step_bytes_b = (uint32_t)dense_rows * row_bytes_b;
    const int slot_row = lane >> 4, slot_chunk = lane & 15;
    int is_tm = walk.tm0, is_tn = walk.tn0, is_step = 0;
    uint32_t is_stage = 0, b_soff = 0;
    uint32_t voff[NB];
    auto set_voff = [&]() {
#pragma unroll
        for (int j = 0; j < NB; j++) {
            const int row = (wave * NB + j) * 4 + slot_row;
            const int col = is_tn * BN + (slot_chunk ^ ((row & 7) << 1)) * 8;
            voff[j] = (col < N && row < dense_rows) ? (uint32_t)row * row_bytes_b + (uint32_t)col * 2u : 0xF0000000u;
        }
    };
    set_voff();
    uint32_t dma_stage = 0;                       // target of the stage being issued
    i32x4 dma_rsrc = rsrc_b;                      // its window of B (rows of the step beyond K fail the range check: zeros)
    uint32_t dma_voff[NB];
    auto stage_begin = [&]() {                    // fixes the addresses of the next stage and advances the cursor
        dma_stage = smem_base + is_stage + wave * (NB * 1024);
        dma_rsrc = buffer_window(p.B, p.b_bytes, b_soff);
#pragma unroll
        for (int j = 0; j < NB; j++) dma_voff[j] = voff[j];
        is_stage = (is_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : is_stage + STAGE_BYTES;
        b_soff += step_bytes_b;
        if (++is_step == S) {
            is_step = 0;
            b_soff = 0;
            walk.next(is_tm, is_tn);
            set_voff();
        }
    };
    auto stage_op = [&](int j) { bdma_b128(dma_voff[j], dma_rsrc, 0, dma_stage + j * 1024); };
    auto issue_stage = [&]() {
        stage_begin();
#pragma unroll
        for (int j = 0; j < NB; j++) stage_op(j);
    };

    // ---- operands (as a consumer) ----
    const int li = lane & 15, kb = lane >> 4;
    const uint32_t col_xor = (uint32_t)(((li & 3) >> 1) << 4);
    const uint32_t col_or = (uint32_t)(li & 1) * 8u;
    const int lane_class = kb * 4 + (li >> 2);
    const uint32_t lane16 = lane * 16, lane4 = lane * 4, gvoff = lane_class * 8;
    // operand sets: x is the one the matrix instructions read; l0 / l1 are the landing sets of the loads, which run two
    // k-steps ahead (an L2 round trip under load is longer than one step)
    struct ASet {
        u32x4 a[4];
        uint32_t i0, i1;
        u32x2 g;
    };
    ASet x, l0 = {}, l1 = {};
    uint32_t base[4];
    auto set_base = [&](u32x2 g) {
        base[0] = ((g.x & 0xffffu) ^ col_xor) | col_or;
        base[1] = ((g.x >> 16) ^ col_xor) | col_or;
        base[2] = ((g.y & 0xffffu) ^ col_xor) | col_or;
        base[3] = ((g.y >> 16) ^ col_xor) | col_or;
    };
    // loader cursor: (tile row, step) of the next operand set to fetch; stops at the last step of the last tile
    int ld_tm = walk.tm0, ld_tn = walk.tn0, ld_step = 0, ld_left = Q;
    uint32_t ld_soff = 0, ld_goff = 0;
    auto load_begin = [&]() {                     // fixes the addresses of the next operand set and advances the cursor
        const uint32_t blk = (uint32_t)((ld_tm * 8 + wave) * S + ld_step);
        ld_goff = blk * 128u;
        ld_soff = blk * (uint32_t)APACK_BLOCK;
        if (ld_left > 1) {          // (past the end the last block is fetched again and never used)
            --ld_left;
            if (++ld_step == S) {
                ld_step = 0;
                walk.next(ld_tm, ld_tn);
            }
        }
    };
    auto load_op = [&](ASet& y, int k) {          // the set's seven loads, in issue order
        if (k == 0) bload_b64(y.g, gvoff, rsrc_g, ld_goff);
        else if (k <= 4) bload_b128(y.a[k - 1], lane16, rsrc_a, ld_soff + (k - 1) * 1024);
        else if (k == 5) bload_b32(y.i0, lane4, rsrc_a, ld_soff + 4096);
        else bload_b32(y.i1, lane4, rsrc_a, ld_soff + 4096 + 256);
    };
    auto load_set = [&](ASet& y) {
        load_begin();
#pragma unroll
        for (int k = 0; k < 7; k++) load_op(y, k);
    };
#define SPATHA_DU_WAIT(CNT, Y) \
    asm volatile("s_waitcnt vmcnt(" #CNT ")" : "+v"(Y.a[0]), "+v"(Y.a[1]), "+v"(Y.a[2]), "+v"(Y.a[3]), "+v"(Y.i0), "+v"(Y.i1), "+v"(Y.g))
    auto take = [&](const ASet& y) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) x.a[mb] = y.a[mb];
        x.i0 = y.i0;
        x.i1 = y.i1;
        set_base(y.g);
    };
    float4_t acc[2][4][4];
    auto zero_acc = [&]() {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) acc[h][a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
    };

    // ---- prologue: three stages and the first two operand sets in flight ----
#pragma unroll
    for (int t = 0; t < PA; t++)
        if (t < Q) issue_stage();
    int issued = Q < PA ? Q : PA;
    load_set(l0);
    load_set(l1);
    SPATHA_DU_WAIT(0, l0);
    SPATHA_DU_WAIT(0, l1);
    take(l0);
    zero_acc();

    int c_tm = walk.tm0, c_tn = walk.tn0, c_step = 0;
    uint32_t c_stage = 0;
    // one k-step: `land` receives the operands of step q + 2, `next` holds those of step q + 1
    auto do_step = [&](ASet& land, ASet& next) {
        __syncthreads();        // stage q has landed for every wave; stage q - 1 is free
        // The step's eleven vector-memory instructions (operands of step q + 2, then this wave's share of stage q + 3)
        // are issued between the groups of matrix instructions: with the memory pipeline at its limit an issue can
        // block for a long time, and the matrix pipe should have work queued meanwhile.
        load_begin();
        const bool more = issued < Q;
        if (more) {
            stage_begin();
            ++issued;
        }
        const char* st = smem + c_stage;
        {
            half8_t a_cur[4];
#pragma unroll
            for (int mb = 0; mb < 4; mb++) a_cur[mb] = __builtin_bit_cast(half8_t, x.a[mb]);
            const uint32_t ix0 = x.i0, ix1 = x.i1;
            auto read_frag = [&](int nb8) {
                half16_t bf;
#pragma unroll
                for (int fb = 0; fb < 4; fb++) {
                    short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, st + (base[fb] ^ (uint32_t)(nb8 << 5))));
                    half4_t h4 = __builtin_bit_cast(half4_t, t4);
                    bf[fb * 4 + 0] = h4[0];
                    bf[fb * 4 + 1] = h4[1];
                    bf[fb * 4 + 2] = h4[2];
                    bf[fb * 4 + 3] = h4[3];
                }
                return bf;
            };
#define SPATHA_MMA4U(NB8, BF)                                                                                          \
    acc[(NB8) >> 2][0][(NB8)&3] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], BF, acc[(NB8) >> 2][0][(NB8)&3], (int)ix0, 0, 0); \
    acc[(NB8) >> 2][1][(NB8)&3] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], BF, acc[(NB8) >> 2][1][(NB8)&3], (int)ix0, 0, 1); \
    acc[(NB8) >> 2][2][(NB8)&3] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], BF, acc[(NB8) >> 2][2][(NB8)&3], (int)ix1, 0, 0); \
    acc[(NB8) >> 2][3][(NB8)&3] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], BF, acc[(NB8) >> 2][3][(NB8)&3], (int)ix1, 0, 1);
            constexpr int DEPTH = 2;        // fragments in flight (three or four measure the same)
            half16_t bf[DEPTH];
#pragma unroll
            for (int k = 0; k < DEPTH; k++) bf[k] = read_frag(k);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int nb8 = 0; nb8 < 8; nb8++) {
                SPATHA_MMA4U(nb8, bf[nb8 % DEPTH])
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (M_ == 8) {
                    if (nb8 == 0) { load_op(land, 0); load_op(land, 1); }
                    else if (nb8 == 1) { load_op(land, 2); load_op(land, 3); }
                    else if (nb8 == 2) { load_op(land, 4); load_op(land, 5); }
                    else if (nb8 == 3) { load_op(land, 6); }
                    else if (more) stage_op(nb8 - 4);
                } else {
                    // two stages: the DMA of the next step's stage goes first, the operand loads behind it
                    if (nb8 < 4) { if (more) { stage_op(2 * nb8); stage_op(2 * nb8 + 1); } }
                    else if (nb8 < 7) { load_op(land, 2 * (nb8 - 4)); load_op(land, 2 * (nb8 - 4) + 1); }
                    else load_op(land, 6);
                }
                __builtin_amdgcn_sched_barrier(0);
                if (nb8 + DEPTH < 8) bf[nb8 % DEPTH] = read_frag(nb8 + DEPTH);
                __builtin_amdgcn_sched_barrier(0);
            }
#undef SPATHA_MMA4U
        }
        c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        // LDS-DMA loads and register loads each retire in order, but not with respect to each other (measured: a wait
        // that leaves the 7 youngest operations, all register loads, in flight returned before older DMA loads had
        // landed).  With at most 7 operations left, at most the 7 youngest of EACH kind are: the operand set of step
        // q + 1 (7 younger register loads) and the DMA of stage q + 1 (8 younger DMA loads) are in.  The two-stage form
        // needs the DMA it issued in this very step and can only wait for everything.
        // Near the end no younger DMA is in flight any more: wait for everything there as well.
        if (M_ == 8 && more) SPATHA_DU_WAIT(7, next);
        else SPATHA_DU_WAIT(0, next);
        take(next);
        if (++c_step == S) {
            c_step = 0;
            const int cm0 = c_tm * BM + wave * 64, cn0 = c_tn * BN;
            char* stg = smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES;
            const int ib = lane >> 4;
#pragma unroll
            for (int wn = 0; wn < 2; wn++) {
                // fused: bias and activation first, always and on one path (a path that skipped them would join this one
                // on all 64 accumulator registers of the block); the write-out itself is then the plain one
                if constexpr (FUSE) fused_bias_act_narrow(acc[wn], p.bias, (int64_t)cm0 + ib * 16, p.act);
                if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED)
                    store_block_transposed_slab<true>(acc[wn], stg, p.C, FUSE ? nullptr : p.bias, (int64_t)cm0, cn0 + wn * 64, p.rows,
                                                      N, lane, true);
                else
                    store_block_row_major_tr<true>(acc[wn], stg, p.C, (int64_t)cm0, cn0 + wn * 64, N, lane, true);
            }
            zero_acc();
            walk.next(c_tm, c_tn);
        }
    };
    for (int q = 0; q < Q; q += 2) {
        do_step(l0, l1);
        if (q + 1 < Q) do_step(l1, l0);
    }
#undef SPATHA_DU_WAIT
}

template <int OUT_LAYOUT, bool FUSE, int M_ = 8>
static hipError_t launch_du(const SpmmParams& p, hipStream_t stream) {
    constexpr int lds = DuCfg<M_>::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    const int cus = p.cus;        // compute units of the plan's device
    void (*kern)(SpmmParams) = spmm_du_kernel<OUT_LAYOUT, FUSE, M_>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        // The kernel's register loads complete asynchronously into named variables; a compiler-made copy of such a
        // variable to scratch memory between the load and its wait would save a value that has not arrived.  An
        // instantiation with any scratch memory is therefore refused.
        hipFuncAttributes fa;
        hipError_t e = hipFuncGetAttributes(&fa, (const void*)kern);
        if (e != hipSuccess) return e;
        if (fa.localSizeBytes != 0) return hipErrorNotSupported;
        e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = p.tiles_m * p.tiles_n;
    int grid = (cus / 8) * 8;
    const int need = ((tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    if (grid < 8) grid = 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(DuCfg<M_>::THREADS), lds, stream, p);
    return hipGetLastError();
}

hipError_t launch_unified(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    const bool t = out_layout == SPATHA_OUT_TRANSPOSED;
    switch (variant) {
        case SPMM_VARIANT_DU512x128_M16:
            if (p.fuse)
                return t ? launch_du<SPATHA_OUT_TRANSPOSED, true, 16>(p, stream) : launch_du<SPATHA_OUT_ROW_MAJOR, true, 16>(p, stream);
            return t ? launch_du<SPATHA_OUT_TRANSPOSED, false, 16>(p, stream) : launch_du<SPATHA_OUT_ROW_MAJOR, false, 16>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace spatha

