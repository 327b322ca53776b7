// Dense-staged kernel with unified waves in two phase groups (m <= 8, rows % 512 == 0): tile 512 x 128.
//
// Same data path as the unified kernel (spmm_unified.hip): eight waves of 64 x 128 each, the packed A operands of a
// wave's rows go from L2 straight into its registers, only the dense B stage (32 KB) lives in LDS and serves all eight
// 64-row blocks, every wave issues an eighth of each stage's DMA.  What differs is WHEN a wave issues its vector-memory
// instructions.  There, all eight waves spread their loads between their groups of matrix instructions; a load whose
// issue blocks (the memory pipeline is the busiest unit of this kernel: 88 wave-instructions, 72 KB per step, through a path that
// delivers about 53 B per clock) then stops that wave's matrix instructions, and since the waves run in lockstep between two barriers, the other
// wave of the SIMD is blocked in the same place.  Here the two waves of a SIMD belong to different phase groups:
//   group X (waves 0-3):  barrier | burst of the step's 11 loads | matrix phase (8 x 4 instructions, reads interleaved)
//   group Y (waves 4-7):  barrier | matrix phase                 | burst
// so that while one wave of a SIMD sits in its burst, the other one feeds the matrix unit, and the memory pipeline
// sees one group's burst in each half of a step.  A burst is always preceded (Y) or followed after the matrix phase (X)
// by a wait for EVERYTHING the wave has in flight (s_waitcnt vmcnt(0)); what it waits for was issued a matrix phase
// earlier.  Waiting for everything sidesteps the ordering question of the unified kernel (register loads and LDS-DMA
// loads do not retire in order with respect to each other, so a partial wait has to be conservative), and it lets two
// operand sets per wave suffice:
//   X, step q: burst = operands of step q + 1 (into the set step q - 1 used) + this wave's share of stage q + 2
//   Y, step q: burst = operands of step q + 2 (into the set step q just used)  + this wave's share of stage q + 2
// Stage q + 2 goes into the slot stage q - 1 occupied, which every wave has left when it passed barrier q: three stages.
// The wait sits ahead of a tile's stores: a wait behind them would wait for the stores too (same counter).
// A finished tile leaves through four LDS slabs per wave (a 64 x 64 block in two LDS round trips); LDS: 3 x 32 KB of
// stages + 8 x 4.6 KB of slabs.

#include "spmm_device.h"

// Development switches, compiled in with -DSPATHA_UP_KNOBS=<bits> for timing experiments only (0 in the library; the
// results are then wrong on purpose):  1 no B stages (matrix phases on whatever the LDS holds)   2 no write-out
//   4 the late group skips its matrix phases   8 a second barrier in the middle of a step   16 no A operands (only
//   the gather table is loaded)   32 write-out without its global stores   64 no matrix instructions
#ifndef SPATHA_UP_KNOBS
#define SPATHA_UP_KNOBS 0
#endif

// Development-only cycle accounting (-DSPATHA_DEV_PROFILE): every wave sums the s_memtime ticks it spends (0) issuing its
// bursts, (1) in matrix phases, (2) in the wait for its loads, (3) at the step barrier, (4) in write-outs; lane 0 writes the
// five sums to prof[(workgroup * 8 + wave) * 8 ..].
#ifdef SPATHA_DEV_PROFILE
#define SPATHA_UP_PROF_DECL long long up_prof_t = __builtin_readcyclecounter(), up_prof_sum[5] = {0, 0, 0, 0, 0};
#define SPATHA_UP_PROF_MARK(SLOT)                                \
    {                                                            \
        const long long now = __builtin_readcyclecounter();      \
        up_prof_sum[SLOT] += now - up_prof_t;                    \
        up_prof_t = now;                                         \
    }
#define SPATHA_UP_PROF_FLUSH                                                              \
    if (p.prof && lane == 0) {                                                            \
        long long* dst = p.prof + ((int64_t)blockIdx.x * 8 + wave) * 8;                   \
        for (int k = 0; k < 5; k++) dst[k] = up_prof_sum[k];                              \
    }
#else
#define SPATHA_UP_PROF_DECL
#define SPATHA_UP_PROF_MARK(SLOT)
#define SPATHA_UP_PROF_FLUSH
#endif

namespace spatha {

namespace {
constexpr int UP_KNOBS = SPATHA_UP_KNOBS;
// tile walks of this kernel: column after column, or tile rows in groups of four (SpmmParams::walk_group)
constexpr int UP_WALK_ROWS = -4;
__device__ __forceinline__ void pload_b128(u32x4& r, uint32_t voff, i32x4 rsrc, uint32_t soff) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2, %3 offen" : "=&v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void pload_b32(uint32_t& r, uint32_t voff, i32x4 rsrc, uint32_t soff) {
    asm volatile("buffer_load_dword %0, %1, %2, %3 offen" : "=&v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
__device__ __forceinline__ void pload_b64(u32x2& r, uint32_t voff, i32x4 rsrc, uint32_t soff) {
    asm volatile("buffer_load_dwordx2 %0, %1, %2, %3 offen" : "=&v"(r) : "v"(voff), "s"(rsrc), "s"(soff) : "memory");
}
}  // namespace

// The whole life of one wave.  LATE is the wave's phase group (false: X, true: Y), a template argument so that each group
// runs straight-line code of its own: an operand set that is in flight must never meet, at a join of two paths, a
// version of itself that is not (the register copy the compiler may place there would copy a value that has not arrived).
template <int OUT_LAYOUT, bool FUSE, bool GROUPED, bool LATE, class Walk>
__device__ __forceinline__ void up_wave(const SpmmParams& p, const Walk& walk, char* smem, uint32_t smem_base, int wave,
                                        int lane) {
    using Cfg = UpCfg;
    constexpr int NB = Cfg::NB;
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::NS, STAGE_BYTES = Cfg::STAGE_BYTES;
    const int S = p.S, N = p.N;
    const int Q = walk.my_tiles * S;
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const i32x4 rsrc_g = make_buffer(p.gtab, p.gtab_bytes);

    // ---- this wave's share of the B stages: 16 of the 128 dense rows ----
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
    int issued = 0;
    auto issue_stage = [&]() {
        if (UP_KNOBS & 1) return;
        if (issued >= Q) return;
        ++issued;
        const uint32_t dst = smem_base + is_stage + wave * (NB * 1024);
        // the step's window of B: rows of the step that lie beyond K fail the range check and arrive as zeros
        const i32x4 rsrc_step = buffer_window(p.B, p.b_bytes, b_soff);
#pragma unroll
        for (int j = 0; j < NB; j++) bdma_b128(voff[j], rsrc_step, 0, dst + j * 1024);
        is_stage = (is_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : is_stage + STAGE_BYTES;
        b_soff += step_bytes_b;
        if (++is_step == S) {
            is_step = 0;
            b_soff = 0;
            walk.next(is_tm, is_tn);
            set_voff();
        }
    };

    // ---- operands ----
    const int li = lane & 15, kb = lane >> 4;
    const uint32_t col_xor = (uint32_t)(((li & 3) >> 1) << 4);
    const uint32_t col_or = (uint32_t)(li & 1) * 8u;
    const int lane_class = kb * 4 + (li >> 2);
    const uint32_t lane16 = lane * 16, lane4 = lane * 4, gvoff = lane_class * 8;
    struct ASet {
        u32x4 a[4];
        uint32_t i0, i1;
        u32x2 g;
    };
    ASet s0 = {}, s1 = {};
    // loader cursor: (tile row, step) of the next operand set to fetch; stops at the last step of the last tile
    int ld_tm = walk.tm0, ld_tn = walk.tn0, ld_step = 0, ld_left = Q;
    auto load_set = [&](ASet& y) {
        const uint32_t blk = (uint32_t)((ld_tm * 8 + wave) * S + ld_step);
        const uint32_t goff = blk * 128u, soff = blk * (uint32_t)APACK_BLOCK;
        if (ld_left > 1) {          // (past the end the last block is fetched again and never used)
            --ld_left;
            if (++ld_step == S) {
                ld_step = 0;
                walk.next(ld_tm, ld_tn);
            }
        }
        pload_b64(y.g, gvoff, rsrc_g, goff);
        if (UP_KNOBS & 16) return;
#pragma unroll
        for (int k = 0; k < 4; k++) pload_b128(y.a[k], lane16, rsrc_a, soff + k * 1024);
        pload_b32(y.i0, lane4, rsrc_a, soff + 4096);
        pload_b32(y.i1, lane4, rsrc_a, soff + 4096 + 256);
    };
    // the wait names both operand sets (in and out), so that the compiler keeps every use of a set behind its wait
#define SPATHA_UP_WAIT_ALL()                                                                                              \
    asm volatile("s_waitcnt vmcnt(0)"                                                                                     \
                 : "+v"(s0.a[0]), "+v"(s0.a[1]), "+v"(s0.a[2]), "+v"(s0.a[3]), "+v"(s0.i0), "+v"(s0.i1), "+v"(s0.g),      \
                   "+v"(s1.a[0]), "+v"(s1.a[1]), "+v"(s1.a[2]), "+v"(s1.a[3]), "+v"(s1.i0), "+v"(s1.i1), "+v"(s1.g)       \
                 :                                                                                                        \
                 : "memory")

    float4_t acc[2][4][4];
    auto zero_acc = [&]() {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) acc[h][a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
    };

    // ---- prologue: stages 0 and 1, operands of step 0 (and of step 1 for the late group) ----
    issue_stage();
    issue_stage();
    load_set(s0);
    if constexpr (LATE) load_set(s1);
    SPATHA_UP_WAIT_ALL();
    zero_acc();

    int c_tm = walk.tm0, c_tn = walk.tn0, c_step = 0;
    uint32_t c_stage = 0;

    // The matrix phase of one k-step: 8 fragments of B (4 transposing reads each), 4 matrix instructions per fragment.
    // Fine interleave: behind every matrix instruction of fragment f goes one read of fragment f + 2, so that the
    // wave's LDS issue runs in the shadow of its own matrix instructions (a matrix instruction occupies the unit for
    // 16 clocks and its issue for 4).  Three fragment buffers in rotation.
    auto matrix_phase = [&](const ASet& x) {
        const uint32_t st = smem_base + c_stage;
        uint32_t base[4];
        base[0] = (((x.g.x & 0xffffu) ^ col_xor) | col_or) + st;      // (stage offsets are multiples of 32 KB: the xor
        base[1] = (((x.g.x >> 16) ^ col_xor) | col_or) + st;          //  of a column-block index below commutes with it)
        base[2] = (((x.g.y & 0xffffu) ^ col_xor) | col_or) + st;
        base[3] = (((x.g.y >> 16) ^ col_xor) | col_or) + st;
        half8_t a_cur[4];
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_cur[mb] = __builtin_bit_cast(half8_t, x.a[mb]);
        const uint32_t ix[2] = {x.i0, x.i1};
        half16_t bf[3];
        // Where the read addresses are computed is a template argument.  A vector ALU instruction BETWEEN two matrix
        // instructions holds the second one back (measured on the matrix phase alone, one wave per SIMD: 952 clocks per
        // step with an xor ahead of every read, 760 with the xors in groups of four, 640 with none), an LDS instruction
        // does not.  GROUPED computes a fragment's four addresses together, ahead of the four matrix instructions its
        // reads follow: 3-4 % faster wherever the clock holds (2:4, 2:5, integer-valued operands).  With Gaussian
        // operands at m >= 7 it does not: the denser matrix phases run into the GPU's power management, launches
        // take anything from 54 to 72 us and the sustained mean is 65-68 us against a steady 58 us with the xors left
        // between the matrix instructions - so that form stays for m > 5 (chosen at launch).
        uint32_t ad[4];
        auto addresses = [&](int nb8) {
#pragma unroll
            for (int fb = 0; fb < 4; fb++) ad[fb] = base[fb] ^ (uint32_t)(nb8 << 5);
        };
        auto read_part = [&](half16_t& dst, int nb8, int fb) {
            const uint32_t addr = GROUPED ? ad[fb] : base[fb] ^ (uint32_t)(nb8 << 5);
            short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)(uintptr_t)addr);
            half4_t h4 = __builtin_bit_cast(half4_t, t4);
            dst[fb * 4 + 0] = h4[0];
            dst[fb * 4 + 1] = h4[1];
            dst[fb * 4 + 2] = h4[2];
            dst[fb * 4 + 3] = h4[3];
        };
#pragma unroll
        for (int k = 0; k < 2; k++) {
            if (GROUPED) addresses(k);
#pragma unroll
            for (int fb = 0; fb < 4; fb++) read_part(bf[k], k, fb);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int nb8 = 0; nb8 < 8; nb8++) {
            if (GROUPED && nb8 + 2 < 8) addresses(nb8 + 2);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                float4_t& c = acc[nb8 >> 2][mb][nb8 & 3];
                if (UP_KNOBS & 64) asm volatile("" ::"v"(bf[nb8 % 3]), "v"(a_cur[mb]), "v"(ix[mb >> 1]));
                else if (mb & 1) c = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[mb], bf[nb8 % 3], c, (int)ix[mb >> 1], 0, 1);
                else c = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[mb], bf[nb8 % 3], c, (int)ix[mb >> 1], 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (nb8 + 2 < 8) read_part(bf[(nb8 + 2) % 3], nb8 + 2, mb);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    // one k-step; `cur` holds its operands, `other` is the wave's second set
    SPATHA_UP_PROF_DECL
    auto do_step = [&](ASet& cur, ASet& other) {
        __syncthreads();        // stage q has landed for every wave; every wave has left stage q - 1
        SPATHA_UP_PROF_MARK(3)
        if constexpr (!LATE) {
            load_set(other);    // operands of step q + 1
            issue_stage();      // share of stage q + 2
            if (UP_KNOBS & 8) __syncthreads();
            SPATHA_UP_PROF_MARK(0)
        }
        if (!(LATE && (UP_KNOBS & 4))) matrix_phase(cur);
        SPATHA_UP_PROF_MARK(1)
        c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        // Everything this wave has in flight, issued one matrix phase ago: X, its burst of this step (operands of step
        // q + 1, share of stage q + 2); Y, its burst of the step before (operands of step q + 1, share of stage q + 1).
        // Always here, never under a condition, and ahead of the tile's stores, which a later wait would sit out too.
        SPATHA_UP_WAIT_ALL();
        SPATHA_UP_PROF_MARK(2)
        if constexpr (LATE) {
            if (UP_KNOBS & 8) __syncthreads();
            load_set(cur);      // operands of step q + 2
            issue_stage();      // share of stage q + 2
            SPATHA_UP_PROF_MARK(0)
        }
        if (++c_step == S) {
            c_step = 0;
            const int cm0 = c_tm * BM + wave * 64, cn0 = c_tn * BN;
            char* stg = smem + Cfg::EPI_BASE + wave * Cfg::WAVE_EPI;
            if (UP_KNOBS & 2) {     // keep the accumulators alive without storing them
                float t = 0.f;
#pragma unroll
                for (int h = 0; h < 2; h++)
#pragma unroll
                    for (int a = 0; a < 4; a++)
#pragma unroll
                        for (int b = 0; b < 4; b++) t += acc[h][a][b][0] + acc[h][a][b][1] + acc[h][a][b][2] + acc[h][a][b][3];
                if (t == 12345.678f) p.C[lane] = 1;
            } else {
#pragma unroll
                for (int wn = 0; wn < 2; wn++) {
                    // fused: bias and activation first, always and on one path (a path that skipped them would join this
                    // one on all 64 accumulator registers of the block); the write-out itself is then the plain one
                    if constexpr (FUSE) fused_bias_act_narrow(acc[wn], p.bias, (int64_t)cm0 + (lane >> 4) * 16, p.act);
                    if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED)
                        store_block_transposed_slab4(acc[wn], stg, p.C, FUSE ? nullptr : p.bias, (int64_t)cm0, cn0 + wn * 64, p.rows, N,
                                                     lane, !(UP_KNOBS & 32));
                    else
                        store_block_row_major_tr4<false>(acc[wn], stg, p.C, (int64_t)cm0, cn0 + wn * 64, N, lane, !(UP_KNOBS & 32), nullptr);
                }
            }
            zero_acc();
            walk.next(c_tm, c_tn);
            SPATHA_UP_PROF_MARK(4)
        }
    };
    for (int q = 0; q < Q; q += 2) {
        do_step(s0, s1);
        if (q + 1 < Q) do_step(s1, s0);
    }
    SPATHA_UP_PROF_FLUSH
#undef SPATHA_UP_WAIT_ALL
}

template <int OUT_LAYOUT, bool FUSE, bool GROUPED, int WALK>
__global__ __launch_bounds__(512) void spmm_up_kernel(SpmmParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalkT<WALK> walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    // (development builds: the workgroups of an XCD start in four groups, skew * 1024 clocks apart, so that their write-outs
    // no longer fall together)
    if (SPATHA_SKEW_ON(p)) {
        const int units = ((blockIdx.x >> 3) & 3) * p.skew;
        for (int i = 0; i < units; i++) __builtin_amdgcn_s_sleep(16);
    }
    if (wave >= 4) up_wave<OUT_LAYOUT, FUSE, GROUPED, true>(p, walk, smem, smem_base, wave, lane);
    else up_wave<OUT_LAYOUT, FUSE, GROUPED, false>(p, walk, smem, smem_base, wave, lane);
}

template <int OUT_LAYOUT, bool FUSE, bool GROUPED, int WALK>
static hipError_t launch_up_walk(const SpmmParams& p, hipStream_t stream) {
    constexpr int lds = UpCfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    const int cus = p.cus;        // compute units of the plan's device
    void (*kern)(SpmmParams) = spmm_up_kernel<OUT_LAYOUT, FUSE, GROUPED, WALK>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        // the kernel's register loads complete asynchronously into named variables: an instantiation that keeps
        // anything in scratch memory could save such a variable before its value has arrived, and is refused
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
    hipLaunchKernelGGL(kern, dim3(grid), dim3(UpCfg::THREADS), lds, stream, p);
    return hipGetLastError();
}

template <int OUT_LAYOUT, bool FUSE, bool GROUPED>
static hipError_t launch_up(const SpmmParams& p, hipStream_t stream) {
    if (p.walk_group == UP_WALK_ROWS && p.tiles_m % 4 == 0) return launch_up_walk<OUT_LAYOUT, FUSE, GROUPED, UP_WALK_ROWS>(p, stream);
    return launch_up_walk<OUT_LAYOUT, FUSE, GROUPED, 1>(p, stream);
}

// largest m that runs the grouped form of the matrix phase
#ifndef SPATHA_UP_GROUPED_MAX_M
#define SPATHA_UP_GROUPED_MAX_M 5
#endif

hipError_t launch_pingpong(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    if (variant != SPMM_VARIANT_UP512x128_S3) return hipErrorInvalidValue;
    // (the plain instantiations carry nothing of the fused write-out; the form of the matrix phase follows m, see there)
    const bool t = out_layout == SPATHA_OUT_TRANSPOSED, grouped = p.m <= SPATHA_UP_GROUPED_MAX_M;
    if (p.fuse) {
        if (grouped) return t ? launch_up<SPATHA_OUT_TRANSPOSED, true, true>(p, stream) : launch_up<SPATHA_OUT_ROW_MAJOR, true, true>(p, stream);
        return t ? launch_up<SPATHA_OUT_TRANSPOSED, true, false>(p, stream) : launch_up<SPATHA_OUT_ROW_MAJOR, true, false>(p, stream);
    }
    if (grouped) return t ? launch_up<SPATHA_OUT_TRANSPOSED, false, true>(p, stream) : launch_up<SPATHA_OUT_ROW_MAJOR, false, true>(p, stream);
    return t ? launch_up<SPATHA_OUT_TRANSPOSED, false, false>(p, stream) : launch_up<SPATHA_OUT_ROW_MAJOR, false, false>(p, stream);
}

}  // namespace spatha
