// Producer / consumer kernels on gathered B stages: consumer waves only read LDS and issue matrix instructions,
// producer waves only compute addresses and issue the global -> LDS DMA.

#include "spmm_device.h"

namespace spatha {

// ---------------------------------------------------------------------------
// Warp-specialised persistent SpMM kernel.
//
// The workgroup has NC = WM*WN consumer waves and NP producer waves.  Consumers do nothing
// but read operands from LDS and issue sparse matrix instructions (and write finished tiles);
// producers do nothing but address arithmetic and DMA issue for the stages NS-1 k-steps
// ahead.  A wave can issue roughly one instruction every few cycles, so keeping the
// bookkeeping out of the consumers' instruction stream is what lets their matrix pipe stay
// busy.  One workgroup barrier per k-step joins the two roles:
//   producer: wait own DMA of stage q | barrier | issue stage q + NS-1
//   consumer:                           barrier | multiply stage q
// Producer pr stands in for the wave (wm = pr / 2, wn = pr % 2) of the 2 x 2 arrangement when
// it comes to which DMA instructions of a stage it issues.
// ---------------------------------------------------------------------------

template <class Cfg, int NP, int PR, bool FINAL_BARRIER = false, class Walk = TileWalk>
__device__ __forceinline__ void ws_producer(const SpmmParams& p, const Walk& walk, char* smem, uint32_t smem_base,
                                            int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1, PA = Cfg::PA;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int WM = BM / 64;
    constexpr int CHUNKS = BN / 8;
    constexpr int RPI = 1024 / ROW_BYTES;
    constexpr int NB_LOADS = 64 / RPI / NP;          // B DMA instructions per producer per stage
    constexpr int A_INSTR = WM * 6;                  // per wave-tile row: 4 operand blocks + 2 index blocks
    constexpr int NA_LOADS = A_INSTR / NP;
    constexpr int LOADS = NB_LOADS + NA_LOADS + 1;
    static_assert(64 % (RPI * NP) == 0 && A_INSTR % NP == 0, "DMA work must split evenly over the producers");
    static_assert((PA - 1) * LOADS < 64, "vmcnt range");

    // k-split: the walk's m-tiles are (row tile, part) pairs, vm = row tile * KS + part, and a part is SC = S / KS k-steps
    // starting at step part * SC (KS = 1: the whole k-loop, vm = row tile)
    const int S = p.S, N = p.N, KS = p.ksplit, SC = S / KS;
    const int Q = walk.my_tiles * SC;
    const int tiles_per_vblock = p.v / BM;
    auto rt_offset = [&](int vm) { return (uint32_t)(((vm / KS) / tiles_per_vblock) * S + (vm % KS) * SC) * 256u; };
    auto a_offset = [&](int vm) { return (uint32_t)(((vm / KS) * WM) * S + (vm % KS) * SC) * (uint32_t)APACK_BLOCK; };
    const i32x4 rsrc_b = make_buffer(p.B, p.b_bytes);
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const i32x4 rsrc_rt = make_buffer(p.rowtab, p.rowtab_bytes);
    const uint32_t row_bytes_b = (uint32_t)N * 2u;
    constexpr uint32_t rt_base = Cfg::RT_BASE + PR * ((PA + 1) * 256);
    const int slot_row = lane / CHUNKS, slot_chunk = lane % CHUNKS;
    int src_chunk[NB_LOADS];
#pragma unroll
    for (int j = 0; j < NB_LOADS; j++) {
        const int rho = (PR * NB_LOADS + j) * RPI + slot_row;
        src_chunk[j] = slot_chunk ^ ((rho & 7) << 1);
    }
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;
    const uint32_t rt_lane_off = (uint32_t)((PR * NB_LOADS) * RPI + slot_row) * 4;

    int is_tm = walk.tm0, is_tn = walk.tn0, is_step = 0;
    uint32_t is_stage = 0;
    uint32_t rt_read = 0;
    int rt_tm = walk.tm0, rt_tn = walk.tn0, rt_step = 0, rt_left = Q - 1;
    uint32_t rt_soff = rt_offset(rt_tm);
    uint32_t a_soff = a_offset(is_tm);    // wave-tile row 0 of the tile, first step of the part
    uint32_t coloff[NB_LOADS];
    auto set_coloff = [&]() {
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const int col = is_tn * BN + src_chunk[j] * 8;
            coloff[j] = (col < N && !SPATHA_KNOB(1)) ? (uint32_t)col * 2u : 0xF0000000u;
        }
    };
    set_coloff();
    auto rt_advance = [&]() {
        if (rt_left > 0) {
            --rt_left;
            rt_soff += 256u;
            if (++rt_step == SC) {
                rt_step = 0;
                walk.next(rt_tm, rt_tn);
                rt_soff = rt_offset(rt_tm);
            }
        }
    };
    auto issue_batch = [&](const uint32_t (&rows)[NB_LOADS]) {
        const uint32_t stage = smem_base + is_stage;
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const uint32_t voff = (rows[j] == 0xffffffffu) ? 0xF0000000u : rows[j] * row_bytes_b + coloff[j];
            bdma_b128(voff, rsrc_b, 0, stage + (PR * NB_LOADS + j) * 1024);
        }
        // the A_INSTR operand / index blocks of the stage, NA_LOADS consecutive ones per producer:
        // instruction a = wm*6 + k; k < 4: operand block k (1 KiB); k >= 4: index block k-4 (256 B)
#pragma unroll
        for (int k = 0; k < NA_LOADS; k++) {
            constexpr int dummy = 0;
            (void)dummy;
            const int a = PR * NA_LOADS + k;
            const int awm = a / 6, ak = a - awm * 6;
            const uint32_t soff = a_soff + (uint32_t)(awm * S) * (uint32_t)APACK_BLOCK;
            const uint32_t dst = stage + B_BYTES + awm * APACK_BLOCK;
            if (ak < 4) bdma_b128(lane16, rsrc_a, soff + ak * 1024, dst + ak * 1024);
            else bdma_b32(lane4, rsrc_a, soff + 4096 + (ak - 4) * 256, dst + 4096 + (ak - 4) * 256);
        }
        const uint32_t rt_write = (rt_read == 0) ? (uint32_t)PA * 256u : rt_read - 256u;
        bdma_b32(lane4, rsrc_rt, rt_soff, smem_base + rt_base + rt_write);
        rt_advance();
        is_stage = (is_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : is_stage + STAGE_BYTES;
        rt_read = (rt_read == (uint32_t)PA * 256u) ? 0u : rt_read + 256u;
        a_soff += (uint32_t)APACK_BLOCK;
        if (++is_step == SC) {
            is_step = 0;
            walk.next(is_tm, is_tn);
            a_soff = a_offset(is_tm);
            set_coloff();
        }
    };
    // prologue: rows of the first PA stages through ordinary loads (nothing is in flight yet)
    {
        uint32_t rows0[PA][NB_LOADS];
        int st_tm = walk.tm0, st_tn = walk.tn0, st_step = 0;
#pragma unroll
        for (int t = 0; t < PA; t++) {
            const int64_t base = ((int64_t)((st_tm / KS) / tiles_per_vblock) * S + (st_tm % KS) * SC + st_step) * 64;
#pragma unroll
            for (int j = 0; j < NB_LOADS; j++)
                rows0[t][j] = (t < Q) ? p.rowtab[base + (PR * NB_LOADS + j) * RPI + slot_row] : 0xffffffffu;
            if (++st_step == SC) { st_step = 0; walk.next(st_tm, st_tn); }
        }
#pragma unroll
        for (int t = 0; t < PA; t++) rt_advance();
#pragma unroll
        for (int t = 0; t < PA; t++)
            if (t < Q) issue_batch(rows0[t]);
    }
    auto issue_from_ring = [&]() {
        uint32_t rows[NB_LOADS];
        const char* rr = smem + rt_base + rt_read + rt_lane_off;
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) rows[j] = *(const uint32_t*)(rr + j * (RPI * 4));
        issue_batch(rows);
    };
    // steady state: PA-1 younger batches stay in flight behind the one being waited for
    const int q_main = Q - PA > 0 ? Q - PA : 0;       // steps that still issue a batch
    for (int q = 0; q < q_main; q++) {
        wait_vmcnt<(PA - 1) * LOADS>();
        __syncthreads();
        if (!SPATHA_KNOB(8)) issue_from_ring();
    }
    // drain: nothing left to issue
    for (int q = q_main; q < Q; q++) {
        wait_stages<LOADS, PA - 1>(Q - 1 - q);
        __syncthreads();
    }
    if (FINAL_BARRIER) __syncthreads();     // (kernels with store waves: the last tile's hand-over)
}

// k-split hand-over of one wave's 64 x 64 block (KS parts of a tile's k-loop, each computed by another workgroup): the wave
// stores its fp32 partial block and takes a ticket; the wave that draws the last ticket adds the parts up IN PART ORDER (its
// own from registers, the others from memory), so the sum does not depend on which part arrives last, and returns true: it
// owns the block's write-out.  No wave ever waits for another.
// The parts of a tile may run on different XCDs, whose L2s do not see each other's lines: partial blocks are written and
// read with the device-scope cache policy (sc1: through the L2 to the memory side), the stores are complete (vmcnt) before
// the ticket is drawn with a device-scope atomic, and the loads are issued behind it.  A device-scope FENCE would do as well
// and costs far more: it writes back and invalidates the XCD's whole L2 (1024 x 4096 x 2048 at 128:2:8: 39.7 us with
// fences, 21.2 us this way, 16.4 us unsplit).  Weaker cache policies (L2-local loads, write-back stores) measure the same
// as these on every shape tried: the hand-over's 4-8 us are its three dependent round trips, not its cache traffic.
// `slot` = index of the (tile, block) among the launch's blocks; partial: [slot][part][16][64] float4; tickets: [slot], zero
// at launch; the wave that draws the last ticket puts the zero back, so a workspace that was cleared once stays usable.
__device__ __forceinline__ bool ksplit_exchange(float4_t (&acc)[4][4], const SpmmParams& p, int64_t slot, int part, int lane) {
    const int KS = p.ksplit;
    constexpr int SC1 = 16;         // cache policy bit of the buffer instructions: device scope
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)p.partial, 0, (int)p.partial_bytes, 0x00020000);
    const uint32_t block0 = (uint32_t)(slot * KS) * 16384u + (uint32_t)lane * 16u;     // part 0 of this block, this lane
    const uint32_t mine = block0 + (uint32_t)part * 16384u;
#pragma unroll
    for (int i = 0; i < 16; i++)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, acc[i >> 2][i & 3]), rsrc, (int)(mine + i * 1024), 0, SC1);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");          // the stores have completed (a wait, no cache operation)
    uint32_t ticket = 0;
    if (lane == 0) ticket = __hip_atomic_fetch_add(p.tickets + slot, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    ticket = (uint32_t)__builtin_amdgcn_readfirstlane((int)ticket);
    if (ticket != (uint32_t)(KS - 1)) return false;
    if (lane == 0) __hip_atomic_store(p.tickets + slot, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");          // (keeps the loads below behind the ticket)
#pragma unroll
    for (int i = 0; i < 16; i++) {
        float4_t t = acc[i >> 2][i & 3];
        if (part != 0) t = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(block0 + i * 1024), 0, SC1));
        for (int q = 1; q < KS; q++) {
            float4_t v = acc[i >> 2][i & 3];
            if (q != part)
                v = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)(block0 + q * 16384 + i * 1024), 0, SC1));
            t += v;
        }
        acc[i >> 2][i & 3] = t;
    }
    return true;
}

template <class Cfg, int WN, int OUT_LAYOUT, class Walk = TileWalk>
__device__ __forceinline__ void ws_consumer(const SpmmParams& p, const Walk& walk, char* smem, int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int EPI_PITCH = Cfg::EPI_PITCH;
    const int S = p.S, N = p.N, KS = p.ksplit, SC = S / KS;
    const int wm = wave / WN, wn = wave - wm * WN;
    float4_t acc[4][4];
    const int li = lane & 15, kb = lane >> 4;
    const int rrow = kb * 4 + (li >> 2);
    const int sw = rrow & 7;
    int tr_off[4];
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int ch = (wn * 8 + nb * 2 + ((li & 3) >> 1)) ^ (sw << 1);
        tr_off[nb] = rrow * ROW_BYTES + ch * 16 + (li & 1) * 8;
    }
    const int a_off = B_BYTES + wm * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + wm * APACK_BLOCK + 4096 + lane * 4;
    const int j16 = lane & 15, ib = lane >> 4;
    int c_tm = walk.tm0, c_tn = walk.tn0;
    uint32_t c_stage = 0;
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++, walk.next(c_tm, c_tn)) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < SC; c_step++) {
            __syncthreads();
            if (!SPATHA_KNOB(16)) mma_stage<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc, [&]() {});
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        }
        const int r_tm = c_tm / KS;          // row tile (the walk's m index counts (row tile, part) pairs)
        if (KS > 1) {
            const int64_t slot = ((int64_t)c_tn * (walk.tiles_m / KS) + r_tm) * Cfg::NC + wave;
            if (!ksplit_exchange(acc, p, slot, c_tm - r_tm * KS, lane)) continue;      // another part's wave writes the block
        }
        const int cm0 = r_tm * BM, cn0 = c_tn * BN;
        if (p.fuse) fused_bias_act(acc, p.bias, (int64_t)cm0 + wm * 64 + ib * 16, p.act);
        const uint16_t* bias = p.fuse ? nullptr : p.bias;
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            store_block_transposed_slab<true>(acc, smem + Cfg::EPI_BASE + wave * (16 * EPI_PITCH), p.C, bias,
                                              (int64_t)cm0 + wm * 64, cn0 + wn * 64, p.rows, N, lane, !SPATHA_KNOB(2));
        } else if (!SPATHA_KNOB(4)) {
            // 16-row slabs through a wave-private LDS buffer -> 128-byte row segments
            char* stg = smem + Cfg::EPI_BASE + wave * (16 * EPI_PITCH);
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
#pragma unroll
                for (int r = 0; r < 4; r++)
#pragma unroll
                    for (int nb = 0; nb < 4; nb++)
                        *(_Float16*)(stg + (r * 4 + ib) * EPI_PITCH + (nb * 16 + j16) * 2) = (_Float16)acc[mb][nb][r];
                __builtin_amdgcn_wave_barrier();
#pragma unroll
                for (int it = 0; it < 2; it++) {
                    const int Lr = it * 8 + (lane >> 3), ch = lane & 7;
                    const int row = 16 * (Lr & 3) + 4 * mb + (Lr >> 2);
                    const int col = cn0 + wn * 64 + ch * 8;
                    u32x4 v = *(const u32x4*)(stg + Lr * EPI_PITCH + ch * 16);
                    if (col < N && !SPATHA_KNOB(2)) store_c16(p.C + ((int64_t)cm0 + wm * 64 + row) * N + col, v);
                }
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
}

template <class Cfg, int WN, int OUT_LAYOUT>
__device__ __forceinline__ void ws_consumer_deferred(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int EPI_PITCH = Cfg::EPI_PITCH;
    const int S = p.S, N = p.N;
    const int wm = wave / WN, wn = wave - wm * WN;
    float4_t acc[4][4];
    uint32_t pend[4][4][2];         // previous tile: [mb][nb][r / 2] = fp16 pair (r even | r odd << 16)
    const int li = lane & 15, kb = lane >> 4;
    const int rrow = kb * 4 + (li >> 2);
    const int sw = rrow & 7;
    int tr_off[4];
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int ch = (wn * 8 + nb * 2 + ((li & 3) >> 1)) ^ (sw << 1);
        tr_off[nb] = rrow * ROW_BYTES + ch * 16 + (li & 1) * 8;
    }
    const int a_off = B_BYTES + wm * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + wm * APACK_BLOCK + 4096 + lane * 4;
    const int j16 = lane & 15, ib = lane >> 4;
    char* stg = smem + Cfg::EPI_BASE + wave * (16 * EPI_PITCH);
    const bool stores_on = !SPATHA_KNOB(2);

    int c_tm = walk.tm0, c_tn = walk.tn0;
    int pm0 = 0, pn0 = 0;           // origin of the tile held in pend
    bool have_pend = false;
    uint32_t c_stage = 0;
    auto flush_part = [&](int part) {
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            const int64_t row0 = (int64_t)pm0 + wm * 64 + ib * 16;
            const int colb = pn0 + wn * 64 + j16;
            if (part == 0) store_block_transposed<0>(pend, p.C, row0, colb, p.rows, N, stores_on);
            else if (part == 1) store_block_transposed<1>(pend, p.C, row0, colb + 16, p.rows, N, stores_on);
            else if (part == 2) store_block_transposed<2>(pend, p.C, row0, colb + 32, p.rows, N, stores_on);
            else store_block_transposed<3>(pend, p.C, row0, colb + 48, p.rows, N, stores_on);
        } else {
            const int64_t rb = (int64_t)pm0 + wm * 64;
            const int cb = pn0 + wn * 64;
            if (part == 0) store_slab_row_major<0, EPI_PITCH>(pend, stg, p.C, rb, cb, N, lane, stores_on);
            else if (part == 1) store_slab_row_major<1, EPI_PITCH>(pend, stg, p.C, rb, cb, N, lane, stores_on);
            else if (part == 2) store_slab_row_major<2, EPI_PITCH>(pend, stg, p.C, rb, cb, N, lane, stores_on);
            else store_slab_row_major<3, EPI_PITCH>(pend, stg, p.C, rb, cb, N, lane, stores_on);
        }
    };
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < S; c_step++) {
            __syncthreads();
            if (!SPATHA_KNOB(16)) mma_stage<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc, [&]() {});
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
            if (have_pend && c_step < 4 && !SPATHA_KNOB(4)) flush_part(c_step);
        }
        // a k-loop shorter than four steps leaves parts of the previous tile unwritten
        if (have_pend && !SPATHA_KNOB(4))
            for (int part = S; part < 4; part++) flush_part(part);
        const int cm0 = c_tm * BM, cn0 = c_tn * BN;
        const bool with_bias = (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) && p.bias;
        u32x4 bias_lo = {0, 0, 0, 0}, bias_hi = {0, 0, 0, 0};
        if (with_bias) {
            const int64_t row0 = (int64_t)cm0 + wm * 64 + ib * 16;
            bias_lo = *(const u32x4*)(p.bias + row0);
            bias_hi = *(const u32x4*)(p.bias + row0 + 8);
        }
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
#pragma unroll
                for (int rp = 0; rp < 2; rp++) {
                    uint32_t w = pack_half2(acc[mb][nb][2 * rp], acc[mb][nb][2 * rp + 1]);
                    if (with_bias) {
                        const uint32_t bw = (mb < 2) ? bias_lo[mb * 2 + rp] : bias_hi[(mb - 2) * 2 + rp];
                        const half2_t sum = __builtin_bit_cast(half2_t, w) + __builtin_bit_cast(half2_t, bw);
                        w = __builtin_bit_cast(uint32_t, sum);
                    }
                    pend[mb][nb][rp] = w;
                }
        pm0 = cm0;
        pn0 = cn0;
        have_pend = true;
        walk.next(c_tm, c_tn);
    }
    if (have_pend && !SPATHA_KNOB(4))
        for (int part = 0; part < 4; part++) flush_part(part);
}

// ---- tall consumer: one wave owns a 128 x 64 tile (two stacked 64-row halves sharing the B
// fragments): 32 matrix instructions per k-step for the same 16 transposing reads, so the
// LDS and issue cost per matrix instruction drops by a third and one consumer per SIMD is enough.
#define SPATHA_MMA8(NB, BF)                                                                                     \
    _Pragma("unroll") for (int h_ = 0; h_ < 2; h_++) {                                                          \
        acc[h_][0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[h_][0], BF, acc[h_][0][NB], (int)ix[h_][0], 0, 0); \
        acc[h_][1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[h_][1], BF, acc[h_][1][NB], (int)ix[h_][0], 0, 1); \
        acc[h_][2][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[h_][2], BF, acc[h_][2][NB], (int)ix[h_][1], 0, 0); \
        acc[h_][3][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[h_][3], BF, acc[h_][3][NB], (int)ix[h_][1], 0, 1); \
    }

template <int ROW_BYTES>
__device__ __forceinline__ void mma_stage_tall(const char* st, int a_off, int i_off, const int (&tr_off)[4],
                                               float4_t (&acc)[2][4][4]) {
    half8_t a_cur[2][4];
    uint32_t ix[2][2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_cur[h][mb] = *(const half8_t*)(st + a_off + h * APACK_BLOCK + mb * 1024);
        ix[h][0] = *(const uint32_t*)(st + i_off + h * APACK_BLOCK);
        ix[h][1] = *(const uint32_t*)(st + i_off + h * APACK_BLOCK + 256);
    }
    half16_t bf0 = read_b_fragment<ROW_BYTES>(st, tr_off[0]);
    half16_t bf1 = read_b_fragment<ROW_BYTES>(st, tr_off[1]);
    __builtin_amdgcn_sched_barrier(0);
    SPATHA_MMA8(0, bf0)
    __builtin_amdgcn_sched_barrier(0);
    bf0 = read_b_fragment<ROW_BYTES>(st, tr_off[2]);
    __builtin_amdgcn_sched_barrier(0);
    SPATHA_MMA8(1, bf1)
    __builtin_amdgcn_sched_barrier(0);
    bf1 = read_b_fragment<ROW_BYTES>(st, tr_off[3]);
    __builtin_amdgcn_sched_barrier(0);
    SPATHA_MMA8(2, bf0)
    SPATHA_MMA8(3, bf1)
}

template <class Cfg, int WN, int OUT_LAYOUT>
__device__ __forceinline__ void ws_consumer_tall(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int EPI_PITCH = Cfg::EPI_PITCH;
    static_assert(BM == 128, "two stacked 64-row halves");
    const int S = p.S, N = p.N, KS = p.ksplit, SC = S / KS;
    const int wn = wave;
    float4_t acc[2][4][4];
    const int li = lane & 15, kb = lane >> 4;
    const int rrow = kb * 4 + (li >> 2);
    const int sw = rrow & 7;
    int tr_off[4];
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int ch = (wn * 8 + nb * 2 + ((li & 3) >> 1)) ^ (sw << 1);
        tr_off[nb] = rrow * ROW_BYTES + ch * 16 + (li & 1) * 8;
    }
    const int a_off = B_BYTES + lane * 16;
    const int i_off = B_BYTES + 4096 + lane * 4;
    const int j16 = lane & 15, ib = lane >> 4;
    int c_tm = walk.tm0, c_tn = walk.tn0;
    uint32_t c_stage = 0;
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) acc[h][a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < SC; c_step++) {
            __syncthreads();
            if (!SPATHA_KNOB(16)) mma_stage_tall<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc);
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        }
        const int r_tm = c_tm / KS;          // row tile (the walk's m index counts (row tile, part) pairs)
        const int cm0 = r_tm * BM, cn0 = c_tn * BN;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            if (KS > 1) {       // the wave's two 64 x 64 blocks are handed over separately: 2 * WN blocks per tile
                const int64_t slot = ((int64_t)c_tn * (walk.tiles_m / KS) + r_tm) * (2 * WN) + wave * 2 + h;
                if (!ksplit_exchange(acc[h], p, slot, c_tm - r_tm * KS, lane)) continue;
            }
            if (p.fuse) fused_bias_act(acc[h], p.bias, (int64_t)cm0 + h * 64 + ib * 16, p.act);
            if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
                if (!SPATHA_KNOB(4))
                    store_block_transposed_slab<true>(acc[h], smem + Cfg::EPI_BASE + wave * (16 * EPI_PITCH), p.C, p.fuse ? nullptr : p.bias,
                                                (int64_t)cm0 + h * 64, cn0 + wn * 64, p.rows, N, lane, !SPATHA_KNOB(2));
            } else if (!SPATHA_KNOB(4)) {
                char* stg = smem + Cfg::EPI_BASE + wave * (16 * EPI_PITCH);
#pragma unroll
                for (int mb = 0; mb < 4; mb++) {
#pragma unroll
                    for (int r = 0; r < 4; r++)
#pragma unroll
                        for (int nb = 0; nb < 4; nb++)
                            *(_Float16*)(stg + (r * 4 + ib) * EPI_PITCH + (nb * 16 + j16) * 2) = (_Float16)acc[h][mb][nb][r];
                    __builtin_amdgcn_wave_barrier();
#pragma unroll
                    for (int it = 0; it < 2; it++) {
                        const int Lr = it * 8 + (lane >> 3), ch = lane & 7;
                        const int row = 16 * (Lr & 3) + 4 * mb + (Lr >> 2);
                        const int col = cn0 + wn * 64 + ch * 8;
                        u32x4 v = *(const u32x4*)(stg + Lr * EPI_PITCH + ch * 16);
                        if (col < N && !SPATHA_KNOB(2)) store_c16(p.C + ((int64_t)cm0 + h * 64 + row) * N + col, v);
                    }
                    __builtin_amdgcn_wave_barrier();
                }
            }
        }
        walk.next(c_tm, c_tn);
    }
}

// Tile 128 x (64 * WN): WN tall consumers + NP producers.
template <int WN, int NS, int NP, int OUT_LAYOUT>
__global__ __launch_bounds__((WN + NP) * 64) void spmm_wst_kernel(SpmmParams p) {
    using Cfg = WsCfg<2, WN, NS, NP>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    if (SPATHA_SKEW_ON(p)) {
        const int units = ((blockIdx.x >> 3) & 7) * p.skew;
        for (int i = 0; i < units; i++) __builtin_amdgcn_s_sleep(16);
    }
    if (wave < WN) {
        ws_consumer_tall<Cfg, WN, OUT_LAYOUT>(p, walk, smem, wave, lane);
    } else {
        const int pr = wave - WN;
        if (pr == 0) ws_producer<Cfg, NP, 0>(p, walk, smem, smem_base, lane);
        else if (pr == 1) ws_producer<Cfg, NP, 1>(p, walk, smem, smem_base, lane);
        else if (NP > 2 && pr == 2) ws_producer<Cfg, NP, (NP > 2 ? 2 : 0)>(p, walk, smem, smem_base, lane);
        else if (NP > 2) ws_producer<Cfg, NP, (NP > 2 ? 3 : 0)>(p, walk, smem, smem_base, lane);
    }
}

template <int WN, int NS, int NP, int OUT_LAYOUT>
static hipError_t launch_wst(const SpmmParams& p, hipStream_t stream) {
    using Cfg = WsCfg<2, WN, NS, NP>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    const int cus = p.cus;        // compute units of the plan's device
    auto kern = spmm_wst_kernel<WN, NS, NP, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int per_cu = (160 * 1024) / lds;
    const int tiles = p.tiles_m * p.tiles_n;
    int grid = ((cus * per_cu) / 8) * 8;
    const int need = ((tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    if (grid < 8) grid = 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3((WN + NP) * 64), lds, stream, p);
    return hipGetLastError();
}

template <int WM, int WN, int NS, int NP, int OUT_LAYOUT, bool DEFER = false, int WALK_GROUP = 1>
__global__ __launch_bounds__((WM * WN + NP) * 64) void spmm_ws_kernel(SpmmParams p) {
    using Cfg = WsCfg<WM, WN, NS, NP>;
    static_assert(NP == 2 || NP == 4, "producer count");
    static_assert(!(DEFER && WALK_GROUP != 1), "the deferred write-out walks column-first only");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalkT<WALK_GROUP> walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    // Workgroups of one XCD start up to 7 * skew apart, so that tiles do not all finish (and
    // hit HBM with their stores) at the same moment on every CU.
    if (SPATHA_SKEW_ON(p)) {
        const int units = ((blockIdx.x >> 3) & 7) * p.skew;
        for (int i = 0; i < units; i++) __builtin_amdgcn_s_sleep(16);      // 16 * 64 clocks
    }
    if (wave < Cfg::NC) {
        if constexpr (DEFER) ws_consumer_deferred<Cfg, WN, OUT_LAYOUT>(p, walk, smem, wave, lane);
        else ws_consumer<Cfg, WN, OUT_LAYOUT>(p, walk, smem, wave, lane);
    } else {
        // the producer index is a template argument: which DMA instructions a producer issues
        // is then fixed at compile time (no branches in its loop)
        const int pr = wave - Cfg::NC;
        if (pr == 0) ws_producer<Cfg, NP, 0>(p, walk, smem, smem_base, lane);
        else if (pr == 1) ws_producer<Cfg, NP, 1>(p, walk, smem, smem_base, lane);
        else if (NP > 2 && pr == 2) ws_producer<Cfg, NP, (NP > 2 ? 2 : 0)>(p, walk, smem, smem_base, lane);
        else if (NP > 2) ws_producer<Cfg, NP, (NP > 2 ? 3 : 0)>(p, walk, smem, smem_base, lane);
    }
}

template <int WM, int WN, int NS, int NP, int OUT_LAYOUT, bool DEFER = false, int WALK_GROUP = 1>
static hipError_t launch_ws(const SpmmParams& p, hipStream_t stream) {
    using Cfg = WsCfg<WM, WN, NS, NP>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    const int cus = p.cus;        // compute units of the plan's device
    auto kern = spmm_ws_kernel<WM, WN, NS, NP, OUT_LAYOUT, DEFER, WALK_GROUP>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int per_cu = (160 * 1024) / lds;
    const int tiles = p.tiles_m * p.tiles_n;
    int grid = cus * per_cu;
    grid = (grid / 8) * 8;
    const int need = ((tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    if (grid < 8) grid = 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::THREADS), lds, stream, p);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// 128 x 128 tiles with a third role: store waves.  A consumer wave that has finished a tile rounds its 64 x 64 block to
// fp16 (bias / activation applied) and leaves it in an LDS staging buffer that holds the whole tile in output order; it then
// starts the next tile at once.  Four store waves pick the tile up behind the next step barrier - each a quarter of it, into
// registers - and write it to C in pieces after the following step barriers, so that the global stores of a tile are spread
// over the next tile's k-loop and never wait on the waves that issue the matrix instructions.  (The producers cannot
// take the stores over: stores in flight would sit in the same counter as the loads they wait for.)
//   consumer: step barriers of tile t | dump t             | step barriers of tile t + 1 | dump t + 1
//   store wave:                                             barrier 0: read t, store 1/n | barrier 1: store 2/n ...
// The staging buffer is free again when the consumers dump the next tile: the store waves have read all of it before they
// join the second step barrier, and a tile has two k-steps or more (the host refuses S = 1 for this kernel).
// ---------------------------------------------------------------------------
// (WswCfg, the LDS layout of this kernel, lives in spmm_device.h beside WsCfg: the kernel registry sizes LDS from it)

template <class Cfg, int OUT_LAYOUT>
__device__ __forceinline__ void wsw_consumer(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1, WN = Cfg::WN;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES, PITCH = Cfg::STG_PITCH;
    const int S = p.S;
    const int wm = wave / WN, wn = wave - wm * WN;
    float4_t acc[4][4];
    const int li = lane & 15, kb = lane >> 4;
    const int rrow = kb * 4 + (li >> 2);
    const int sw = rrow & 7;
    int tr_off[4];
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int ch = (wn * 8 + nb * 2 + ((li & 3) >> 1)) ^ (sw << 1);
        tr_off[nb] = rrow * ROW_BYTES + ch * 16 + (li & 1) * 8;
    }
    const int a_off = B_BYTES + wm * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + wm * APACK_BLOCK + 4096 + lane * 4;
    const int j16 = lane & 15, ib = lane >> 4;
    char* stg = smem + Cfg::EPI_BASE;
    int c_tm = walk.tm0, c_tn = walk.tn0;
    uint32_t c_stage = 0;
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < S; c_step++) {
            __syncthreads();
            mma_stage<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc, [&]() {});
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        }
        const int cm0 = c_tm * BM;
        // lane (j16, ib) holds column nb*16 + j16, rows ib*16 + mb*4 + 0..3 of the wave's block
        if (p.fuse) fused_bias_act(acc, p.bias, (int64_t)cm0 + wm * 64 + ib * 16, p.act);
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            // staging [tile column][tile row]: four consecutive rows of one column are 8 contiguous bytes.  (The bias of
            // this layout is added by the store waves: a load from global memory here would sit in the consumers' path.)
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                const int row = wm * 64 + ib * 16 + mb * 4;
#pragma unroll
                for (int nb = 0; nb < 4; nb++) {
                    half4_t h4;
#pragma unroll
                    for (int r = 0; r < 4; r++) h4[r] = (_Float16)acc[mb][nb][r];
                    *(half4_t*)(stg + (wn * 64 + nb * 16 + j16) * PITCH + row * 2) = h4;
                }
            }
        } else {
            // staging: per consumer block eight slabs of [64 block columns][8 rows] (slab 2*mb + ib/2 holds rows
            // 16*ib + 4*mb + r of the lane groups ib = 2*(ib/2), 2*(ib/2) + 1), 16 bytes per slab row: a lane's four
            // rows of one column are one 8-byte write, and a store wave gets row-major pieces back with transposing reads
            char* blk = stg + wave * 8192;
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                char* slab = blk + (mb * 2 + (ib >> 1)) * 1024;
#pragma unroll
                for (int nb = 0; nb < 4; nb++) {
                    half4_t h4;
#pragma unroll
                    for (int r = 0; r < 4; r++) h4[r] = (_Float16)acc[mb][nb][r];
                    *(half4_t*)(slab + (nb * 16 + j16) * 16 + (ib & 1) * 8) = h4;
                }
            }
        }
        walk.next(c_tm, c_tn);
    }
    __syncthreads();        // the last tile's hand-over
}

template <class Cfg, int OUT_LAYOUT>
__device__ __forceinline__ void wsw_storer(const SpmmParams& p, const TileWalk& walk, char* smem, int sw, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, PITCH = Cfg::STG_PITCH;
    const int S = p.S, N = p.N;
    const char* stg = smem + Cfg::EPI_BASE;
    // this wave's quarter of the staged tile, 8 pieces of 1 KB (16 bytes per lane).  Transposed output: BN / 4 staging rows
    // (tile columns of BM rows), a piece = RPP of them.  Row-major output: the block of consumer wave `sw`, a piece = one
    // slab = 8 rows x 128 bytes, read back row-major with transposing reads.
    constexpr int LPR = BM * 2 / 16, RPP = 64 / LPR;        // lanes per staging row, staging rows per piece
    const int srow = sw * (BN / 4) + lane / LPR, chunk = lane % LPR;
    const int li = lane & 15, kb = lane >> 4;
    const int rd_off = (8 * (2 * kb + ((li & 3) >> 1)) + (li >> 2)) * 16 + (li & 1) * 8;
    const int q_lo = 4 * ((li >> 2) & 1) + (li & 3);
    const int blk_row0 = (sw / Cfg::WN) * 64, blk_col = (sw % Cfg::WN) * 64 + 8 * (2 * kb + (li >> 3));
    const int pieces_per_step = S >= 4 ? 2 : (S == 3 ? 3 : 4);
    // (stores through asm statements: a store the compiler knows of would be waited for at the next step barrier, and every
    // wave of the workgroup with it)
    u32x4 held[8];
    int h_tm = 0, h_tn = 0, next_piece = 8;          // tile held in registers; 8 = nothing left to store
    auto load_tile = [&](int tm, int tn) {
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            // a lane's pieces are eight consecutive rows of several columns: one 16-byte piece of the bias serves them all
            // (fp16 addition on the rounded product, as everywhere)
            u32x4 b8 = {0, 0, 0, 0};
            const bool with_bias = !p.fuse && p.bias;
            if (with_bias) b8 = *(const u32x4*)(p.bias + tm * BM + chunk * 8);
#pragma unroll
            for (int i = 0; i < 8; i++) {
                u32x4 v = *(const u32x4*)(stg + (srow + RPP * i) * PITCH + chunk * 16);
                if (with_bias) v = __builtin_bit_cast(u32x4, __builtin_bit_cast(half8_t, v) + __builtin_bit_cast(half8_t, b8));
                held[i] = v;
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                const char* slab = stg + sw * 8192 + i * 1024 + rd_off;
                const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, slab));
                const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, slab + 4 * 16));
                held[i].x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
                held[i].y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
                held[i].z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
                held[i].w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
            }
        }
        h_tm = tm;
        h_tn = tn;
        next_piece = 0;
    };
    auto store_pieces = [&](int count) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (i >= next_piece && i < next_piece + count) {
                if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
                    const int col = h_tn * BN + srow + RPP * i;         // staging row = tile column
                    if (col < N) store_c16<true>(p.C + (int64_t)col * p.rows + h_tm * BM + chunk * 8, held[i]);
                } else {
                    const int q = 8 * (i & 1) + q_lo;                  // piece i: slab of mb = i / 2, lane groups 2*(i & 1), + 1
                    const int row = blk_row0 + 16 * (q >> 2) + 4 * (i >> 1) + (q & 3);
                    const int col = h_tn * BN + blk_col;
                    if (col < N) store_c16<true>(p.C + ((int64_t)h_tm * BM + row) * N + col, held[i]);
                }
            }
        }
        next_piece += count;
    };
    int c_tm = walk.tm0, c_tn = walk.tn0;
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
        for (int c_step = 0; c_step < S; c_step++) {
            __syncthreads();
            // (the tile before that one is stored by now: its pieces went out over at most four steps, and S >= 2)
            if (c_step == 0 && c_tile > 0) load_tile(h_tm, h_tn);
            if (next_piece < 8) store_pieces(pieces_per_step);
        }
        // the coordinates of the tile the consumers are about to dump
        h_tm = c_tm;
        h_tn = c_tn;
        walk.next(c_tm, c_tn);
    }
    __syncthreads();        // the last tile's hand-over
    load_tile(h_tm, h_tn);
    store_pieces(8);
}

template <int WM, int WN, int NS, int NP, int OUT_LAYOUT>
__global__ __launch_bounds__((8 + NP) * 64) void spmm_wsw_kernel(SpmmParams p) {
    using Cfg = WswCfg<WM, WN, NS, NP>;
    static_assert((NP == 2 || NP == 4) && Cfg::THREADS == (8 + NP) * 64, "wave counts");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    if (wave < Cfg::NC) {
        wsw_consumer<Cfg, OUT_LAYOUT>(p, walk, smem, wave, lane);
    } else if (wave < Cfg::NC + NP) {
        const int pr = wave - Cfg::NC;
        if (pr == 0) ws_producer<Cfg, NP, 0, true>(p, walk, smem, smem_base, lane);
        else if (pr == 1) ws_producer<Cfg, NP, 1, true>(p, walk, smem, smem_base, lane);
        else if (NP > 2 && pr == 2) ws_producer<Cfg, NP, (NP > 2 ? 2 : 0), true>(p, walk, smem, smem_base, lane);
        else if (NP > 2) ws_producer<Cfg, NP, (NP > 2 ? 3 : 0), true>(p, walk, smem, smem_base, lane);
    } else {
        wsw_storer<Cfg, OUT_LAYOUT>(p, walk, smem, wave - Cfg::NC - NP, lane);
    }
}

template <int WM, int WN, int NS, int NP, int OUT_LAYOUT>
static hipError_t launch_wsw(const SpmmParams& p, hipStream_t stream) {
    using Cfg = WswCfg<WM, WN, NS, NP>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    if (p.S < 2) return hipErrorInvalidValue;
    const int cus = p.cus;        // compute units of the plan's device
    auto kern = spmm_wsw_kernel<WM, WN, NS, NP, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = p.tiles_m * p.tiles_n;
    int grid = (cus / 8) * 8;
    const int need = ((tiles + 7) / 8) * 8;
    if (grid > need) grid = need;
    if (grid < 8) grid = 8;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(Cfg::THREADS), lds, stream, p);
    return hipGetLastError();
}

hipError_t launch_warpspec(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    const bool t = out_layout == SPATHA_OUT_TRANSPOSED;
    switch (variant) {
        case SPMM_VARIANT_W128x128_S3:
            if (p.walk_group == 0)
                return t ? launch_ws<2, 2, 3, 4, SPATHA_OUT_TRANSPOSED, false, 0>(p, stream)
                         : launch_ws<2, 2, 3, 4, SPATHA_OUT_ROW_MAJOR, false, 0>(p, stream);
            return t ? launch_ws<2, 2, 3, 4, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_ws<2, 2, 3, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_W128x256_S3:
            return t ? launch_ws<2, 4, 3, 4, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_ws<2, 4, 3, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_W64x256_S3:
            return t ? launch_ws<1, 4, 3, 2, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_ws<1, 4, 3, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_D64x256_S3:
            return t ? launch_ws<1, 4, 3, 2, SPATHA_OUT_TRANSPOSED, true>(p, stream)
                     : launch_ws<1, 4, 3, 2, SPATHA_OUT_ROW_MAJOR, true>(p, stream);
        case SPMM_VARIANT_T128x256_S3:
            return t ? launch_wst<4, 3, 4, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_wst<4, 3, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_WS128x128_S3:
            return t ? launch_wsw<2, 2, 3, 4, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_wsw<2, 2, 3, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_WS64x256_S3:
            return t ? launch_wsw<1, 4, 3, 2, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_wsw<1, 4, 3, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace spatha

