// Producer / consumer kernels on dense-staged B (m <= 8): a stage holds all 16 m dense B rows of a k-step once for
// every 64-row (or 32-row) block of the tile, and each consumer picks its rows through its read addresses.

#include "spmm_device.h"

namespace spatha {

// ---------------------------------------------------------------------------
// Dense-staged kernel for m <= 8 (tile 256 x 128 = four 64-row blocks; pays off most at V = 64).
//
// With 64-row blocks a gathered B stage serves only 64 rows of C, and the L2 -> LDS traffic
// per output element doubles.  Here the producers stage ALL 16*m dense B rows of a k-step
// (m <= 8: at most 128 rows x 256 B) once for the four V blocks of the tile, and each
// consumer picks its V block's 4-of-m rows through the ADDRESSES of its transposing reads:
// gtab holds, per (64-row block, k-step, lane class), the LDS byte offset of the row a lane has to
// read for each of its four fragments (row * 256 + swizzle), built once per matrix.
// Rows beyond K come back as zeros from the buffer range check (the producers' descriptor is the
// window of B that starts at the step's first row, so the check sees the row's true distance from
// the end of B), so padding groups (whose column offsets are 0) and tail groups need no special case.
// With four consumer waves, wave w owns rows 128*(w/2) .. +127 (two 64-row blocks) x columns
// 64*(w%2) .. +63; with eight, rows 64*(w/2) .. +63 (two waves per SIMD hide each other's LDS
// latency and barrier waits).  Producers need no row table: B rows are consecutive.
// ---------------------------------------------------------------------------

template <class Cfg, int M, int NP, int PR>
__device__ __forceinline__ void ds_producer(const SpmmParams& p, const TileWalk& walk, uint32_t smem_base, int lane) {
    constexpr int BN = Cfg::BN, NS = Cfg::PA + 1, PA = Cfg::PA;
    constexpr int B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int NB_LOADS = (4 * M) / NP;           // 4 rows per DMA instruction
    constexpr int NA_LOADS = 24 / NP;                // 4 wave-tile rows x (4 operand + 2 index blocks)
    constexpr int LOADS = NB_LOADS + NA_LOADS;
    static_assert((4 * M) % NP == 0 && 24 % NP == 0, "DMA work must split evenly over the producers");
    static_assert((PA - 1) * LOADS < 64, "vmcnt range");
    const int S = p.S, N = p.N;
    const int Q = walk.my_tiles * S;
    const i32x4 rsrc_b = make_buffer(p.B, p.b_bytes);
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const uint32_t row_bytes_b = (uint32_t)N * 2u;
    const int dense_rows = 16 * p.m;                 // rows of B one k-step spans (<= 16 * M)
    const uint32_t step_bytes_b = (uint32_t)dense_rows * row_bytes_b;
    const int slot_row = lane >> 4, slot_chunk = lane & 15;
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;

    int is_tm = walk.tm0, is_tn = walk.tn0, is_step = 0;
    uint32_t is_stage = 0, b_soff = 0;
    uint32_t a_soff = (uint32_t)((is_tm * 4) * S) * (uint32_t)APACK_BLOCK;
    int issue_left = Q;
    uint32_t voff[NB_LOADS];
    auto set_voff = [&]() {
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const int row = (PR * NB_LOADS + j) * 4 + slot_row;             // dense row inside the stage
            const int col = is_tn * BN + (slot_chunk ^ ((row & 7) << 1)) * 8;
            voff[j] = (col < N && row < dense_rows && !SPATHA_KNOB(1)) ? (uint32_t)row * row_bytes_b + (uint32_t)col * 2u
                                                                       : 0xF0000000u;
        }
    };
    set_voff();
    auto issue_batch = [&]() {
        const uint32_t stage = smem_base + is_stage;
        // the step's window of B: rows of the step that lie beyond K fail the range check and arrive as zeros
        const i32x4 rsrc_step = buffer_window(p.B, p.b_bytes, b_soff);
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) bdma_b128(voff[j], rsrc_step, 0, stage + (PR * NB_LOADS + j) * 1024);
#pragma unroll
        for (int k = 0; k < NA_LOADS; k++) {
            const int a = PR * NA_LOADS + k;
            const int awm = a / 6, ak = a - awm * 6;
            const uint32_t soff = a_soff + (uint32_t)(awm * S) * (uint32_t)APACK_BLOCK;
            const uint32_t dst = stage + B_BYTES + awm * APACK_BLOCK;
            if (ak < 4) bdma_b128(lane16, rsrc_a, soff + ak * 1024, dst + ak * 1024);
            else bdma_b32(lane4, rsrc_a, soff + 4096 + (ak - 4) * 256, dst + 4096 + (ak - 4) * 256);
        }
        --issue_left;
        is_stage = (is_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : is_stage + STAGE_BYTES;
        a_soff += (uint32_t)APACK_BLOCK;
        b_soff += step_bytes_b;
        if (++is_step == S) {
            is_step = 0;
            b_soff = 0;
            walk.next(is_tm, is_tn);
            a_soff = (uint32_t)((is_tm * 4) * S) * (uint32_t)APACK_BLOCK;
            set_voff();
        }
    };
#pragma unroll
    for (int t = 0; t < PA; t++)
        if (t < Q) issue_batch();
    const int q_main = Q - PA > 0 ? Q - PA : 0;
    // STAGE_EPI: the barrier the consumers hold after the last step of every tile, before they take that step's stage
    // for their write-out (the refill of that stage is issued after the NEXT step barrier, which they reach afterwards)
    int bar_step = 0;
    auto tile_end_barrier = [&]() {
        if (Cfg::STAGE_EPI && ++bar_step == S) {
            bar_step = 0;
            __syncthreads();
        }
    };
    for (int q = 0; q < q_main; q++) {
        wait_vmcnt<(PA - 1) * LOADS>();
        __syncthreads();
        if (!SPATHA_KNOB(8)) issue_batch();
        tile_end_barrier();
    }
    for (int q = q_main; q < Q; q++) {
        wait_stages<LOADS, PA - 1>(Q - 1 - q);
        __syncthreads();
        tile_end_barrier();
    }
}

template <class Cfg, int OUT_LAYOUT>
__device__ __forceinline__ void ds_consumer(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    const int S = p.S, N = p.N;
    constexpr int H = Cfg::H;
    const int rb0 = (wave >> 1) * H, wn = wave & 1;      // first 64-row block of this wave, column half
    float4_t acc[H][4][4];
    const int li = lane & 15, kb = lane >> 4;
    // fixed part of a transposing-read address: column chunk (wn*8 + (li%4)/2) and the 8-byte half
    const uint32_t col_xor = (uint32_t)((wn * 8 + ((li & 3) >> 1)) << 4);
    const uint32_t col_or = (uint32_t)(li & 1) * 8u;
    const int a_off = B_BYTES + rb0 * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + rb0 * APACK_BLOCK + 4096 + lane * 4;
    const int j16 = lane & 15, ib = lane >> 4;
    // gather table: [64-row block][step][kb][c = (li/4)][fb] u16 -> this lane's 8 bytes per (block, step)
    const int lane_class = kb * 4 + (li >> 2);
    auto gtab_ptr = [&](int tm, int h, int step) {
        const int64_t vb = (int64_t)tm * 4 + rb0 + h;
        return (const u32x2*)(p.gtab + ((vb * S + step) * 16 + lane_class) * 4);
    };

    int c_tm = walk.tm0, c_tn = walk.tn0;
    int n_tm = c_tm, n_tn = c_tn;       // tile of the NEXT step's table entries
    SPATHA_PROF_DECL
    uint32_t c_stage = 0, epi_stage = 0;
    u32x2 g_next[H];
    // LDS offsets of this step's four fragments (per 64-row block): computed at the end of the previous step,
    // behind its matrix instructions, so that the first reads can issue right after the barrier
    uint32_t base[H][4];
    auto set_base = [&](int h, u32x2 g) {
        base[h][0] = ((g.x & 0xffffu) ^ col_xor) | col_or;
        base[h][1] = ((g.x >> 16) ^ col_xor) | col_or;
        base[h][2] = ((g.y & 0xffffu) ^ col_xor) | col_or;
        base[h][3] = ((g.y >> 16) ^ col_xor) | col_or;
    };
#pragma unroll
    for (int h = 0; h < H; h++) set_base(h, *gtab_ptr(c_tm, h, 0));
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
#pragma unroll
        for (int h = 0; h < H; h++)
#pragma unroll
            for (int a = 0; a < 4; a++)
#pragma unroll
                for (int b = 0; b < 4; b++) acc[h][a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < S; c_step++) {
            // table entries of the next step (next tile after the last step; clamped at the very end)
            int ns = c_step + 1;
            if (ns == S) {
                ns = 0;
                if (c_tile + 1 < walk.my_tiles) walk.next(n_tm, n_tn);
            }
            if (!SPATHA_KNOB(32) || ns == 0) {      // (development knob 32: table entries only ahead of a tile's stores)
#pragma unroll
                for (int h = 0; h < H; h++) g_next[h] = *gtab_ptr(n_tm, h, ns);
            }
            SPATHA_PROF_MARK(0)
            __syncthreads();
            SPATHA_PROF_MARK(1)
            if (!SPATHA_KNOB(16)) {
                const char* st = smem + c_stage;
#pragma unroll
                for (int h = 0; h < H; h++) {
                    half8_t a_cur[4];
#pragma unroll
                    for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(st + a_off + h * APACK_BLOCK + mb * 1024);
                    const uint32_t i0 = *(const uint32_t*)(st + i_off + h * APACK_BLOCK);
                    const uint32_t i1 = *(const uint32_t*)(st + i_off + h * APACK_BLOCK + 256);
                    auto read_frag = [&](int nb) {
                        half16_t bf;
#pragma unroll
                        for (int fb = 0; fb < 4; fb++) {
                            short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, st + (base[h][fb] ^ (uint32_t)(nb << 5))));
                            half4_t h4 = __builtin_bit_cast(half4_t, t4);
                            bf[fb * 4 + 0] = h4[0];
                            bf[fb * 4 + 1] = h4[1];
                            bf[fb * 4 + 2] = h4[2];
                            bf[fb * 4 + 3] = h4[3];
                        }
                        return bf;
                    };
                    half16_t bf0 = read_frag(0);
                    half16_t bf1 = read_frag(1);
                    __builtin_amdgcn_sched_barrier(0);
#define SPATHA_MMA4H(NB, BF)                                                                                          \
    acc[h][0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], BF, acc[h][0][NB], (int)i0, 0, 0);             \
    acc[h][1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], BF, acc[h][1][NB], (int)i0, 0, 1);             \
    acc[h][2][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], BF, acc[h][2][NB], (int)i1, 0, 0);             \
    acc[h][3][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], BF, acc[h][3][NB], (int)i1, 0, 1);
                    SPATHA_MMA4H(0, bf0)
                    __builtin_amdgcn_sched_barrier(0);
                    bf0 = read_frag(2);
                    __builtin_amdgcn_sched_barrier(0);
                    SPATHA_MMA4H(1, bf1)
                    __builtin_amdgcn_sched_barrier(0);
                    bf1 = read_frag(3);
                    __builtin_amdgcn_sched_barrier(0);
                    SPATHA_MMA4H(2, bf0)
                    SPATHA_MMA4H(3, bf1)
#undef SPATHA_MMA4H
                }
            }
            epi_stage = c_stage;
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
#pragma unroll
            for (int h = 0; h < H; h++) set_base(h, g_next[h]);
        }
        const int cm0 = c_tm * BM + rb0 * 64, cn0 = c_tn * BN;
        SPATHA_PROF_MARK(0)
        if constexpr (Cfg::STAGE_EPI) {
            __syncthreads();            // every consumer is done with the last stage: it is the write-out's until the next step barrier
            SPATHA_PROF_MARK(1)
            char* stg = smem + epi_stage + wave * WAVE_EPI_BYTES;
            const bool pre = p.fuse && (p.act != SPATHA_ACT_NONE || OUT_LAYOUT == SPATHA_OUT_TRANSPOSED);
            if (pre) fused_bias_act(acc[0], p.bias, (int64_t)cm0 + ib * 16, p.act);
            if (!SPATHA_KNOB(4)) {
                if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED)
                    store_block_transposed_slab4(acc[0], stg, p.C, p.fuse ? nullptr : p.bias, (int64_t)cm0, cn0 + wn * 64, p.rows, N,
                                                 lane, !SPATHA_KNOB(2));
                else if (p.fuse && !pre && p.bias)
                    store_block_row_major_tr4<true>(acc[0], stg, p.C, (int64_t)cm0, cn0 + wn * 64, N, lane, !SPATHA_KNOB(2), p.bias);
                else
                    store_block_row_major_tr4<false>(acc[0], stg, p.C, (int64_t)cm0, cn0 + wn * 64, N, lane, !SPATHA_KNOB(2), nullptr);
            }
        } else
#pragma unroll
        for (int h = 0; h < H; h++) {
            // a bias alone rides in the row-major write-out itself (packed fp16 additions); anything else goes first
            const bool pre = p.fuse && (p.act != SPATHA_ACT_NONE || OUT_LAYOUT == SPATHA_OUT_TRANSPOSED);
            if (pre) fused_bias_act(acc[h], p.bias, (int64_t)cm0 + h * 64 + ib * 16, p.act);
            if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
                if (!SPATHA_KNOB(4))
                    store_block_transposed_slab<true>(acc[h], smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES, p.C, p.fuse ? nullptr : p.bias,
                                                (int64_t)cm0 + h * 64, cn0 + wn * 64, p.rows, N, lane, !SPATHA_KNOB(2));
            } else if (!SPATHA_KNOB(4)) {
                // two copies, so that the plain path carries nothing of the bias path
                if (p.fuse && !pre && p.bias)
                    store_block_row_major_tr<Cfg::NC == 8, Cfg::NC == 8>(acc[h], smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES, p.C,
                                                                         (int64_t)cm0 + h * 64, cn0 + wn * 64, N, lane,
                                                                         !SPATHA_KNOB(2), p.bias);
                else
                    store_block_row_major_tr<Cfg::NC == 8>(acc[h], smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES, p.C,
                                                           (int64_t)cm0 + h * 64, cn0 + wn * 64, N, lane, !SPATHA_KNOB(2), nullptr);
            }
        }
        SPATHA_PROF_MARK(2)
        walk.next(c_tm, c_tn);
    }
    SPATHA_PROF_FLUSH
}

// Accumulators in half-tile order (lane group a = lane / 16 holds, in register mb = 2h + b, tile rows 32h + 8a + 4b + r)
// -> standard order (lane group g holds, in register mb', rows 16g + 4mb' + r), so that every write-out routine
// applies: the value of (g, mb') sits in lane group 2(g % 2) + mb'/2, register 2(g / 2) + mb' % 2.  Two lane
// permutes per value (one per candidate source register), the lane's own g picks.
__device__ __forceinline__ void half_to_standard_order(float4_t (&acc)[4][4], int lane) {
    const int g = lane >> 4, j = lane & 15;
    // the permutation stays inside a column block nb: sixteen temporaries at a time
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        float out[4][4];
#pragma unroll
        for (int mbp = 0; mbp < 4; mbp++) {
            const int addr = (((2 * (g & 1) + (mbp >> 1)) << 4) | j) << 2;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float s0 = acc[mbp & 1][nb][r], s1 = acc[2 + (mbp & 1)][nb][r];
                const int v0 = __builtin_amdgcn_ds_bpermute(addr, __float_as_int(s0));
                const int v1 = __builtin_amdgcn_ds_bpermute(addr, __float_as_int(s1));
                out[mbp][r] = __int_as_float((g >> 1) ? v1 : v0);
            }
        }
#pragma unroll
        for (int mb = 0; mb < 4; mb++) acc[mb][nb] = (float4_t){out[mb][0], out[mb][1], out[mb][2], out[mb][3]};
        __builtin_amdgcn_sched_barrier(0);
    }
}

// Consumer of the dense-staged kernel for V = 32 (96, 160, ...): eight 64 x 64 waves as in ds_consumer, but a wave's
// 64 rows span two V blocks.  The operands are packed in half-tile order (see spmm_half_kernel): instructions 0, 1
// multiply a fragment gathered with the first half's table entry, instructions 2, 3 one gathered with the second's
// (gtab then has one entry per 32-row block).  The dense B stage is the same, so the fill traffic does not grow with
// the smaller V; only the consumers read twice as many fragments.
template <class Cfg, int OUT_LAYOUT>
__device__ __forceinline__ void ds_consumer_half(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    static_assert(Cfg::NC == 8, "one 64-row block per consumer wave");
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    const int S = p.S, N = p.N;
    const int rb0 = wave >> 1, wn = wave & 1;
    float4_t acc[4][4];
    const int li = lane & 15, kb = lane >> 4;
    const uint32_t col_xor = (uint32_t)((wn * 8 + ((li & 3) >> 1)) << 4);
    const uint32_t col_or = (uint32_t)(li & 1) * 8u;
    const int a_off = B_BYTES + rb0 * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + rb0 * APACK_BLOCK + 4096 + lane * 4;
    const int ib = lane >> 4;
    const int lane_class = kb * 4 + (li >> 2);
    auto gtab_ptr = [&](int tm, int half, int step) {
        const int64_t vb = ((int64_t)tm * 4 + rb0) * 2 + half;          // 32-row block
        return (const u32x2*)(p.gtab + ((vb * S + step) * 16 + lane_class) * 4);
    };
    int c_tm = walk.tm0, c_tn = walk.tn0;
    int n_tm = c_tm, n_tn = c_tn;
    uint32_t c_stage = 0;
    u32x2 g_next[2];
    uint32_t base[2][4];
    auto set_base = [&](int h, u32x2 g) {
        base[h][0] = ((g.x & 0xffffu) ^ col_xor) | col_or;
        base[h][1] = ((g.x >> 16) ^ col_xor) | col_or;
        base[h][2] = ((g.y & 0xffffu) ^ col_xor) | col_or;
        base[h][3] = ((g.y >> 16) ^ col_xor) | col_or;
    };
    set_base(0, *gtab_ptr(c_tm, 0, 0));
    set_base(1, *gtab_ptr(c_tm, 1, 0));
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < S; c_step++) {
            int ns = c_step + 1;
            if (ns == S) {
                ns = 0;
                if (c_tile + 1 < walk.my_tiles) walk.next(n_tm, n_tn);
            }
            g_next[0] = *gtab_ptr(n_tm, 0, ns);
            g_next[1] = *gtab_ptr(n_tm, 1, ns);
            __syncthreads();
            const char* st = smem + c_stage;
            half8_t a_cur[4];
#pragma unroll
            for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(st + a_off + mb * 1024);
            const uint32_t i0 = *(const uint32_t*)(st + i_off);
            const uint32_t i1 = *(const uint32_t*)(st + i_off + 256);
            auto read_frag = [&](int h, int nb) {
                half16_t bf;
#pragma unroll
                for (int fb = 0; fb < 4; fb++) {
                    short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, st + (base[h][fb] ^ (uint32_t)(nb << 5))));
                    half4_t h4 = __builtin_bit_cast(half4_t, t4);
                    bf[fb * 4 + 0] = h4[0];
                    bf[fb * 4 + 1] = h4[1];
                    bf[fb * 4 + 2] = h4[2];
                    bf[fb * 4 + 3] = h4[3];
                }
                return bf;
            };
            // three fragments in flight at most (the register budget of three waves per SIMD): the next block's first-half
            // fragment is requested before the current first-half instructions, its second-half one before the second-half ones
            half16_t lo = read_frag(0, 0), hi = read_frag(1, 0);
#define SPATHA_HALF_STEP(NB)                                    \
    {                                                           \
        half16_t lo_n, hi_n;                                    \
        __builtin_amdgcn_sched_barrier(0);                      \
        if (NB < 3) lo_n = read_frag(0, NB + 1);                \
        __builtin_amdgcn_sched_barrier(0);                      \
        SPATHA_MMA2LO(NB, lo)                                   \
        __builtin_amdgcn_sched_barrier(0);                      \
        if (NB < 3) hi_n = read_frag(1, NB + 1);                \
        __builtin_amdgcn_sched_barrier(0);                      \
        SPATHA_MMA2HI(NB, hi)                                   \
        if (NB < 3) { lo = lo_n; hi = hi_n; }                   \
    }
            SPATHA_HALF_STEP(0)
            SPATHA_HALF_STEP(1)
            SPATHA_HALF_STEP(2)
            SPATHA_HALF_STEP(3)
#undef SPATHA_HALF_STEP
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
            set_base(0, g_next[0]);
            set_base(1, g_next[1]);
        }
        const int cm0 = c_tm * BM + rb0 * 64, cn0 = c_tn * BN;
        half_to_standard_order(acc, lane);
        const bool pre = p.fuse && (p.act != SPATHA_ACT_NONE || OUT_LAYOUT == SPATHA_OUT_TRANSPOSED);
        if (pre) fused_bias_act(acc, p.bias, (int64_t)cm0 + ib * 16, p.act);
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED)
            store_block_transposed_slab<true>(acc, smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES, p.C, p.fuse ? nullptr : p.bias,
                                        (int64_t)cm0, cn0 + wn * 64, p.rows, N, lane, true);
        else
            store_block_row_major_tr<true>(acc, smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES, p.C, (int64_t)cm0, cn0 + wn * 64, N,
                                           lane, true, (p.fuse && !pre) ? p.bias : nullptr);
        walk.next(c_tm, c_tn);
    }
}

// Ping-pong consumer of the dense-staged kernel (eight 64 x 64 consumer waves, two per SIMD).
// Waves 0-3 ("early") read a stage's operands right after its barrier and multiply as the
// fragments arrive.  Waves 4-7 ("late") run one phase behind: after the barrier of step s they
// first issue the 16 matrix instructions of step s-1 from registers, re-loading each fragment's
// registers from stage s as soon as the instructions that read it are issued, and reach the
// next barrier once stage s sits in registers.  On every SIMD one wave's LDS latency is thus
// covered by the other wave's matrix work, with a single register set per wave.
template <class Cfg, int OUT_LAYOUT, bool LATE>
__device__ __forceinline__ void ds_consumer_pp(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    static_assert(Cfg::NC == 8, "ping-pong needs two consumer waves per SIMD");
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    const int S = p.S, N = p.N;
    const int rb0 = wave & 3, wn = (wave >> 2) & 1;      // 64-row block, column half (= phase group)
    float4_t acc[4][4];
    SPATHA_PROF_DECL
    const int li = lane & 15, kb = lane >> 4;
    const uint32_t col_xor = (uint32_t)((wn * 8 + ((li & 3) >> 1)) << 4);
    const uint32_t col_or = (uint32_t)(li & 1) * 8u;
    const int a_off = B_BYTES + rb0 * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + rb0 * APACK_BLOCK + 4096 + lane * 4;
    const int j16 = lane & 15, ib = lane >> 4;
    const int lane_class = kb * 4 + (li >> 2);
    auto gtab_ptr = [&](int tm, int step) {
        const int64_t vb = (int64_t)tm * 4 + rb0;
        return (const u32x2*)(p.gtab + ((vb * S + step) * 16 + lane_class) * 4);
    };
    auto zero_acc = [&]() {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
    };
    half8_t a_cur[4];
    uint32_t i0 = 0, i1 = 0;
    half16_t bf[4];
    uint32_t base[4];
    auto set_base = [&](u32x2 g) {
        base[0] = ((g.x & 0xffffu) ^ col_xor) | col_or;
        base[1] = ((g.x >> 16) ^ col_xor) | col_or;
        base[2] = ((g.y & 0xffffu) ^ col_xor) | col_or;
        base[3] = ((g.y >> 16) ^ col_xor) | col_or;
    };
    auto read_frag = [&](const char* st, int nb) {
#pragma unroll
        for (int fb = 0; fb < 4; fb++) {
            short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, st + (base[fb] ^ (uint32_t)(nb << 5))));
            half4_t h4 = __builtin_bit_cast(half4_t, t4);
            bf[nb][fb * 4 + 0] = h4[0];
            bf[nb][fb * 4 + 1] = h4[1];
            bf[nb][fb * 4 + 2] = h4[2];
            bf[nb][fb * 4 + 3] = h4[3];
        }
    };
    auto read_a = [&](const char* st) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(st + a_off + mb * 1024);
        i0 = *(const uint32_t*)(st + i_off);
        i1 = *(const uint32_t*)(st + i_off + 256);
    };
#define SPATHA_MMA4P(NB)                                                                                         \
    acc[0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], bf[NB], acc[0][NB], (int)i0, 0, 0);          \
    acc[1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], bf[NB], acc[1][NB], (int)i0, 0, 1);          \
    acc[2][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], bf[NB], acc[2][NB], (int)i1, 0, 0);          \
    acc[3][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], bf[NB], acc[3][NB], (int)i1, 0, 1);
    auto write_out = [&](int tm, int tn) {
        const int cm0 = tm * BM + rb0 * 64, cn0 = tn * BN;
        SPATHA_PROF_MARK(0)
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            const int64_t row0 = (int64_t)cm0 + ib * 16;
            half8_t bias_lo, bias_hi;
            if (p.bias) {
                bias_lo = *(const half8_t*)(p.bias + row0);
                bias_hi = *(const half8_t*)(p.bias + row0 + 8);
            }
#pragma unroll
            for (int nb = 0; nb < 4; nb++) {
                const int col = cn0 + wn * 64 + nb * 16 + j16;
                half8_t lo, hi;
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
#pragma unroll
                    for (int r = 0; r < 4; r++) {
                        lo[mb * 4 + r] = (_Float16)acc[mb][nb][r];
                        hi[mb * 4 + r] = (_Float16)acc[mb + 2][nb][r];
                    }
                if (p.bias) {
                    lo = lo + bias_lo;
                    hi = hi + bias_hi;
                }
                if (col < N && !SPATHA_KNOB(2)) {
                    uint16_t* dst = p.C + (int64_t)col * p.rows + row0;
                    *(half8_t*)dst = lo;
                    *(half8_t*)(dst + 8) = hi;
                }
            }
        } else if (!SPATHA_KNOB(4)) {
            store_block_row_major_tr<true>(acc, smem + Cfg::EPI_BASE + wave * Cfg::SLAB_BYTES, p.C, (int64_t)cm0,
                                           cn0 + wn * 64, N, lane, !SPATHA_KNOB(2));
        }
        SPATHA_PROF_MARK(2)
    };

    int c_tm = walk.tm0, c_tn = walk.tn0;
    int n_tm = c_tm, n_tn = c_tn;       // tile of the NEXT step's table entries
    int o_tm = c_tm, o_tn = c_tn;       // late waves: tile whose last step is still in registers
    uint32_t c_stage = 0;
    u32x2 g_next = *gtab_ptr(c_tm, 0);
    set_base(g_next);
    zero_acc();
    if (LATE) {
#pragma unroll
        for (int k = 0; k < 4; k++) {
            a_cur[k] = (half8_t)(_Float16)0.f;
            bf[k] = (half16_t)(_Float16)0.f;
        }
    }
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
        for (int c_step = 0; c_step < S; c_step++) {
            int ns = c_step + 1;
            if (ns == S) {
                ns = 0;
                if (c_tile + 1 < walk.my_tiles) walk.next(n_tm, n_tn);
            }
            g_next = *gtab_ptr(n_tm, ns);
            SPATHA_PROF_MARK(0)
            __syncthreads();
            SPATHA_PROF_MARK(1)
            const char* st = smem + c_stage;
            if (!LATE) {
                if (!SPATHA_KNOB(16)) {
                    read_a(st);
                    read_frag(st, 0);
                    read_frag(st, 1);
                    __builtin_amdgcn_sched_barrier(0);
                    SPATHA_MMA4P(0)
                    __builtin_amdgcn_sched_barrier(0);
                    read_frag(st, 2);
                    __builtin_amdgcn_sched_barrier(0);
                    SPATHA_MMA4P(1)
                    __builtin_amdgcn_sched_barrier(0);
                    read_frag(st, 3);
                    __builtin_amdgcn_sched_barrier(0);
                    SPATHA_MMA4P(2)
                    SPATHA_MMA4P(3)
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else if (!SPATHA_KNOB(16)) {
                // registers hold the previous step (all zeros before the first one)
                SPATHA_MMA4P(0)
                __builtin_amdgcn_sched_barrier(0);
                read_frag(st, 0);
                __builtin_amdgcn_sched_barrier(0);
                SPATHA_MMA4P(1)
                __builtin_amdgcn_sched_barrier(0);
                read_frag(st, 1);
                __builtin_amdgcn_sched_barrier(0);
                SPATHA_MMA4P(2)
                __builtin_amdgcn_sched_barrier(0);
                read_frag(st, 2);
                __builtin_amdgcn_sched_barrier(0);
                SPATHA_MMA4P(3)
                __builtin_amdgcn_sched_barrier(0);
                read_frag(st, 3);
                read_a(st);
                __builtin_amdgcn_sched_barrier(0);
                if (c_step == 0 && c_tile > 0) {
                    // that was the last step of the previous tile
                    write_out(o_tm, o_tn);
                    zero_acc();
                }
                o_tm = c_tm;
                o_tn = c_tn;
            }
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
            set_base(g_next);
        }
        if (!LATE) write_out(c_tm, c_tn), zero_acc();
        walk.next(c_tm, c_tn);
    }
    if (LATE) {
        if (!SPATHA_KNOB(16)) {
            SPATHA_MMA4P(0)
            SPATHA_MMA4P(1)
            SPATHA_MMA4P(2)
            SPATHA_MMA4P(3)
        }
        write_out(o_tm, o_tn);
    }
#undef SPATHA_MMA4P
    SPATHA_PROF_FLUSH
}

template <int M, int NS, int NP, int OUT_LAYOUT>
__global__ __launch_bounds__((8 + NP) * 64) void spmm_dspp_kernel(SpmmParams p) {
    using Cfg = DsCfg<M, NS, NP, 8>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    if (wave < 4) {
        ds_consumer_pp<Cfg, OUT_LAYOUT, false>(p, walk, smem, wave, lane);
    } else if (wave < 8) {
        ds_consumer_pp<Cfg, OUT_LAYOUT, true>(p, walk, smem, wave, lane);
    } else {
        const int pr = wave - 8;
        if (pr == 0) ds_producer<Cfg, M, NP, 0>(p, walk, smem_base, lane);
        else if (pr == 1) ds_producer<Cfg, M, NP, 1>(p, walk, smem_base, lane);
        else if (pr == 2) ds_producer<Cfg, M, NP, 2>(p, walk, smem_base, lane);
        else ds_producer<Cfg, M, NP, 3>(p, walk, smem_base, lane);
    }
}

template <int M, int NS, int NP, int NC, int OUT_LAYOUT, bool HALF = false>
__global__ __launch_bounds__((NC + NP) * 64) void spmm_ds_kernel(SpmmParams p) {
    using Cfg = DsCfg<M, NS, NP, NC, (NC == 8 && !HALF)>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    if (SPATHA_SKEW_ON(p)) {
        // workgroups of one XCD start up to 7 * skew * 1024 clocks apart (write-out bursts spread over time)
        const int units = ((blockIdx.x >> 3) & 7) * p.skew;
        for (int i = 0; i < units; i++) __builtin_amdgcn_s_sleep(16);
    }
    if (wave < NC) {
        if constexpr (HALF) ds_consumer_half<Cfg, OUT_LAYOUT>(p, walk, smem, wave, lane);
        else ds_consumer<Cfg, OUT_LAYOUT>(p, walk, smem, wave, lane);
    } else {
        const int pr = wave - NC;
        if (pr == 0) ds_producer<Cfg, M, NP, 0>(p, walk, smem_base, lane);
        else if (pr == 1) ds_producer<Cfg, M, NP, 1>(p, walk, smem_base, lane);
        else if (pr == 2) ds_producer<Cfg, M, NP, 2>(p, walk, smem_base, lane);
        else ds_producer<Cfg, M, NP, 3>(p, walk, smem_base, lane);
    }
}

template <int M, int NS, int NP, int NC, int OUT_LAYOUT, bool PINGPONG = false, bool HALF = false>
static hipError_t launch_ds(const SpmmParams& p, hipStream_t stream) {
    using Cfg = DsCfg<M, NS, NP, NC>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    static_assert(!PINGPONG || NC == 8, "ping-pong needs eight consumer waves");
    const int cus = p.cus;        // compute units of the plan's device
    void (*kern)(SpmmParams);
    if constexpr (PINGPONG) kern = spmm_dspp_kernel<M, NS, NP, OUT_LAYOUT>;
    else kern = spmm_ds_kernel<M, NS, NP, NC, OUT_LAYOUT, HALF>;
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

hipError_t launch_densestage(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    const bool t = out_layout == SPATHA_OUT_TRANSPOSED;
    switch (variant) {
        case SPMM_VARIANT_DS256x128_S3_C8:
            return t ? launch_ds<8, 3, 4, 8, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_ds<8, 3, 4, 8, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_DS256x128_S3_PP:
            return t ? launch_ds<8, 3, 4, 8, SPATHA_OUT_TRANSPOSED, true>(p, stream)
                     : launch_ds<8, 3, 4, 8, SPATHA_OUT_ROW_MAJOR, true>(p, stream);
        case SPMM_VARIANT_DSH256x128_S3_C8:
            return t ? launch_ds<8, 3, 4, 8, SPATHA_OUT_TRANSPOSED, false, true>(p, stream)
                     : launch_ds<8, 3, 4, 8, SPATHA_OUT_ROW_MAJOR, false, true>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace spatha

