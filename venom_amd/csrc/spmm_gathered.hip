// Kernels that gather the B rows of each V-row block into their LDS stages (any m): the register-staged first
// kernel, the global -> LDS DMA pipeline, its half-tile form for V = 32, 96, ... and the persistent pipeline.

#include "spmm_device.h"

namespace spatha {

// ---------------------------------------------------------------------------
// Main SpMM kernel.  Workgroup = WM x WN waves, each owning a 64 x 64 tile of C.
// ---------------------------------------------------------------------------
template <int WM, int WN, int OUT_LAYOUT>
__global__ __launch_bounds__(WM* WN * 64) void spmm_kernel(SpmmParams p) {
    constexpr int NT = WM * WN * 64;
    constexpr int BM = WM * 64, BN = WN * 64;
    constexpr int PITCH_B = BN * 2 + 32;             // bytes per gathered-B row in LDS
    constexpr int STAGE_B = 64 * PITCH_B;
    constexpr int CHUNKS_PER_ROW = BN / 8;           // 16-byte chunks
    constexpr int B_LOADS = 64 * CHUNKS_PER_ROW / NT;  // per thread per step
    constexpr int ROWS_PER_PASS = NT / CHUNKS_PER_ROW;
    static_assert(64 * CHUNKS_PER_ROW % NT == 0, "tile/threads");
    constexpr int PITCH_C = 144;                      // bytes per staged C row (64 halfs + pad)

    extern __shared__ __attribute__((aligned(16))) char smem[];

    // --- tile assignment: workgroups that are resident on one XCD (id % 8) walk the
    //     m-tiles of the same B column panel, so the panel is read from that XCD's L2.
    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) >> 3;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int tile = xcd * chunk + local;
    if (local >= chunk || tile >= tiles) return;
    const int tile_n = tile / p.tiles_m, tile_m = tile - tile_n * p.tiles_m;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WN, wn = wave - wm * WN;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int S = p.S, N = p.N;

    const int64_t wt = (int64_t)(m0 / 64 + wm);                       // wave tile index along rows
    const char* a_blk = (const char*)p.apack + ((int64_t)wt * S) * APACK_BLOCK;   // + s*APACK_BLOCK
    const uint32_t* rt = p.rowtab + (int64_t)(m0 / p.v) * S * 64;

    // B loader coordinates
    const int bc = tid % CHUNKS_PER_ROW;            // 16-byte chunk inside the row
    const int br = tid / CHUNKS_PER_ROW;            // first LDS row handled
    const int bcol = n0 + bc * 8;
    const bool bcol_ok = bcol < N;
    const uint16_t* bbase = p.B + bcol;

    u32x4 breg[B_LOADS];
    u32x4 areg[4];
    u32x2 ireg;
    uint32_t rows_next[B_LOADS];

    auto load_rows = [&](int s) {
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) rows_next[i] = rt[s * 64 + br + i * ROWS_PER_PASS];
    };
    auto load_global = [&](int s) {
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) {
            uint32_t row = rows_next[i];
            u32x4 z = {0u, 0u, 0u, 0u};
            breg[i] = (row != 0xffffffffu && bcol_ok && !SPATHA_KNOB(1)) ? *(const u32x4*)(bbase + (int64_t)row * N) : z;
        }
#pragma unroll
        for (int mb = 0; mb < 4; mb++) areg[mb] = *(const u32x4*)(a_blk + (int64_t)s * APACK_BLOCK + mb * 1024 + lane * 16);
        ireg.x = *(const uint32_t*)(a_blk + (int64_t)s * APACK_BLOCK + 4096 + lane * 4);
        ireg.y = *(const uint32_t*)(a_blk + (int64_t)s * APACK_BLOCK + 4096 + 256 + lane * 4);
    };
    auto store_lds = [&](int stage) {
        char* base = smem + stage * STAGE_B + br * PITCH_B + bc * 16;
#pragma unroll
        for (int i = 0; i < B_LOADS; i++) *(u32x4*)(base + i * ROWS_PER_PASS * PITCH_B) = breg[i];
    };

    float4_t acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

    // transposing-read address of this lane: block kb = lane/16 reads rows fb*16 + kb*4 + (i/4),
    // columns wn*64 + nb*16 + 4*(i%4)
    const int li = lane & 15, kb = lane >> 4;
    const int tr_off = (kb * 4 + (li >> 2)) * PITCH_B + (wn * 64 + (li & 3) * 4) * 2;

    load_rows(0);
    load_global(0);
    if (S > 1) load_rows(1);
    store_lds(0);
    half8_t a_cur[4];
    uint32_t i_cur[2];
#pragma unroll
    for (int mb = 0; mb < 4; mb++) a_cur[mb] = __builtin_bit_cast(half8_t, areg[mb]);
    i_cur[0] = ireg.x;
    i_cur[1] = ireg.y;
    __syncthreads();

    for (int s = 0; s < S; s++) {
        const bool more = (s + 1) < S;
        if (more) {
            load_global(s + 1);
            if (s + 2 < S) load_rows(s + 2);
        }
        const char* bst = smem + (s & 1) * STAGE_B + tr_off;
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            half16_t bf;
#pragma unroll
            for (int fb = 0; fb < 4; fb++) {
                short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, bst + fb * 16 * PITCH_B + nb * 32));
                half4_t h4 = __builtin_bit_cast(half4_t, t4);
                bf[fb * 4 + 0] = h4[0];
                bf[fb * 4 + 1] = h4[1];
                bf[fb * 4 + 2] = h4[2];
                bf[fb * 4 + 3] = h4[3];
            }
            acc[0][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], bf, acc[0][nb], (int)i_cur[0], 0, 0);
            acc[1][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], bf, acc[1][nb], (int)i_cur[0], 0, 1);
            acc[2][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], bf, acc[2][nb], (int)i_cur[1], 0, 0);
            acc[3][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], bf, acc[3][nb], (int)i_cur[1], 0, 1);
        }
        if (more) {
            store_lds((s + 1) & 1);
#pragma unroll
            for (int mb = 0; mb < 4; mb++) a_cur[mb] = __builtin_bit_cast(half8_t, areg[mb]);
            i_cur[0] = ireg.x;
            i_cur[1] = ireg.y;
        }
        __syncthreads();
    }

    // ------------------------------------------------------------------ epilogue
    const int j = lane & 15, ib = lane >> 4;
    if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
        // lane holds, per nb, 16 consecutive matrix rows (16*ib + 0..15) of column 16*nb + j
        const int64_t row0 = (int64_t)m0 + wm * 64 + ib * 16;
        half8_t bias_lo, bias_hi;
        if (p.bias) {
            bias_lo = *(const half8_t*)(p.bias + row0);
            bias_hi = *(const half8_t*)(p.bias + row0 + 8);
        }
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            const int col = n0 + wn * 64 + nb * 16 + j;
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
            if (col < N) {
                uint16_t* dst = p.C + (int64_t)col * p.rows + row0;
                *(half8_t*)dst = lo;
                *(half8_t*)(dst + 8) = hi;
            }
        }
    } else {
        // stage the wave's 64 x 64 tile in LDS (rows reordered so that the four lane blocks
        // write to disjoint banks), then write 128-byte row segments
        char* st = smem + wave * (64 * PITCH_C);
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int L = (4 * mb + r) * 4 + ib;
#pragma unroll
                for (int nb = 0; nb < 4; nb++)
                    *(_Float16*)(st + L * PITCH_C + (nb * 16 + j) * 2) = (_Float16)acc[mb][nb][r];
            }
        // wave-private staging: no workgroup barrier needed, only the wave's own LDS writes
        __builtin_amdgcn_s_waitcnt(0xc07f);   // lgkmcnt(0)
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int L = it * 8 + (lane >> 3), ch = lane & 7;
            const int row = 16 * (L & 3) + (L >> 2);
            const int col = n0 + wn * 64 + ch * 8;
            u32x4 v = *(const u32x4*)(st + L * PITCH_C + ch * 16);
            if (col < N && !SPATHA_KNOB(2)) store_c16(p.C + ((int64_t)m0 + wm * 64 + row) * N + col, v);
        }
    }
}

// ---------------------------------------------------------------------------
// Pipelined SpMM kernel.  Everything the k-loop consumes -- the gathered B rows, the packed
// A operands and their index words -- is copied global -> LDS by the DMA path
// (global_load_lds_dwordx4 / _dword: no VGPR staging, no LDS store instructions) NS-1
// k-steps ahead of the step being multiplied.  One workgroup barrier per k-step.
//
// The DMA loads are issued from inline assembly on purpose: the compiler's wait-count
// insertion treats every LDS read as a possible alias of every outstanding LDS-DMA write and
// would drain the whole queue (vmcnt(0)) before the first read of each step, which removes
// the overlap this kernel exists for.  No other vector-memory instruction is issued inside
// the loop, so the explicit s_waitcnt vmcnt(k) below is the only bookkeeping: a wave issues
// exactly LOADS_PER_STAGE DMA instructions per stage, in stage order.  The asm statements carry
// no "memory" clobber (it would stop the compiler from reading the row table with scalar
// loads); they are volatile, so they keep their order relative to each other and to the
// workgroup barrier, which is what separates a stage's DMA writes from its LDS reads.
//
// LDS layout of one stage:
//   [0, 64*BN*2)                gathered B rows, row pitch BN*2 bytes (a DMA instruction writes
//                               1 KiB contiguous, so rows cannot be padded); bank conflicts of
//                               the transposing reads are avoided by XOR-ing the 16-byte chunk
//                               index of row rho with 2*(rho % 8) on the GLOBAL side of the copy
//   [.., + WM*APACK_BLOCK)      per 64-row wave tile: 4 KiB A operands + 512 B index words
// ---------------------------------------------------------------------------

template <int WM, int WN, int NS, int OUT_LAYOUT>
__global__ __launch_bounds__(WM* WN * 64) void spmm_pipe_kernel(SpmmParams p) {
    constexpr int NW = WM * WN;
    constexpr int BM = WM * 64, BN = WN * 64;
    constexpr int ROW_BYTES = BN * 2;
    constexpr int B_BYTES = 64 * ROW_BYTES;
    constexpr int STAGE_BYTES = B_BYTES + WM * APACK_BLOCK;
    constexpr int CHUNKS = BN / 8;                   // 16-byte chunks per row
    constexpr int ROWS_PER_INST = 1024 / ROW_BYTES;  // rows one DMA instruction covers (4 or 2)
    constexpr int NB_LOADS = 64 / ROWS_PER_INST / NW;  // B DMA instructions per wave per stage
    constexpr int NA_X4 = 4 / WN > 0 ? 4 / WN : 1;   // A-operand DMA instructions per wave per stage
    constexpr int LOADS_PER_STAGE = NB_LOADS + NA_X4 + 1;
    constexpr int PA = NS - 1;                       // prefetch distance in k-steps
    constexpr int PITCH_C = 144;
    static_assert(WN == 1 || WN == 2 || WN == 4, "A operand split");
    static_assert(64 % (ROWS_PER_INST * NW) == 0, "rows per step must split over the waves");
    static_assert((NS - 2) * LOADS_PER_STAGE < 64, "vmcnt range");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    uint32_t* lds_rt = (uint32_t*)(smem + NS * STAGE_BYTES);      // row table of this V block: S*64 words

    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) >> 3;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int tile = xcd * chunk + local;
    if (local >= chunk || tile >= tiles) return;
    const int tile_n = tile / p.tiles_m, tile_m = tile - tile_n * p.tiles_m;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave - wm * WN;
    const int m0 = tile_m * BM, n0 = tile_n * BN;
    const int S = p.S, N = p.N;

    const char* a_src = (const char*)p.apack + ((int64_t)(m0 / 64 + wm) * S) * APACK_BLOCK;
    const uint32_t* rt = p.rowtab + (int64_t)(m0 / p.v) * S * 64;

    // ---- B loader: this lane's slot in each of the wave's NB_LOADS instructions
    const int slot_row = lane / CHUNKS;
    const int slot_chunk = lane % CHUNKS;
    int64_t b_col_off[NB_LOADS];                     // byte offset of the source chunk inside a B row, or -1
    const char* zero_src = (const char*)p.zeros + lane * 16;
#pragma unroll
    for (int j = 0; j < NB_LOADS; j++) {
        const int rho = (wave * NB_LOADS + j) * ROWS_PER_INST + slot_row;
        const int src_chunk = slot_chunk ^ ((rho & 7) << 1);
        const int col = n0 + src_chunk * 8;
        b_col_off[j] = (col < N) ? (int64_t)col * 2 : -1;
    }
    auto issue_stage = [&](int s) {
        const uint32_t stage = smem_base + (s % NS) * STAGE_BYTES;
        uint32_t rows[NB_LOADS];
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) rows[j] = lds_rt[s * 64 + (wave * NB_LOADS + j) * ROWS_PER_INST + slot_row];
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const int inst = wave * NB_LOADS + j;
            const bool ok = (rows[j] != 0xffffffffu) && (b_col_off[j] >= 0) && !SPATHA_KNOB(1);
            const char* src = (const char*)p.B + (int64_t)rows[j] * N * 2 + b_col_off[j];
            src = ok ? src : zero_src;
            dma_b128(src, stage + inst * 1024);
        }
        // A operands of wave tile wm: the WN waves of the row split the 4 operand blocks; the
        // two index blocks go to waves with even / odd wn (duplicates write identical bytes)
        const char* ab = a_src + (int64_t)s * APACK_BLOCK;
        const uint32_t a_lds = stage + B_BYTES + wm * APACK_BLOCK;
#pragma unroll
        for (int k = 0; k < NA_X4; k++) {
            const int mb = (WN >= 4) ? wn : wn * NA_X4 + k;
            dma_b128(ab + mb * 1024 + lane * 16, a_lds + mb * 1024);
        }
        const int d = wn & 1;
        dma_b32(ab + 4096 + d * 256 + lane * 4, a_lds + 4096 + d * 256);
        if (WN == 1) dma_b32(ab + 4096 + 256 + lane * 4, a_lds + 4096 + 256);
    };
    constexpr int L = LOADS_PER_STAGE + (WN == 1 ? 1 : 0);

    float4_t acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

    // transposing-read offsets: row fb*16 + kb*4 + i/4; 16-byte chunk (wn*8 + nb*2 + (i%4)/2) ^ swizzle
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

    // ---- the V-block's row table goes to LDS once (ordinary loads, before any DMA is in flight:
    //      a vector load inside the loop would make the compiler drain the DMA queue)
    for (int i = tid; i < S * 64; i += NW * 64) lds_rt[i] = rt[i];
    __syncthreads();

    // ---- prologue: NS-1 stages in flight
#pragma unroll
    for (int t = 0; t < PA; t++)
        if (t < S) issue_stage(t);

    for (int s = 0; s < S; s++) {
        // stages after s that this wave has already issued may stay in flight
        const int later = (S - 1 - s) < (NS - 2) ? (S - 1 - s) : (NS - 2);
        wait_stages<L, NS - 2>(later);
        __syncthreads();          // stage s is complete for every wave; stage s-1 is no longer read
        mma_stage<ROW_BYTES>(smem + (s % NS) * STAGE_BYTES, a_off, i_off, tr_off, acc, [&]() {
            if (s + PA < S) issue_stage(s + PA);
        });
    }

    // ------------------------------------------------------------------ epilogue
    const int j = lane & 15, ib = lane >> 4;
    if (p.fuse) fused_bias_act(acc, p.bias, (int64_t)m0 + wm * 64 + ib * 16, p.act);
    const uint16_t* bias = p.fuse ? nullptr : p.bias;
    if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
        __syncthreads();                 // every wave is done reading the stages: their memory becomes the slabs
        store_block_transposed_slab<true>(acc, smem + wave * TT_SLAB_BYTES, p.C, bias, (int64_t)m0 + wm * 64, n0 + wn * 64,
                                          p.rows, N, lane, true);
    } else if (!SPATHA_KNOB(4)) {
        __syncthreads();                 // every wave is done reading the stages
        char* stg = smem + wave * (64 * PITCH_C);
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int Lr = (4 * mb + r) * 4 + ib;
#pragma unroll
                for (int nb = 0; nb < 4; nb++)
                    *(_Float16*)(stg + Lr * PITCH_C + (nb * 16 + j) * 2) = (_Float16)acc[mb][nb][r];
            }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int Lr = it * 8 + (lane >> 3), ch = lane & 7;
            const int row = 16 * (Lr & 3) + (Lr >> 2);
            const int col = n0 + wn * 64 + ch * 8;
            u32x4 v = *(const u32x4*)(stg + Lr * PITCH_C + ch * 16);
            // (256-wide tiles: written through, 0-13 % faster on the BERT-large / GPT-2-large layer shapes; the 128-wide ones lose)
            if (col < N && !SPATHA_KNOB(2)) store_c16<(WN >= 4)>(p.C + ((int64_t)m0 + wm * 64 + row) * N + col, v);
        }
    }
}

template <int WM, int WN, int NS, int OUT_LAYOUT>
static hipError_t launch_pipe(const SpmmParams& p, hipStream_t stream) {
    constexpr int BN = WN * 64;
    constexpr int stage_bytes = NS * (64 * BN * 2 + WM * APACK_BLOCK);
    static_assert(stage_bytes >= WM * WN * 64 * 144, "the epilogue staging reuses the stage buffers");
    const int lds = stage_bytes + p.S * 256;
    if (lds > 160 * 1024) return hipErrorInvalidValue;     // callers check with spmm_variant_fits first
    auto kern = spmm_pipe_kernel<WM, WN, NS, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) / 8;
    hipLaunchKernelGGL(kern, dim3(chunk * 8), dim3(WM * WN * 64), lds, stream, p);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Pipelined kernel for V = 32 (any V that is a multiple of 32 but not of 64).
//
// A 64-row wave tile then spans two V blocks, each with its own column-loc, so a stage holds TWO
// gathered sets of 64 B rows and the packed operands use the "half tile" row order: instruction
// row (mb, 4*ib + r) holds tile row 32*(mb/2) + 8*ib + 4*(mb%2) + r, so that instructions 0, 1
// multiply the first set and instructions 2, 3 the second.  A lane ends up with two runs of 8
// consecutive matrix rows (8*ib .. +7 and 32 + 8*ib .. +7) of one output column.
// The row tables of the tile's two halves sit in LDS as 16-bit row numbers (0xffff = zero row).
// Tile 64 x (64*WN), one wave per 64 columns; everything else as in spmm_pipe_kernel.
// ---------------------------------------------------------------------------
// Fused epilogue (t = fp16(acc) + bias[row], then the activation in fp32) for the half-tile operand order: the lane's
// values of instruction mb are tile rows 32*(mb/2) + 8*ib + 4*(mb%2) + r.  `hi_rows` is false for the padded second half
// of a last tile (rows % 64 == 32), whose bias entries do not exist.
template <int ACT>
__device__ __forceinline__ void fused_bias_act_half_impl(float4_t (&acc)[4][4], const uint16_t* bias, int64_t m0, int ib,
                                                         bool hi_rows) {
#pragma unroll
    for (int mb = 0; mb < 4; mb++) {
        half4_t bv = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
        if (bias && (mb < 2 || hi_rows)) bv = *(const half4_t*)(bias + m0 + 32 * (mb >> 1) + 8 * ib + 4 * (mb & 1));
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            float4_t v = acc[mb][nb];
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const float t = (float)((_Float16)v[r] + bv[r]);
                v[r] = ACT == SPATHA_ACT_GELU ? act_gelu_erf(t) : ACT == SPATHA_ACT_GELU_TANH ? act_gelu_tanh(t) : t;
            }
            acc[mb][nb] = v;
            if (ACT != SPATHA_ACT_NONE) __builtin_amdgcn_sched_barrier(0);
        }
    }
}
__device__ __forceinline__ void fused_bias_act_half(float4_t (&acc)[4][4], const uint16_t* bias, int64_t m0, int ib, bool hi_rows,
                                                    int act) {
    if (act == SPATHA_ACT_GELU) fused_bias_act_half_impl<SPATHA_ACT_GELU>(acc, bias, m0, ib, hi_rows);
    else if (act == SPATHA_ACT_GELU_TANH) fused_bias_act_half_impl<SPATHA_ACT_GELU_TANH>(acc, bias, m0, ib, hi_rows);
    else fused_bias_act_half_impl<SPATHA_ACT_NONE>(acc, bias, m0, ib, hi_rows);
}

template <int WN, int NS, int OUT_LAYOUT>
__global__ __launch_bounds__(WN * 64) void spmm_half_kernel(SpmmParams p) {
    constexpr int BN = WN * 64;
    constexpr int ROW_BYTES = BN * 2;
    constexpr int B_BYTES = 64 * ROW_BYTES;          // one gathered set
    constexpr int STAGE_BYTES = 2 * B_BYTES + APACK_BLOCK;
    constexpr int CHUNKS = BN / 8;
    constexpr int RPI = 1024 / ROW_BYTES;            // rows one DMA instruction covers
    constexpr int NB_LOADS = 128 / RPI / WN;         // B DMA instructions per wave per stage (both sets)
    constexpr int NA_X4 = 4 / WN;
    constexpr int L = NB_LOADS + NA_X4 + 1;
    constexpr int PA = NS - 1;
    constexpr int PITCH_C = 144;
    static_assert(WN == 2 || WN == 4, "A operand split");
    static_assert((NS - 2) * L < 64, "vmcnt range");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    uint16_t* lds_rt = (uint16_t*)(smem + NS * STAGE_BYTES);      // [S][2 halves][64] row numbers

    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) >> 3;
    const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3;
    const int tile = xcd * chunk + local;
    if (local >= chunk || tile >= tiles) return;
    const int tile_n = tile / p.tiles_m, tile_m = tile - tile_n * p.tiles_m;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wn = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m0 = tile_m * 64, n0 = tile_n * BN;
    const int S = p.S, N = p.N;
    const char* a_src = (const char*)p.apack + ((int64_t)tile_m * S) * APACK_BLOCK;

    const int slot_row = lane / CHUNKS;
    const int slot_chunk = lane % CHUNKS;
    int64_t b_col_off[NB_LOADS];
    const char* zero_src = (const char*)p.zeros + lane * 16;
#pragma unroll
    for (int j = 0; j < NB_LOADS; j++) {
        const int rho = (wn * NB_LOADS + j) * RPI + slot_row;          // 0..127; the swizzle only sees rho % 8
        const int src_chunk = slot_chunk ^ ((rho & 7) << 1);
        const int col = n0 + src_chunk * 8;
        b_col_off[j] = (col < N) ? (int64_t)col * 2 : -1;
    }
    auto issue_stage = [&](int s) {
        const uint32_t stage = smem_base + (s % NS) * STAGE_BYTES;
        uint32_t rows[NB_LOADS];
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) rows[j] = lds_rt[s * 128 + (wn * NB_LOADS + j) * RPI + slot_row];
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const int inst = wn * NB_LOADS + j;
            const bool ok = (rows[j] != 0xffffu) && (b_col_off[j] >= 0);
            const char* src = (const char*)p.B + (int64_t)rows[j] * N * 2 + b_col_off[j];
            src = ok ? src : zero_src;
            dma_b128(src, stage + inst * 1024);                        // set 1 starts at B_BYTES = 64 rows
        }
        const char* ab = a_src + (int64_t)s * APACK_BLOCK;
        const uint32_t a_lds = stage + 2 * B_BYTES;
#pragma unroll
        for (int k = 0; k < NA_X4; k++) {
            const int mb = (WN >= 4) ? wn : wn * NA_X4 + k;
            dma_b128(ab + mb * 1024 + lane * 16, a_lds + mb * 1024);
        }
        const int d = wn & 1;
        dma_b32(ab + 4096 + d * 256 + lane * 4, a_lds + 4096 + d * 256);
    };

    float4_t acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

    const int li = lane & 15, kb = lane >> 4;
    const int rrow = kb * 4 + (li >> 2);
    const int sw = rrow & 7;
    int tr_off[4];
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        const int ch = (wn * 8 + nb * 2 + ((li & 3) >> 1)) ^ (sw << 1);
        tr_off[nb] = rrow * ROW_BYTES + ch * 16 + (li & 1) * 8;
    }
    const int a_off = 2 * B_BYTES + lane * 16;
    const int i_off = 2 * B_BYTES + 4096 + lane * 4;

    // ---- row tables of the two halves -> LDS (ordinary loads, before any DMA is in flight)
    {
        const uint32_t* rt0 = p.rowtab + (int64_t)(m0 / p.v) * S * 64;
        const uint32_t* rt1 = p.rowtab + (int64_t)((m0 + 32) / p.v) * S * 64;
        const bool second_half = m0 + 32 < p.rows;      // rows % 64 == 32: the last tile's second half is padding
        for (int i = tid; i < S * 128; i += WN * 64) {
            const int s = i >> 7, rho = i & 63;
            const uint32_t r = (i & 64) ? (second_half ? rt1[s * 64 + rho] : 0xffffffffu) : rt0[s * 64 + rho];
            lds_rt[i] = (r == 0xffffffffu) ? (uint16_t)0xffffu : (uint16_t)r;
        }
    }
    __syncthreads();

#pragma unroll
    for (int t = 0; t < PA; t++)
        if (t < S) issue_stage(t);

    for (int s = 0; s < S; s++) {
        const int later = (S - 1 - s) < (NS - 2) ? (S - 1 - s) : (NS - 2);
        wait_stages<L, NS - 2>(later);
        __syncthreads();
        const char* st = smem + (s % NS) * STAGE_BYTES;
        half8_t a_cur[4];
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(st + a_off + mb * 1024);
        const uint32_t i0 = *(const uint32_t*)(st + i_off), i1 = *(const uint32_t*)(st + i_off + 256);
        half16_t lo0 = read_b_fragment<ROW_BYTES>(st, tr_off[0]);
        half16_t hi0 = read_b_fragment<ROW_BYTES>(st + B_BYTES, tr_off[0]);
        half16_t lo1 = read_b_fragment<ROW_BYTES>(st, tr_off[1]);
        half16_t hi1 = read_b_fragment<ROW_BYTES>(st + B_BYTES, tr_off[1]);
        __builtin_amdgcn_sched_barrier(0);
        if (s + PA < S) issue_stage(s + PA);
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA2LO(0, lo0)
        SPATHA_MMA2HI(0, hi0)
        __builtin_amdgcn_sched_barrier(0);
        lo0 = read_b_fragment<ROW_BYTES>(st, tr_off[2]);
        hi0 = read_b_fragment<ROW_BYTES>(st + B_BYTES, tr_off[2]);
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA2LO(1, lo1)
        SPATHA_MMA2HI(1, hi1)
        __builtin_amdgcn_sched_barrier(0);
        lo1 = read_b_fragment<ROW_BYTES>(st, tr_off[3]);
        hi1 = read_b_fragment<ROW_BYTES>(st + B_BYTES, tr_off[3]);
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA2LO(2, lo0)
        SPATHA_MMA2HI(2, hi0)
        SPATHA_MMA2LO(3, lo1)
        SPATHA_MMA2HI(3, hi1)
    }

    // ------------------------------------------------------------------ write-out
    const int j = lane & 15, ib = lane >> 4;
    const bool hi_rows = m0 + 32 < p.rows;
    if (p.fuse) fused_bias_act_half(acc, p.bias, m0, ib, hi_rows, p.act);
    const uint16_t* bias = p.fuse ? nullptr : p.bias;         // the plain transposed write-out adds the bias itself
    if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
        // per output column the lane holds rows 8*ib .. +7 (instructions 0, 1) and 32 + 8*ib .. +7 (2, 3)
        const int64_t row_lo = (int64_t)m0 + ib * 8, row_hi = row_lo + 32;
        half8_t bias_lo, bias_hi = {};
        if (bias) {
            bias_lo = *(const half8_t*)(bias + row_lo);
            if (hi_rows) bias_hi = *(const half8_t*)(bias + row_hi);
        }
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            const int col = n0 + wn * 64 + nb * 16 + j;
            half8_t lo, hi;
#pragma unroll
            for (int mb = 0; mb < 2; mb++)
#pragma unroll
                for (int r = 0; r < 4; r++) {
                    lo[mb * 4 + r] = (_Float16)acc[mb][nb][r];
                    hi[mb * 4 + r] = (_Float16)acc[mb + 2][nb][r];
                }
            if (bias) {
                lo = lo + bias_lo;
                hi = hi + bias_hi;
            }
            if (col < N) {
                uint16_t* dst = p.C + (int64_t)col * p.rows;
                *(half8_t*)(dst + row_lo) = lo;
                if (hi_rows) *(half8_t*)(dst + row_hi) = hi;
            }
        }
    } else {
        __syncthreads();                 // every wave is done reading the stages
        char* stg = smem + wn * (64 * PITCH_C);
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
                const int Lr = (4 * mb + r) * 4 + ib;
#pragma unroll
                for (int nb = 0; nb < 4; nb++)
                    *(_Float16*)(stg + Lr * PITCH_C + (nb * 16 + j) * 2) = (_Float16)acc[mb][nb][r];
            }
        __builtin_amdgcn_s_waitcnt(0xc07f);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < 8; it++) {
            const int Lr = it * 8 + (lane >> 3), ch = lane & 7;
            // slab row Lr = (4*mb + r)*4 + ib  ->  tile row 32*(mb/2) + 8*ib + 4*(mb%2) + r
            const int row = 32 * (Lr >> 5) + 8 * (Lr & 3) + 4 * ((Lr >> 4) & 1) + ((Lr >> 2) & 3);
            const int col = n0 + wn * 64 + ch * 8;
            u32x4 v = *(const u32x4*)(stg + Lr * PITCH_C + ch * 16);
            if (col < N && m0 + row < p.rows) store_c16(p.C + ((int64_t)m0 + row) * N + col, v);
        }
    }
}

template <int WN, int NS, int OUT_LAYOUT>
static hipError_t launch_half(const SpmmParams& p, hipStream_t stream) {
    constexpr int stage_bytes = half_stage_bytes<WN, NS>();
    static_assert(stage_bytes >= WN * 64 * 144, "the write-out staging reuses the stage buffers");
    const int lds = stage_bytes + p.S * 256;
    if (lds > 160 * 1024) return hipErrorInvalidValue;
    auto kern = spmm_half_kernel<WN, NS, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) / 8;
    hipLaunchKernelGGL(kern, dim3(chunk * 8), dim3(WN * 64), lds, stream, p);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Persistent pipelined SpMM kernel.
//
// One workgroup per CU slot walks a list of C tiles; the k-steps of all its tiles form one
// flat sequence, and the DMA pipeline (NS LDS stages, NS-1 steps ahead) runs across tile
// boundaries, so the load latency at the start of a tile and the store latency at its end
// are hidden behind the neighbouring tiles' work.
//
// All loads inside the loop are buffer loads with the LDS modifier (buffer_load_dword[x4] ...
// offen lds) issued from inline assembly (see the note on spmm_pipe_kernel).  A buffer
// descriptor's bounds check returns zero for an out-of-range offset; zero rows of B (padding
// groups, columns beyond K, columns beyond N) are therefore requested at offset 0xF0000000.
//
// Per k-step each wave issues one batch, always in this order and always complete:
//   NB_LOADS x  b128   gathered B rows of stage f = q + NS-1      -> stage f % NS
//   NA_X4    x  b128   A operands of stage f                       -> stage f % NS
//   1        x  b32    index words of stage f                      -> stage f % NS
//   1        x  b32    row table of stage f + NS-1 (this wave's private ring)
// and waits with s_waitcnt vmcnt(k * LOADS) for the batch issued NS-1 steps earlier.
// ---------------------------------------------------------------------------

template <int WM, int WN, int NS, int OUT_LAYOUT>
__global__ __launch_bounds__(WM* WN * 64) void spmm_persist_kernel(SpmmParams p) {
    using Cfg = PersistCfg<WM, WN, NS>;
    constexpr int NW = Cfg::NW, BM = Cfg::BM, BN = Cfg::BN;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int CHUNKS = BN / 8;
    constexpr int RPI = 1024 / ROW_BYTES;            // rows one DMA instruction covers (4 or 2)
    constexpr int NB_LOADS = 64 / RPI / NW;
    constexpr int NA_X4 = 4 / WN > 0 ? 4 / WN : 1;
    constexpr int LOADS = NB_LOADS + NA_X4 + 2;
    constexpr int PA = Cfg::PA;
    constexpr int EPI_PITCH = Cfg::EPI_PITCH;
    static_assert(WN == 2 || WN == 4, "A operand split");
    static_assert(64 % (RPI * NW) == 0, "rows per step must split over the waves");
    static_assert((PA - 1) * LOADS < 64, "vmcnt range");

    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave - wm * WN;
    const int S = p.S, N = p.N;

    // ---- this workgroup's tile list: XCD x (= id % 8) owns a contiguous range of tile ids
    //      (id -> n-tile major, m-tile minor); its workgroups take them round robin.  Tile
    //      coordinates advance by a fixed (dm, dn) with carry: no division per tile.
    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) >> 3;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
    const int first = xcd * chunk;
    const int last = (first + chunk) < tiles ? (first + chunk) : tiles;      // exclusive
    int my_tiles = 0;
    if (first + slot < last) my_tiles = (last - first - slot + slots - 1) / slots;
    if (my_tiles == 0) return;
    const int Q = my_tiles * S;
    const int step_dn = slots / p.tiles_m, step_dm = slots - step_dn * p.tiles_m;
    const int tn0 = (first + slot) / p.tiles_m, tm0 = (first + slot) - tn0 * p.tiles_m;
    auto next_tile = [&](int& tm, int& tn) {
        tm += step_dm;
        tn += step_dn;
        if (tm >= p.tiles_m) { tm -= p.tiles_m; tn += 1; }
    };
    const int tiles_per_vblock = p.v / BM;           // V % BM == 0 is checked on the host

    const i32x4 rsrc_b = make_buffer(p.B, p.b_bytes);
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const i32x4 rsrc_rt = make_buffer(p.rowtab, p.rowtab_bytes);
    const uint32_t row_bytes_b = (uint32_t)N * 2u;

    // ---- LDS regions
    constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    const uint32_t rt_base = EPI_BASE + Cfg::EPI_BYTES + wave * ((PA + 1) * 256);

    // ---- B loader slots of this lane
    const int slot_row = lane / CHUNKS;
    const int slot_chunk = lane % CHUNKS;
    int src_chunk[NB_LOADS];
#pragma unroll
    for (int j = 0; j < NB_LOADS; j++) {
        const int rho = (wave * NB_LOADS + j) * RPI + slot_row;
        src_chunk[j] = slot_chunk ^ ((rho & 7) << 1);
    }
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;
    const uint32_t rt_lane_off = (uint32_t)((wave * NB_LOADS) * RPI + slot_row) * 4;   // + j*RPI*4

    // ---- issue state (all scalar except coloff): stage f = next batch to issue
    int is_tm = tm0, is_tn = tn0, is_step = 0;
    uint32_t is_stage = 0;                                   // byte offset of the LDS stage for f
    uint32_t a_soff = (uint32_t)((is_tm * (BM / 64) + wm) * S) * (uint32_t)APACK_BLOCK;
    int issue_left = Q;                                      // batches not yet issued
    uint32_t rt_read = 0;                                    // ring slot (bytes) holding the rows of stage f
    // row-table state: stage f + PA (clamped to the last stage)
    int rt_tm = tm0, rt_tn = tn0, rt_step = 0, rt_left = Q - 1;   // advances still allowed
    uint32_t rt_soff = (uint32_t)((rt_tm / tiles_per_vblock) * S) * 256u;
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
            if (++rt_step == S) {
                rt_step = 0;
                next_tile(rt_tm, rt_tn);
                rt_soff = (uint32_t)((rt_tm / tiles_per_vblock) * S) * 256u;
            }
        }
    };

    // issues the batch of stage f with the given rows and moves the issue state to f + 1
    auto issue_batch = [&](const uint32_t (&rows)[NB_LOADS]) {
        const uint32_t stage = smem_base + is_stage;
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const uint32_t voff = (rows[j] == 0xffffffffu) ? 0xF0000000u : rows[j] * row_bytes_b + coloff[j];
            bdma_b128(voff, rsrc_b, 0, stage + (wave * NB_LOADS + j) * 1024);
        }
        const uint32_t a_lds = stage + B_BYTES + wm * APACK_BLOCK;
#pragma unroll
        for (int k = 0; k < NA_X4; k++) {
            const int mb = (WN >= 4) ? wn : wn * NA_X4 + k;
            bdma_b128(lane16, rsrc_a, a_soff + mb * 1024, a_lds + mb * 1024);
        }
        const int d = wn & 1;
        bdma_b32(lane4, rsrc_a, a_soff + 4096 + d * 256, a_lds + 4096 + d * 256);
        // row table of stage f + PA goes to the ring slot just before the one read now
        const uint32_t rt_write = (rt_read == 0) ? (uint32_t)PA * 256u : rt_read - 256u;
        bdma_b32(lane4, rsrc_rt, rt_soff, smem_base + rt_base + rt_write);
        rt_advance();
        // advance to stage f + 1
        --issue_left;
        is_stage = (is_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : is_stage + STAGE_BYTES;
        rt_read = (rt_read == (uint32_t)PA * 256u) ? 0u : rt_read + 256u;
        a_soff += (uint32_t)APACK_BLOCK;
        if (++is_step == S) {
            is_step = 0;
            next_tile(is_tm, is_tn);
            a_soff = (uint32_t)((is_tm * (BM / 64) + wm) * S) * (uint32_t)APACK_BLOCK;
            set_coloff();
        }
    };

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

    // ---- prologue: the first PA batches take their rows through ordinary loads (nothing is in
    //      flight yet); the row-table cursor starts PA stages ahead of the issue cursor.
    {
        uint32_t rows0[PA][NB_LOADS];
        int st_tm = tm0, st_tn = tn0, st_step = 0;
#pragma unroll
        for (int t = 0; t < PA; t++) {
            const int64_t base = ((int64_t)(st_tm / tiles_per_vblock) * S + st_step) * 64;
#pragma unroll
            for (int j = 0; j < NB_LOADS; j++)
                rows0[t][j] = (t < Q) ? p.rowtab[base + (wave * NB_LOADS + j) * RPI + slot_row] : 0xffffffffu;
            if (++st_step == S) { st_step = 0; next_tile(st_tm, st_tn); }
        }
#pragma unroll
        for (int t = 0; t < PA; t++) rt_advance();
#pragma unroll
        for (int t = 0; t < PA; t++)
            if (t < Q) issue_batch(rows0[t]);
    }

    const int j16 = lane & 15, ib = lane >> 4;
    int c_tm = tm0, c_tn = tn0;
    int q_left = Q;                 // steps not yet multiplied
    uint32_t c_stage = 0;           // byte offset of the stage multiplied next
    for (int c_tile = 0; c_tile < my_tiles; c_tile++) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < S; c_step++) {
            // batches issued after the one needed now may stay in flight
            if (q_left > PA - 1) wait_vmcnt<(PA - 1) * LOADS>();
            else wait_stages<LOADS, PA - 1>(q_left - 1);
            --q_left;
            __syncthreads();
            mma_stage<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc, [&]() {
                if (issue_left > 0) {
                    uint32_t rows[NB_LOADS];
                    const char* rr = smem + rt_base + rt_read + rt_lane_off;
#pragma unroll
                    for (int j = 0; j < NB_LOADS; j++) rows[j] = *(const uint32_t*)(rr + j * (RPI * 4));
                    issue_batch(rows);
                }
            });
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        }
        // ------------------------------------------------ tile finished: write it out
        const int cm0 = c_tm * BM, cn0 = c_tn * BN;
        if (p.fuse) fused_bias_act(acc, p.bias, (int64_t)cm0 + wm * 64 + ib * 16, p.act);
        const uint16_t* bias = p.fuse ? nullptr : p.bias;
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            const int64_t row0 = (int64_t)cm0 + wm * 64 + ib * 16;
            half8_t bias_lo, bias_hi;
            if (bias) {
                bias_lo = *(const half8_t*)(bias + row0);
                bias_hi = *(const half8_t*)(bias + row0 + 8);
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
                if (bias) {
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
            // 16-row slabs through a wave-private LDS buffer -> 128-byte row segments
            char* stg = smem + EPI_BASE + wave * (16 * EPI_PITCH);
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
        next_tile(c_tm, c_tn);
    }
}

template <int WM, int WN, int NS, int OUT_LAYOUT>
static hipError_t launch_persist(const SpmmParams& p, hipStream_t stream) {
    using Cfg = PersistCfg<WM, WN, NS>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    const int cus = p.cus;        // compute units of the plan's device
    auto kern = spmm_persist_kernel<WM, WN, NS, OUT_LAYOUT>;
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
    hipLaunchKernelGGL(kern, dim3(grid), dim3(WM * WN * 64), lds, stream, p);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Host-side launchers
// ---------------------------------------------------------------------------
template <int WM, int WN, int OUT_LAYOUT>
static hipError_t launch_variant(const SpmmParams& p, hipStream_t stream) {
    constexpr int BN = WN * 64;
    constexpr int stage_bytes = 2 * 64 * (BN * 2 + 32);
    constexpr int epi_bytes = WM * WN * 64 * 144;
    constexpr int lds = stage_bytes > epi_bytes ? stage_bytes : epi_bytes;
    auto kern = spmm_kernel<WM, WN, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set && lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = p.tiles_m * p.tiles_n;
    const int chunk = (tiles + 7) / 8;
    hipLaunchKernelGGL(kern, dim3(chunk * 8), dim3(WM * WN * 64), lds, stream, p);
    return hipGetLastError();
}

hipError_t launch_gathered(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    const bool t = out_layout == SPATHA_OUT_TRANSPOSED;
    switch (variant) {
        case SPMM_VARIANT_128x128:
            return t ? launch_variant<2, 2, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_variant<2, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_64x256:
            return t ? launch_variant<1, 4, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_variant<1, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_P128x128_S3:
            return t ? launch_pipe<2, 2, 3, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_pipe<2, 2, 3, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_P64x256_S2:
            return t ? launch_pipe<1, 4, 2, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_pipe<1, 4, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_R64x256_S3:
            return t ? launch_persist<1, 4, 3, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_persist<1, 4, 3, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_H64x256_S2:
            return t ? launch_half<4, 2, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_half<4, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_H64x128_S3:
            return t ? launch_half<2, 3, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_half<2, 3, SPATHA_OUT_ROW_MAJOR>(p, stream);
        case SPMM_VARIANT_H64x128_S2:
            return t ? launch_half<2, 2, SPATHA_OUT_TRANSPOSED>(p, stream) : launch_half<2, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace spatha

