// gfx950 (CDNA4) kernels of the V:N:M SpMM:  C = A_vnm * B, fp16 in, fp32 accumulate.
//
// The contraction runs on v_smfmac_f32_16x16x64_f16: A (16 rows x 64 logical k,
// stored 2:4 compressed as 8 halfs per lane) times B (64 k x 16 columns, 16 halfs
// per lane) with a 16-bit index field per lane that says, for each kept pair,
// which 2 of the 4 B values of its group it multiplies.
//
// Operand mapping of that instruction (measured on the hardware with one-hot
// operands, not taken from documentation):
//   A lane l      : row i = l % 16, quarter kq = l / 16; element e = 2*g' + j is
//                   kept value j of the lane's pair g' (0..3)
//   idx           : bits [4*g' + 2*j, +2) of the 16-bit half selected by ABID
//   B lane l      : column l % 16, kb = l / 16; element f belongs to the pair
//                   (kq = 2*(f/8) + kb/2, g' = 2*(kb%2) + (f%8)/4), position f % 4
//   D lane l      : column l % 16, rows 4*(l/16) + 0..3 in the 4 result registers
// So if the 16 groups of one 64-k step are numbered gamma = 4*fb + kb
// (fb = f/4), lane block kb needs, for fb = 0..3, the four B rows of group
// gamma: exactly what four transposing LDS reads deliver when the gathered B rows
// of a step sit in LDS in natural order (row 4*gamma + c).
//
// ds_read_b64_tr_b16 (measured): inside each block of 16 lanes, lane i supplies
// the address of 4 consecutive halfs; lanes 4e..4e+3 together form a 16-half
// row e; lane i receives column i of rows 0..3.
//
// Data layout produced once per matrix by pack_kernel (all "derived copies"):
//   apack  [rows/64][S] blocks of APACK_BLOCK = 4608 bytes, S = ceil(Ksp/32) k-steps:
//            half [4 mb][64 lanes][8]             A operands
//            u32  [2 d][64 lanes]                 idx fields: word d = mb 2d | mb 2d+1 << 16
//   rowtab u32  [rows/V][S*64]                    B row feeding LDS row rho of step s
//                                                 (group*m + column-loc, or ~0 = zero row)
// Inside a 64-row wave tile the sparse-instruction row (mb, i = 4*ib + r) holds
// matrix row 16*ib + 4*mb + r, so that one lane ends up with 16 consecutive
// matrix rows of one output column (contiguous 32 bytes of the transposed output).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "spmm_kernels.h"

namespace spatha {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// Development knobs (time accounting: parts of a kernel switched off, results then wrong on purpose) exist only in
// builds with -DSPATHA_DEV_PROFILE; in the product they are compile-time false.
#ifdef SPATHA_DEV_PROFILE
#define SPATHA_KNOB(bit) (p.debug & (bit))
#define SPATHA_SKEW_ON(p) ((p).skew > 0)
#else
#define SPATHA_KNOB(bit) false
#define SPATHA_SKEW_ON(p) false
#endif

// Row-major stores of C: 16 bytes per lane.  Built with -DSPATHA_OUT_32B (the counterpart of the reference's OUT_32B
// ablation switch, CMakeLists.txt:25-33) the same bytes leave as four 4-byte stores, to measure what the wide
// stores are worth; assembly, so that the compiler cannot merge them again.
template <bool WRITE_THROUGH = false>
__device__ __forceinline__ void store_c16(uint16_t* dst, u32x4 v) {
#ifdef SPATHA_OUT_32B
    asm volatile(
        "global_store_dword %0, %1, off\n\t"
        "global_store_dword %0, %2, off offset:4\n\t"
        "global_store_dword %0, %3, off offset:8\n\t"
        "global_store_dword %0, %4, off offset:12" ::"v"(dst), "v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w)
        : "memory");
#else
    // WRITE_THROUGH (sc1): the result goes through to memory instead of staying in the XCD's L2, where it would push
    // out the operand panels the other workgroups of the XCD are re-reading.  Pays in the dense-staged kernels
    // (4096 x 1024 x 16384 at 64:2:8: 63.7 -> 62.2 us row-major, 66.3 -> 60.7 us transposed + bias) and in the tall
    // kernel's transposed write-out (1024 x 4096 x 16384 at 128:2:16: 33 -> 30.4 us), not in the 128 x 128 tiles
    // (37.7 -> 39.3 us at 128:2:32); the non-temporal hint costs 3 us everywhere.
    // The s_nop covers the two wait states that the hardware needs between a store of more than 64 bits and a VALU
    // write of its data registers: the compiler inserts them for its own stores, not after an asm statement.
    if (WRITE_THROUGH) asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" ::"v"(dst), "v"(v) : "memory");
    else *(u32x4*)dst = v;
#endif
}

// "Dynamic LDS limit raised" flags, one per (kernel, device): the attribute is a per-device property of a kernel.
static bool& lds_attr_flag(const void* kern) {
    struct Entry { const void* kern; bool set[16]; };
    static Entry table[256] = {};
    static std::mutex lock;
    int dev = 0;
    (void)hipGetDevice(&dev);
    std::lock_guard<std::mutex> guard(lock);
    int i = 0;
    while (i < 255 && table[i].kern && table[i].kern != kern) i++;
    table[i].kern = kern;
    return table[i].set[dev & 15];
}

// ---------------------------------------------------------------------------
// pack_kernel: canonical (values, metadata, columns) -> (apack, ipack, rowtab)
// One thread per (wave tile, step, mb, lane) for apack/ipack; rowtab separately.
// ---------------------------------------------------------------------------
__global__ void pack_a_kernel(const uint16_t* __restrict__ values, const uint32_t* __restrict__ metadata, int rows,
                              int ksp, int S, int half_tiles, uint16_t* __restrict__ apack) {
    const int64_t total = (int64_t)(rows / 64) * S * 4 * 64;
    const int ngroups = ksp / 2;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int lane = (int)(t & 63);
        int mb = (int)((t >> 6) & 3);
        int64_t ws = t >> 8;                 // wave tile * S + step
        int s = (int)(ws % S);
        int64_t wt = ws / S;
        int i = lane & 15, kq = lane >> 4;
        int ib = i >> 2, rr = i & 3;
        // matrix row; half_tiles: the order of the V = 32 kernels (instructions 0, 1 = rows 0..31 of the tile)
        int64_t r = wt * 64 + (half_tiles ? 32 * (mb >> 1) + 8 * ib + 4 * (mb & 1) + rr : 16 * ib + 4 * mb + rr);
        // canonical coordinates of the row
        int64_t R16 = r >> 4;
        int q = (int)((r >> 2) & 3), p = (int)((r >> 1) & 1), sbit = (int)(r & 1);
        uint16_t vals[8];
        uint32_t idx16 = 0;
#pragma unroll
        for (int gp = 0; gp < 4; gp++) {
            int fb = (kq >> 1) * 2 + (gp & 1);
            int kb = (kq & 1) * 2 + (gp >> 1);
            int g = s * 16 + fb * 4 + kb;                 // global group
            if (g < ngroups) {
                int tt = g >> 2, u = g & 3;
                int64_t vi = R16 * 16 * (int64_t)ksp + (int64_t)tt * 128 + q * 32 + u * 8 + p * 4 + sbit * 2;
                vals[2 * gp] = values[vi];
                vals[2 * gp + 1] = values[vi + 1];
                int64_t wi = (r >> 5) * (int64_t)(ksp >> 3) * 16 + (int64_t)tt * 16 + ((r >> 4) & 1) * 8 + q * 2 + p;
                uint32_t nib = (metadata[wi] >> (sbit * 16 + u * 4)) & 0xfu;
                idx16 |= nib << (4 * gp);
            } else {
                vals[2 * gp] = 0;
                vals[2 * gp + 1] = 0;
                idx16 |= 0x4u << (4 * gp);                // positions (0,1): harmless, values are zero
            }
        }
        u32x4 out;
        out.x = vals[0] | ((uint32_t)vals[1] << 16);
        out.y = vals[2] | ((uint32_t)vals[3] << 16);
        out.z = vals[4] | ((uint32_t)vals[5] << 16);
        out.w = vals[6] | ((uint32_t)vals[7] << 16);
        char* blk = (char*)apack + ws * APACK_BLOCK;
        *(u32x4*)(blk + mb * 1024 + lane * 16) = out;
        // index words: [d][lane] dwords after the operands, 16 bits per mb (mb = 2d + half)
        *(uint16_t*)(blk + 4096 + (mb >> 1) * 256 + lane * 4 + (mb & 1) * 2) = (uint16_t)idx16;
    }
}

__global__ void pack_rowtab_kernel(const uint32_t* __restrict__ columns, int rows, int cols, int m, int v, int ksp,
                                   int S, uint32_t* __restrict__ rowtab) {
    const int ngroups = ksp / 2;
    const int64_t total = (int64_t)(rows / v) * S * 64;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int rho = (int)(t & 63);
        int64_t bs = t >> 6;
        int s = (int)(bs % S);
        int64_t b = bs / S;
        int g = s * 16 + (rho >> 2), c = rho & 3;
        uint32_t row = 0xffffffffu;
        if (g < ngroups) {
            int64_t k = (int64_t)g * m + columns[b * ngroups * 4 + (int64_t)g * 4 + c];
            if (k < cols) row = (uint32_t)k;
        }
        rowtab[t] = row;
    }
}

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
    const char* a_blk = (const char*)p.apack + (wt * S) * APACK_BLOCK;   // + s*APACK_BLOCK
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
// Fused epilogue ahead of a write-out, for a lane that holds rows row16 + 4*mb + r (standard operand order) of
// its output columns:  t = fp16(acc);  t += bias[row] (one fp16 addition, as in the reference's fused bias,
// end2end blockwise_kernel.h:324-341);  t = act(t), evaluated in fp32.  The write-out's own conversion to fp16 is
// then exact without an activation and the single rounding of the activation's value with one.
// Used when SpmmParams::fuse is set (row-major output with a bias, or any activation); the write-out is then
// given no bias.
// ---------------------------------------------------------------------------
// x * Phi(x) = max(x, 0) - a * Phi(-a), a = |x|: only the lower tail is evaluated, where Phi keeps its relative accuracy
// (1 + erf(x / sqrt 2) would cancel), as 2^P(a) with P the degree-7 interpolant of log2 Phi(-a) on [0, 5.75] (relative
// error of Phi below 5e-6; beyond 5.75 the term is under half the smallest fp16 subnormal).  Checked on the CPU over
// every fp16 input: 99.4 % of the fp16 results equal the rounded exact value, none is more than one step away.
// 14 instructions + one exponential (the erfc form with a reciprocal and an exponential needed 27 issue slots).
__device__ __forceinline__ float act_gelu_erf(float x) {
    const float a = fabsf(x);
    const float ac = fminf(a, 5.75f);
    float p = fmaf(ac, -1.920561127e-06f, 6.327379007e-05f);
    p = fmaf(ac, p, -9.432987473e-04f);
    p = fmaf(ac, p, 8.555782832e-03f);
    p = fmaf(ac, p, -5.405129916e-02f);
    p = fmaf(ac, p, -4.583827060e-01f);
    p = fmaf(ac, p, -1.151278015e+00f);
    p = fmaf(ac, p, -9.999938734e-01f);
    const float tail = a > 5.75f ? 0.0f : a * __builtin_amdgcn_exp2f(p);
    return fmaxf(x, 0.0f) - tail;
}
__device__ __forceinline__ float act_gelu_tanh(float x) {
    // 0.5 (1 + tanh u) = 1 / (1 + exp(-2u)): no cancellation for negative x; exp -> inf gives -0, exp -> 0 gives x
    const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
    return x * __frcp_rn(1.0f + __expf(-2.0f * u));
}
template <int ACT>
__device__ __forceinline__ void fused_bias_act_impl(float4_t (&acc)[4][4], const uint16_t* bias, int64_t row16) {
    // one (mb, nb) group of four values at a time, fenced, so that the scheduler does not interleave all 64 chains
    // of the activation and run out of registers next to the accumulators
#pragma unroll
    for (int mb = 0; mb < 4; mb++) {
        half4_t bv = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
        if (bias) bv = *(const half4_t*)(bias + row16 + 4 * mb);
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
__device__ __forceinline__ void fused_bias_act(float4_t (&acc)[4][4], const uint16_t* bias, int64_t row16, int act) {
    if (act == SPATHA_ACT_GELU) fused_bias_act_impl<SPATHA_ACT_GELU>(acc, bias, row16);
    else if (act == SPATHA_ACT_GELU_TANH) fused_bias_act_impl<SPATHA_ACT_GELU_TANH>(acc, bias, row16);
    else fused_bias_act_impl<SPATHA_ACT_NONE>(acc, bias, row16);
}

// ---------------------------------------------------------------------------
// One k-step of a wave's 64 x 64 tile out of an LDS stage: 4 A operands + index words,
// 4 B fragments (16 transposing reads), 16 sparse matrix instructions.  The B fragments are
// double buffered in registers and `between` (the next stage's DMA issue) runs after the
// first reads have been sent, so that LDS latency overlaps address arithmetic and matrix work
// instead of being paid once per fragment.
// ---------------------------------------------------------------------------
template <int ROW_BYTES>
__device__ __forceinline__ half16_t read_b_fragment(const char* st, int off) {
    half16_t bf;
#pragma unroll
    for (int fb = 0; fb < 4; fb++) {
        short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, st + off + fb * 16 * ROW_BYTES));
        half4_t h4 = __builtin_bit_cast(half4_t, t4);
        bf[fb * 4 + 0] = h4[0];
        bf[fb * 4 + 1] = h4[1];
        bf[fb * 4 + 2] = h4[2];
        bf[fb * 4 + 3] = h4[3];
    }
    return bf;
}

#define SPATHA_MMA4(NB, BF)                                                                                   \
    acc[0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], BF, acc[0][NB], (int)i0, 0, 0);           \
    acc[1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], BF, acc[1][NB], (int)i0, 0, 1);           \
    acc[2][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], BF, acc[2][NB], (int)i1, 0, 0);           \
    acc[3][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], BF, acc[3][NB], (int)i1, 0, 1);

template <int ROW_BYTES, class Between>
__device__ __forceinline__ void mma_stage(const char* st, int a_off, int i_off, const int (&tr_off)[4],
                                          float4_t (&acc)[4][4], Between&& between) {
    half8_t a_cur[4];
#pragma unroll
    for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(st + a_off + mb * 1024);
    const uint32_t i0 = *(const uint32_t*)(st + i_off), i1 = *(const uint32_t*)(st + i_off + 256);
    half16_t bf0 = read_b_fragment<ROW_BYTES>(st, tr_off[0]);
    half16_t bf1 = read_b_fragment<ROW_BYTES>(st, tr_off[1]);
    __builtin_amdgcn_sched_barrier(0);
    between();
    __builtin_amdgcn_sched_barrier(0);
    SPATHA_MMA4(0, bf0)
    __builtin_amdgcn_sched_barrier(0);
    bf0 = read_b_fragment<ROW_BYTES>(st, tr_off[2]);
    __builtin_amdgcn_sched_barrier(0);
    SPATHA_MMA4(1, bf1)
    __builtin_amdgcn_sched_barrier(0);
    bf1 = read_b_fragment<ROW_BYTES>(st, tr_off[3]);
    __builtin_amdgcn_sched_barrier(0);
    SPATHA_MMA4(2, bf0)
    SPATHA_MMA4(3, bf1)
}

constexpr int TT_PITCH = 144;                      // 64 rows x 2 B + 16 B pad (keeps 16-byte alignment)
constexpr int TT_SLAB_BYTES = 8 * TT_PITCH;        // per wave
// Transposed write-out (C^T[N][rows], + bias) of one wave's 64 x 64 block through an LDS slab of 8 columns x 64 rows,
// so that every store instruction covers whole 128-byte lines (defined further down).
template <bool WRITE_THROUGH = false>
__device__ __forceinline__ void store_block_transposed_slab(const float4_t (&acc)[4][4], char* stg, uint16_t* C,
                                                            const uint16_t* bias, int64_t row0, int col0, int rows_total, int N,
                                                            int lane, bool stores_on);

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
// (s_nop: one wait state between the write of m0 and the LDS-DMA instruction that reads it; the compiler does not
// look inside an asm statement for that.)
__device__ __forceinline__ void dma_b128(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "m0");
}
__device__ __forceinline__ void dma_b32(const void* gptr, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds_addr), "v"(gptr) : "m0");
}
template <int N_>
__device__ __forceinline__ void wait_vmcnt() {
    static_assert(N_ >= 0 && N_ < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N_));
}
template <int L, int MAXK>
__device__ __forceinline__ void wait_stages(int k) {
    // wait until at most k stages (k * L loads) of this wave are still in flight
    if constexpr (MAXK == 0) {
        wait_vmcnt<0>();
    } else {
        if (k >= MAXK) wait_vmcnt<MAXK * L>();
        else wait_stages<L, MAXK - 1>(k);
    }
}

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
#define SPATHA_MMA2LO(NB, BF)                                                                                 \
    acc[0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], BF, acc[0][NB], (int)i0, 0, 0);           \
    acc[1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], BF, acc[1][NB], (int)i0, 0, 1);
#define SPATHA_MMA2HI(NB, BF)                                                                                 \
    acc[2][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], BF, acc[2][NB], (int)i1, 0, 0);           \
    acc[3][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], BF, acc[3][NB], (int)i1, 0, 1);

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
        for (int i = tid; i < S * 128; i += WN * 64) {
            const int s = i >> 7, rho = i & 63;
            const uint32_t r = ((i & 64) ? rt1 : rt0)[s * 64 + rho];
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
    if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
        // per output column the lane holds rows 8*ib .. +7 (instructions 0, 1) and 32 + 8*ib .. +7 (2, 3)
        const int64_t row_lo = (int64_t)m0 + ib * 8, row_hi = row_lo + 32;
        half8_t bias_lo, bias_hi;
        if (p.bias) {
            bias_lo = *(const half8_t*)(p.bias + row_lo);
            bias_hi = *(const half8_t*)(p.bias + row_hi);
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
                uint16_t* dst = p.C + (int64_t)col * p.rows;
                *(half8_t*)(dst + row_lo) = lo;
                *(half8_t*)(dst + row_hi) = hi;
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
            if (col < N) store_c16(p.C + ((int64_t)m0 + row) * N + col, v);
        }
    }
}

template <int WN, int NS>
constexpr int half_stage_bytes() { return NS * (2 * 64 * WN * 128 + APACK_BLOCK); }

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
typedef int i32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ i32x4 make_buffer(const void* base, uint32_t bytes) {
    const uint64_t a = (uint64_t)(uintptr_t)base;
    i32x4 r;
    r.x = __builtin_amdgcn_readfirstlane((int)(uint32_t)a);
    r.y = __builtin_amdgcn_readfirstlane((int)((uint32_t)(a >> 32) & 0xffffu));   // stride 0: raw buffer
    r.z = __builtin_amdgcn_readfirstlane((int)bytes);
    r.w = 0x00020000;
    return r;
}
// Descriptor of the part of a buffer that starts `off` bytes in (off is wave-uniform).  The range check of a raw buffer
// compares the vector offset (plus the instruction's immediate) with the record count and leaves the scalar offset
// out, so a window that moves through the buffer is expressed here, in base and count, never as a scalar offset.
__device__ __forceinline__ i32x4 buffer_window(const void* base, uint32_t bytes, uint32_t off) {
    return make_buffer((const char*)base + off, off < bytes ? bytes - off : 0u);
}
__device__ __forceinline__ void bdma_b128(uint32_t voff, i32x4 rsrc, uint32_t soff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc),
                 "s"(soff)
                 : "m0");
}
__device__ __forceinline__ void bdma_b32(uint32_t voff, i32x4 rsrc, uint32_t soff, uint32_t lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, %3 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc),
                 "s"(soff)
                 : "m0");
}

template <int WM, int WN, int NS>
struct PersistCfg {
    static constexpr int NW = WM * WN;
    static constexpr int BM = WM * 64, BN = WN * 64;
    static constexpr int ROW_BYTES = BN * 2;
    static constexpr int B_BYTES = 64 * ROW_BYTES;
    static constexpr int STAGE_BYTES = B_BYTES + WM * APACK_BLOCK;
    static constexpr int PA = NS - 1;
    static constexpr int EPI_PITCH = 144;
    static constexpr int EPI_BYTES = NW * 16 * EPI_PITCH;          // one 16-row slab per wave at a time
    static constexpr int RT_BYTES = NW * (PA + 1) * 256;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + EPI_BYTES + RT_BYTES;
};

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
    static int cus = 0;
    auto kern = spmm_persist_kernel<WM, WN, NS, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        int dev = 0;
        if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
        if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
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
template <int WM, int WN, int NS, int NP>
struct WsCfg {
    static constexpr int NC = WM * WN;
    static constexpr int BM = WM * 64, BN = WN * 64;
    static constexpr int ROW_BYTES = BN * 2;
    static constexpr int B_BYTES = 64 * ROW_BYTES;
    static constexpr int STAGE_BYTES = B_BYTES + WM * APACK_BLOCK;
    static constexpr int PA = NS - 1;
    static constexpr int EPI_PITCH = 144;
    static constexpr int EPI_BYTES = NC * 16 * EPI_PITCH;
    static constexpr int RT_BYTES = NP * (PA + 1) * 256;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + EPI_BYTES + RT_BYTES;
    static constexpr int THREADS = (NC + NP) * 64;
    static constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    static constexpr uint32_t RT_BASE = EPI_BASE + EPI_BYTES;
};

// Tile walk shared by both roles: XCD x (= workgroup id % 8) owns a contiguous range of tile
// ids (id -> n-tile major, m-tile minor) and its workgroups take them round robin; the
// coordinates advance by a fixed (dm, dn) with carry, so no division per tile.
struct TileWalk {
    int my_tiles, tm0, tn0, step_dm, step_dn, tiles_m;
    __device__ __forceinline__ void init(int tiles_m_, int tiles_n_) {
        tiles_m = tiles_m_;
        const int tiles = tiles_m_ * tiles_n_;
        const int chunk = (tiles + 7) >> 3;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
        const int first = xcd * chunk;
        const int last = (first + chunk) < tiles ? (first + chunk) : tiles;
        my_tiles = 0;
        if (first + slot < last) my_tiles = (last - first - slot + slots - 1) / slots;
        step_dn = slots / tiles_m;
        step_dm = slots - step_dn * tiles_m;
        tn0 = (first + slot) / tiles_m;
        tm0 = (first + slot) - tn0 * tiles_m;
    }
    __device__ __forceinline__ void next(int& tm, int& tn) const {
        tm += step_dm;
        tn += step_dn;
        if (tm >= tiles_m) { tm -= tiles_m; tn += 1; }
    }
};

template <class Cfg, int NP, int PR>
__device__ __forceinline__ void ws_producer(const SpmmParams& p, const TileWalk& walk, char* smem, uint32_t smem_base,
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

    const int S = p.S, N = p.N;
    const int Q = walk.my_tiles * S;
    const int tiles_per_vblock = p.v / BM;
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
    uint32_t rt_soff = (uint32_t)((rt_tm / tiles_per_vblock) * S) * 256u;
    uint32_t a_soff = (uint32_t)((is_tm * WM) * S) * (uint32_t)APACK_BLOCK;    // wave-tile row 0 of the tile
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
                walk.next(rt_tm, rt_tn);
                rt_soff = (uint32_t)((rt_tm / tiles_per_vblock) * S) * 256u;
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
        if (++is_step == S) {
            is_step = 0;
            walk.next(is_tm, is_tn);
            a_soff = (uint32_t)((is_tm * WM) * S) * (uint32_t)APACK_BLOCK;
            set_coloff();
        }
    };
    // prologue: rows of the first PA stages through ordinary loads (nothing is in flight yet)
    {
        uint32_t rows0[PA][NB_LOADS];
        int st_tm = walk.tm0, st_tn = walk.tn0, st_step = 0;
#pragma unroll
        for (int t = 0; t < PA; t++) {
            const int64_t base = ((int64_t)(st_tm / tiles_per_vblock) * S + st_step) * 64;
#pragma unroll
            for (int j = 0; j < NB_LOADS; j++)
                rows0[t][j] = (t < Q) ? p.rowtab[base + (PR * NB_LOADS + j) * RPI + slot_row] : 0xffffffffu;
            if (++st_step == S) { st_step = 0; walk.next(st_tm, st_tn); }
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
}

template <class Cfg, int WN, int OUT_LAYOUT>
__device__ __forceinline__ void ws_consumer(const SpmmParams& p, const TileWalk& walk, char* smem, int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, NS = Cfg::PA + 1;
    constexpr int ROW_BYTES = Cfg::ROW_BYTES, B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int EPI_PITCH = Cfg::EPI_PITCH;
    const int S = p.S, N = p.N;
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
    for (int c_tile = 0; c_tile < walk.my_tiles; c_tile++) {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
        for (int c_step = 0; c_step < S; c_step++) {
            __syncthreads();
            if (!SPATHA_KNOB(16)) mma_stage<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc, [&]() {});
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        }
        const int cm0 = c_tm * BM, cn0 = c_tn * BN;
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
        walk.next(c_tm, c_tn);
    }
}

// ---- deferred write-out -------------------------------------------------------------------
// A finished 64 x 64 wave tile is rounded to fp16 pairs (32 registers) and written one quarter
// per k-step of the NEXT tile: the stores of a tile are then spread over the following tile's
// matrix work instead of stalling every consumer on a burst that all CUs issue together.
__device__ __forceinline__ uint32_t pack_half2(float a, float b) {
    half2_t h = {(_Float16)a, (_Float16)b};
    return __builtin_bit_cast(uint32_t, h);
}

// rows 4*MB..4*MB+3 (+16*ib) of the pending wave tile -> row-major C through the wave's LDS slab
template <int MB, int EPI_PITCH>
__device__ __forceinline__ void store_slab_row_major(const uint32_t (&pend)[4][4][2], char* stg, uint16_t* C, int64_t row_base,
                                                     int col_base, int N, int lane, bool enable) {
    const int j16 = lane & 15, ib = lane >> 4;
#pragma unroll
    for (int rp = 0; rp < 2; rp++)
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            uint32_t w = pend[MB][nb][rp];
            asm volatile("" : "+v"(w));      // keeps the >> 16 below from being hoisted out of the k-loop (32 registers)
            *(uint16_t*)(stg + ((2 * rp) * 4 + ib) * EPI_PITCH + (nb * 16 + j16) * 2) = (uint16_t)w;
            *(uint16_t*)(stg + ((2 * rp + 1) * 4 + ib) * EPI_PITCH + (nb * 16 + j16) * 2) = (uint16_t)(w >> 16);
        }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < 2; it++) {
        const int Lr = it * 8 + (lane >> 3), ch = lane & 7;
        const int row = 16 * (Lr & 3) + 4 * MB + (Lr >> 2);
        const int col = col_base + ch * 8;
        u32x4 v = *(const u32x4*)(stg + Lr * EPI_PITCH + ch * 16);
        if (col < N && enable) store_c16(C + (row_base + row) * N + col, v);
    }
    __builtin_amdgcn_wave_barrier();
}

// column block NB of the pending wave tile -> transposed output (32 contiguous bytes per lane)
template <int NB>
__device__ __forceinline__ void store_block_transposed(const uint32_t (&pend)[4][4][2], uint16_t* C, int64_t row0, int col,
                                                       int rows_total, int N, bool enable) {
    u32x4 lo = {pend[0][NB][0], pend[0][NB][1], pend[1][NB][0], pend[1][NB][1]};
    u32x4 hi = {pend[2][NB][0], pend[2][NB][1], pend[3][NB][0], pend[3][NB][1]};
    if (col < N && enable) {
        uint16_t* dst = C + (int64_t)col * rows_total + row0;
        *(u32x4*)dst = lo;
        *(u32x4*)(dst + 8) = hi;
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

// Transposed write-out (C^T[N][rows], + bias) of one wave's 64 x 64 block through an LDS slab of 8 columns x 64 rows.
// Straight from the accumulators a lane could only store 16-byte pieces 32 bytes apart; through the slab every
// store instruction writes 8 output rows (columns of C) x 128 contiguous bytes.
template <bool WRITE_THROUGH>
__device__ __forceinline__ void store_block_transposed_slab(const float4_t (&acc)[4][4], char* stg, uint16_t* C,
                                                            const uint16_t* bias, int64_t row0, int col0, int rows_total, int N,
                                                            int lane, bool stores_on) {
    const int j16 = lane & 15, ib = lane >> 4;     // as accumulator lane: column j16 of a 16-column block, rows 16*ib + 4*mb + r
    const int rn = lane >> 3, rc = lane & 7;       // as reader: slab column rn, 16-byte chunk rc (rows 8*rc .. 8*rc + 7)
    half4_t b4[4];
    if (bias) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) b4[mb] = *(const half4_t*)(bias + row0 + 16 * ib + 4 * mb);
    }
#pragma unroll
    for (int nb = 0; nb < 4; nb++) {
        half4_t h4[4];
#pragma unroll
        for (int mb = 0; mb < 4; mb++) {
#pragma unroll
            for (int r = 0; r < 4; r++) h4[mb][r] = (_Float16)acc[mb][nb][r];
            if (bias) h4[mb] = h4[mb] + b4[mb];
        }
#pragma unroll
        for (int hf = 0; hf < 2; hf++) {
            if ((j16 >> 3) == hf) {
#pragma unroll
                for (int mb = 0; mb < 4; mb++) *(half4_t*)(stg + (j16 & 7) * TT_PITCH + (16 * ib + 4 * mb) * 2) = h4[mb];
            }
            __builtin_amdgcn_wave_barrier();
            const u32x4 v = *(const u32x4*)(stg + rn * TT_PITCH + rc * 16);
            __builtin_amdgcn_wave_barrier();
            const int col = col0 + nb * 16 + hf * 8 + rn;
            if (col < N && stores_on) store_c16<WRITE_THROUGH>(C + (int64_t)col * rows_total + row0 + rc * 8, v);
        }
    }
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
    const int S = p.S, N = p.N;
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
        for (int c_step = 0; c_step < S; c_step++) {
            __syncthreads();
            if (!SPATHA_KNOB(16)) mma_stage_tall<ROW_BYTES>(smem + c_stage, a_off, i_off, tr_off, acc);
            c_stage = (c_stage + STAGE_BYTES == NS * STAGE_BYTES) ? 0u : c_stage + STAGE_BYTES;
        }
        const int cm0 = c_tm * BM, cn0 = c_tn * BN;
#pragma unroll
        for (int h = 0; h < 2; h++) {
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
    static int cus = 0;
    auto kern = spmm_wst_kernel<WN, NS, NP, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        int dev = 0;
        if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
        if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
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

// Row-major write-out of one wave's 64 x 64 block through a column-major LDS slab.
// A lane holds, per (mb, nb), rows 16*ib + 4*mb + r (r = 0..3) of column nb*16 + j16: four
// consecutive slab rows q = 4*ib + r of one column, i.e. ONE 8-byte LDS write into slab[col][q]
// (TR_PITCH bytes per column).  The transposing read gives result lanes 4k..4k+3 of a 16-lane
// block the four halfs of the 8-byte chunks that lanes k, 4+k, 8+k, 12+k address, so the chunk
// addresses are chosen per lane such that result lane (kb, 4k+x) ends up with slab row
// 8*s + 4*(k%2) + x and columns 8*(2*kb + k/2) .. +3 (+4 for the second read): one global store
// instruction then covers 8 rows x 128 contiguous bytes.
// Development-only cycle accounting (compiled in with -DSPATHA_DEV_PROFILE): each consumer wave sums the
// s_memtime ticks it spends (0) computing, (1) waiting at the step barrier, (2) in the write-out, and
// lane 0 writes the three sums to prof[(block * 16 + wave) * 4 ..].
#ifdef SPATHA_DEV_PROFILE
#define SPATHA_PROF_DECL long long prof_t = __builtin_readcyclecounter(), prof_sum[3] = {0, 0, 0};
#define SPATHA_PROF_MARK(SLOT)                                   \
    {                                                            \
        const long long now = __builtin_readcyclecounter();      \
        prof_sum[SLOT] += now - prof_t;                          \
        prof_t = now;                                            \
    }
#define SPATHA_PROF_FLUSH                                                                 \
    if (p.prof && lane == 0) {                                                            \
        long long* dst = p.prof + ((int64_t)blockIdx.x * 16 + wave) * 4;                  \
        dst[0] = prof_sum[0];                                                             \
        dst[1] = prof_sum[1];                                                             \
        dst[2] = prof_sum[2];                                                             \
    }
#else
#define SPATHA_PROF_DECL
#define SPATHA_PROF_MARK(SLOT)
#define SPATHA_PROF_FLUSH
#endif

constexpr int TR_PITCH = 40;                       // 16 rows x 2 B + 8 B pad
constexpr int TR_SLAB_BYTES = 64 * TR_PITCH;       // per wave, all 16 slab rows at once
constexpr int TR8_PITCH = 16;                      // 8 rows x 2 B
constexpr int TR8_SLAB_BYTES = 64 * TR8_PITCH;     // per wave, 8 slab rows at a time (ROWS8: half the lanes write)
// BIAS_VIA_SLAB (needs ROWS8 and 128 spare bytes behind the slab): the block's 64 bias values are fetched once, ahead of
// the first store, and the phases read them from LDS; a bias load inside a phase would make that phase wait on the
// vector-memory counter, i.e. for every store issued so far.
template <bool ROWS8, bool BIAS_VIA_SLAB = false>
__device__ __forceinline__ void store_block_row_major_tr(const float4_t (&acc)[4][4], char* stg, uint16_t* C, int64_t row0,
                                                         int col0, int N, int lane, bool stores_on,
                                                         const uint16_t* bias = nullptr) {
    static_assert(!BIAS_VIA_SLAB || ROWS8, "the spare bytes sit behind the 8-row slab");
    constexpr int PITCH = ROWS8 ? TR8_PITCH : TR_PITCH;
    if (BIAS_VIA_SLAB && bias) {
        if (lane < 32) *(uint32_t*)(stg + TR8_SLAB_BYTES + lane * 4) = *(const uint32_t*)(bias + row0 + lane * 2);
        __builtin_amdgcn_wave_barrier();
    }
    const int j16 = lane & 15, ib = lane >> 4;     // as accumulator lane: column j16, rows 4*ib + r
    const int li = lane & 15, kb = lane >> 4;
    // as chunk supplier: source row e = li/4, chunk k = li%4
    const int rd_off = (8 * (2 * kb + ((li & 3) >> 1)) + (li >> 2)) * PITCH + (li & 1) * 8;
    // as result lane: k = li/4, x = li%4
    const int q_lo = 4 * ((li >> 2) & 1) + (li & 3);
    const int out_col = col0 + 8 * (2 * kb + (li >> 3));
    const bool live = out_col < N && stores_on;
    // Eight phases (mb, half of the slab rows).  LDS operations of one wave execute in order, so the slab can be
    // rewritten for the next phase as soon as this phase's reads are ISSUED; the global store of a phase is issued
    // one phase late, behind the next phase's LDS traffic, so that no phase waits for a full LDS round trip.
    u32x4 held = {0u, 0u, 0u, 0u};
    int held_row = 0;
#pragma unroll
    for (int ph = 0; ph < 8; ph++) {
        const int mb = ph >> 1, sidx = ph & 1;
        if (ROWS8 || sidx == 0) {
            half4_t h4[4];
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
#pragma unroll
                for (int r = 0; r < 4; r++) h4[nb][r] = (_Float16)acc[mb][nb][r];
            if (bias) {          // fp16 addition on the rounded product, rows row0 + 16*ib + 4*mb + r
                const half4_t bv = BIAS_VIA_SLAB ? *(const half4_t*)(stg + TR8_SLAB_BYTES + (16 * ib + 4 * mb) * 2)
                                                 : *(const half4_t*)(bias + row0 + 16 * ib + 4 * mb);
#pragma unroll
                for (int nb = 0; nb < 4; nb++) h4[nb] = h4[nb] + bv;
            }
            if (ROWS8) {
                if ((ib >> 1) == sidx) {
#pragma unroll
                    for (int nb = 0; nb < 4; nb++) *(half4_t*)(stg + (nb * 16 + j16) * PITCH + (ib & 1) * 8) = h4[nb];
                }
            } else {
#pragma unroll
                for (int nb = 0; nb < 4; nb++) *(half4_t*)(stg + (nb * 16 + j16) * PITCH + ib * 8) = h4[nb];
            }
        }
        __builtin_amdgcn_wave_barrier();
        const int roff = rd_off + (ROWS8 ? 0 : sidx * 16);
        short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, stg + roff));
        short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, stg + roff + 4 * PITCH));
        __builtin_amdgcn_wave_barrier();
        if (ph > 0 && live) store_c16<true>(C + (row0 + held_row) * N + out_col, held);
        held.x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
        held.y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
        held.z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
        held.w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
        const int q = 8 * sidx + q_lo;
        held_row = 16 * (q >> 2) + 4 * mb + (q & 3);
    }
    if (live) store_c16<true>(C + (row0 + held_row) * N + out_col, held);
    __builtin_amdgcn_wave_barrier();
}

// The same two write-outs with four slabs per wave (stg: 4 slabs, then 128 bytes for the block's bias values): four
// phases' LDS writes and transposing / row reads are in flight before the first store waits for its data, so a 64 x 64
// block costs two LDS round trips instead of eight.
template <bool WITH_BIAS>
__device__ __forceinline__ void store_block_row_major_tr4(const float4_t (&acc)[4][4], char* stg, uint16_t* C, int64_t row0,
                                                          int col0, int N, int lane, bool stores_on, const uint16_t* bias) {
    constexpr int PITCH = TR8_PITCH, SLAB = TR8_SLAB_BYTES;
    const int j16 = lane & 15, ib = lane >> 4;
    const int li = lane & 15, kb = lane >> 4;
    const int rd_off = (8 * (2 * kb + ((li & 3) >> 1)) + (li >> 2)) * PITCH + (li & 1) * 8;
    const int q_lo = 4 * ((li >> 2) & 1) + (li & 3);
    const int out_col = col0 + 8 * (2 * kb + (li >> 3));
    const bool live = out_col < N && stores_on;
    char* bias_lds = stg + 4 * TT_SLAB_BYTES;
    if (WITH_BIAS) {
        if (lane < 32) *(uint32_t*)(bias_lds + lane * 4) = *(const uint32_t*)(bias + row0 + lane * 2);
        __builtin_amdgcn_wave_barrier();
    }
#pragma unroll
    for (int grp = 0; grp < 2; grp++) {
#pragma unroll
        for (int mb2 = 0; mb2 < 2; mb2++) {
            const int mb = grp * 2 + mb2;
            half4_t h4[4];
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
#pragma unroll
                for (int r = 0; r < 4; r++) h4[nb][r] = (_Float16)acc[mb][nb][r];
            if (WITH_BIAS) {     // fp16 addition on the rounded product, rows row0 + 16*ib + 4*mb + r
                const half4_t bv = *(const half4_t*)(bias_lds + (16 * ib + 4 * mb) * 2);
#pragma unroll
                for (int nb = 0; nb < 4; nb++) h4[nb] = h4[nb] + bv;
            }
            // slab 2*mb2 + sidx takes the rows of lane groups ib = 2*sidx, 2*sidx + 1
            char* slab = stg + (mb2 * 2 + (ib >> 1)) * SLAB;
#pragma unroll
            for (int nb = 0; nb < 4; nb++) *(half4_t*)(slab + (nb * 16 + j16) * PITCH + (ib & 1) * 8) = h4[nb];
        }
        __builtin_amdgcn_wave_barrier();
        short4_t lo[4], hi[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            lo[k] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, stg + k * SLAB + rd_off));
            hi[k] = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, stg + k * SLAB + rd_off + 4 * PITCH));
        }
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int mb = grp * 2 + (k >> 1), sidx = k & 1;
            const int q = 8 * sidx + q_lo;
            const int row = 16 * (q >> 2) + 4 * mb + (q & 3);
            u32x4 v;
            v.x = (uint32_t)(uint16_t)lo[k][0] | ((uint32_t)(uint16_t)lo[k][1] << 16);
            v.y = (uint32_t)(uint16_t)lo[k][2] | ((uint32_t)(uint16_t)lo[k][3] << 16);
            v.z = (uint32_t)(uint16_t)hi[k][0] | ((uint32_t)(uint16_t)hi[k][1] << 16);
            v.w = (uint32_t)(uint16_t)hi[k][2] | ((uint32_t)(uint16_t)hi[k][3] << 16);
            if (live) store_c16<true>(C + (row0 + row) * N + out_col, v);
        }
    }
    __builtin_amdgcn_wave_barrier();
}

__device__ __forceinline__ void store_block_transposed_slab4(const float4_t (&acc)[4][4], char* stg, uint16_t* C,
                                                             const uint16_t* bias, int64_t row0, int col0, int rows_total, int N,
                                                             int lane, bool stores_on) {
    const int j16 = lane & 15, ib = lane >> 4;     // as accumulator lane: column j16 of a 16-column block, rows 16*ib + 4*mb + r
    const int rn = lane >> 3, rc = lane & 7;       // as reader: slab column rn, 16-byte chunk rc (rows 8*rc .. 8*rc + 7)
    half4_t b4[4];
    if (bias) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) b4[mb] = *(const half4_t*)(bias + row0 + 16 * ib + 4 * mb);
    }
#pragma unroll
    for (int grp = 0; grp < 2; grp++) {
#pragma unroll
        for (int nb2 = 0; nb2 < 2; nb2++) {
            const int nb = grp * 2 + nb2;
            // slab 2*nb2 + hf takes the columns j16 = 8*hf .. 8*hf + 7 of block nb
            char* slab = stg + (nb2 * 2 + (j16 >> 3)) * TT_SLAB_BYTES;
#pragma unroll
            for (int mb = 0; mb < 4; mb++) {
                half4_t h4;
#pragma unroll
                for (int r = 0; r < 4; r++) h4[r] = (_Float16)acc[mb][nb][r];
                if (bias) h4 = h4 + b4[mb];
                *(half4_t*)(slab + (j16 & 7) * TT_PITCH + (16 * ib + 4 * mb) * 2) = h4;
            }
        }
        __builtin_amdgcn_wave_barrier();
        u32x4 v[4];
#pragma unroll
        for (int k = 0; k < 4; k++) v[k] = *(const u32x4*)(stg + k * TT_SLAB_BYTES + rn * TT_PITCH + rc * 16);
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const int col = col0 + (grp * 2 + (k >> 1)) * 16 + (k & 1) * 8 + rn;
            if (col < N && stores_on) store_c16<true>(C + (int64_t)col * rows_total + row0 + rc * 8, v[k]);
        }
    }
    __builtin_amdgcn_wave_barrier();
}

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
// STAGE_EPI: the consumers write a tile out through the memory of the stage they consumed last (a workgroup barrier at
// the end of every tile, which the producers join, makes it theirs until the next step barrier): room for four slabs
// per wave, so that a 64 x 64 block leaves in two LDS round trips instead of eight.
constexpr int WAVE_EPI_BYTES = 4 * TT_SLAB_BYTES + 128;      // four slabs of the larger kind + the block's bias values
template <int M, int NS, int NP, int NC_, bool STAGE_EPI_ = false>
struct DsCfg {
    static constexpr bool STAGE_EPI = STAGE_EPI_;
    static constexpr int NC = NC_;                 // consumer waves: 4 (128 x 64 each) or 8 (64 x 64 each)
    static constexpr int H = 8 / NC;               // 64-row blocks per consumer wave
    static_assert(NC == 4 || NC == 8, "consumer waves");
    static constexpr int BM = 256, BN = 128;
    static constexpr int ROW_BYTES = BN * 2;
    static constexpr int DENSE_ROWS = 16 * M;
    static constexpr int B_BYTES = DENSE_ROWS * ROW_BYTES;
    static constexpr int STAGE_BYTES = B_BYTES + 4 * APACK_BLOCK;
    static constexpr int PA = NS - 1;
    static constexpr int SLAB_BYTES = NC == 4 ? TR_SLAB_BYTES : (TR8_SLAB_BYTES > TT_SLAB_BYTES ? TR8_SLAB_BYTES : TT_SLAB_BYTES);
    static_assert(NC == 4 || SLAB_BYTES >= TR8_SLAB_BYTES + 128, "room for the block's bias values behind the 8-row slab");
    static constexpr int EPI_BYTES = NC * SLAB_BYTES;
    static constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + EPI_BYTES;
    static constexpr int THREADS = (NC + NP) * 64;
    static_assert(!STAGE_EPI || (NC == 8 && NC * WAVE_EPI_BYTES <= STAGE_BYTES), "the write-out slabs must fit one stage");
};

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
    static int cus = 0;
    void (*kern)(SpmmParams);
    if constexpr (PINGPONG) kern = spmm_dspp_kernel<M, NS, NP, OUT_LAYOUT>;
    else kern = spmm_ds_kernel<M, NS, NP, NC, OUT_LAYOUT, HALF>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        int dev = 0;
        if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
        if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
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
// M_ = 8: 32 KB stages, four of them; M_ = 16 (m <= 16): 64 KB stages, two of them - the stage for step q + 1 is issued
// at the head of step q and has that step to land.
template <int M_>
struct DuCfg {
    static_assert(M_ == 8 || M_ == 16, "dense rows per group a stage is sized for");
    static constexpr int BM = 512, BN = 128, M = M_, NS = M_ == 8 ? 4 : 2, PA = NS - 1;
    static constexpr int NB = M_ / 2;              // DMA instructions per wave and stage (4 rows x 256 B each)
    static constexpr int ROW_BYTES = BN * 2;
    static constexpr int STAGE_BYTES = 16 * M * ROW_BYTES;
    static constexpr int SLAB_BYTES = TT_SLAB_BYTES;
    static_assert(SLAB_BYTES >= TR8_SLAB_BYTES + 128, "slab");
    static constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + 8 * SLAB_BYTES;
    static constexpr int THREADS = 512;
};

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
            // a bias alone rides in the row-major write-out itself (packed fp16 additions); anything else goes first
            const bool pre = FUSE && (p.act != SPATHA_ACT_NONE || OUT_LAYOUT == SPATHA_OUT_TRANSPOSED);
#pragma unroll
            for (int wn = 0; wn < 2; wn++) {
                if (FUSE && pre) fused_bias_act(acc[wn], p.bias, (int64_t)cm0 + ib * 16, p.act);
                if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED)
                    store_block_transposed_slab<true>(acc[wn], stg, p.C, FUSE ? nullptr : p.bias, (int64_t)cm0, cn0 + wn * 64, p.rows,
                                                      N, lane, true);
                else if (FUSE && !pre && p.bias)
                    store_block_row_major_tr<true, true>(acc[wn], stg, p.C, (int64_t)cm0, cn0 + wn * 64, N, lane, true, p.bias);
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
    static int cus = 0;
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
        int dev = 0;
        if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
        if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
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

// ---------------------------------------------------------------------------
// Dense-staged kernel without workgroup barriers in the main loop ("flag-synchronised").
//
// A step of the barrier-synchronised kernels above costs the matrix pipes several hundred idle
// clocks: every wave has to issue its last instruction of the step before any wave may start the
// next one.  Here each stage of the ring carries two monotonic counters in LDS instead:
//   full[stage]  += 1 by every producer wave once its share of the stage has landed (vmcnt),
//   empty[stage] += 1 by every consumer wave once it has read the stage into registers.
// A consumer polls full >= NP * (use + 1) before reading, a producer polls empty >= NC * use
// before overwriting, so waves only ever wait for data, never for each other.  Polls are
// bounded (SPIN_LIMIT) so that a logic error ends in wrong results, not in a hang.
// The gather table travels with the stage (512 B per k-step, tile-major copy of it), so consumer
// waves issue no global loads at all and never wait for their own stores.
// ---------------------------------------------------------------------------
constexpr int SPIN_LIMIT = 1 << 20;

template <int SLEEP = 1>
__device__ __forceinline__ void flag_wait(uint32_t lds_addr, uint32_t target) {
    for (int spin = 0; spin < SPIN_LIMIT; spin++) {
        uint32_t v;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(lds_addr) : "memory");
        if ((int)((uint32_t)__builtin_amdgcn_readfirstlane((int)v) - target) >= 0) break;
        __builtin_amdgcn_s_sleep(SLEEP);
    }
}

// all LDS reads of this wave have landed -> bump the counter (one lane)
__device__ __forceinline__ void flag_signal(uint32_t lds_addr, int lane) {
    if (lane == 0) {
        const uint32_t one = 1;
        asm volatile("s_waitcnt lgkmcnt(0)\n\tds_add_u32 %0, %1" ::"v"(lds_addr), "v"(one) : "memory");
    }
}

template <int M, int NS, int NP>
struct DsfCfg {
    static constexpr int NC = 8;
    static constexpr int BM = 256, BN = 128;
    static constexpr int B_BYTES = 16 * M * BN * 2;
    static constexpr int GT_OFF = B_BYTES + 4 * APACK_BLOCK;
    static constexpr int GT_BYTES = 512;
    static constexpr int STAGE_BYTES = GT_OFF + GT_BYTES;
    static constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    static constexpr int EPI_BYTES = NC * TR8_SLAB_BYTES;
    static constexpr uint32_t FLAG_BASE = EPI_BASE + EPI_BYTES;     // full[NS], empty[NS]
    static constexpr int LDS_BYTES = FLAG_BASE + 64;
    static constexpr int THREADS = (NC + NP) * 64;
};

template <class Cfg, int M, int NS, int NP, int PR>
__device__ __forceinline__ void dsf_producer(const SpmmParams& p, const TileWalk& walk, uint32_t smem_base, int lane) {
    constexpr int BN = Cfg::BN;
    constexpr int B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    constexpr int NB_LOADS = (4 * M) / NP;
    constexpr int NA_LOADS = 24 / NP;
    constexpr int NG_LOADS = PR < 2 ? 1 : 0;         // the 512-byte gather table slice: two 256-byte pieces
    constexpr int LOADS = NB_LOADS + NA_LOADS + NG_LOADS;
    static_assert((4 * M) % NP == 0 && 24 % NP == 0 && NP >= 2, "DMA work must split evenly over the producers");
    const int S = p.S, N = p.N;
    const int Q = walk.my_tiles * S;
    const i32x4 rsrc_b = make_buffer(p.B, p.b_bytes);
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const i32x4 rsrc_g = make_buffer(p.gtab_tiles, p.gtab_tiles_bytes);
    const uint32_t row_bytes_b = (uint32_t)N * 2u;
    const int dense_rows = 16 * p.m;
    const uint32_t step_bytes_b = (uint32_t)dense_rows * row_bytes_b;
    const int slot_row = lane >> 4, slot_chunk = lane & 15;
    const uint32_t lane16 = lane * 16, lane4 = lane * 4;
    const uint32_t full_base = smem_base + Cfg::FLAG_BASE, empty_base = full_base + NS * 4;

    int is_tm = walk.tm0, is_tn = walk.tn0, is_step = 0;
    uint32_t b_soff = 0;
    uint32_t a_soff = (uint32_t)((is_tm * 4) * S) * (uint32_t)APACK_BLOCK;
    uint32_t g_soff = (uint32_t)(is_tm * S) * 512u + PR * 256u;
    uint32_t voff[NB_LOADS];
    auto set_voff = [&]() {
#pragma unroll
        for (int j = 0; j < NB_LOADS; j++) {
            const int row = (PR * NB_LOADS + j) * 4 + slot_row;
            const int col = is_tn * BN + (slot_chunk ^ ((row & 7) << 1)) * 8;
            voff[j] = (col < N && row < dense_rows && !SPATHA_KNOB(1)) ? (uint32_t)row * row_bytes_b + (uint32_t)col * 2u
                                                                       : 0xF0000000u;
        }
    };
    set_voff();
    int st = 0, prev_st = 0;            // ring slot of the batch being issued / of the one before it
    uint32_t use = 0;                   // how often slot `st` has been filled before
    bool pending = false;               // a batch is in flight whose stage has not been published yet
    for (int q = 0; q < Q; q++) {
        if (use > 0) {
            // if the slot is still being read, publish what is in flight first: a consumer must never wait for a
            // stage that has landed only because this wave waits for another one to drain
            uint32_t v;
            asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(v) : "v"(empty_base + st * 4) : "memory");
            if ((int)((uint32_t)__builtin_amdgcn_readfirstlane((int)v) - (uint32_t)Cfg::NC * use) < 0) {
                if (pending) {
                    wait_vmcnt<0>();
                    flag_signal(full_base + prev_st * 4, lane);
                    pending = false;
                }
                flag_wait(empty_base + st * 4, (uint32_t)Cfg::NC * use);
            }
        }
        if (!SPATHA_KNOB(8)) {
            const uint32_t stage = smem_base + st * STAGE_BYTES;
            const i32x4 rsrc_step = buffer_window(p.B, p.b_bytes, b_soff);      // rows of the step beyond K: zeros
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
            if (NG_LOADS) bdma_b32(lane4, rsrc_g, g_soff, stage + Cfg::GT_OFF + PR * 256);
        }
        a_soff += (uint32_t)APACK_BLOCK;
        b_soff += step_bytes_b;
        g_soff += 512u;
        if (++is_step == S) {
            is_step = 0;
            b_soff = 0;
            walk.next(is_tm, is_tn);
            a_soff = (uint32_t)((is_tm * 4) * S) * (uint32_t)APACK_BLOCK;
            g_soff = (uint32_t)(is_tm * S) * 512u + PR * 256u;
            set_voff();
        }
        if (pending) {
            // everything but the batch just issued has landed: publish the previous batch
            if (!SPATHA_KNOB(8)) wait_vmcnt<LOADS>();
            flag_signal(full_base + prev_st * 4, lane);
        }
        pending = true;
        prev_st = st;
        if (++st == NS) {
            st = 0;
            ++use;
        }
    }
    wait_vmcnt<0>();
    if (pending) flag_signal(full_base + prev_st * 4, lane);
}

// Consumer of the flag-synchronised kernel.  All operands are read one step ahead: while the 16
// matrix instructions of step q issue, every fragment's registers are re-loaded from the stage
// of step q+1 as soon as the instructions that read them are out; the A operands go to a second
// register set early in the step.  The counter of stage q+1 is requested (not waited for) behind
// the first four instructions of step q and checked behind the next four: LDS reads return in
// order, so by then the operand reads of step q, issued a whole step earlier, have long landed and
// the check costs no LDS round trip.  A stage is handed back to the producers as soon as it sits
// in registers, before it is multiplied, and the next tile's first stage loads while this tile
// is written out.
template <class Cfg, int NS, int NP, int OUT_LAYOUT>
__device__ __forceinline__ void dsf_consumer(const SpmmParams& p, const TileWalk& walk, char* smem, uint32_t smem_base,
                                             int wave, int lane) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN;
    constexpr int B_BYTES = Cfg::B_BYTES, STAGE_BYTES = Cfg::STAGE_BYTES;
    const int S = p.S, N = p.N;
    const int Q = walk.my_tiles * S;
    const int rb0 = wave & 3, wn = (wave >> 2) & 1;      // 64-row block, column half
    float4_t acc[4][4];
    SPATHA_PROF_DECL
    const int li = lane & 15, kb = lane >> 4;
    const uint32_t col_xor = (uint32_t)((wn * 8 + ((li & 3) >> 1)) << 4);
    const uint32_t col_or = (uint32_t)(li & 1) * 8u;
    const int a_off = B_BYTES + rb0 * APACK_BLOCK + lane * 16;
    const int i_off = B_BYTES + rb0 * APACK_BLOCK + 4096 + lane * 4;
    const int g_off = Cfg::GT_OFF + rb0 * 128 + (kb * 4 + (li >> 2)) * 8;
    const int j16 = lane & 15, ib = lane >> 4;
    const uint32_t full_base = smem_base + Cfg::FLAG_BASE, empty_base = full_base + NS * 4;

    half8_t a_cur[4];
    uint32_t i0, i1;
    half16_t bf[4];
    uint32_t base[4];
    auto set_base = [&](u32x2 g) {
        base[0] = ((g.x & 0xffffu) ^ col_xor) | col_or;
        base[1] = ((g.x >> 16) ^ col_xor) | col_or;
        base[2] = ((g.y & 0xffffu) ^ col_xor) | col_or;
        base[3] = ((g.y >> 16) ^ col_xor) | col_or;
    };
    auto read_frag = [&](const char* stg, int nb) {
#pragma unroll
        for (int fb = 0; fb < 4; fb++) {
            short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, stg + (base[fb] ^ (uint32_t)(nb << 5))));
            half4_t h4 = __builtin_bit_cast(half4_t, t4);
            bf[nb][fb * 4 + 0] = h4[0];
            bf[nb][fb * 4 + 1] = h4[1];
            bf[nb][fb * 4 + 2] = h4[2];
            bf[nb][fb * 4 + 3] = h4[3];
        }
    };
    auto read_a = [&](const char* stg) {
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(stg + a_off + mb * 1024);
        i0 = *(const uint32_t*)(stg + i_off);
        i1 = *(const uint32_t*)(stg + i_off + 256);
    };
#define SPATHA_MMA4F(NB)                                                                                 \
    acc[0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], bf[NB], acc[0][NB], (int)i0, 0, 0);  \
    acc[1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], bf[NB], acc[1][NB], (int)i0, 0, 1);  \
    acc[2][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[2], bf[NB], acc[2][NB], (int)i1, 0, 0);  \
    acc[3][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[3], bf[NB], acc[3][NB], (int)i1, 0, 1);
    auto zero_acc = [&]() {
#pragma unroll
        for (int a = 0; a < 4; a++)
#pragma unroll
            for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
    };

    int c_tm = walk.tm0, c_tn = walk.tn0, c_step = 0;
    int st = 0;
    uint32_t use = 0;
    zero_acc();
    half8_t a_nxt[4];
    uint32_t j0, j1;
    // prologue: stage of step 0 into registers
    flag_wait(full_base, (uint32_t)NP);
    {
        const char* stg = smem;
        set_base(*(const u32x2*)(stg + g_off));
        read_a(stg);
        read_frag(stg, 0);
        read_frag(stg, 1);
        read_frag(stg, 2);
        read_frag(stg, 3);
    }
    for (int q = 0; q < Q; q++) {
        int nst = st + 1;
        uint32_t nuse = use;
        if (nst == NS) {
            nst = 0;
            ++nuse;
        }
        const bool have_next = q + 1 < Q;
        // after the last step there is nothing to prefetch: re-read the current stage (never overwritten again)
        const char* stg = smem + (have_next ? nst : st) * STAGE_BYTES;
        const uint32_t flag_addr = full_base + (have_next ? nst : st) * 4;
        const uint32_t target = (uint32_t)NP * ((have_next ? nuse : use) + 1);
        SPATHA_PROF_MARK(0)
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA4F(0)
        __builtin_amdgcn_sched_barrier(0);
        // counter and gather-table entry of the next stage, requested behind the first instructions of this step
        uint32_t flag;
        asm volatile("ds_read_b32 %0, %1" : "=v"(flag) : "v"(flag_addr) : "memory");
        u32x2 g = *(const u32x2*)(stg + g_off);
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA4F(1)
        __builtin_amdgcn_sched_barrier(0);
        // LDS reads return in order: with the counter, everything of this step's stage has landed as well
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(flag), "+v"(g)::"memory");
        if ((int)((uint32_t)__builtin_amdgcn_readfirstlane((int)flag) - target) < 0) {
            SPATHA_PROF_MARK(0)
            flag_wait(flag_addr, target);
            g = *(const u32x2*)(stg + g_off);
            SPATHA_PROF_MARK(1)
        }
        flag_signal(empty_base + st * 4, lane);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_nxt[mb] = *(const half8_t*)(stg + a_off + mb * 1024);
        j0 = *(const uint32_t*)(stg + i_off);
        j1 = *(const uint32_t*)(stg + i_off + 256);
        set_base(g);
        read_frag(stg, 0);
        read_frag(stg, 1);
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA4F(2)
        __builtin_amdgcn_sched_barrier(0);
        read_frag(stg, 2);
        __builtin_amdgcn_sched_barrier(0);
        SPATHA_MMA4F(3)
        __builtin_amdgcn_sched_barrier(0);
        read_frag(stg, 3);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a_cur[mb] = a_nxt[mb];
        i0 = j0;
        i1 = j1;
        st = nst;
        use = nuse;
        if (++c_step == S) {
            c_step = 0;
            const int cm0 = c_tm * BM + rb0 * 64, cn0 = c_tn * BN;
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
                store_block_row_major_tr<true>(acc, smem + Cfg::EPI_BASE + wave * TR8_SLAB_BYTES, p.C, (int64_t)cm0,
                                               cn0 + wn * 64, N, lane, !SPATHA_KNOB(2));
            }
            SPATHA_PROF_MARK(2)
            zero_acc();
            walk.next(c_tm, c_tn);
        }
    }
#undef SPATHA_MMA4F
    SPATHA_PROF_FLUSH
}

template <int M, int NS, int NP, int OUT_LAYOUT>
__global__ __launch_bounds__((8 + NP) * 64) void spmm_dsf_kernel(SpmmParams p) {
    using Cfg = DsfCfg<M, NS, NP>;
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    if (tid < 16) *(uint32_t*)(smem + Cfg::FLAG_BASE + tid * 4) = 0u;
    __syncthreads();
    if (wave < 8) {
        dsf_consumer<Cfg, NS, NP, OUT_LAYOUT>(p, walk, smem, smem_base, wave, lane);
    } else {
        const int pr = wave - 8;
        if (pr == 0) dsf_producer<Cfg, M, NS, NP, 0>(p, walk, smem_base, lane);
        else if (pr == 1) dsf_producer<Cfg, M, NS, NP, 1>(p, walk, smem_base, lane);
        else if (pr == 2) dsf_producer<Cfg, M, NS, NP, 2>(p, walk, smem_base, lane);
        else dsf_producer<Cfg, M, NS, NP, 3>(p, walk, smem_base, lane);
    }
}

template <int M, int NS, int NP, int OUT_LAYOUT>
static hipError_t launch_dsf(const SpmmParams& p, hipStream_t stream) {
    using Cfg = DsfCfg<M, NS, NP>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    static int cus = 0;
    auto kern = spmm_dsf_kernel<M, NS, NP, OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        int dev = 0;
        if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
        if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
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

// tile-major copy of the gather table for the flag-synchronised kernel:
// [256-row tile][step][64-row block in tile][kb][c][fb] u16, 512 contiguous bytes per (tile, step)
__global__ void pack_gtab_tiles_kernel(const uint32_t* __restrict__ columns, int rows, int m, int v, int ksp, int S,
                                       uint16_t* __restrict__ gtab) {
    const int ngroups = ksp / 2;
    const int64_t total = (int64_t)(rows / 256) * S * 256;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int fb = (int)(t & 3), c = (int)((t >> 2) & 3), kb = (int)((t >> 4) & 3), rb = (int)((t >> 6) & 3);
        const int64_t ts = t >> 8;
        const int s = (int)(ts % S);
        const int64_t tile = ts / S;
        const int64_t b = (tile * 256 + rb * 64) / v;
        const int gamma = fb * 4 + kb;
        const int g = s * 16 + gamma;
        uint32_t d = (uint32_t)gamma * m;
        if (g < ngroups) d += columns[b * ngroups * 4 + (int64_t)g * 4 + c];
        gtab[t] = (uint16_t)(d * 256u + (d & 7u) * 32u);
    }
}

hipError_t launch_pack_gtab_tiles(const uint32_t* columns, int rows, int m, int v, int ksp, int S, uint16_t* gtab,
                                  hipStream_t stream) {
    int64_t total = (int64_t)(rows / 256) * S * 256;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 65535 * 8) blocks = 65535 * 8;
    hipLaunchKernelGGL(pack_gtab_tiles_kernel, dim3(blocks), dim3(256), 0, stream, columns, rows, m, v, ksp, S, gtab);
    return hipGetLastError();
}

// ---------------------------------------------------------------------------
// Skinny-N kernel (N <= 64): the product is bound by streaming A from HBM, not by the matrix units.
// One workgroup per 64-row tile; its four waves split the k-steps (wave w takes steps w, w+4, ...),
// so that 4 * rows/64 waves keep loads in flight, and add their fp32 partial tiles through LDS at the
// end in a fixed order.  No LDS staging of B: a lane fetches the 16 elements of its B fragment
// straight from global memory (B is small and stays in L2) through a buffer descriptor whose bounds
// check returns the zeros of padding rows and of columns beyond N.  Operands of step i+1 and the row
// table of step i+2 are requested before step i is multiplied.
// ---------------------------------------------------------------------------
template <int NB, int OUT_LAYOUT>
__global__ __launch_bounds__(256) void spmm_skinny_kernel(SpmmParams p) {
    __shared__ float4_t red[4][4][NB][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = blockIdx.x;
    const int S = p.S, N = p.N;
    const int li = lane & 15, kb = lane >> 4;
    const int64_t vb = ((int64_t)tile * 64) / p.v;
    const char* a_tile = (const char*)p.apack + (int64_t)tile * S * APACK_BLOCK;
    const uint32_t* rt_block = p.rowtab + vb * S * 64;
    __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)p.B, 0, (int)p.b_bytes, 0x00020000);
    const uint32_t row_bytes = (uint32_t)N * 2u;

    float4_t acc[4][NB];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < NB; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

    auto clamp_step = [&](int st) { return st < S ? st : S - 1; };
    auto load_rt = [&](int st, u32x4 (&rt)[4]) {
        const uint32_t* q = rt_block + (int64_t)clamp_step(st) * 64 + 4 * kb;
#pragma unroll
        for (int fb = 0; fb < 4; fb++) rt[fb] = *(const u32x4*)(q + 16 * fb);
    };
    auto load_a = [&](int st, half8_t (&a)[4], uint32_t& i0, uint32_t& i1) {
        const char* q = a_tile + (int64_t)clamp_step(st) * APACK_BLOCK;
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a[mb] = *(const half8_t*)(q + mb * 1024 + lane * 16);
        i0 = *(const uint32_t*)(q + 4096 + lane * 4);
        i1 = *(const uint32_t*)(q + 4352 + lane * 4);
    };
    auto load_b = [&](const u32x4 (&rt)[4], half16_t (&bf)[NB]) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const int col = nb * 16 + li;
#pragma unroll
            for (int fb = 0; fb < 4; fb++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t row = rt[fb][j];
                    const uint32_t voff = (row != 0xFFFFFFFFu && col < N) ? row * row_bytes + (uint32_t)col * 2u : 0xF0000000u;
                    const uint16_t h = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc_b, (int)voff, 0, 0);
                    bf[nb][fb * 4 + j] = __builtin_bit_cast(_Float16, h);
                }
        }
    };

    u32x4 rt1[4], rt2[4];
    half8_t a0[4], a1[4];
    uint32_t i00, i01, i10, i11;
    half16_t b0[NB], b1[NB];
    int st = wave;
    load_rt(st, rt1);
    load_a(st, a0, i00, i01);
    load_b(rt1, b0);
    load_rt(st + 4, rt1);
    for (; st < S; st += 4) {
        load_rt(st + 8, rt2);
        load_a(st + 4, a1, i10, i11);
        load_b(rt1, b1);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            acc[0][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[0], b0[nb], acc[0][nb], (int)i00, 0, 0);
            acc[1][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[1], b0[nb], acc[1][nb], (int)i00, 0, 1);
            acc[2][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[2], b0[nb], acc[2][nb], (int)i01, 0, 0);
            acc[3][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[3], b0[nb], acc[3][nb], (int)i01, 0, 1);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            a0[k] = a1[k];
            rt1[k] = rt2[k];
        }
        i00 = i10;
        i01 = i11;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) b0[nb] = b1[nb];
    }
#pragma unroll
    for (int mb = 0; mb < 4; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) red[wave][mb][nb][lane] = acc[mb][nb];
    __syncthreads();
    // wave w finishes instruction-row block mb = w: rows 16*ib + 4*mb + r of the tile, column nb*16 + li
    const int mb = wave, ib = kb;
    const int64_t row0 = (int64_t)tile * 64 + 16 * ib + 4 * mb;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        float4_t sum = ((red[0][mb][nb][lane] + red[1][mb][nb][lane]) + red[2][mb][nb][lane]) + red[3][mb][nb][lane];
        const int col = nb * 16 + li;
        half4_t h4;
#pragma unroll
        for (int r = 0; r < 4; r++) h4[r] = (_Float16)sum[r];
        if (col >= N || SPATHA_KNOB(2)) continue;
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            if (p.bias) h4 = h4 + *(const half4_t*)(p.bias + row0);
            *(half4_t*)(p.C + (int64_t)col * p.rows + row0) = h4;
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++) *(_Float16*)(p.C + (row0 + r) * N + col) = h4[r];
        }
    }
}

template <int OUT_LAYOUT>
static hipError_t launch_skinny(const SpmmParams& p, hipStream_t stream) {
    const int nb = (p.N + 15) / 16;
    const dim3 grid(p.rows / 64), block(256);
    if (nb <= 1) hipLaunchKernelGGL((spmm_skinny_kernel<1, OUT_LAYOUT>), grid, block, 0, stream, p);
    else if (nb == 2) hipLaunchKernelGGL((spmm_skinny_kernel<2, OUT_LAYOUT>), grid, block, 0, stream, p);
    else if (nb == 3) hipLaunchKernelGGL((spmm_skinny_kernel<3, OUT_LAYOUT>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((spmm_skinny_kernel<4, OUT_LAYOUT>), grid, block, 0, stream, p);
    return hipGetLastError();
}

// gather table of the dense-staged kernel: [64-row block][step][kb][c][fb] u16 = LDS byte offset of dense
// row d = gamma*m + column-loc (gamma = 4*fb + kb): d*256 + (d % 8)*32 (the swizzle of that row)
__global__ void pack_gtab_kernel(const uint32_t* __restrict__ columns, int rows, int m, int v, int ksp, int S,
                                 int block_rows, uint16_t* __restrict__ gtab) {
    const int ngroups = ksp / 2;
    const int64_t total = (int64_t)(rows / block_rows) * S * 64;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int fb = (int)(t & 3), c = (int)((t >> 2) & 3), kb = (int)((t >> 4) & 3);
        const int64_t bs = t >> 6;
        const int s = (int)(bs % S);
        const int64_t b = (bs / S) * block_rows / v;          // V block of this 64-row (or, for V = 32, 32-row) block
        const int gamma = fb * 4 + kb;
        const int g = s * 16 + gamma;
        uint32_t d = (uint32_t)gamma * m;
        if (g < ngroups) d += columns[b * ngroups * 4 + (int64_t)g * 4 + c];
        gtab[t] = (uint16_t)(d * 256u + (d & 7u) * 32u);
    }
}

hipError_t launch_pack_gtab(const uint32_t* columns, int rows, int m, int v, int ksp, int S, int block_rows, uint16_t* gtab,
                            hipStream_t stream) {
    int64_t total = (int64_t)(rows / block_rows) * S * 64;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 65535 * 8) blocks = 65535 * 8;
    hipLaunchKernelGGL(pack_gtab_kernel, dim3(blocks), dim3(256), 0, stream, columns, rows, m, v, ksp, S, block_rows, gtab);
    return hipGetLastError();
}

template <int WM, int WN, int NS, int NP, int OUT_LAYOUT, bool DEFER = false>
__global__ __launch_bounds__((WM * WN + NP) * 64) void spmm_ws_kernel(SpmmParams p) {
    using Cfg = WsCfg<WM, WN, NS, NP>;
    static_assert(NP == 2 || NP == 4, "producer count");
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    TileWalk walk;
    walk.init(p.tiles_m, p.tiles_n);
    if (walk.my_tiles == 0) return;
    // Workgroups of one XCD start up to 7 * skew apart, so that tiles do not all finish (and
    // hit HBM with their stores) at the same moment on every CU.
    if (SPATHA_SKEW_ON(p)) {
        const int units = ((blockIdx.x >> 3) & 7) * p.skew;
        for (int i = 0; i < units; i++) __builtin_amdgcn_s_sleep(16);      // 16 * 64 clocks
    }
    if (wave < Cfg::NC) {
        if (DEFER) ws_consumer_deferred<Cfg, WN, OUT_LAYOUT>(p, walk, smem, wave, lane);
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

template <int WM, int WN, int NS, int NP, int OUT_LAYOUT, bool DEFER = false>
static hipError_t launch_ws(const SpmmParams& p, hipStream_t stream) {
    using Cfg = WsCfg<WM, WN, NS, NP>;
    constexpr int lds = Cfg::LDS_BYTES;
    static_assert(lds <= 160 * 1024, "LDS budget");
    static int cus = 0;
    auto kern = spmm_ws_kernel<WM, WN, NS, NP, OUT_LAYOUT, DEFER>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return e;
        int dev = 0;
        if ((e = hipGetDevice(&dev)) != hipSuccess) return e;
        if ((e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev)) != hipSuccess) return e;
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

const char* spmm_variant_name(int variant) {
    switch (variant) {
        case SPMM_VARIANT_128x128: return "smfmac16x16x64_wg256_tile128x128";
        case SPMM_VARIANT_64x256: return "smfmac16x16x64_wg256_tile64x256";
        case SPMM_VARIANT_P128x128_S4: return "smfmac16x16x64_ldsdirect_tile128x128_4stage";
        case SPMM_VARIANT_P128x128_S3: return "smfmac16x16x64_ldsdirect_tile128x128_3stage";
        case SPMM_VARIANT_P64x256_S2: return "smfmac16x16x64_ldsdirect_tile64x256_2stage";
        case SPMM_VARIANT_P64x256_S3: return "smfmac16x16x64_ldsdirect_tile64x256_3stage";
        case SPMM_VARIANT_P128x128_S6: return "smfmac16x16x64_ldsdirect_tile128x128_6stage";
        case SPMM_VARIANT_P64x256_S4: return "smfmac16x16x64_ldsdirect_tile64x256_4stage";
        case SPMM_VARIANT_R128x128_S4: return "smfmac16x16x64_persistent_tile128x128_4stage";
        case SPMM_VARIANT_R128x128_S5: return "smfmac16x16x64_persistent_tile128x128_5stage";
        case SPMM_VARIANT_R128x128_S2: return "smfmac16x16x64_persistent_tile128x128_2stage";
        case SPMM_VARIANT_R64x256_S3: return "smfmac16x16x64_persistent_tile64x256_3stage";
        case SPMM_VARIANT_R64x256_S4: return "smfmac16x16x64_persistent_tile64x256_4stage";
        case SPMM_VARIANT_W128x128_S5: return "smfmac16x16x64_warpspec_tile128x128_5stage";
        case SPMM_VARIANT_W128x128_S3: return "smfmac16x16x64_warpspec_tile128x128_3stage";
        case SPMM_VARIANT_W128x128_S2: return "smfmac16x16x64_warpspec_tile128x128_2stage";
        case SPMM_VARIANT_W128x256_S3: return "smfmac16x16x64_warpspec_tile128x256_3stage";
        case SPMM_VARIANT_W64x256_S2: return "smfmac16x16x64_warpspec_tile64x256_2stage";
        case SPMM_VARIANT_W64x256_S3: return "smfmac16x16x64_warpspec_tile64x256_3stage";
        case SPMM_VARIANT_D128x256_S3: return "smfmac16x16x64_warpspec_deferred_tile128x256_3stage";
        case SPMM_VARIANT_D128x128_S3: return "smfmac16x16x64_warpspec_deferred_tile128x128_3stage";
        case SPMM_VARIANT_D128x128_S5: return "smfmac16x16x64_warpspec_deferred_tile128x128_5stage";
        case SPMM_VARIANT_D64x256_S3: return "smfmac16x16x64_warpspec_deferred_tile64x256_3stage";
        case SPMM_VARIANT_T128x256_S3: return "smfmac16x16x64_warpspec_tall_tile128x256_3stage";
        case SPMM_VARIANT_T128x128_S4: return "smfmac16x16x64_warpspec_tall_tile128x128_4stage";
        case SPMM_VARIANT_T128x128_S5: return "smfmac16x16x64_warpspec_tall_tile128x128_5stage";
        case SPMM_VARIANT_DS256x128_S3: return "smfmac16x16x64_warpspec_densestage_tile256x128_3stage";
        case SPMM_VARIANT_DS256x128_S2: return "smfmac16x16x64_warpspec_densestage_tile256x128_2stage";
        case SPMM_VARIANT_DS256x128_S3_C8: return "smfmac16x16x64_warpspec_densestage_tile256x128_3stage_8consumers";
        case SPMM_VARIANT_DS256x128_S3_PP: return "smfmac16x16x64_warpspec_densestage_tile256x128_3stage_pingpong";
        case SPMM_VARIANT_DSF256x128_S3: return "smfmac16x16x64_warpspec_densestage_flagsync_tile256x128_3stage";
        case SPMM_VARIANT_SKINNY: return "smfmac16x16x64_skinny_tile64xN_splitk4";
        case SPMM_VARIANT_H64x256_S2: return "smfmac16x16x64_halftile_ldsdirect_tile64x256_2stage";
        case SPMM_VARIANT_H64x128_S3: return "smfmac16x16x64_halftile_ldsdirect_tile64x128_3stage";
        case SPMM_VARIANT_H64x128_S2: return "smfmac16x16x64_halftile_ldsdirect_tile64x128_2stage";
        case SPMM_VARIANT_DSH256x128_S3_C8: return "smfmac16x16x64_halftile_densestage_tile256x128_3stage_8consumers";
        case SPMM_VARIANT_DU512x128_S4: return "smfmac16x16x64_unified_densestage_aregs_tile512x128_4stage";
        case SPMM_VARIANT_DU512x128_M16: return "smfmac16x16x64_unified_densestage_aregs_tile512x128_m16_2stage";
        default: return nullptr;
    }
}

// LDS bytes the variant needs for S k-steps (pipelined variants keep the row table in LDS)
int spmm_variant_lds(int variant, int S) {
    switch (variant) {
        case SPMM_VARIANT_P128x128_S4: return 4 * (64 * 128 * 2 + 2 * APACK_BLOCK) + S * 256;
        case SPMM_VARIANT_P128x128_S3: return 3 * (64 * 128 * 2 + 2 * APACK_BLOCK) + S * 256;
        case SPMM_VARIANT_P128x128_S6: return 6 * (64 * 128 * 2 + 2 * APACK_BLOCK) + S * 256;
        case SPMM_VARIANT_P64x256_S2: return 2 * (64 * 256 * 2 + APACK_BLOCK) + S * 256;
        case SPMM_VARIANT_P64x256_S3: return 3 * (64 * 256 * 2 + APACK_BLOCK) + S * 256;
        case SPMM_VARIANT_P64x256_S4: return 4 * (64 * 256 * 2 + APACK_BLOCK) + S * 256;
        case SPMM_VARIANT_R128x128_S4: return PersistCfg<2, 2, 4>::LDS_BYTES;
        case SPMM_VARIANT_R128x128_S5: return PersistCfg<2, 2, 5>::LDS_BYTES;
        case SPMM_VARIANT_R128x128_S2: return PersistCfg<2, 2, 2>::LDS_BYTES;
        case SPMM_VARIANT_R64x256_S3: return PersistCfg<1, 4, 3>::LDS_BYTES;
        case SPMM_VARIANT_R64x256_S4: return PersistCfg<1, 4, 4>::LDS_BYTES;
        case SPMM_VARIANT_W128x128_S5: return WsCfg<2, 2, 5, 4>::LDS_BYTES;
        case SPMM_VARIANT_W128x128_S3: return WsCfg<2, 2, 3, 4>::LDS_BYTES;
        case SPMM_VARIANT_W128x128_S2: return WsCfg<2, 2, 2, 4>::LDS_BYTES;
        case SPMM_VARIANT_W128x256_S3: return WsCfg<2, 4, 3, 4>::LDS_BYTES;
        case SPMM_VARIANT_W64x256_S2: return WsCfg<1, 4, 2, 2>::LDS_BYTES;
        case SPMM_VARIANT_W64x256_S3: return WsCfg<1, 4, 3, 2>::LDS_BYTES;
        case SPMM_VARIANT_D128x256_S3: return WsCfg<2, 4, 3, 4>::LDS_BYTES;
        case SPMM_VARIANT_D128x128_S3: return WsCfg<2, 2, 3, 4>::LDS_BYTES;
        case SPMM_VARIANT_D128x128_S5: return WsCfg<2, 2, 5, 4>::LDS_BYTES;
        case SPMM_VARIANT_D64x256_S3: return WsCfg<1, 4, 3, 2>::LDS_BYTES;
        case SPMM_VARIANT_T128x256_S3: return WsCfg<2, 4, 3, 4>::LDS_BYTES;
        case SPMM_VARIANT_T128x128_S4: return WsCfg<2, 2, 4, 2>::LDS_BYTES;
        case SPMM_VARIANT_T128x128_S5: return WsCfg<2, 2, 5, 4>::LDS_BYTES;
        case SPMM_VARIANT_DS256x128_S3: return DsCfg<8, 3, 4, 4>::LDS_BYTES;
        case SPMM_VARIANT_DS256x128_S2: return DsCfg<8, 2, 4, 4>::LDS_BYTES;
        case SPMM_VARIANT_DS256x128_S3_C8: return DsCfg<8, 3, 4, 8>::LDS_BYTES;
        case SPMM_VARIANT_DS256x128_S3_PP: return DsCfg<8, 3, 4, 8>::LDS_BYTES;
        case SPMM_VARIANT_DSF256x128_S3: return DsfCfg<8, 3, 4>::LDS_BYTES;
        case SPMM_VARIANT_SKINNY: return 64 * 1024;
        case SPMM_VARIANT_H64x256_S2: return half_stage_bytes<4, 2>() + S * 256;
        case SPMM_VARIANT_H64x128_S3: return half_stage_bytes<2, 3>() + S * 256;
        case SPMM_VARIANT_H64x128_S2: return half_stage_bytes<2, 2>() + S * 256;
        case SPMM_VARIANT_DSH256x128_S3_C8: return DsCfg<8, 3, 4, 8>::LDS_BYTES;
        case SPMM_VARIANT_DU512x128_S4: return DuCfg<8>::LDS_BYTES;
        case SPMM_VARIANT_DU512x128_M16: return DuCfg<16>::LDS_BYTES;
        case SPMM_VARIANT_128x128: case SPMM_VARIANT_64x256: return 1;
        default: return 0;
    }
}

int spmm_variant_bm(int variant) {
    switch (variant) {
        case SPMM_VARIANT_128x128: case SPMM_VARIANT_P128x128_S4: case SPMM_VARIANT_P128x128_S3: case SPMM_VARIANT_P128x128_S6:
        case SPMM_VARIANT_R128x128_S4: case SPMM_VARIANT_R128x128_S5: case SPMM_VARIANT_R128x128_S2:
        case SPMM_VARIANT_W128x128_S5: case SPMM_VARIANT_W128x128_S3: case SPMM_VARIANT_W128x128_S2: case SPMM_VARIANT_W128x256_S3:
        case SPMM_VARIANT_D128x256_S3: case SPMM_VARIANT_D128x128_S3: case SPMM_VARIANT_D128x128_S5:
        case SPMM_VARIANT_T128x256_S3: case SPMM_VARIANT_T128x128_S4: case SPMM_VARIANT_T128x128_S5: return 128;
        case SPMM_VARIANT_R64x256_S3: case SPMM_VARIANT_R64x256_S4: case SPMM_VARIANT_W64x256_S2: case SPMM_VARIANT_W64x256_S3: case SPMM_VARIANT_D64x256_S3:
        case SPMM_VARIANT_64x256: case SPMM_VARIANT_P64x256_S2: case SPMM_VARIANT_P64x256_S3: case SPMM_VARIANT_P64x256_S4:
        case SPMM_VARIANT_SKINNY: case SPMM_VARIANT_H64x256_S2: case SPMM_VARIANT_H64x128_S3: case SPMM_VARIANT_H64x128_S2: return 64;
        case SPMM_VARIANT_DS256x128_S3: case SPMM_VARIANT_DS256x128_S2: case SPMM_VARIANT_DS256x128_S3_C8: case SPMM_VARIANT_DS256x128_S3_PP: case SPMM_VARIANT_DSF256x128_S3: case SPMM_VARIANT_DSH256x128_S3_C8: return 256;
        case SPMM_VARIANT_DU512x128_S4: case SPMM_VARIANT_DU512x128_M16: return 512;
        default: return 0;
    }
}
int spmm_variant_bn(int variant) {
    switch (variant) {
        case SPMM_VARIANT_128x128: case SPMM_VARIANT_P128x128_S4: case SPMM_VARIANT_P128x128_S3: case SPMM_VARIANT_P128x128_S6:
        case SPMM_VARIANT_R128x128_S4: case SPMM_VARIANT_R128x128_S5: case SPMM_VARIANT_R128x128_S2:
        case SPMM_VARIANT_W128x128_S5: case SPMM_VARIANT_W128x128_S3: case SPMM_VARIANT_W128x128_S2:
        case SPMM_VARIANT_D128x128_S3: case SPMM_VARIANT_D128x128_S5: case SPMM_VARIANT_T128x128_S4: case SPMM_VARIANT_T128x128_S5:
        case SPMM_VARIANT_DS256x128_S3: case SPMM_VARIANT_DS256x128_S2: case SPMM_VARIANT_DS256x128_S3_C8: case SPMM_VARIANT_DS256x128_S3_PP: case SPMM_VARIANT_DSF256x128_S3:
        case SPMM_VARIANT_H64x128_S3: case SPMM_VARIANT_H64x128_S2: case SPMM_VARIANT_DSH256x128_S3_C8:
        case SPMM_VARIANT_DU512x128_S4: case SPMM_VARIANT_DU512x128_M16: return 128;
        case SPMM_VARIANT_SKINNY: return 64;
        case SPMM_VARIANT_H64x256_S2: return 256;
        case SPMM_VARIANT_D128x256_S3: case SPMM_VARIANT_D64x256_S3: case SPMM_VARIANT_T128x256_S3:
        case SPMM_VARIANT_R64x256_S3: case SPMM_VARIANT_R64x256_S4: case SPMM_VARIANT_W64x256_S2: case SPMM_VARIANT_W64x256_S3: case SPMM_VARIANT_W128x256_S3:
        case SPMM_VARIANT_64x256: case SPMM_VARIANT_P64x256_S2: case SPMM_VARIANT_P64x256_S3: case SPMM_VARIANT_P64x256_S4: return 256;
        default: return 0;
    }
}

hipError_t launch_spmm(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    if (variant == SPMM_VARIANT_128x128) {
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_variant<2, 2, SPATHA_OUT_TRANSPOSED>(p, stream)
                                                   : launch_variant<2, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
    }
    if (variant == SPMM_VARIANT_64x256) {
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_variant<1, 4, SPATHA_OUT_TRANSPOSED>(p, stream)
                                                   : launch_variant<1, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
    }
#define SPATHA_PIPE_CASE(ID, WM_, WN_, NS_)                                                             \
    if (variant == ID)                                                                                  \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_pipe<WM_, WN_, NS_, SPATHA_OUT_TRANSPOSED>(p, stream) \
                                                   : launch_pipe<WM_, WN_, NS_, SPATHA_OUT_ROW_MAJOR>(p, stream);
    SPATHA_PIPE_CASE(SPMM_VARIANT_P128x128_S4, 2, 2, 4)
    SPATHA_PIPE_CASE(SPMM_VARIANT_P128x128_S3, 2, 2, 3)
    SPATHA_PIPE_CASE(SPMM_VARIANT_P64x256_S2, 1, 4, 2)
    SPATHA_PIPE_CASE(SPMM_VARIANT_P64x256_S3, 1, 4, 3)
    SPATHA_PIPE_CASE(SPMM_VARIANT_P128x128_S6, 2, 2, 6)
    SPATHA_PIPE_CASE(SPMM_VARIANT_P64x256_S4, 1, 4, 4)
#undef SPATHA_PIPE_CASE
#define SPATHA_PERSIST_CASE(ID, WM_, WN_, NS_)                                                          \
    if (variant == ID)                                                                                  \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_persist<WM_, WN_, NS_, SPATHA_OUT_TRANSPOSED>(p, stream) \
                                                   : launch_persist<WM_, WN_, NS_, SPATHA_OUT_ROW_MAJOR>(p, stream);
    SPATHA_PERSIST_CASE(SPMM_VARIANT_R128x128_S4, 2, 2, 4)
    SPATHA_PERSIST_CASE(SPMM_VARIANT_R128x128_S5, 2, 2, 5)
    SPATHA_PERSIST_CASE(SPMM_VARIANT_R128x128_S2, 2, 2, 2)
    SPATHA_PERSIST_CASE(SPMM_VARIANT_R64x256_S3, 1, 4, 3)
    SPATHA_PERSIST_CASE(SPMM_VARIANT_R64x256_S4, 1, 4, 4)
#undef SPATHA_PERSIST_CASE
#define SPATHA_WS_CASE(ID, WM_, WN_, NS_, NP_)                                                          \
    if (variant == ID)                                                                                  \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_ws<WM_, WN_, NS_, NP_, SPATHA_OUT_TRANSPOSED>(p, stream) \
                                                   : launch_ws<WM_, WN_, NS_, NP_, SPATHA_OUT_ROW_MAJOR>(p, stream);
    SPATHA_WS_CASE(SPMM_VARIANT_W128x128_S5, 2, 2, 5, 4)
    SPATHA_WS_CASE(SPMM_VARIANT_W128x128_S3, 2, 2, 3, 4)
    SPATHA_WS_CASE(SPMM_VARIANT_W128x128_S2, 2, 2, 2, 4)
    SPATHA_WS_CASE(SPMM_VARIANT_W128x256_S3, 2, 4, 3, 4)
    SPATHA_WS_CASE(SPMM_VARIANT_W64x256_S2, 1, 4, 2, 2)
    SPATHA_WS_CASE(SPMM_VARIANT_W64x256_S3, 1, 4, 3, 2)
#undef SPATHA_WS_CASE
#define SPATHA_WSD_CASE(ID, WM_, WN_, NS_, NP_)                                                         \
    if (variant == ID)                                                                                  \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_ws<WM_, WN_, NS_, NP_, SPATHA_OUT_TRANSPOSED, true>(p, stream) \
                                                   : launch_ws<WM_, WN_, NS_, NP_, SPATHA_OUT_ROW_MAJOR, true>(p, stream);
    SPATHA_WSD_CASE(SPMM_VARIANT_D128x256_S3, 2, 4, 3, 4)
    SPATHA_WSD_CASE(SPMM_VARIANT_D128x128_S3, 2, 2, 3, 4)
    SPATHA_WSD_CASE(SPMM_VARIANT_D128x128_S5, 2, 2, 5, 4)
    SPATHA_WSD_CASE(SPMM_VARIANT_D64x256_S3, 1, 4, 3, 2)
#undef SPATHA_WSD_CASE
#define SPATHA_WST_CASE(ID, WN_, NS_, NP_)                                                              \
    if (variant == ID)                                                                                  \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_wst<WN_, NS_, NP_, SPATHA_OUT_TRANSPOSED>(p, stream) \
                                                   : launch_wst<WN_, NS_, NP_, SPATHA_OUT_ROW_MAJOR>(p, stream);
    SPATHA_WST_CASE(SPMM_VARIANT_T128x256_S3, 4, 3, 4)
    SPATHA_WST_CASE(SPMM_VARIANT_T128x128_S4, 2, 4, 2)
    SPATHA_WST_CASE(SPMM_VARIANT_T128x128_S5, 2, 5, 4)
#undef SPATHA_WST_CASE
#define SPATHA_DS_CASE(V, NS, NC)                                                                              \
    if (variant == V)                                                                                          \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_ds<8, NS, 4, NC, SPATHA_OUT_TRANSPOSED>(p, stream) \
                                                   : launch_ds<8, NS, 4, NC, SPATHA_OUT_ROW_MAJOR>(p, stream);
    SPATHA_DS_CASE(SPMM_VARIANT_DS256x128_S3, 3, 4)
    SPATHA_DS_CASE(SPMM_VARIANT_DS256x128_S2, 2, 4)
    SPATHA_DS_CASE(SPMM_VARIANT_DS256x128_S3_C8, 3, 8)
#undef SPATHA_DS_CASE
#define SPATHA_HALF_CASE(ID, WN_, NS_)                                                                  \
    if (variant == ID)                                                                                  \
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_half<WN_, NS_, SPATHA_OUT_TRANSPOSED>(p, stream) \
                                                   : launch_half<WN_, NS_, SPATHA_OUT_ROW_MAJOR>(p, stream);
    SPATHA_HALF_CASE(SPMM_VARIANT_H64x256_S2, 4, 2)
    SPATHA_HALF_CASE(SPMM_VARIANT_H64x128_S3, 2, 3)
    SPATHA_HALF_CASE(SPMM_VARIANT_H64x128_S2, 2, 2)
#undef SPATHA_HALF_CASE
    if (variant == SPMM_VARIANT_SKINNY)
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_skinny<SPATHA_OUT_TRANSPOSED>(p, stream)
                                                   : launch_skinny<SPATHA_OUT_ROW_MAJOR>(p, stream);
    if (variant == SPMM_VARIANT_DSH256x128_S3_C8)
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_ds<8, 3, 4, 8, SPATHA_OUT_TRANSPOSED, false, true>(p, stream)
                                                   : launch_ds<8, 3, 4, 8, SPATHA_OUT_ROW_MAJOR, false, true>(p, stream);
    // (no fused write-out: that instantiation needs scratch memory, which the kernel's asynchronous register loads rule out)
    if (variant == SPMM_VARIANT_DU512x128_S4) {
        if (p.fuse) return hipErrorNotSupported;
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_du<SPATHA_OUT_TRANSPOSED, false>(p, stream)
                                                   : launch_du<SPATHA_OUT_ROW_MAJOR, false>(p, stream);
    }
    if (variant == SPMM_VARIANT_DU512x128_M16) {
        if (p.fuse) return hipErrorNotSupported;
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_du<SPATHA_OUT_TRANSPOSED, false, 16>(p, stream)
                                                   : launch_du<SPATHA_OUT_ROW_MAJOR, false, 16>(p, stream);
    }
    if (variant == SPMM_VARIANT_DSF256x128_S3)
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_dsf<8, 3, 4, SPATHA_OUT_TRANSPOSED>(p, stream)
                                                   : launch_dsf<8, 3, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
    if (variant == SPMM_VARIANT_DS256x128_S3_PP)
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_ds<8, 3, 4, 8, SPATHA_OUT_TRANSPOSED, true>(p, stream)
                                                   : launch_ds<8, 3, 4, 8, SPATHA_OUT_ROW_MAJOR, true>(p, stream);
    return hipErrorInvalidValue;
}

hipError_t launch_pack(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                       int m, int v, int ksp, int S, int half_tiles, uint16_t* apack, uint32_t* rowtab, hipStream_t stream) {
    int64_t total_a = (int64_t)(rows / 64) * S * 256;
    int blocks_a = (int)((total_a + 255) / 256);
    if (blocks_a > 65535 * 8) blocks_a = 65535 * 8;
    hipLaunchKernelGGL(pack_a_kernel, dim3(blocks_a), dim3(256), 0, stream, values, metadata, rows, ksp, S, half_tiles, apack);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    int64_t total_r = (int64_t)(rows / v) * S * 64;
    int blocks_r = (int)((total_r + 255) / 256);
    if (blocks_r > 65535 * 8) blocks_r = 65535 * 8;
    hipLaunchKernelGGL(pack_rowtab_kernel, dim3(blocks_r), dim3(256), 0, stream, columns, rows, cols, m, v, ksp, S, rowtab);
    return hipGetLastError();
}

}  // namespace spatha
