// Device code shared by the SpMM kernel families of this library (gfx950): operand types, the write-out routines,
// buffer-descriptor helpers, the persistent tile walk and the compile-time configurations whose LDS sizes the
// dispatcher also needs.  Included by every spmm_*.hip source; everything here is a template or force-inlined.
//
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

#pragma once

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
// The same with the choice of the activation inside the loop (one uniform branch per group of four values): the two
// paths then join on four registers, not on the 64 of the whole block - for kernels that have no registers to spare
// for the copies such a join can cost.
__device__ __forceinline__ void fused_bias_act_narrow(float4_t (&acc)[4][4], const uint16_t* bias, int64_t row16, int act) {
#pragma unroll
    for (int mb = 0; mb < 4; mb++) {
        half4_t bv = {(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
        if (bias) bv = *(const half4_t*)(bias + row16 + 4 * mb);
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            float4_t v = acc[mb][nb];
#pragma unroll
            for (int r = 0; r < 4; r++) v[r] = (float)((_Float16)v[r] + bv[r]);
            if (act == SPATHA_ACT_GELU) {
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = act_gelu_erf(v[r]);
            } else if (act == SPATHA_ACT_GELU_TANH) {
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = act_gelu_tanh(v[r]);
            }
            acc[mb][nb] = v;
            __builtin_amdgcn_sched_barrier(0);
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

// the two halves of a half-tile step (V a multiple of 32 only): instructions 0, 1 multiply the first gathered set, 2, 3 the second
#define SPATHA_MMA2LO(NB, BF)                                                                                 \
    acc[0][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[0], BF, acc[0][NB], (int)i0, 0, 0);           \
    acc[1][NB] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a_cur[1], BF, acc[1][NB], (int)i0, 0, 1);
#define SPATHA_MMA2HI(NB, BF)                                                                                 \
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

template <int WN, int NS>
constexpr int half_stage_bytes() { return NS * (2 * 64 * WN * 128 + APACK_BLOCK); }

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

// LDS layout of the producer / consumer kernel with store waves (spmm_wsw_kernel, spmm_warpspec.hip): the stages of
// WsCfg, a staging buffer that holds one whole finished tile, and the row-table slots.
template <int WM_, int WN_, int NS, int NP_>
struct WswCfg {
    static_assert(WM_ * WN_ == 4, "four consumer waves, four store waves");
    static constexpr int WM = WM_, WN = WN_, NP = NP_;
    static constexpr int NC = 4, NSW = 4;
    static constexpr int BM = WM * 64, BN = WN * 64;
    static constexpr int ROW_BYTES = BN * 2;
    static constexpr int B_BYTES = 64 * ROW_BYTES;
    static constexpr int STAGE_BYTES = B_BYTES + WM * APACK_BLOCK;
    static constexpr int PA = NS - 1;
    static constexpr int STG_PITCH = BM * 2 + 16;                   // transposed output: a tile column (BM rows) + 16 B
    // the staging buffer: row-major output 4 blocks x 8 slabs x 1 KB, transposed output BN tile columns
    static constexpr int EPI_BYTES = BN * STG_PITCH > 4 * 8192 ? BN * STG_PITCH : 4 * 8192;
    static constexpr int RT_BYTES = NP * (PA + 1) * 256;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + EPI_BYTES + RT_BYTES;
    static constexpr int THREADS = (NC + NP + NSW) * 64;
    static constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    static constexpr uint32_t RT_BASE = EPI_BASE + EPI_BYTES;
};

// LDS layout of the tile-and-a-half kernel (spmm_onehalf.hip): per k-step an F sub-stage (64 gathered B rows of 256 columns
// + two operand blocks) and an H sub-stage (64 gathered B rows of 128 columns + two operand blocks), two of each, and a
// row-table ring of four slots.
struct OhCfg {
    static constexpr int ROW_BYTES = 512, HROW_BYTES = 256;
    static constexpr int B_BYTES = 64 * ROW_BYTES, HB_BYTES = 64 * HROW_BYTES;
    static constexpr int F_BYTES = B_BYTES + 2 * APACK_BLOCK;
    static constexpr int H_BYTES = HB_BYTES + 2 * APACK_BLOCK;
    static constexpr int PAIR = F_BYTES + H_BYTES;
    static constexpr int RT_BASE = 2 * PAIR;
    static constexpr int LDS_BYTES = RT_BASE + 4 * 256;
};

// Tile walk shared by both roles: XCD x (= workgroup id % 8) owns a contiguous range of tile
// ids (id -> n-tile major, m-tile minor) and its workgroups take them round robin; the
// coordinates advance by a fixed (dm, dn) with carry, so no division per tile.
// The tiles of a launch in walk order, eight consecutive chunks of them for the eight XCDs (workgroup id % 8), within a chunk
// workgroup j of an XCD takes tiles j, j + workgroups, ...  The order decides what the workgroups of an XCD share in its L2.
// GROUP == 1: through a tile column's row tiles, column after column (index tn * tiles_m + tm): the XCD works on one column
// tile of B at a time and streams A past it.
// GROUP == 0: through a tile row's column tiles first (index tm * tiles_n + tn); GROUP == g > 1: the same within groups of g
// tile columns (tiles_n a multiple of g): the workgroups of an XCD then work on fewer tile rows at a time, g column tiles of
// each - the packed A operands of a tile row enter that XCD's L2 once instead of once per XCD that holds one of its column
// tiles.  Pays where tile rows of A are large against tile columns of B.
// GROUP == -h < 0: tile rows in groups of h (tiles_m a multiple of h), within a group column after column: an XCD only ever
// sees h tile rows of A (they stay in its L2 for the whole launch when they fit) and reads more tile columns of B instead.
template <int GROUP>
struct TileWalkT {
    int my_tiles, tm0, tn0, step_dm, step_dn, tiles_m, tiles_n, stride;
    // tile number `t` of the walk -> tile coordinates (wave-uniform, kept in scalar registers: they end up in scalar operands)
    __device__ __forceinline__ void locate(int t, int& tm, int& tn) const {
        if constexpr (GROUP >= 0) {
            const int g = GROUP == 0 ? tiles_n : GROUP, per_group = tiles_m * g;
            const int grp = t / per_group, rem = t - grp * per_group;
            const int row = rem / g;
            tm = __builtin_amdgcn_readfirstlane(row);
            tn = __builtin_amdgcn_readfirstlane(grp * g + (rem - row * g));
        } else {
            constexpr int h = -GROUP;
            const int per_group = tiles_n * h;
            const int grp = t / per_group, rem = t - grp * per_group;
            const int col = rem / h;
            tn = __builtin_amdgcn_readfirstlane(col);
            tm = __builtin_amdgcn_readfirstlane(grp * h + (rem - col * h));
        }
    }
    __device__ __forceinline__ int number(int tm, int tn) const {
        if constexpr (GROUP >= 0) {
            const int g = GROUP == 0 ? tiles_n : GROUP, grp = tn / g;
            return grp * tiles_m * g + tm * g + (tn - grp * g);
        } else {
            constexpr int h = -GROUP;
            const int grp = tm / h;
            return grp * tiles_n * h + tn * h + (tm - grp * h);
        }
    }
    __device__ __forceinline__ void init(int tiles_m_, int tiles_n_) {
        tiles_m = tiles_m_;
        tiles_n = tiles_n_;
        const int tiles = tiles_m_ * tiles_n_;
        const int chunk = (tiles + 7) >> 3;
        const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3, slots = gridDim.x >> 3;
        const int first = xcd * chunk;
        const int last = (first + chunk) < tiles ? (first + chunk) : tiles;
        my_tiles = 0;
        if (first + slot < last) my_tiles = (last - first - slot + slots - 1) / slots;
        stride = slots;
        if constexpr (GROUP == 1) {
            step_dn = slots / tiles_m;
            step_dm = slots - step_dn * tiles_m;
            tn0 = (first + slot) / tiles_m;
            tm0 = (first + slot) - tn0 * tiles_m;
        } else {
            step_dm = step_dn = 0;
            locate(first + slot, tm0, tn0);
        }
    }
    __device__ __forceinline__ void next(int& tm, int& tn) const {
        if constexpr (GROUP == 1) {
            tm += step_dm;
            tn += step_dn;
            if (tm >= tiles_m) { tm -= tiles_m; tn += 1; }
        } else {
            locate(number(tm, tn) + stride, tm, tn);
        }
    }
};
using TileWalk = TileWalkT<1>;

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
template <bool ROWS8, bool BIAS_VIA_SLAB = false, bool WRITE_THROUGH = true>
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
        if (ph > 0 && live) store_c16<WRITE_THROUGH>(C + (row0 + held_row) * N + out_col, held);
        held.x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
        held.y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
        held.z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
        held.w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
        const int q = 8 * sidx + q_lo;
        held_row = 16 * (q >> 2) + 4 * mb + (q & 3);
    }
    if (live) store_c16<WRITE_THROUGH>(C + (row0 + held_row) * N + out_col, held);
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

// The unified kernel in two phase groups (spmm_pingpong.hip): m <= 8, three 32 KB stages.
struct UpCfg {
    static constexpr int BM = 512, BN = 128, M = 8, NS = 3;
    static constexpr int NB = 4;                   // DMA instructions per wave and stage (4 rows x 256 B each)
    static constexpr int STAGE_BYTES = 16 * M * BN * 2;
    static constexpr int WAVE_EPI = WAVE_EPI_BYTES;            // four write-out slabs per wave
    static constexpr uint32_t EPI_BASE = NS * STAGE_BYTES;
    static constexpr int LDS_BYTES = NS * STAGE_BYTES + 8 * WAVE_EPI;
    static constexpr int THREADS = 512;
};

}  // namespace spatha

