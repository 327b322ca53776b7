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
//   apack  half [rows/64][S][4 mb][64 lanes][8]   A operands, S = ceil(Ksp/32) k-steps
//   ipack  u32  [rows/64][S][64 lanes][2]         idx fields: word d = mb 2d | mb 2d+1 << 16
//   rowtab u32  [rows/V][S*64]                    B row feeding LDS row rho of step s
//                                                 (group*m + column-loc, or ~0 = zero row)
// Inside a 64-row wave tile the sparse-instruction row (mb, i = 4*ib + r) holds
// matrix row 16*ib + 4*mb + r, so that one lane ends up with 16 consecutive
// matrix rows of one output column (contiguous 32 bytes of the transposed output).

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace spatha {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

// ---------------------------------------------------------------------------
// pack_kernel: canonical (values, metadata, columns) -> (apack, ipack, rowtab)
// One thread per (wave tile, step, mb, lane) for apack/ipack; rowtab separately.
// ---------------------------------------------------------------------------
__global__ void pack_a_kernel(const uint16_t* __restrict__ values, const uint32_t* __restrict__ metadata, int rows,
                              int ksp, int S, uint16_t* __restrict__ apack, uint32_t* __restrict__ ipack) {
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
        int64_t r = wt * 64 + 16 * ib + 4 * mb + rr;      // matrix row
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
        *(u32x4*)(apack + t * 8) = out;
        // idx: [wt][s][lane][2] words, 16 bits per mb
        uint16_t* ip16 = (uint16_t*)ipack;
        ip16[((ws * 64 + lane) * 2 + (mb >> 1)) * 2 + (mb & 1)] = (uint16_t)idx16;
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
    const u32x4* a_ptr = (const u32x4*)p.apack + (wt * S) * 256 + lane;   // + s*256 + mb*64
    const u32x2* i_ptr = (const u32x2*)p.ipack + (wt * S) * 64 + lane;    // + s*64
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
            breg[i] = (row != 0xffffffffu && bcol_ok) ? *(const u32x4*)(bbase + (int64_t)row * N) : z;
        }
#pragma unroll
        for (int mb = 0; mb < 4; mb++) areg[mb] = a_ptr[(int64_t)s * 256 + mb * 64];
        ireg = i_ptr[(int64_t)s * 64];
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
            if (col < N) *(u32x4*)(p.C + ((int64_t)m0 + wm * 64 + row) * N + col) = v;
        }
    }
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
    static bool attr_set = false;
    auto kern = spmm_kernel<WM, WN, OUT_LAYOUT>;
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
        default: return nullptr;
    }
}

int spmm_variant_bm(int variant) { return variant == SPMM_VARIANT_128x128 ? 128 : variant == SPMM_VARIANT_64x256 ? 64 : 0; }
int spmm_variant_bn(int variant) { return variant == SPMM_VARIANT_128x128 ? 128 : variant == SPMM_VARIANT_64x256 ? 256 : 0; }

hipError_t launch_spmm(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    if (variant == SPMM_VARIANT_128x128) {
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_variant<2, 2, SPATHA_OUT_TRANSPOSED>(p, stream)
                                                   : launch_variant<2, 2, SPATHA_OUT_ROW_MAJOR>(p, stream);
    }
    if (variant == SPMM_VARIANT_64x256) {
        return out_layout == SPATHA_OUT_TRANSPOSED ? launch_variant<1, 4, SPATHA_OUT_TRANSPOSED>(p, stream)
                                                   : launch_variant<1, 4, SPATHA_OUT_ROW_MAJOR>(p, stream);
    }
    return hipErrorInvalidValue;
}

hipError_t launch_pack(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                       int m, int v, int ksp, int S, uint16_t* apack, uint32_t* ipack, uint32_t* rowtab,
                       hipStream_t stream) {
    int64_t total_a = (int64_t)(rows / 64) * S * 256;
    int blocks_a = (int)((total_a + 255) / 256);
    if (blocks_a > 65535 * 8) blocks_a = 65535 * 8;
    hipLaunchKernelGGL(pack_a_kernel, dim3(blocks_a), dim3(256), 0, stream, values, metadata, rows, ksp, S, apack, ipack);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    int64_t total_r = (int64_t)(rows / v) * S * 64;
    int blocks_r = (int)((total_r + 255) / 256);
    if (blocks_r > 65535 * 8) blocks_r = 65535 * 8;
    hipLaunchKernelGGL(pack_rowtab_kernel, dim3(blocks_r), dim3(256), 0, stream, columns, rows, cols, m, v, ksp, S, rowtab);
    return hipGetLastError();
}

}  // namespace spatha
