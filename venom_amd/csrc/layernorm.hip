// out = LayerNorm(x + residual) over the last dimension of a [tokens, hidden] fp16 matrix, in one pass over memory:
// the two elementwise kernels (addition, normalisation) that follow the attention-output and FFN-down projections of
// every encoder layer in the end-to-end models (reference harness: end2end/bert_pytorch.py:170-219 runs the stock
// BertSelfOutput / BertOutput modules, `LayerNorm(dropout(dense(h)) + input)`).
// Numerics follow the two kernels they replace: the sum is rounded to fp16 first (packed fp16 addition = one rounding of
// the exact sum), then mean, biased variance, 1/sqrt(var + eps) and the affine map are evaluated in fp32 and the result
// is rounded to fp16 once.
// One wave per token: a lane holds the token's 8-value chunks lane, lane + 64, ... in registers (two passes over
// registers for mean and variance, no re-read), wave-wide sums through DPP-style lane exchanges.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace spatha {

typedef uint32_t ln_u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 ln_half2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ ln_half2 as_half2(uint32_t w) { return __builtin_bit_cast(ln_half2, w); }
__device__ __forceinline__ uint32_t as_u32(ln_half2 h) { return __builtin_bit_cast(uint32_t, h); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

template <int NJ>
__global__ __launch_bounds__(256) void add_layernorm_f16_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual,
                                                                const uint16_t* __restrict__ gamma,
                                                                const uint16_t* __restrict__ beta, float eps, int tokens,
                                                                int hidden, uint16_t* __restrict__ out) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t token = (int64_t)blockIdx.x * 4 + wave;
    if (token >= tokens) return;
    const int chunks = hidden >> 3;
    const uint16_t* xr = x + token * hidden;
    const uint16_t* rr = residual ? residual + token * hidden : nullptr;
    float s[NJ][8];
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int c = lane + 64 * j;
        if (c < chunks) {
            // (vector elements go through scalars: a bit cast applied to an indexed vector element reads element 0)
            const ln_u32x4 av = *(const ln_u32x4*)(xr + c * 8);
            uint32_t a[4] = {av.x, av.y, av.z, av.w};
            if (rr) {
                const ln_u32x4 bv = *(const ln_u32x4*)(rr + c * 8);
                const uint32_t b[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const ln_half2 t = as_half2(a[k]) + as_half2(b[k]);
                    a[k] = as_u32(t);
                }
            }
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const ln_half2 t = as_half2(a[k]);
                s[j][2 * k] = (float)t[0];
                s[j][2 * k + 1] = (float)t[1];
                sum += s[j][2 * k] + s[j][2 * k + 1];
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) s[j][k] = 0.f;
        }
    }
    const float mean = wave_sum(sum) / (float)hidden;
    float sq = 0.f;
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        if (lane + 64 * j < chunks) {
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float d = s[j][k] - mean;
                sq += d * d;
            }
        }
    }
    const float rstd = rsqrtf(wave_sum(sq) / (float)hidden + eps);
#pragma unroll
    for (int j = 0; j < NJ; j++) {
        const int c = lane + 64 * j;
        if (c < chunks) {
            const ln_u32x4 gv = *(const ln_u32x4*)(gamma + c * 8);
            const ln_u32x4 bv = *(const ln_u32x4*)(beta + c * 8);
            const uint32_t g[4] = {gv.x, gv.y, gv.z, gv.w}, b[4] = {bv.x, bv.y, bv.z, bv.w};
            uint32_t ow[4];
#pragma unroll
            for (int k = 0; k < 4; k++) {
                const ln_half2 g2 = as_half2(g[k]), b2 = as_half2(b[k]);
                ln_half2 y;
                y[0] = (_Float16)((s[j][2 * k] - mean) * rstd * (float)g2[0] + (float)b2[0]);
                y[1] = (_Float16)((s[j][2 * k + 1] - mean) * rstd * (float)g2[1] + (float)b2[1]);
                ow[k] = as_u32(y);
            }
            const ln_u32x4 o = {ow[0], ow[1], ow[2], ow[3]};
            *(ln_u32x4*)(out + token * hidden + c * 8) = o;
        }
    }
}

// The same normalisation, written twice: row-major as above and FEATURE-MAJOR, out_t[hidden][tokens] - the layout the next
// V:N:M projection takes as its right-hand side (the reference's layer makes that copy with `x.T.contiguous()` in front of
// every SpMM, end2end/bert_pytorch.py:87, :130-134).  A workgroup of eight waves normalises TOK tokens (TOK / 8 per wave),
// leaves the fp16 results in an LDS tile [TOK][hidden + 4] (8-byte writes; the pitch of 2 (mod 64) words keeps the column
// reads below free of bank conflicts) and then writes the tile out by columns: a lane gathers the 8 tokens of one feature
// and stores them as 16 bytes, four (TOK = 32) lanes side by side covering 64 contiguous bytes of a feature's row.
template <int NJ, int TOK>
__global__ __launch_bounds__(512) void add_layernorm_f16_t_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ residual,
                                                                  const uint16_t* __restrict__ gamma, const uint16_t* __restrict__ beta,
                                                                  float eps, int tokens, int hidden, uint16_t* __restrict__ out,
                                                                  uint16_t* __restrict__ out_t) {
    extern __shared__ __attribute__((aligned(16))) uint16_t ln_tile[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int chunks = hidden >> 3;
    const int pitch = hidden + 4;                    // halfs
    const int64_t tok0 = (int64_t)blockIdx.x * TOK;
    constexpr int PER_WAVE = TOK / 8;
    // all of the wave's tokens are fetched before the first one is reduced: 2 * PER_WAVE * NJ loads of 16 bytes in flight per lane
    ln_u32x4 xa[PER_WAVE][NJ], xb[PER_WAVE][NJ];
#pragma unroll
    for (int t = 0; t < PER_WAVE; t++) {
        const int64_t token = tok0 + wave * PER_WAVE + t;
        const bool live = token < tokens;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int c = lane + 64 * j;
            const ln_u32x4 zero = {0u, 0u, 0u, 0u};
            xa[t][j] = (live && c < chunks) ? *(const ln_u32x4*)(x + token * hidden + c * 8) : zero;
            xb[t][j] = (live && c < chunks && residual) ? *(const ln_u32x4*)(residual + token * hidden + c * 8) : zero;
        }
    }
#pragma unroll
    for (int t = 0; t < PER_WAVE; t++) {
        const int local = wave * PER_WAVE + t;
        const int64_t token = tok0 + local;
        if (token >= tokens) break;
        float s[NJ][8];
        float sum = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int c = lane + 64 * j;
            if (c < chunks) {
                uint32_t a[4] = {xa[t][j].x, xa[t][j].y, xa[t][j].z, xa[t][j].w};
                if (residual) {
                    // (x + 0 would not be the identity for -0: the addition runs only with a residual)
                    const uint32_t b[4] = {xb[t][j].x, xb[t][j].y, xb[t][j].z, xb[t][j].w};
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        const ln_half2 tt = as_half2(a[k]) + as_half2(b[k]);
                        a[k] = as_u32(tt);
                    }
                }
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const ln_half2 tt = as_half2(a[k]);
                    s[j][2 * k] = (float)tt[0];
                    s[j][2 * k + 1] = (float)tt[1];
                    sum += s[j][2 * k] + s[j][2 * k + 1];
                }
            } else {
#pragma unroll
                for (int k = 0; k < 8; k++) s[j][k] = 0.f;
            }
        }
        const float mean = wave_sum(sum) / (float)hidden;
        float sq = 0.f;
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            if (lane + 64 * j < chunks) {
#pragma unroll
                for (int k = 0; k < 8; k++) {
                    const float d = s[j][k] - mean;
                    sq += d * d;
                }
            }
        }
        const float rstd = rsqrtf(wave_sum(sq) / (float)hidden + eps);
#pragma unroll
        for (int j = 0; j < NJ; j++) {
            const int c = lane + 64 * j;
            if (c < chunks) {
                const ln_u32x4 gv = *(const ln_u32x4*)(gamma + c * 8);
                const ln_u32x4 bv = *(const ln_u32x4*)(beta + c * 8);
                const uint32_t g[4] = {gv.x, gv.y, gv.z, gv.w}, b[4] = {bv.x, bv.y, bv.z, bv.w};
                uint32_t ow[4];
#pragma unroll
                for (int k = 0; k < 4; k++) {
                    const ln_half2 g2 = as_half2(g[k]), b2 = as_half2(b[k]);
                    ln_half2 y;
                    y[0] = (_Float16)((s[j][2 * k] - mean) * rstd * (float)g2[0] + (float)b2[0]);
                    y[1] = (_Float16)((s[j][2 * k + 1] - mean) * rstd * (float)g2[1] + (float)b2[1]);
                    ow[k] = as_u32(y);
                }
                const ln_u32x4 o = {ow[0], ow[1], ow[2], ow[3]};
                *(ln_u32x4*)(out + token * hidden + c * 8) = o;
                uint32_t* dst = (uint32_t*)(ln_tile + local * pitch + c * 8);      // 8-byte aligned: pitch % 4 == 0
                *(uint2*)dst = make_uint2(ow[0], ow[1]);
                *(uint2*)(dst + 2) = make_uint2(ow[2], ow[3]);
            }
        }
    }
    __syncthreads();
    // by columns: item = (feature f, piece p of 8 tokens)
    constexpr int PIECES = TOK / 8;
    const int items = hidden * PIECES;
    for (int idx = threadIdx.x; idx < items; idx += 512) {
        const int p = idx % PIECES, f = idx / PIECES;
        const int64_t token = tok0 + p * 8;
        if (token >= tokens) continue;                  // (tokens % 8 == 0: a piece is all there or not at all)
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            const uint32_t lo = ln_tile[(p * 8 + 2 * k) * pitch + f], hi = ln_tile[(p * 8 + 2 * k + 1) * pitch + f];
            w[k] = lo | (hi << 16);
        }
        const ln_u32x4 o = {w[0], w[1], w[2], w[3]};
        *(ln_u32x4*)(out_t + (int64_t)f * tokens + token) = o;
    }
}

template <int NJ, int TOK>
static hipError_t launch_ln_t(const uint16_t* x, const uint16_t* residual, const uint16_t* gamma, const uint16_t* beta, float eps,
                              int tokens, int hidden, uint16_t* out, uint16_t* out_t, hipStream_t stream) {
    const int lds = TOK * (hidden + 4) * 2;
    auto kern = add_layernorm_f16_t_kernel<NJ, TOK>;
    if (lds > 48 * 1024) {
        static bool raised[16] = {};
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        if (!raised[dev & 15]) {
            e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
            if (e != hipSuccess) return e;
            raised[dev & 15] = true;
        }
    }
    hipLaunchKernelGGL(kern, dim3((tokens + TOK - 1) / TOK), dim3(512), lds, stream, x, residual, gamma, beta, eps, tokens, hidden, out,
                       out_t);
    return hipGetLastError();
}

// hidden <= 1024: 32 tokens per workgroup (66 KB of LDS); <= 2048: 16; <= 4096: 8
hipError_t launch_add_layernorm_f16_t(const uint16_t* x, const uint16_t* residual, const uint16_t* gamma, const uint16_t* beta,
                                      float eps, int tokens, int hidden, uint16_t* out, uint16_t* out_t, hipStream_t stream) {
    if (hidden <= 512) return launch_ln_t<1, 32>(x, residual, gamma, beta, eps, tokens, hidden, out, out_t, stream);
    if (hidden <= 1024) return launch_ln_t<2, 32>(x, residual, gamma, beta, eps, tokens, hidden, out, out_t, stream);
    if (hidden <= 2048) return launch_ln_t<4, 16>(x, residual, gamma, beta, eps, tokens, hidden, out, out_t, stream);
    return launch_ln_t<8, 8>(x, residual, gamma, beta, eps, tokens, hidden, out, out_t, stream);
}

hipError_t launch_add_layernorm_f16(const uint16_t* x, const uint16_t* residual, const uint16_t* gamma, const uint16_t* beta,
                                    float eps, int tokens, int hidden, uint16_t* out, hipStream_t stream) {
    const dim3 grid((tokens + 3) / 4), block(256);
    const int nj = (hidden / 8 + 63) / 64;
    if (nj <= 1) hipLaunchKernelGGL(add_layernorm_f16_kernel<1>, grid, block, 0, stream, x, residual, gamma, beta, eps, tokens, hidden, out);
    else if (nj <= 2) hipLaunchKernelGGL(add_layernorm_f16_kernel<2>, grid, block, 0, stream, x, residual, gamma, beta, eps, tokens, hidden, out);
    else if (nj <= 4) hipLaunchKernelGGL(add_layernorm_f16_kernel<4>, grid, block, 0, stream, x, residual, gamma, beta, eps, tokens, hidden, out);
    else hipLaunchKernelGGL(add_layernorm_f16_kernel<8>, grid, block, 0, stream, x, residual, gamma, beta, eps, tokens, hidden, out);
    return hipGetLastError();
}

}  // namespace spatha
