// Dense fp16 GEMM on gfx950 MFMA: C[rows x N] = A[rows x cols] * B[cols x N], fp32
// accumulation, fp16 output.  It plays the role of the dense library GEMM in the
// reference benchmark: the comparison point and the --check product.  It is a plain
// 128x128 tile kernel (v_mfma_f32_16x16x32_f16, B staged through LDS and read with the
// transposing LDS load), not a tuned one.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace spatha {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

#define LDS_PTR(T, p) ((__attribute__((address_space(3))) T*)(p))

__global__ __launch_bounds__(256) void dense_gemm_kernel(const uint16_t* __restrict__ A, const uint16_t* __restrict__ B,
                                                         int rows, int cols, int N, uint16_t* __restrict__ C) {
    constexpr int PITCH_B = 128 * 2 + 32;
    constexpr int PITCH_C = 144;
    __shared__ __attribute__((aligned(16))) char smem[4 * 64 * PITCH_C];   // >= 32 * PITCH_B
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int m0 = blockIdx.y * 128, n0 = blockIdx.x * 128;
    const int li = lane & 15, kb = lane >> 4;

    float4_t acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

    // B loader: 32 rows x 16 chunks = 512 chunks, 2 per thread
    const int bc = tid & 15, br = tid >> 4;
    const int bcol = n0 + bc * 8;
    const int tr_off = (kb * 8 + (li >> 2)) * PITCH_B + (wn * 64 + (li & 3) * 4) * 2;

    for (int k0 = 0; k0 < cols; k0 += 32) {
        u32x4 breg[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            int k = k0 + br + i * 16;
            u32x4 z = {0u, 0u, 0u, 0u};
            breg[i] = (k < cols && bcol < N) ? *(const u32x4*)(B + (int64_t)k * N + bcol) : z;
        }
        half8_t af[4];
#pragma unroll
        for (int mb = 0; mb < 4; mb++) {
            int r = m0 + wm * 64 + mb * 16 + li;
            int k = k0 + kb * 8;
            u32x4 z = {0u, 0u, 0u, 0u};
            u32x4 v = (r < rows && k < cols) ? *(const u32x4*)(A + (int64_t)r * cols + k) : z;
            af[mb] = __builtin_bit_cast(half8_t, v);
        }
        __syncthreads();
#pragma unroll
        for (int i = 0; i < 2; i++) *(u32x4*)(smem + (br + i * 16) * PITCH_B + bc * 16) = breg[i];
        __syncthreads();
#pragma unroll
        for (int nb = 0; nb < 4; nb++) {
            half8_t bf;
#pragma unroll
            for (int h = 0; h < 2; h++) {
                short4_t t4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(short4_t, smem + tr_off + h * 4 * PITCH_B + nb * 32));
                half4_t h4 = __builtin_bit_cast(half4_t, t4);
                bf[h * 4 + 0] = h4[0]; bf[h * 4 + 1] = h4[1]; bf[h * 4 + 2] = h4[2]; bf[h * 4 + 3] = h4[3];
            }
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
                acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[mb], bf, acc[mb][nb], 0, 0, 0);
        }
    }
    __syncthreads();
    // epilogue through wave-private LDS staging
    const int j = lane & 15, ib = lane >> 4;
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
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < 8; it++) {
        const int L = it * 8 + (lane >> 3), ch = lane & 7;
        const int row = m0 + wm * 64 + (L >> 4) * 16 + (L & 3) * 4 + ((L >> 2) & 3);   // mb, ib, r
        const int col = n0 + wn * 64 + ch * 8;
        u32x4 v = *(const u32x4*)(st + L * PITCH_C + ch * 16);
        if (row < rows && col < N) *(u32x4*)(C + (int64_t)row * N + col) = v;
    }
}

hipError_t launch_dense_gemm(const uint16_t* A, const uint16_t* B, int rows, int cols, int N, uint16_t* C,
                             hipStream_t stream) {
    dim3 grid((N + 127) / 128, (rows + 127) / 128);
    hipLaunchKernelGGL(dense_gemm_kernel, grid, dim3(256), 0, stream, A, B, rows, cols, N, C);
    return hipGetLastError();
}

}  // namespace spatha
