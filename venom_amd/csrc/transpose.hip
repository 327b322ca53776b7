// out[c][r] = in[r][c] for fp16 matrices: the `dense.contiguous()` of a transposed activation that the
// PyTorch layer performs before every SpMM (reference: end2end/bert_pytorch.py:85-87, :130-134).
// A generic strided-copy kernel moves 2 bytes per lane on one side; this one moves 16 bytes per lane on
// both sides through a 64 x 64 LDS tile.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace spatha {

typedef uint32_t tr_u32x4 __attribute__((ext_vector_type(4)));

constexpr int TT = 64;            // tile edge
constexpr int TP = TT + 2;        // LDS pitch in halfs (odd number of 32-bit words: conflict-free column reads)

__global__ __launch_bounds__(256) void transpose_f16_kernel(const uint16_t* __restrict__ in, int rows, int cols,
                                                            uint16_t* __restrict__ out) {
    __shared__ uint16_t tile[TT * TP];
    const int tid = threadIdx.x;
    const int64_t r0 = (int64_t)blockIdx.y * TT, c0 = (int64_t)blockIdx.x * TT;
    const bool vec_in = (cols % 8 == 0), vec_out = (rows % 8 == 0);
    // load: 8 lanes x 16 B per row, 32 rows per pass
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        const int r = pass * 32 + (tid >> 3), c = (tid & 7) * 8;
        uint16_t v[8];
        if (r0 + r < rows) {
            const uint16_t* src = in + (r0 + r) * cols + c0 + c;
            if (vec_in && c0 + c + 8 <= cols) {
                *(tr_u32x4*)v = *(const tr_u32x4*)src;
            } else {
#pragma unroll
                for (int k = 0; k < 8; k++) v[k] = (c0 + c + k < cols) ? src[k] : (uint16_t)0;
            }
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++) v[k] = 0;
        }
#pragma unroll
        for (int k = 0; k < 8; k++) tile[r * TP + c + k] = v[k];
    }
    __syncthreads();
    // store: output row = input column; 8 lanes x 16 B per output row
#pragma unroll
    for (int pass = 0; pass < 2; pass++) {
        const int c = pass * 32 + (tid >> 3), r = (tid & 7) * 8;
        if (c0 + c >= cols) continue;
        uint16_t v[8];
#pragma unroll
        for (int k = 0; k < 8; k++) v[k] = tile[(r + k) * TP + c];
        uint16_t* dst = out + (c0 + c) * rows + r0 + r;
        if (vec_out && r0 + r + 8 <= rows) {
            *(tr_u32x4*)dst = *(const tr_u32x4*)v;
        } else {
#pragma unroll
            for (int k = 0; k < 8; k++)
                if (r0 + r + k < rows) dst[k] = v[k];
        }
    }
}

hipError_t launch_transpose_f16(const uint16_t* in, int rows, int cols, uint16_t* out, hipStream_t stream) {
    dim3 grid((cols + TT - 1) / TT, (rows + TT - 1) / TT);
    hipLaunchKernelGGL(transpose_f16_kernel, grid, dim3(256), 0, stream, in, rows, cols, out);
    return hipGetLastError();
}

}  // namespace spatha
