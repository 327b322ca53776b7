// Launch interface between the C ABI layer and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include "../../include/spatha.h"

namespace spatha {

struct SpmmParams {
    const uint16_t* apack;    // packed A operands
    const uint32_t* ipack;    // packed sparse-index fields
    const uint32_t* rowtab;   // gathered B row per LDS row
    const uint16_t* B;        // cols x N, row-major
    const uint16_t* bias;     // rows, or null
    uint16_t* C;              // rows x N, or N x rows when transposed
    int rows, cols, N, S, v;
    int tiles_m, tiles_n;
};

enum { SPMM_VARIANT_AUTO = 0, SPMM_VARIANT_128x128 = 1, SPMM_VARIANT_64x256 = 2, SPMM_VARIANT_COUNT = 3 };

const char* spmm_variant_name(int variant);
int spmm_variant_bm(int variant);
int spmm_variant_bn(int variant);

hipError_t launch_spmm(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);

hipError_t launch_pack(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                       int m, int v, int ksp, int S, uint16_t* apack, uint32_t* ipack, uint32_t* rowtab,
                       hipStream_t stream);

hipError_t launch_dense_gemm(const uint16_t* A, const uint16_t* B, int rows, int cols, int N, uint16_t* C,
                             hipStream_t stream);

}  // namespace spatha
