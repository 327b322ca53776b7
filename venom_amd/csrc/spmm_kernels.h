// Launch interface between the C ABI layer and the gfx950 kernels.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stdint.h>

#include "../../include/spatha.h"

namespace spatha {

enum { APACK_BLOCK = 4096 + 512 };

struct SpmmParams {
    const uint16_t* apack;    // packed A operands + sparse-index words, APACK_BLOCK bytes per (64 rows, k-step)
    const uint32_t* rowtab;   // gathered B row per LDS row
    const uint16_t* gtab;     // dense-staged kernels: LDS offset per (64-row block, step, lane class, fragment), or null
    const uint16_t* gtab_tiles;  // the same table, tile-major (512 B per 256-row tile and step), or null
    uint32_t gtab_tiles_bytes;
    uint32_t gtab_bytes;      // size of gtab (buffer descriptor of the unified dense-staged kernel)
    const uint16_t* B;        // cols x N, row-major
    const uint16_t* bias;     // rows, or null
    const void* zeros;        // >= 1 KiB of zero bytes (source of zero-filled B rows)
    uint16_t* C;              // rows x N, or N x rows when transposed
    int rows, cols, N, S, v;
    int m;                    // dense columns per group (dense-staged kernels)
    uint32_t b_bytes, apack_bytes, rowtab_bytes;   // sizes for buffer descriptors (persistent kernels)
    int tiles_m, tiles_n;
    int skew;                 // start-up skew between workgroups, in units of 1024 clocks (0 = none)
    long long* prof;          // development cycle-accounting buffer (SPATHA_DEV_PROFILE builds), else null
    int fuse;                 // 1: bias and activation are applied ahead of the write-out (fused_bias_act)
    int act;                  // SPATHA_ACT_*
    int debug;                // development knobs (0 in production): 1 = skip B loads, 2 = skip C stores
};

enum {
    SPMM_VARIANT_AUTO = 0,
    SPMM_VARIANT_128x128 = 1,      // register-staged, 2 LDS stages
    SPMM_VARIANT_64x256 = 2,
    SPMM_VARIANT_P128x128_S4 = 3,  // direct-to-LDS pipeline
    SPMM_VARIANT_P128x128_S3 = 4,
    SPMM_VARIANT_P64x256_S2 = 5,
    SPMM_VARIANT_P64x256_S3 = 6,
    SPMM_VARIANT_P128x128_S6 = 7,
    SPMM_VARIANT_P64x256_S4 = 8,
    SPMM_VARIANT_R128x128_S4 = 9,  // persistent, pipeline runs across tiles
    SPMM_VARIANT_R128x128_S5 = 10,
    SPMM_VARIANT_R128x128_S2 = 11,
    SPMM_VARIANT_R64x256_S3 = 12,
    SPMM_VARIANT_R64x256_S4 = 13,
    SPMM_VARIANT_W128x128_S5 = 14,  // persistent + producer/consumer wave specialisation
    SPMM_VARIANT_W128x128_S3 = 15,
    SPMM_VARIANT_W128x128_S2 = 16,
    SPMM_VARIANT_W128x256_S3 = 17,
    SPMM_VARIANT_W64x256_S2 = 18,
    SPMM_VARIANT_W64x256_S3 = 19,
    SPMM_VARIANT_D128x256_S3 = 20,  // wave-specialised + write-out deferred into the next tile
    SPMM_VARIANT_D128x128_S3 = 21,
    SPMM_VARIANT_D128x128_S5 = 22,
    SPMM_VARIANT_D64x256_S3 = 23,
    SPMM_VARIANT_T128x256_S3 = 24,  // wave-specialised, each consumer wave owns 128 x 64
    SPMM_VARIANT_T128x128_S4 = 25,
    SPMM_VARIANT_T128x128_S5 = 26,
    SPMM_VARIANT_DS256x128_S3 = 27,  // m <= 8: all 16*m dense B rows of a k-step staged once for four 64-row blocks
    SPMM_VARIANT_DS256x128_S2 = 28,
    SPMM_VARIANT_DS256x128_S3_C8 = 29,  // eight 64 x 64 consumer waves (two per SIMD)
    SPMM_VARIANT_DS256x128_S3_PP = 30,  // eight consumers in two phase groups (ping-pong)
    SPMM_VARIANT_DSF256x128_S3 = 31,    // dense-staged, LDS flag counters instead of workgroup barriers
    SPMM_VARIANT_SKINNY = 32,           // N <= 64: one 64-row tile per workgroup, k split over four waves, B straight from L2
    SPMM_VARIANT_H64x256_S2 = 33,       // V % 64 != 0: a 64-row tile spans two V blocks, two gathered B sets per stage
    SPMM_VARIANT_H64x128_S3 = 34,
    SPMM_VARIANT_H64x128_S2 = 35,
    SPMM_VARIANT_DSH256x128_S3_C8 = 36, // V % 64 != 0, m <= 8: dense-staged B, two gather-table entries per consumer wave
    SPMM_VARIANT_DU512x128_S4 = 37,     // m <= 8, rows % 512 == 0: eight unified 64 x 128 waves, A operands in registers, only B staged
    SPMM_VARIANT_DU512x128_M16 = 38,    // the same for 8 < m <= 16: 64 KB stages, two of them
    SPMM_VARIANT_COUNT = 39
};

const char* spmm_variant_name(int variant);
int spmm_variant_bm(int variant);
int spmm_variant_bn(int variant);
int spmm_variant_lds(int variant, int S);

hipError_t launch_spmm(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);

hipError_t launch_pack(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                       int m, int v, int ksp, int S, int half_tiles, uint16_t* apack, uint32_t* rowtab, hipStream_t stream);

// Search phase of the magnitude selector on the GPU (select_gpu.hip): one entry per (V-row block, group) task,
// block-major, groups in the order full groups then the tail group (if it has three or more columns).
struct SelectWinner {
    int best[4];    // winning column subset, ascending; zeros when no subset has a positive total
    int any;
};
hipError_t launch_select_winners(const float* dense_abs_dev, int rows, int cols, int m, int v, SelectWinner* out_dev,
                                 hipStream_t stream);

hipError_t launch_pack_gtab(const uint32_t* columns, int rows, int m, int v, int ksp, int S, int block_rows, uint16_t* gtab,
                            hipStream_t stream);

hipError_t launch_pack_gtab_tiles(const uint32_t* columns, int rows, int m, int v, int ksp, int S, uint16_t* gtab,
                                  hipStream_t stream);

hipError_t launch_transpose_f16(const uint16_t* in, int rows, int cols, uint16_t* out, hipStream_t stream);
hipError_t launch_add_layernorm_f16(const uint16_t* x, const uint16_t* residual, const uint16_t* gamma, const uint16_t* beta,
                                    float eps, int tokens, int hidden, uint16_t* out, hipStream_t stream);

hipError_t launch_dense_gemm(const uint16_t* A, const uint16_t* B, int rows, int cols, int N, uint16_t* C,
                             hipStream_t stream);

}  // namespace spatha
