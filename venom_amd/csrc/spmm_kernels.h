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
    uint32_t gtab_bytes;      // size of gtab (buffer descriptor of the unified dense-staged kernel)
    const uint16_t* B;        // cols x N, row-major
    const uint16_t* bias;     // rows, or null
    const void* zeros;        // >= 1 KiB of zero bytes (source of zero-filled B rows)
    uint16_t* C;              // rows x N, or N x rows when transposed
    int rows, cols, N, S, v;
    int m;                    // dense columns per group (dense-staged kernels)
    uint32_t b_bytes, apack_bytes, rowtab_bytes;   // sizes for buffer descriptors (persistent kernels)
    int tiles_m, tiles_n;
    int cus;                  // compute units of the device the launch goes to (grid size of the persistent kernels)
    int walk_group;           // order of the tile walk (TileWalkT): 1 column tiles one after the other (default); 0 a tile row's
                              // column tiles first (kernel 6 only); -4 tile rows in groups of four (kernel 18 only)
    // k-split (producer/consumer kernels 6 and 10 only; 1 everywhere else): tiles_m then counts (row tile, part) pairs and
    // every part runs S / ksplit k-steps; fp32 partial blocks and one ticket per 64 x 64 block live in the caller's workspace
    int ksplit;
    float* partial;
    uint32_t partial_bytes;
    uint32_t* tickets;
    int skew;                 // start-up skew between workgroups, in units of 1024 clocks (0 = none)
    long long* prof;          // development cycle-accounting buffer (SPATHA_DEV_PROFILE builds), else null
    int fuse;                 // 1: bias and activation are applied ahead of the write-out (fused_bias_act)
    int act;                  // SPATHA_ACT_*
    int debug;                // development knobs (0 in production): 1 = skip B loads, 2 = skip C stores
};

enum {
    SPMM_VARIANT_AUTO = 0,
    // gathered B stages (any m)
    SPMM_VARIANT_128x128 = 1,           // register-staged, 2 LDS stages: first kernel, fallback
    SPMM_VARIANT_64x256 = 2,
    SPMM_VARIANT_P128x128_S3 = 3,       // global -> LDS DMA pipeline, 3 stages
    SPMM_VARIANT_P64x256_S2 = 4,
    SPMM_VARIANT_R64x256_S3 = 5,        // persistent: the pipeline runs across tile boundaries
    SPMM_VARIANT_W128x128_S3 = 6,       // persistent + producer / consumer waves
    SPMM_VARIANT_W128x256_S3 = 7,
    SPMM_VARIANT_W64x256_S3 = 8,
    SPMM_VARIANT_D64x256_S3 = 9,        // ... with the write-out deferred into the next tile's steps
    SPMM_VARIANT_T128x256_S3 = 10,      // ... each consumer wave owns 128 x 64
    // dense-staged B (m <= 8): all 16 m dense rows of a k-step staged once for the tile's 64-row blocks
    SPMM_VARIANT_DS256x128_S3_C8 = 11,  // eight 64 x 64 consumer waves + four producers
    SPMM_VARIANT_DS256x128_S3_PP = 12,  // the eight consumers in two phase groups
    SPMM_VARIANT_SKINNY = 13,           // N <= 64: one 64-row tile per workgroup, k split over four waves, B straight from L2
    // V % 64 != 0: a 64-row tile spans two V blocks
    SPMM_VARIANT_H64x256_S2 = 14,       // two gathered B sets per stage
    SPMM_VARIANT_H64x128_S3 = 15,
    SPMM_VARIANT_H64x128_S2 = 16,
    SPMM_VARIANT_DSH256x128_S3_C8 = 17, // m <= 8: dense-staged B, two gather-table entries per consumer wave
    // unified waves, A operands in registers, only B staged (rows % 512 == 0)
    SPMM_VARIANT_UP512x128_S3 = 18,     // m <= 8: the eight waves in two phase groups (burst of loads / matrix phase)
    SPMM_VARIANT_DU512x128_M16 = 19,    // 8 < m <= 16: one phase group, 64 KB stages, two of them
    SPMM_VARIANT_WS128x128_S3 = 20,     // id 6 with store waves: finished tiles leave through an LDS staging buffer and a third role
    SPMM_VARIANT_WS64x256_S3 = 21,      // id 8 with store waves
    SPMM_VARIANT_OH192x256 = 22,        // V % 128 == 0: a whole 128 x 256 tile and a 64-row half of another one per workgroup, one k-loop
    SPMM_VARIANT_COUNT = 23
};

const char* spmm_variant_name(int variant);
int spmm_variant_bm(int variant);
int spmm_variant_bn(int variant);
int spmm_variant_lds(int variant, int S);

hipError_t launch_spmm(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);

// one launch switch per kernel family (spmm_gathered.hip, spmm_warpspec.hip, spmm_densestage.hip, spmm_unified.hip,
// spmm_skinny.hip, spmm_pingpong.hip, spmm_onehalf.hip); hipErrorInvalidValue for an id of another family
hipError_t launch_gathered(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);
hipError_t launch_warpspec(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);
hipError_t launch_densestage(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);
hipError_t launch_unified(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);
hipError_t launch_skinny_family(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);
hipError_t launch_pingpong(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);
hipError_t launch_onehalf(int variant, int out_layout, const SpmmParams& p, hipStream_t stream);

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

// words of 32 bits set to zero by a kernel (tickets of a k-split launch; a kernel, so that the launch can be recorded into a graph)
hipError_t launch_clear_words(uint32_t* words, int count, hipStream_t stream);

hipError_t launch_pack_gtab(const uint32_t* columns, int rows, int m, int v, int ksp, int S, int block_rows, uint16_t* gtab,
                            hipStream_t stream);

hipError_t launch_transpose_f16(const uint16_t* in, int rows, int cols, uint16_t* out, hipStream_t stream);
hipError_t launch_add_layernorm_f16(const uint16_t* x, const uint16_t* residual, const uint16_t* gamma, const uint16_t* beta,
                                    float eps, int tokens, int hidden, uint16_t* out, hipStream_t stream);

hipError_t launch_add_layernorm_f16_t(const uint16_t* x, const uint16_t* residual, const uint16_t* gamma, const uint16_t* beta,
                                      float eps, int tokens, int hidden, uint16_t* out, uint16_t* out_t, hipStream_t stream);

hipError_t launch_dense_gemm(const uint16_t* A, const uint16_t* B, int rows, int cols, int N, uint16_t* C,
                             hipStream_t stream);

}  // namespace spatha
