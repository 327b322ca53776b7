// Kernel registry: name, tile shape and LDS need per kernel id, and the launch switch over the kernel families.

#include "spmm_device.h"

namespace spatha {

namespace {
struct VariantInfo {
    int id;
    const char* name;
    int bm, bn;
    int lds;            // LDS bytes, without the row table the per-tile pipelines keep there (rt_per_step bytes per k-step)
    int rt_per_step;
    hipError_t (*launch)(int, int, const SpmmParams&, hipStream_t);
};

const VariantInfo kVariants[] = {
    {SPMM_VARIANT_OH192x256, "smfmac16x16x64_warpspec_tile_and_a_half_192x256_4slots", 128, 256, OhCfg::LDS_BYTES, 0, launch_onehalf},
    {SPMM_VARIANT_128x128, "smfmac16x16x64_wg256_tile128x128", 128, 128, 1, 0, launch_gathered},
    {SPMM_VARIANT_64x256, "smfmac16x16x64_wg256_tile64x256", 64, 256, 1, 0, launch_gathered},
    {SPMM_VARIANT_P128x128_S3, "smfmac16x16x64_ldsdirect_tile128x128_3stage", 128, 128, 3 * (64 * 128 * 2 + 2 * APACK_BLOCK), 256,
     launch_gathered},
    {SPMM_VARIANT_P64x256_S2, "smfmac16x16x64_ldsdirect_tile64x256_2stage", 64, 256, 2 * (64 * 256 * 2 + APACK_BLOCK), 256,
     launch_gathered},
    {SPMM_VARIANT_R64x256_S3, "smfmac16x16x64_persistent_tile64x256_3stage", 64, 256, PersistCfg<1, 4, 3>::LDS_BYTES, 0,
     launch_gathered},
    {SPMM_VARIANT_W128x128_S3, "smfmac16x16x64_warpspec_tile128x128_3stage", 128, 128, WsCfg<2, 2, 3, 4>::LDS_BYTES, 0,
     launch_warpspec},
    {SPMM_VARIANT_W128x256_S3, "smfmac16x16x64_warpspec_tile128x256_3stage", 128, 256, WsCfg<2, 4, 3, 4>::LDS_BYTES, 0,
     launch_warpspec},
    {SPMM_VARIANT_W64x256_S3, "smfmac16x16x64_warpspec_tile64x256_3stage", 64, 256, WsCfg<1, 4, 3, 2>::LDS_BYTES, 0, launch_warpspec},
    {SPMM_VARIANT_D64x256_S3, "smfmac16x16x64_warpspec_deferred_tile64x256_3stage", 64, 256, WsCfg<1, 4, 3, 2>::LDS_BYTES, 0,
     launch_warpspec},
    {SPMM_VARIANT_WS128x128_S3, "smfmac16x16x64_warpspec_storewaves_tile128x128_3stage", 128, 128,
     WswCfg<2, 2, 3, 4>::LDS_BYTES, 0, launch_warpspec},
    {SPMM_VARIANT_WS64x256_S3, "smfmac16x16x64_warpspec_storewaves_tile64x256_3stage", 64, 256,
     WswCfg<1, 4, 3, 2>::LDS_BYTES, 0, launch_warpspec},
    {SPMM_VARIANT_T128x256_S3, "smfmac16x16x64_warpspec_tall_tile128x256_3stage", 128, 256, WsCfg<2, 4, 3, 4>::LDS_BYTES, 0,
     launch_warpspec},
    {SPMM_VARIANT_DS256x128_S3_C8, "smfmac16x16x64_warpspec_densestage_tile256x128_3stage_8consumers", 256, 128,
     DsCfg<8, 3, 4, 8>::LDS_BYTES, 0, launch_densestage},
    {SPMM_VARIANT_DS256x128_S3_PP, "smfmac16x16x64_warpspec_densestage_tile256x128_3stage_pingpong", 256, 128,
     DsCfg<8, 3, 4, 8>::LDS_BYTES, 0, launch_densestage},
    {SPMM_VARIANT_SKINNY, "smfmac16x16x64_skinny_tile64xN_splitk4", 64, 64, 64 * 1024, 0, launch_skinny_family},
    {SPMM_VARIANT_H64x256_S2, "smfmac16x16x64_halftile_ldsdirect_tile64x256_2stage", 64, 256, half_stage_bytes<4, 2>(), 256,
     launch_gathered},
    {SPMM_VARIANT_H64x128_S3, "smfmac16x16x64_halftile_ldsdirect_tile64x128_3stage", 64, 128, half_stage_bytes<2, 3>(), 256,
     launch_gathered},
    {SPMM_VARIANT_H64x128_S2, "smfmac16x16x64_halftile_ldsdirect_tile64x128_2stage", 64, 128, half_stage_bytes<2, 2>(), 256,
     launch_gathered},
    {SPMM_VARIANT_DSH256x128_S3_C8, "smfmac16x16x64_halftile_densestage_tile256x128_3stage_8consumers", 256, 128,
     DsCfg<8, 3, 4, 8>::LDS_BYTES, 0, launch_densestage},
    {SPMM_VARIANT_UP512x128_S3, "smfmac16x16x64_unified_pingpong_densestage_aregs_tile512x128_3stage", 512, 128, UpCfg::LDS_BYTES, 0,
     launch_pingpong},
    {SPMM_VARIANT_DU512x128_M16, "smfmac16x16x64_unified_densestage_aregs_tile512x128_m16_2stage", 512, 128, DuCfg<16>::LDS_BYTES, 0,
     launch_unified},
};

const VariantInfo* find(int variant) {
    for (const VariantInfo& v : kVariants)
        if (v.id == variant) return &v;
    return nullptr;
}
}  // namespace

const char* spmm_variant_name(int variant) {
    const VariantInfo* v = find(variant);
    return v ? v->name : nullptr;
}

// LDS bytes the variant needs for S k-steps (the per-tile pipelines keep the row table in LDS)
int spmm_variant_lds(int variant, int S) {
    const VariantInfo* v = find(variant);
    return v ? v->lds + S * v->rt_per_step : 0;
}

int spmm_variant_bm(int variant) {
    const VariantInfo* v = find(variant);
    return v ? v->bm : 0;
}

int spmm_variant_bn(int variant) {
    const VariantInfo* v = find(variant);
    return v ? v->bn : 0;
}

hipError_t launch_spmm(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    const VariantInfo* v = find(variant);
    return v ? v->launch(variant, out_layout, p, stream) : hipErrorInvalidValue;
}

}  // namespace spatha
