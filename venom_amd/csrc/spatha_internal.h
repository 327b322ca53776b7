// Plan object of the SpMM and the pieces of its life cycle that more than one source file of the library needs.
#pragma once

#include <hip/hip_runtime_api.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/spatha.h"

struct spatha_spmm_plan {
    spatha_vnm_geometry geo;
    int S;                 // k-steps of 64 compressed B rows
    int half_tiles;        // V % 64 != 0: operands packed in the order of the half-tile kernels
    int device;
    int cus;               // compute units of that device
    uint16_t* apack;
    uint32_t* rowtab;
    void* zeros;           // 1 KiB of zeros on the device
    uint16_t* gtab;        // gather table of the dense-staged kernels (m <= 8, rows % 256 == 0), or null
    size_t gtab_bytes;
    size_t apack_bytes, rowtab_bytes;
};

namespace spatha {

// sizes of a plan's derived copies (a size of 0: the copy is not made for this shape)
struct PlanLayout {
    int S, half_tiles;
    size_t apack_bytes, rowtab_bytes, gtab_bytes;
};
void plan_layout(int rows, int m, int v, int ksp, PlanLayout* out);

// fills the derived copies a plan points to from the canonical arrays (pack kernels on `stream`)
hipError_t plan_pack(const spatha_spmm_plan* plan, const uint16_t* values_dev, const uint32_t* metadata_dev,
                     const uint32_t* columns_dev, hipStream_t stream);

// the argument checks and the kernel choice of plan_run alone: nothing is launched; *chosen (may be null) gets the kernel id
int plan_run_check(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev, const uint16_t* out_dev,
                   int out_layout, int activation, bool fused_entry, int variant, int* chosen);

// argument checks, kernel choice and launch shared by every run entry point; returns a spatha_status.  With a workspace
// (device memory of at least the size split_workspace_bytes names) the automatic choice may split k-loops over workgroups.
int plan_run(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev, uint16_t* out_dev,
             int out_layout, int activation, bool fused_entry, int variant, void* stream, void* workspace = nullptr,
             size_t workspace_bytes = 0);

// records a HIP error for spatha_last_hip_error and returns SPATHA_ERR_HIP
int note_hip_error(hipError_t e);

}  // namespace spatha
