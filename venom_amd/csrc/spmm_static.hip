// spatha_spmm_run_noalloc: one SpMM from the canonical arrays with no allocation of any kind.
//
// spatha_spmm_plan_create allocates the derived copies of A that the kernels read (packed operands, row table, gather
// tables, a block of zeros) with hipMalloc.  Callers that cannot allocate (code under HIP graph capture, serving loops,
// harnesses that forbid it) get this entry point instead: the same pack kernels write the same copies into a fixed
// array in device memory that is part of the library's code object, and the same SpMM kernels read them from there.
// Every GPU the library runs on holds the array (SCRATCH_BYTES) from the first call until the process ends.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "spatha_internal.h"
#include "spmm_kernels.h"

namespace {

constexpr size_t SCRATCH_BYTES = 8u << 20;       // 8 MiB: A up to e.g. 4096 x 1024 or 1024 x 4096 at 2:8, 4096 x 1024 at 2:4
constexpr int MAX_DEVICES = 16;

// Device memory of the derived copies.  In host code this name only stands for the symbol; its address on a device
// comes from hipGetSymbolAddress (below) and is what every kernel argument uses.
static __device__ __align__(256) unsigned char scratch[SCRATCH_BYTES];

std::mutex g_lock;
unsigned char* g_scratch_ptr[MAX_DEVICES] = {};

// Address of the current device's copy of the array (each device has its own), looked up once per device.
hipError_t scratch_address(int device, unsigned char** out) {
    std::lock_guard<std::mutex> guard(g_lock);
    if (!g_scratch_ptr[device]) {
        void* ptr = nullptr;
        hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return e;
        g_scratch_ptr[device] = (unsigned char*)ptr;
    }
    *out = g_scratch_ptr[device];
    return hipSuccess;
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

}  // namespace

extern "C" int spatha_spmm_run_noalloc(int rows, int cols, int n, int m, int v, const uint16_t* values_dev,
                                       const uint32_t* metadata_dev, const uint32_t* columns_dev, const uint16_t* B_dev, int N,
                                       const uint16_t* bias_dev, uint16_t* out_dev, int out_layout, void* stream) {
    spatha_vnm_geometry geo;
    int st = spatha_vnm_geometry_init(rows, cols, n, m, v, &geo);
    if (st) return st;
    if (!values_dev || !metadata_dev || !columns_dev) return SPATHA_ERR_BAD_ARGUMENT;
    spatha::PlanLayout lay;
    spatha::plan_layout(rows, m, v, geo.ksp, &lay);
    // [zeros 1 KiB][packed operands][row table][gather table], each at a multiple of 256 bytes
    const size_t off_apack = 1024;
    const size_t off_rowtab = off_apack + align256(lay.apack_bytes);
    const size_t off_gtab = off_rowtab + align256(lay.rowtab_bytes);
    const size_t need = off_gtab + align256(lay.gtab_bytes);
    if (need > SCRATCH_BYTES) return SPATHA_ERR_TOO_LARGE;      // the matrix's derived copies do not fit the fixed array

    int ndev = 0, dev = -1;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev == 0) return SPATHA_ERR_NO_DEVICE;
    if ((e = hipGetDevice(&dev)) != hipSuccess) return spatha::note_hip_error(e);
    if (dev < 0 || dev >= MAX_DEVICES) return SPATHA_ERR_UNSUPPORTED;
    unsigned char* base = nullptr;
    if ((e = scratch_address(dev, &base)) != hipSuccess) return spatha::note_hip_error(e);

    spatha_spmm_plan plan;
    plan.geo = geo;
    plan.S = lay.S;
    plan.half_tiles = lay.half_tiles;
    plan.device = dev;
    plan.cus = 0;
    if (hipDeviceGetAttribute(&plan.cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) plan.cus = 0;
    plan.zeros = base;
    plan.apack = (uint16_t*)(base + off_apack);
    plan.rowtab = (uint32_t*)(base + off_rowtab);
    plan.gtab = lay.gtab_bytes ? (uint16_t*)(base + off_gtab) : nullptr;
    plan.apack_bytes = lay.apack_bytes; plan.rowtab_bytes = lay.rowtab_bytes;
    plan.gtab_bytes = lay.gtab_bytes;

    // every argument check and the kernel choice come before the first launch: a call that is going to be refused must
    // not have touched the array another (valid) call may be about to read
    if ((st = spatha::plan_run_check(&plan, B_dev, N, bias_dev, out_dev, out_layout, SPATHA_ACT_NONE, false, 0, nullptr)) != SPATHA_OK)
        return st;

    // The array keeps what the last call left: the block of zeros is cleared again, everything else is rewritten in
    // full by the pack kernels (every byte the SpMM kernels read for this shape).
    // (a kernel, not hipMemsetAsync: the call may be recorded into a graph by its caller)
    if ((e = spatha::launch_clear_words((uint32_t*)base, 256, (hipStream_t)stream)) != hipSuccess) return spatha::note_hip_error(e);
    if ((e = spatha::plan_pack(&plan, values_dev, metadata_dev, columns_dev, (hipStream_t)stream)) != hipSuccess)
        return spatha::note_hip_error(e);
    return spatha::plan_run(&plan, B_dev, N, bias_dev, out_dev, out_layout, SPATHA_ACT_NONE, false, 0, stream);
}
