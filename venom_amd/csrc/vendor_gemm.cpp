// Dense fp16 GEMM of the vendor library (hipBLASLt), the baseline behind the driver's gemm_time / speedup columns.
// Counterpart of the reference's cuBLAS wrapper (src/gemm/cublas_gemm.cpp:54-96): C = A * B, all row-major, fp16
// operands, fp32 compute, fp16 result, computed as the column-major product C^T = B^T * A^T like there (:70-79).
// Part of the benchmark_spmm driver only; the library itself does not link hipBLASLt.

#include "vendor_gemm.h"

#include <hip/hip_runtime_api.h>
#include <hipblaslt/hipblaslt.h>

#include <new>

struct VendorGemm {
    hipblasLtHandle_t handle = nullptr;
    hipblasLtMatmulDesc_t desc = nullptr;
    hipblasLtMatrixLayout_t lay_b = nullptr, lay_a = nullptr, lay_c = nullptr;
    hipblasLtMatmulPreference_t pref = nullptr;
    hipblasLtMatmulAlgo_t algo;
    void* workspace = nullptr;
    size_t workspace_bytes = 0;
};

void vendor_gemm_destroy(VendorGemm* g) {
    if (!g) return;
    if (g->pref) (void)hipblasLtMatmulPreferenceDestroy(g->pref);
    if (g->lay_a) (void)hipblasLtMatrixLayoutDestroy(g->lay_a);
    if (g->lay_b) (void)hipblasLtMatrixLayoutDestroy(g->lay_b);
    if (g->lay_c) (void)hipblasLtMatrixLayoutDestroy(g->lay_c);
    if (g->desc) (void)hipblasLtMatmulDescDestroy(g->desc);
    if (g->handle) (void)hipblasLtDestroy(g->handle);
    if (g->workspace) (void)hipFree(g->workspace);
    delete g;
}

VendorGemm* vendor_gemm_create(int rows, int cols, int n) {
    VendorGemm* g = new (std::nothrow) VendorGemm();
    if (!g) return nullptr;
    g->workspace_bytes = 64u << 20;
    bool ok = hipblasLtCreate(&g->handle) == HIPBLAS_STATUS_SUCCESS &&
              hipblasLtMatmulDescCreate(&g->desc, HIPBLAS_COMPUTE_32F, HIP_R_32F) == HIPBLAS_STATUS_SUCCESS;
    hipblasOperation_t op_n = HIPBLAS_OP_N;
    ok = ok && hipblasLtMatmulDescSetAttribute(g->desc, HIPBLASLT_MATMUL_DESC_TRANSA, &op_n, sizeof(op_n)) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatmulDescSetAttribute(g->desc, HIPBLASLT_MATMUL_DESC_TRANSB, &op_n, sizeof(op_n)) == HIPBLAS_STATUS_SUCCESS;
    // column-major views: B^T is n x cols (ld n), A^T is cols x rows (ld cols), C^T is n x rows (ld n)
    ok = ok && hipblasLtMatrixLayoutCreate(&g->lay_b, HIP_R_16F, (uint64_t)n, (uint64_t)cols, (int64_t)n) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatrixLayoutCreate(&g->lay_a, HIP_R_16F, (uint64_t)cols, (uint64_t)rows, (int64_t)cols) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatrixLayoutCreate(&g->lay_c, HIP_R_16F, (uint64_t)n, (uint64_t)rows, (int64_t)n) == HIPBLAS_STATUS_SUCCESS;
    ok = ok && hipMalloc(&g->workspace, g->workspace_bytes) == hipSuccess;
    ok = ok && hipblasLtMatmulPreferenceCreate(&g->pref) == HIPBLAS_STATUS_SUCCESS &&
         hipblasLtMatmulPreferenceSetAttribute(g->pref, HIPBLASLT_MATMUL_PREF_MAX_WORKSPACE_BYTES, &g->workspace_bytes,
                                               sizeof(g->workspace_bytes)) == HIPBLAS_STATUS_SUCCESS;
    if (ok) {
        hipblasLtMatmulHeuristicResult_t result[1];
        int found = 0;
        ok = hipblasLtMatmulAlgoGetHeuristic(g->handle, g->desc, g->lay_b, g->lay_a, g->lay_c, g->lay_c, g->pref, 1, result,
                                             &found) == HIPBLAS_STATUS_SUCCESS && found > 0;
        if (ok) g->algo = result[0].algo;
    }
    if (!ok) {
        vendor_gemm_destroy(g);
        return nullptr;
    }
    return g;
}

int vendor_gemm_run(VendorGemm* g, const void* A_dev, const void* B_dev, void* C_dev, void* stream) {
    const float alpha = 1.f, beta = 0.f;
    hipblasStatus_t st = hipblasLtMatmul(g->handle, g->desc, &alpha, B_dev, g->lay_b, A_dev, g->lay_a, &beta, C_dev, g->lay_c,
                                         C_dev, g->lay_c, &g->algo, g->workspace, g->workspace_bytes, (hipStream_t)stream);
    return st == HIPBLAS_STATUS_SUCCESS ? 0 : 1;
}
