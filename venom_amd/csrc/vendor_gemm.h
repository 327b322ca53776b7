// Vendor dense GEMM (hipBLASLt) for the benchmark driver: C[rows x n] = A[rows x cols] * B[cols x n], row-major fp16,
// fp32 compute.  vendor_gemm_create returns null when the library or a kernel for the shape is not available.
#pragma once

struct VendorGemm;

VendorGemm* vendor_gemm_create(int rows, int cols, int n);
int vendor_gemm_run(VendorGemm* g, const void* A_dev, const void* B_dev, void* C_dev, void* stream);
void vendor_gemm_destroy(VendorGemm* g);
