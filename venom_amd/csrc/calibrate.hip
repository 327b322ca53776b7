// Machine calibration kernels for bench.py --calibrate (library of their own, libspatha_calibrate.so; not part of the
// SpMM path and not declared in include/spatha.h).  They measure what bounds the SpMM kernels from outside:
//   spatha_calibrate_store   writes a rows x N fp16 matrix once, in the SpMM kernels' own tile order and store shape:
//                            the rate (and socket power) at which the chip takes the C matrix when nothing else runs
//   spatha_calibrate_smfmac  sparse matrix instructions on register operands only (the matrix phase of the 512 x 128
//                            kernel without its LDS reads and loads): the instruction rate (and socket power) the chip
//                            sustains for the operand values given - under its power limit that is well below the nominal
//                            peak for Gaussian operands; with either shape of the instruction
// Both return a hipError_t as int.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// 512 x 128 tiles, eight row tiles of a column panel in a row (the SpMM kernels' order); a wave owns 64 rows of its tile and
// writes them 8 rows x 128 bytes per instruction, write-through (the row-major write-out's stores)
__global__ __launch_bounds__(512) void store_kernel(uint16_t* C, int rows, int N, int seed) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int tiles_m = rows / 512, tiles = tiles_m * (N / 128);
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        const int tm = tile % tiles_m, tn = tile / tiles_m;
        u32x4 v;                  // pseudo-random bits: the power drawn depends on how many bits toggle
        v.x = (uint32_t)tile * 2654435761u ^ (uint32_t)lane * 40503u ^ (uint32_t)seed;
        v.y = v.x * 1664525u + 1013904223u;
        v.z = v.y * 1664525u + 1013904223u;
        v.w = v.z * 1664525u + 1013904223u;
        for (int half = 0; half < 2; half++)
            for (int r8 = 0; r8 < 8; r8++) {
                const int64_t row = (int64_t)tm * 512 + wave * 64 + r8 * 8 + (lane >> 3);
                uint16_t* dst = C + row * N + tn * 128 + half * 64 + (lane & 7) * 8;
                asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
                v.x += 0x9e3779b9u;
                v.z ^= v.x;
            }
    }
}

// every wave: 4 A operands (16 x 32 stored values each) and 8 B fragments (64 x 16) in registers, 32 matrix
// instructions per pass on 32 accumulator blocks - two waves per SIMD as in the SpMM kernel
__global__ __launch_bounds__(512) void smfmac_kernel(const _Float16* A, const _Float16* B, float* out, int passes) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    half8_t a[4];
    half16_t b[8];
    for (int i = 0; i < 4; i++) a[i] = *(const half8_t*)(A + (t * 4 + i) * 8);
    for (int i = 0; i < 8; i++) b[i] = *(const half16_t*)(B + (t * 8 + i) * 16);
    float4_t acc[8][4];
    for (int i = 0; i < 8; i++)
        for (int j = 0; j < 4; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    const int idx = 0x44444444;     // stored values 0 and 1 of every group of four sit at positions 0 and 1
    for (int p = 0; p < passes; p++) {
#pragma unroll
        for (int nb = 0; nb < 8; nb++)
#pragma unroll
            for (int mb = 0; mb < 4; mb++)
                acc[nb][mb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[mb], b[nb], acc[nb][mb], idx, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 8; i++)
        for (int j = 0; j < 4; j++) s += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    out[t] = s;
#endif
}

// the same wave tile (64 x 128, 64 k per pass) on the 32 x 32 x 32 sparse instruction: 2 x 4 blocks of 32 x 32, two
// k-halves, 16 instructions per pass, each twice the work of a 16 x 16 x 64 one
__global__ __launch_bounds__(512) void smfmac32_kernel(const _Float16* A, const _Float16* B, float* out, int passes) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    half8_t a[4];       // 2 row blocks x 2 k-halves
    half16_t b[8];      // 4 column blocks x 2 k-halves
    for (int i = 0; i < 4; i++) a[i] = *(const half8_t*)(A + (t * 4 + i) * 8);
    for (int i = 0; i < 8; i++) b[i] = *(const half16_t*)(B + (t * 8 + i) * 16);
    float16_t acc[2][4];
    for (int i = 0; i < 2; i++)
        for (int j = 0; j < 4; j++)
            for (int k = 0; k < 16; k++) acc[i][j][k] = 0.f;
    const int idx = 0x44444444;
    for (int p = 0; p < passes; p++) {
#pragma unroll
        for (int kh = 0; kh < 2; kh++)
#pragma unroll
            for (int nb = 0; nb < 4; nb++)
#pragma unroll
                for (int mb = 0; mb < 2; mb++)
                    acc[mb][nb] = __builtin_amdgcn_smfmac_f32_32x32x32_f16(a[mb * 2 + kh], b[nb * 2 + kh], acc[mb][nb], idx, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 2; i++)
        for (int j = 0; j < 4; j++)
            for (int k = 0; k < 16; k++) s += acc[i][j][k];
    out[t] = s;
#endif
}

}  // namespace

extern "C" {

// dst: rows x N fp16 (rows a multiple of 512, N of 128), written once by `workgroups` workgroups of 512 threads
int spatha_calibrate_store(uint16_t* dst, int rows, int N, int workgroups, int seed, void* stream) {
    if (!dst || rows <= 0 || N <= 0 || rows % 512 != 0 || N % 128 != 0 || workgroups <= 0) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(store_kernel, dim3(workgroups), dim3(512), 0, (hipStream_t)stream, dst, rows, N, seed);
    return (int)hipGetLastError();
}

// a: workgroups * 512 * 32 fp16, b: workgroups * 512 * 128 fp16, out: workgroups * 512 floats; per wave and pass 32
// instructions 16 x 16 x 64 (shape 16) or 16 instructions 32 x 32 x 32 (shape 32): the same work either way
int spatha_calibrate_smfmac(const uint16_t* a, const uint16_t* b, float* out, int workgroups, int passes, int shape, void* stream) {
    if (!a || !b || !out || workgroups <= 0 || passes <= 0 || (shape != 16 && shape != 32)) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL(shape == 32 ? smfmac32_kernel : smfmac_kernel, dim3(workgroups), dim3(512), 0, (hipStream_t)stream, (const _Float16*)a, (const _Float16*)b,
                       out, passes);
    return (int)hipGetLastError();
}

}  // extern "C"
