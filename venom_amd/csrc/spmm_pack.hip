// One-time packing of the canonical arrays into the copies the kernels read (operands in matrix-instruction
// order, row tables, gather tables).

#include "spmm_device.h"

namespace spatha {

// ---------------------------------------------------------------------------
// pack_kernel: canonical (values, metadata, columns) -> (apack, ipack, rowtab)
// One thread per (wave tile, step, mb, lane) for apack/ipack; rowtab separately.
// ---------------------------------------------------------------------------
__global__ void pack_a_kernel(const uint16_t* __restrict__ values, const uint32_t* __restrict__ metadata, int rows,
                              int ksp, int S, int half_tiles, uint16_t* __restrict__ apack) {
    // (rows % 64 == 32 with V a multiple of 32 only: the last wave tile's second half is padding, packed as zeros)
    const int64_t total = (int64_t)((rows + 63) / 64) * S * 4 * 64;
    const int ngroups = ksp / 2;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int lane = (int)(t & 63);
        int mb = (int)((t >> 6) & 3);
        int64_t ws = t >> 8;                 // wave tile * S + step
        int s = (int)(ws % S);
        int64_t wt = ws / S;
        int i = lane & 15, kq = lane >> 4;
        int ib = i >> 2, rr = i & 3;
        // matrix row; half_tiles: the order of the V = 32 kernels (instructions 0, 1 = rows 0..31 of the tile)
        int64_t r = wt * 64 + (half_tiles ? 32 * (mb >> 1) + 8 * ib + 4 * (mb & 1) + rr : 16 * ib + 4 * mb + rr);
        // canonical coordinates of the row
        int64_t R16 = r >> 4;
        int q = (int)((r >> 2) & 3), p = (int)((r >> 1) & 1), sbit = (int)(r & 1);
        uint16_t vals[8];
        uint32_t idx16 = 0;
#pragma unroll
        for (int gp = 0; gp < 4; gp++) {
            int fb = (kq >> 1) * 2 + (gp & 1);
            int kb = (kq & 1) * 2 + (gp >> 1);
            int g = s * 16 + fb * 4 + kb;                 // global group
            if (g < ngroups && r < rows) {
                int tt = g >> 2, u = g & 3;
                int64_t vi = R16 * 16 * (int64_t)ksp + (int64_t)tt * 128 + q * 32 + u * 8 + p * 4 + sbit * 2;
                vals[2 * gp] = values[vi];
                vals[2 * gp + 1] = values[vi + 1];
                int64_t wi = (r >> 5) * (int64_t)(ksp >> 3) * 16 + (int64_t)tt * 16 + ((r >> 4) & 1) * 8 + q * 2 + p;
                uint32_t nib = (metadata[wi] >> (sbit * 16 + u * 4)) & 0xfu;
                idx16 |= nib << (4 * gp);
            } else {
                vals[2 * gp] = 0;
                vals[2 * gp + 1] = 0;
                idx16 |= 0x4u << (4 * gp);                // positions (0,1): harmless, values are zero
            }
        }
        u32x4 out;
        out.x = vals[0] | ((uint32_t)vals[1] << 16);
        out.y = vals[2] | ((uint32_t)vals[3] << 16);
        out.z = vals[4] | ((uint32_t)vals[5] << 16);
        out.w = vals[6] | ((uint32_t)vals[7] << 16);
        char* blk = (char*)apack + ws * APACK_BLOCK;
        *(u32x4*)(blk + mb * 1024 + lane * 16) = out;
        // index words: [d][lane] dwords after the operands, 16 bits per mb (mb = 2d + half)
        *(uint16_t*)(blk + 4096 + (mb >> 1) * 256 + lane * 4 + (mb & 1) * 2) = (uint16_t)idx16;
    }
}

__global__ void pack_rowtab_kernel(const uint32_t* __restrict__ columns, int rows, int cols, int m, int v, int ksp,
                                   int S, uint32_t* __restrict__ rowtab) {
    const int ngroups = ksp / 2;
    const int64_t total = (int64_t)(rows / v) * S * 64;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        int rho = (int)(t & 63);
        int64_t bs = t >> 6;
        int s = (int)(bs % S);
        int64_t b = bs / S;
        int g = s * 16 + (rho >> 2), c = rho & 3;
        uint32_t row = 0xffffffffu;
        if (g < ngroups) {
            int64_t k = (int64_t)g * m + columns[b * ngroups * 4 + (int64_t)g * 4 + c];
            if (k < cols) row = (uint32_t)k;
        }
        rowtab[t] = row;
    }
}

// gather table of the dense-staged kernel: [64-row block][step][kb][c][fb] u16 = LDS byte offset of dense
// row d = gamma*m + column-loc (gamma = 4*fb + kb): d*256 + (d % 8)*32 (the swizzle of that row)
__global__ void pack_gtab_kernel(const uint32_t* __restrict__ columns, int rows, int m, int v, int ksp, int S,
                                 int block_rows, uint16_t* __restrict__ gtab) {
    const int ngroups = ksp / 2;
    const int64_t total = (int64_t)(rows / block_rows) * S * 64;
    for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < total; t += (int64_t)gridDim.x * blockDim.x) {
        const int fb = (int)(t & 3), c = (int)((t >> 2) & 3), kb = (int)((t >> 4) & 3);
        const int64_t bs = t >> 6;
        const int s = (int)(bs % S);
        const int64_t b = (bs / S) * block_rows / v;          // V block of this 64-row (or, for V = 32, 32-row) block
        const int gamma = fb * 4 + kb;
        const int g = s * 16 + gamma;
        uint32_t d = (uint32_t)gamma * m;
        if (g < ngroups) d += columns[b * ngroups * 4 + (int64_t)g * 4 + c];
        gtab[t] = (uint16_t)(d * 256u + (d & 7u) * 32u);
    }
}

hipError_t launch_pack_gtab(const uint32_t* columns, int rows, int m, int v, int ksp, int S, int block_rows, uint16_t* gtab,
                            hipStream_t stream) {
    int64_t total = (int64_t)(rows / block_rows) * S * 64;
    int blocks = (int)((total + 255) / 256);
    if (blocks > 65535 * 8) blocks = 65535 * 8;
    hipLaunchKernelGGL(pack_gtab_kernel, dim3(blocks), dim3(256), 0, stream, columns, rows, m, v, ksp, S, block_rows, gtab);
    return hipGetLastError();
}

hipError_t launch_pack(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                       int m, int v, int ksp, int S, int half_tiles, uint16_t* apack, uint32_t* rowtab, hipStream_t stream) {
    int64_t total_a = (int64_t)((rows + 63) / 64) * S * 256;
    int blocks_a = (int)((total_a + 255) / 256);
    if (blocks_a > 65535 * 8) blocks_a = 65535 * 8;
    hipLaunchKernelGGL(pack_a_kernel, dim3(blocks_a), dim3(256), 0, stream, values, metadata, rows, ksp, S, half_tiles, apack);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    int64_t total_r = (int64_t)(rows / v) * S * 64;
    int blocks_r = (int)((total_r + 255) / 256);
    if (blocks_r > 65535 * 8) blocks_r = 65535 * 8;
    hipLaunchKernelGGL(pack_rowtab_kernel, dim3(blocks_r), dim3(256), 0, stream, columns, rows, cols, m, v, ksp, S, rowtab);
    return hipGetLastError();
}

__global__ void clear_words_kernel(uint32_t* words, int count) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < count) words[i] = 0u;
}

hipError_t launch_clear_words(uint32_t* words, int count, hipStream_t stream) {
    if (count <= 0) return hipSuccess;
    hipLaunchKernelGGL(clear_words_kernel, dim3((count + 255) / 256), dim3(256), 0, stream, words, count);
    return hipGetLastError();
}

}  // namespace spatha
