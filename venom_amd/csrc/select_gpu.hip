// Magnitude selector, search phase on the GPU: for every (V-row block, m-column group) the subset of 4 (3 in a
// three-column tail) columns that maximises the sum over the block's rows of the two largest magnitudes
// (group_n_m2 / func, end2end/grouped_nmv_tensor.py:81-343).  The totals are accumulated exactly as the host code
// does it (fp32, row by row, largest then second largest, no fused operations), subsets are ranked in lexicographic
// order and only a strictly larger total replaces the best one, so the winner is the host's winner bit for bit.
// One workgroup per task: the V x width block of magnitudes sits in LDS, every thread walks a contiguous range of
// subset ranks, a workgroup reduction keeps the largest total and, among equals, the lowest rank.

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "spmm_kernels.h"

namespace spatha {

namespace {
__device__ __forceinline__ unsigned long long binom(int n, int k) {      // k <= 4
    if (k < 0 || n < k) return 0ull;
    unsigned long long r = 1ull;
    for (int i = 0; i < k; i++) r = r * (unsigned long long)(n - i) / (unsigned long long)(i + 1);
    return r;
}
}  // namespace

__global__ __launch_bounds__(256) void select_winners_kernel(const float* __restrict__ dense_abs, int cols, int m, int v,
                                                             int full, int rem, int per_block, SelectWinner* __restrict__ out) {
    extern __shared__ float tile[];                 // [v][width]
    __shared__ float red_total[256];
    __shared__ unsigned long long red_rank[256];
    const int task = blockIdx.x, tid = threadIdx.x;
    const int b = task / per_block, gi = task - b * per_block;
    const int width = gi < full ? m : rem;
    const int take = (gi < full || rem != 3) ? 4 : 3;
    const float* base = dense_abs + (int64_t)b * v * cols + (int64_t)gi * m;
    for (int i = tid; i < v * width; i += 256) {
        const int r = i / width, c = i - r * width;
        tile[i] = base[(int64_t)r * cols + c];
    }
    __syncthreads();
    const unsigned long long nsub = binom(width, take);
    const unsigned long long chunk = (nsub + 255ull) / 256ull;
    unsigned long long rank = chunk * (unsigned long long)tid;
    const unsigned long long end = rank + chunk < nsub ? rank + chunk : nsub;
    float best = 0.f;
    unsigned long long best_rank = ~0ull;
    if (rank < nsub) {
        // unrank: the rank-th subset of {0..width-1} of size `take` in lexicographic order
        int pick[4] = {0, 0, 0, 0};
        {
            unsigned long long left = rank;
            int c = 0;
            for (int i = 0; i < take; i++) {
                while (true) {
                    const unsigned long long below = binom(width - 1 - c, take - 1 - i);   // subsets that keep c at position i
                    if (left < below) break;
                    left -= below;
                    c++;
                }
                pick[i] = c++;
            }
        }
        for (; rank < end; rank++) {
            float total = 0.f;
            if (take == 4) {
                const float* t0 = tile + pick[0];
                const float* t1 = tile + pick[1];
                const float* t2 = tile + pick[2];
                const float* t3 = tile + pick[3];
                for (int r = 0; r < v; r++) {
                    const float a = t0[r * width], bb = t1[r * width], c = t2[r * width], d = t3[r * width];
                    const float h1 = fmaxf(a, bb), l1 = fminf(a, bb), h2 = fmaxf(c, d), l2 = fminf(c, d);
                    const float top1 = fmaxf(h1, h2), top2 = fmaxf(fminf(h1, h2), fmaxf(l1, l2));
                    total = __fadd_rn(total, top1);
                    total = __fadd_rn(total, top2);
                }
            } else {
                const float* t0 = tile + pick[0];
                const float* t1 = tile + pick[1];
                const float* t2 = tile + pick[2];
                for (int r = 0; r < v; r++) {
                    const float a = t0[r * width], bb = t1[r * width], c = t2[r * width];
                    const float h1 = fmaxf(a, bb), l1 = fminf(a, bb);
                    const float top1 = fmaxf(h1, c), top2 = fmaxf(fminf(h1, c), l1);
                    total = __fadd_rn(total, top1);
                    total = __fadd_rn(total, top2);
                }
            }
            if (total > best) {
                best = total;
                best_rank = rank;
            }
            // next subset in lexicographic order
            int i = take - 1;
            while (i >= 0 && pick[i] == width - take + i) i--;
            if (i >= 0) {
                pick[i]++;
                for (int k = i + 1; k < take; k++) pick[k] = pick[k - 1] + 1;
            }
        }
    }
    red_total[tid] = best;
    red_rank[tid] = best_rank;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if (tid < s) {
            const float ot = red_total[tid + s];
            const unsigned long long orank = red_rank[tid + s];
            if (ot > red_total[tid] || (ot == red_total[tid] && orank < red_rank[tid])) {
                red_total[tid] = ot;
                red_rank[tid] = orank;
            }
        }
        __syncthreads();
    }
    if (tid == 0) {
        SelectWinner w;
        w.any = red_rank[0] != ~0ull && red_total[0] > 0.f;
        w.best[0] = w.best[1] = w.best[2] = w.best[3] = 0;
        if (w.any) {
            unsigned long long left = red_rank[0];
            int c = 0;
            for (int i = 0; i < take; i++) {
                while (true) {
                    const unsigned long long below = binom(width - 1 - c, take - 1 - i);
                    if (left < below) break;
                    left -= below;
                    c++;
                }
                w.best[i] = c++;
            }
        }
        out[task] = w;
    }
}

hipError_t launch_select_winners(const float* dense_abs_dev, int rows, int cols, int m, int v, SelectWinner* out_dev,
                                 hipStream_t stream) {
    const int blocks = rows / v, full = cols / m, rem = cols % m;
    const int per_block = full + ((rem >= 3) ? 1 : 0);
    const int tasks = blocks * per_block;
    if (tasks == 0) return hipSuccess;
    const int widest = full > 0 ? m : rem;
    const size_t lds = (size_t)v * widest * sizeof(float);
    if (lds > 150 * 1024) return hipErrorInvalidValue;
    if (lds > 48 * 1024) {
        hipError_t e = hipFuncSetAttribute((const void*)select_winners_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(select_winners_kernel, dim3(tasks), dim3(256), lds, stream, dense_abs_dev, cols, m, v, full, rem,
                       per_block, out_dev);
    return hipGetLastError();
}

}  // namespace spatha
