// Kernel for few columns of B (N <= 64): streaming A is all that matters.

#include "spmm_device.h"

namespace spatha {

// ---------------------------------------------------------------------------
// Skinny-N kernel (N <= 64): the product is bound by streaming A from HBM, not by the matrix units.
// One workgroup per 64-row tile; its four waves split the k-steps (wave w takes steps w, w+4, ...),
// so that 4 * rows/64 waves keep loads in flight, and add their fp32 partial tiles through LDS at the
// end in a fixed order.  No LDS staging of B: a lane fetches the 16 elements of its B fragment
// straight from global memory (B is small and stays in L2) through a buffer descriptor whose bounds
// check returns the zeros of padding rows and of columns beyond N.  Operands of step i+1 and the row
// table of step i+2 are requested before step i is multiplied.
// ---------------------------------------------------------------------------
template <int NB, int OUT_LAYOUT>
__global__ __launch_bounds__(256) void spmm_skinny_kernel(SpmmParams p) {
    __shared__ float4_t red[4][4][NB][64];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int tile = blockIdx.x;
    const int S = p.S, N = p.N;
    const int li = lane & 15, kb = lane >> 4;
    const int64_t vb = ((int64_t)tile * 64) / p.v;
    const char* a_tile = (const char*)p.apack + (int64_t)tile * S * APACK_BLOCK;
    const uint32_t* rt_block = p.rowtab + vb * S * 64;
    __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc((void*)p.B, 0, (int)p.b_bytes, 0x00020000);
    const uint32_t row_bytes = (uint32_t)N * 2u;

    float4_t acc[4][NB];
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < NB; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};

    auto clamp_step = [&](int st) { return st < S ? st : S - 1; };
    auto load_rt = [&](int st, u32x4 (&rt)[4]) {
        const uint32_t* q = rt_block + (int64_t)clamp_step(st) * 64 + 4 * kb;
#pragma unroll
        for (int fb = 0; fb < 4; fb++) rt[fb] = *(const u32x4*)(q + 16 * fb);
    };
    auto load_a = [&](int st, half8_t (&a)[4], uint32_t& i0, uint32_t& i1) {
        const char* q = a_tile + (int64_t)clamp_step(st) * APACK_BLOCK;
#pragma unroll
        for (int mb = 0; mb < 4; mb++) a[mb] = *(const half8_t*)(q + mb * 1024 + lane * 16);
        i0 = *(const uint32_t*)(q + 4096 + lane * 4);
        i1 = *(const uint32_t*)(q + 4352 + lane * 4);
    };
    auto load_b = [&](const u32x4 (&rt)[4], half16_t (&bf)[NB]) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            const int col = nb * 16 + li;
#pragma unroll
            for (int fb = 0; fb < 4; fb++)
#pragma unroll
                for (int j = 0; j < 4; j++) {
                    const uint32_t row = rt[fb][j];
                    const uint32_t voff = (row != 0xFFFFFFFFu && col < N) ? row * row_bytes + (uint32_t)col * 2u : 0xF0000000u;
                    const uint16_t h = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc_b, (int)voff, 0, 0);
                    bf[nb][fb * 4 + j] = __builtin_bit_cast(_Float16, h);
                }
        }
    };

    u32x4 rt1[4], rt2[4];
    half8_t a0[4], a1[4];
    uint32_t i00, i01, i10, i11;
    half16_t b0[NB], b1[NB];
    int st = wave;
    load_rt(st, rt1);
    load_a(st, a0, i00, i01);
    load_b(rt1, b0);
    load_rt(st + 4, rt1);
    for (; st < S; st += 4) {
        load_rt(st + 8, rt2);
        load_a(st + 4, a1, i10, i11);
        load_b(rt1, b1);
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            acc[0][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[0], b0[nb], acc[0][nb], (int)i00, 0, 0);
            acc[1][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[1], b0[nb], acc[1][nb], (int)i00, 0, 1);
            acc[2][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[2], b0[nb], acc[2][nb], (int)i01, 0, 0);
            acc[3][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a0[3], b0[nb], acc[3][nb], (int)i01, 0, 1);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            a0[k] = a1[k];
            rt1[k] = rt2[k];
        }
        i00 = i10;
        i01 = i11;
#pragma unroll
        for (int nb = 0; nb < NB; nb++) b0[nb] = b1[nb];
    }
#pragma unroll
    for (int mb = 0; mb < 4; mb++)
#pragma unroll
        for (int nb = 0; nb < NB; nb++) red[wave][mb][nb][lane] = acc[mb][nb];
    __syncthreads();
    // wave w finishes instruction-row block mb = w: rows 16*ib + 4*mb + r of the tile, column nb*16 + li
    const int mb = wave, ib = kb;
    const int64_t row0 = (int64_t)tile * 64 + 16 * ib + 4 * mb;
#pragma unroll
    for (int nb = 0; nb < NB; nb++) {
        float4_t sum = ((red[0][mb][nb][lane] + red[1][mb][nb][lane]) + red[2][mb][nb][lane]) + red[3][mb][nb][lane];
        const int col = nb * 16 + li;
        half4_t h4;
#pragma unroll
        for (int r = 0; r < 4; r++) h4[r] = (_Float16)sum[r];
        if (col >= N || SPATHA_KNOB(2)) continue;
        if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
            if (p.bias) h4 = h4 + *(const half4_t*)(p.bias + row0);
            *(half4_t*)(p.C + (int64_t)col * p.rows + row0) = h4;
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++) *(_Float16*)(p.C + (row0 + r) * N + col) = h4[r];
        }
    }
}

template <int OUT_LAYOUT>
static hipError_t launch_skinny(const SpmmParams& p, hipStream_t stream) {
    const int nb = (p.N + 15) / 16;
    const dim3 grid(p.rows / 64), block(256);
    if (nb <= 1) hipLaunchKernelGGL((spmm_skinny_kernel<1, OUT_LAYOUT>), grid, block, 0, stream, p);
    else if (nb == 2) hipLaunchKernelGGL((spmm_skinny_kernel<2, OUT_LAYOUT>), grid, block, 0, stream, p);
    else if (nb == 3) hipLaunchKernelGGL((spmm_skinny_kernel<3, OUT_LAYOUT>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((spmm_skinny_kernel<4, OUT_LAYOUT>), grid, block, 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_skinny_family(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    if (variant != SPMM_VARIANT_SKINNY) return hipErrorInvalidValue;
    return out_layout == SPATHA_OUT_TRANSPOSED ? launch_skinny<SPATHA_OUT_TRANSPOSED>(p, stream)
                                               : launch_skinny<SPATHA_OUT_ROW_MAJOR>(p, stream);
}

}  // namespace spatha

