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
// NB = 1, 2 or 4 column blocks of 16.  Column block nb holds the columns NB * j + nb (j = 0 .. 15), not 16 * nb + j: lane j of
// a block then needs NB ADJACENT columns of every gathered row, one load of 2 * NB bytes instead of NB loads of 2 bytes - 16
// vector-memory instructions per k-step whatever N (with a load per element, 32 columns cost 39 us on the GPT-3 FFN matrix
// where 16 cost 30).  N is a multiple of 8, so the NB columns of a lane lie all inside N or all outside.
// ---------------------------------------------------------------------------
// LEAN (four column blocks only): see the main loop.  (The lean form is compiled for three waves per SIMD - three workgroups
// of four waves per CU - which it reaches with 158 registers.)
template <int NB, int OUT_LAYOUT, bool LEAN = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(LEAN ? 3 : 2))) void spmm_skinny_kernel(SpmmParams p) {
    // (the partial tiles are added up two column blocks at a time: 32 KB of LDS, so that three or more workgroups share a CU)
    constexpr int RB = NB < 2 ? NB : 2;
    __shared__ float4_t red[4][4][RB][64];
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
    static_assert(NB == 1 || NB == 2 || NB == 4, "column blocks per tile");
    const int col0 = NB * li;       // this lane's NB columns: col0 + nb
    auto load_b = [&](const u32x4 (&rt)[4], half16_t (&bf)[NB]) {
#pragma unroll
        for (int fb = 0; fb < 4; fb++)
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const uint32_t row = rt[fb][j];
                const uint32_t voff = (row != 0xFFFFFFFFu && col0 < N) ? row * row_bytes + (uint32_t)col0 * 2u : 0xF0000000u;
                if constexpr (NB == 1) {
                    const uint16_t h = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc_b, (int)voff, 0, 0);
                    bf[0][fb * 4 + j] = __builtin_bit_cast(_Float16, h);
                } else if constexpr (NB == 2) {
                    const uint32_t w = __builtin_amdgcn_raw_buffer_load_b32(rsrc_b, (int)voff, 0, 0);
                    bf[0][fb * 4 + j] = __builtin_bit_cast(_Float16, (uint16_t)w);
                    bf[1][fb * 4 + j] = __builtin_bit_cast(_Float16, (uint16_t)(w >> 16));
                } else {
                    const u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(rsrc_b, (int)voff, 0, 0);
                    bf[0][fb * 4 + j] = __builtin_bit_cast(_Float16, (uint16_t)w.x);
                    bf[1][fb * 4 + j] = __builtin_bit_cast(_Float16, (uint16_t)(w.x >> 16));
                    bf[2][fb * 4 + j] = __builtin_bit_cast(_Float16, (uint16_t)w.y);
                    bf[3][fb * 4 + j] = __builtin_bit_cast(_Float16, (uint16_t)(w.y >> 16));
                }
            }
    };

    auto multiply = [&](const half8_t (&a)[4], uint32_t i0, uint32_t i1, const half16_t (&b)[NB]) {
#pragma unroll
        for (int nb = 0; nb < NB; nb++) {
            acc[0][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[0], b[nb], acc[0][nb], (int)i0, 0, 0);
            acc[1][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[1], b[nb], acc[1][nb], (int)i0, 0, 1);
            acc[2][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[2], b[nb], acc[2][nb], (int)i1, 0, 0);
            acc[3][nb] = __builtin_amdgcn_smfmac_f32_16x16x64_f16(a[3], b[nb], acc[3][nb], (int)i1, 0, 1);
        }
    };
    int st = wave;
    if constexpr (!LEAN) {
        u32x4 rt1[4], rt2[4];
        half8_t a0[4], a1[4];
        uint32_t i00, i01, i10, i11;
        half16_t b0[NB], b1[NB];
        load_rt(st, rt1);
        load_a(st, a0, i00, i01);
        load_b(rt1, b0);
        load_rt(st + 4, rt1);
        for (; st < S; st += 4) {
            load_rt(st + 8, rt2);
            load_a(st + 4, a1, i10, i11);
            load_b(rt1, b1);
            multiply(a0, i00, i01, b0);
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
    } else {
        // Four column blocks with every operand double-buffered need 192 registers: two workgroups per CU.  With more than two
        // 64-row tiles per CU (GPT-3 FFN matrix: three) this form runs instead: only B is double-buffered, the A operands and
        // the row table of the next step are requested behind this step's matrix instructions, into the registers those have
        // just read; three workgroups per CU, whose loads cover one another's waits (38 against 40.5 us there; with one tile
        // per CU or less and long k-loops it is the slower form, 33.5 against 31.2 us on 12288 x 12288 at 64:2:8; with a wave's
        // share of the k-loop at four steps or less its shorter prologue wins again: 5.4 against 5.7 us on 4096 x 1024).
        u32x4 rt1[4];
        half8_t a0[4];
        uint32_t i00, i01;
        half16_t b0[NB], b1[NB];
        load_rt(st, rt1);
        load_a(st, a0, i00, i01);
        load_b(rt1, b0);
        load_rt(st + 4, rt1);
        for (; st < S; st += 4) {
            load_b(rt1, b1);
            multiply(a0, i00, i01, b0);
            load_a(st + 4, a0, i00, i01);
            load_rt(st + 8, rt1);
#pragma unroll
            for (int nb = 0; nb < NB; nb++) b0[nb] = b1[nb];
        }
    }
    // wave w finishes instruction-row block mb = w: rows 16*ib + 4*mb + r of the tile, column NB*li + nb
    const int out_mb = wave, ib = kb;
    const int64_t row0 = (int64_t)tile * 64 + 16 * ib + 4 * out_mb;
#pragma unroll
    for (int nb0 = 0; nb0 < NB; nb0 += RB) {
        if (nb0) __syncthreads();       // the pass before has been read
#pragma unroll
        for (int mb = 0; mb < 4; mb++)
#pragma unroll
            for (int nb = 0; nb < RB; nb++) red[wave][mb][nb][lane] = acc[mb][nb0 + nb];
        __syncthreads();
#pragma unroll
        for (int nb = 0; nb < RB; nb++) {
            float4_t sum = ((red[0][out_mb][nb][lane] + red[1][out_mb][nb][lane]) + red[2][out_mb][nb][lane]) + red[3][out_mb][nb][lane];
            const int col = col0 + nb0 + nb;
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
}

template <int OUT_LAYOUT>
static hipError_t launch_skinny(const SpmmParams& p, hipStream_t stream) {
    const dim3 grid(p.rows / 64), block(256);
    if (p.N <= 16) hipLaunchKernelGGL((spmm_skinny_kernel<1, OUT_LAYOUT>), grid, block, 0, stream, p);
    else if (p.N <= 32) hipLaunchKernelGGL((spmm_skinny_kernel<2, OUT_LAYOUT>), grid, block, 0, stream, p);
    else if (p.rows / 64 > 2 * p.cus || p.S <= 16) hipLaunchKernelGGL((spmm_skinny_kernel<4, OUT_LAYOUT, true>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((spmm_skinny_kernel<4, OUT_LAYOUT>), grid, block, 0, stream, p);
    return hipGetLastError();
}

hipError_t launch_skinny_family(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    if (variant != SPMM_VARIANT_SKINNY) return hipErrorInvalidValue;
    return out_layout == SPATHA_OUT_TRANSPOSED ? launch_skinny<SPATHA_OUT_TRANSPOSED>(p, stream)
                                               : launch_skinny<SPATHA_OUT_ROW_MAJOR>(p, stream);
}

}  // namespace spatha

