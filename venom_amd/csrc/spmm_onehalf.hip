// One and a half row tiles per workgroup, walked through k together (V a multiple of 128).
//
// When 128-row tiles number about one and a half times the CUs, whole tiles leave half the chip idle in their second
// round, and a second launch for the rest streams all of B through every XCD's L2 once more.  Here a workgroup takes one
// whole row tile (128 rows x 256 columns) AND one 128-column half of another row tile, and runs both k-loops as one: the
// workgroups of an XCD stay in step through k, so a gathered row of B enters the XCD's L2 once per launch, and every CU
// has the same amount of work.  With T row tiles, F = ceil(2T / 3) workgroups per column tile take the tiles 0 .. F-1;
// the remaining T - F tiles are cut in two column halves and workgroup f < 2 (T - F) adds one of them (the two halves of a
// tile go to workgroups eight apart, i.e. on the same XCD, where T - F is a multiple of eight: the tile's rows of A then
// enter one L2).  A column half needs half of each gathered B row; a row half would need all of it for half the rows.
//
// A k-step is two sub-stages: F (64 gathered B rows x 256 columns of the whole tile's V block + two operand blocks) and H
// (64 gathered B rows x 128 columns of the other tile's V block + its two operand blocks).  Four LDS slots, F_a H_a F_b H_b;
// sub-stage s lives in slot s % 4 and two sub-stages are in flight behind the one being multiplied.  One workgroup barrier
// per sub-stage.
//
// Sixteen waves: what limits a wave here is per wave - about 20 B per clock of transposing LDS reads, one LDS-DMA
// instruction per ~60 clocks - so the work is spread over as many waves as the register file allows at 128 registers.
// Twelve consumer waves own one 64 x 64 block each (eight on the whole tile, four on the column half); a wave multiplies the
// first two 16-column fragments of its sub-stage in the interval after the sub-stage's barrier and the other two in the
// next interval (operands of A kept in registers), so that all twelve read LDS in every interval.  Four producer waves
// issue the A blocks and the row table; EVERY wave issues the B-row DMA of four rows of each sub-stage (two instructions
// in F, one in H).
//
//   barrier s   : sub-stage s has landed (every wave waited for its own share), readers of sub-stage s - 2 are done
//   all waves   : issue their share of sub-stage s + 2 into slot (s + 2) % 4 = slot of s - 2
//   F consumers : s even: fragments 0, 1 of F_(s/2)        s odd: fragments 2, 3 of F_((s-1)/2)
//   H consumers : s odd:  fragments 0, 1 of H_((s-1)/2)    s even: fragments 2, 3 of H_(s/2 - 1)

#include "spmm_device.h"

namespace spatha {

namespace {

constexpr int OH_ROW_BYTES = OhCfg::ROW_BYTES, OH_B_BYTES = OhCfg::B_BYTES, OH_F_BYTES = OhCfg::F_BYTES;
constexpr int OH_HROW_BYTES = OhCfg::HROW_BYTES, OH_HB_BYTES = OhCfg::HB_BYTES;
constexpr int OH_PAIR = OhCfg::PAIR, OH_RT_BASE = OhCfg::RT_BASE, OH_LDS = OhCfg::LDS_BYTES;
constexpr int OH_EPI_PITCH = 144;                               // write-out staging (in the slots, after the last barrier)
constexpr int OH_NC = 12, OH_NP = 4;
static_assert(OH_LDS <= 160 * 1024, "LDS budget");
static_assert(OH_NC * 16 * OH_EPI_PITCH <= OH_F_BYTES, "staging of the consumers fits the first slot");

// Two DMA instructions of 1 KiB behind ONE write of m0: the instruction's immediate offset moves the LDS destination
// (m0 + offset + lane * 16) and the memory address alike, so the second instruction uses a descriptor whose base lies
// 1 KiB below the buffer's (and whose size is 1 KiB more): base' + voff + 1 KiB = base + voff, and the range check
// voff + 1 KiB < size + 1 KiB is the buffer's own.
__device__ __forceinline__ void bdma2_b128(uint32_t v0, uint32_t v1, i32x4 r0, i32x4 r1, uint32_t lds_addr) {
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
        "buffer_load_dwordx4 %1, %3, 0 offen lds\n\t"
        "buffer_load_dwordx4 %2, %4, 0 offen offset:1024 lds" ::"s"(lds_addr),
        "v"(v0), "v"(v1), "s"(r0), "s"(r1)
        : "m0");
}

__device__ __forceinline__ uint32_t oh_slot(int s) { return (uint32_t)(((s >> 1) & 1) * OH_PAIR + (s & 1) * OH_F_BYTES); }

// A wave's share of the B rows of every sub-stage: rows 4 w .. 4 w + 3 (F: two DMA instructions of two 512-byte rows each;
// H: one instruction of four 256-byte rows).
struct OhRows {
    i32x4 r0, r1;
    uint32_t row_bytes_b;
    int col_f, col_h, n_cols, lane_, wave_;
    bool has_extra;
    __device__ __forceinline__ void init(const SpmmParams& p, int wave, int lane, int tn, int extra_half, bool has_extra_) {
        r0 = make_buffer(p.B, p.b_bytes);
        r1 = make_buffer((const char*)p.B - 1024, p.b_bytes + 1024u);
        row_bytes_b = (uint32_t)p.N * 2u;
        col_f = tn * 256;
        col_h = tn * 256 + extra_half * 128;
        n_cols = SPATHA_KNOB(1) ? 0 : p.N;
        lane_ = lane;
        wave_ = wave;
        has_extra = has_extra_;
    }
    // byte offset of the lane's 16-byte chunk inside a B row (the chunk order of an LDS row is swizzled by the row's low
    // bits); computed at issue time, registers are what this kernel is short of
    __device__ __forceinline__ uint32_t coloff_f(int i) const {
        const int rho = (wave_ * 2 + i) * 2 + (lane_ >> 5);
        const int col = col_f + ((lane_ & 31) ^ ((rho & 7) << 1)) * 8;
        return col < n_cols ? (uint32_t)col * 2u : 0xF0000000u;
    }
    __device__ __forceinline__ uint32_t coloff_h() const {
        const int rho = wave_ * 4 + (lane_ >> 4);
        const int col = col_h + ((lane_ & 15) ^ ((rho & 7) << 1)) * 8;
        return col < n_cols ? (uint32_t)col * 2u : 0xF0000000u;
    }
    __device__ __forceinline__ void issue_f(uint32_t row0, uint32_t row1, int s, uint32_t smem_base) const {
        const uint32_t v0 = (row0 == 0xffffffffu) ? 0xF0000000u : row0 * row_bytes_b + coloff_f(0);
        const uint32_t v1 = (row1 == 0xffffffffu) ? 0xF0000000u : row1 * row_bytes_b + coloff_f(1);
        bdma2_b128(v0, v1, r0, r1, smem_base + oh_slot(s) + (uint32_t)wave_ * 2048u);
    }
    __device__ __forceinline__ void issue_h(uint32_t row, int s, uint32_t smem_base) const {
        const uint32_t v = (row == 0xffffffffu) ? 0xF0000000u : row * row_bytes_b + coloff_h();
        bdma_b128(v, r0, 0, smem_base + oh_slot(s) + (uint32_t)wave_ * 1024u);
    }
    // sub-stage s >= 2: the rows come from the ring slot that the row-table DMA of sub-stage s - 2 filled
    __device__ __forceinline__ void issue_from_ring(const char* smem, int s, uint32_t smem_base) const {
        const char* rr = smem + OH_RT_BASE + (s & 3) * 256;
        if (!(s & 1)) {
            const char* e = rr + ((wave_ * 2) * 2 + (lane_ >> 5)) * 4;
            issue_f(*(const uint32_t*)e, *(const uint32_t*)(e + 8), s, smem_base);
        } else {
            const uint32_t row = *(const uint32_t*)(rr + (wave_ * 4 + (lane_ >> 4)) * 4);
            issue_h(has_extra ? row : 0xffffffffu, s, smem_base);
        }
    }
    // sub-stages 0 and 1: rows through ordinary loads (vb: V block whose row table applies)
    __device__ __forceinline__ void issue_first(const SpmmParams& p, int s, uint32_t vb, uint32_t smem_base) const {
        const uint32_t* rt = p.rowtab + (int64_t)vb * p.S * 64;
        if (!(s & 1)) {
            const int e = (wave_ * 2) * 2 + (lane_ >> 5);
            issue_f(rt[e], rt[e + 2], s, smem_base);
        } else {
            issue_h(has_extra ? rt[wave_ * 4 + (lane_ >> 4)] : 0xffffffffu, s, smem_base);
        }
    }
};

// full_block: 64-row block (rows / 64) the whole tile starts at; extra_block: the same of the tile whose column half
// `extra_half` the workgroup adds, < 0: none
template <int PR>
__device__ __forceinline__ void oh_producer(const SpmmParams& p, char* smem, uint32_t smem_base, int lane, int full_block,
                                            int extra_block, int extra_half, int tn) {
    // beside its share of the B rows: three of the twelve operand / index blocks of every sub-stage, and (producer 3) the
    // row-table entry two sub-stages on
    constexpr int N_A = 3 + (PR == 3);
    const int S = p.S;
    const int blocks_per_v = p.v / 64;
    const bool has_extra = extra_block >= 0;
    const i32x4 rsrc_a = make_buffer(p.apack, p.apack_bytes);
    const i32x4 rsrc_rt = make_buffer(p.rowtab, p.rowtab_bytes);
    const uint32_t lane16 = SPATHA_KNOB(32) ? 0xF0000000u : lane * 16, lane4 = SPATHA_KNOB(32) ? 0xF0000000u : lane * 4;
    // (integer division runs on the vector unit: back into scalar registers, the DMA's scalar offsets are built from these)
    const uint32_t vb_f = (uint32_t)__builtin_amdgcn_readfirstlane(full_block / blocks_per_v);
    const uint32_t vb_h = has_extra ? (uint32_t)__builtin_amdgcn_readfirstlane(extra_block / blocks_per_v) : 0u;
    OhRows part;
    part.init(p, OH_NC + PR, lane, tn, extra_half, has_extra);

    // the A blocks of sub-stage s (k-step s / 2; s even: F, s odd: H) and the row-table entry of sub-stage s + 2.
    // Producer PR: instructions 3 PR .. 3 PR + 2 of the twelve (row half = instruction / 6; inside a row half 0 .. 3: 1 KiB of
    // operands each, 4, 5: 256 B of index words each)
    auto issue_a = [&](int s) {
        const int k = s >> 1;
        const bool extra = s & 1;
        const uint32_t a_dst = smem_base + oh_slot(s) + (extra ? OH_HB_BYTES : OH_B_BYTES);
        const int block0 = extra ? (has_extra ? extra_block : 0) : full_block;
        const uint32_t v16 = (extra && !has_extra) ? 0xF0000000u : lane16, v4 = (extra && !has_extra) ? 0xF0000000u : lane4;
#pragma unroll
        for (int i = 0; i < 3; i++) {
            const int a = PR * 3 + i, hf = a / 6, ak = a - hf * 6;
            const uint32_t soff = (uint32_t)__builtin_amdgcn_readfirstlane(((block0 + hf) * S + k) * (int)APACK_BLOCK);
            const uint32_t dst = a_dst + hf * APACK_BLOCK;
            if (ak < 4) bdma_b128(v16, rsrc_a, soff + ak * 1024, dst + ak * 1024);
            else bdma_b32(v4, rsrc_a, soff + 4096 + (ak - 4) * 256, dst + 4096 + (ak - 4) * 256);
        }
        if (PR == 3) {
            const bool more = k + 1 < S && (!extra || has_extra);
            const uint32_t rt_src =
                (uint32_t)__builtin_amdgcn_readfirstlane((int)(((extra ? vb_h : vb_f) * (uint32_t)S + (uint32_t)(more ? k + 1 : 0)) * 256u));
            bdma_b32(more ? lane * 4u : 0xF0000000u, rsrc_rt, rt_src, smem_base + OH_RT_BASE + ((s + 2) & 3) * 256);
        }
    };
    // everything of sub-stage s is issued before anything of sub-stage s + 1: a wait then names how many instructions of
    // the younger sub-stage may still be in flight (B share: two instructions in F, one in H)
    part.issue_first(p, 0, vb_f, smem_base);
    issue_a(0);
    part.issue_first(p, 1, vb_h, smem_base);
    issue_a(1);
    for (int k = 0; k + 1 < S; k++) {
        wait_vmcnt<1 + N_A>();          // sub-stage 2k has landed, 2k + 1 (H) may be on its way
        __syncthreads();
        part.issue_from_ring(smem, 2 * k + 2, smem_base);
        issue_a(2 * k + 2);
        wait_vmcnt<2 + N_A>();          // sub-stage 2k + 1 has landed, 2k + 2 (F) may be on its way
        __syncthreads();
        part.issue_from_ring(smem, 2 * k + 3, smem_base);
        issue_a(2 * k + 3);
    }
    wait_vmcnt<1 + N_A>();
    __syncthreads();
    wait_vmcnt<0>();
    __syncthreads();
    __syncthreads();                    // the H consumers' last fragments
    __syncthreads();                    // the slots become write-out staging
}

template <int OUT_LAYOUT>
__device__ __forceinline__ void oh_consumer(const SpmmParams& p, char* smem, uint32_t smem_base, int wave, int lane, int full_block,
                                            int extra_block, int extra_half, int tn) {
    const int S = p.S, N = p.N;
    const bool on_extra = wave >= 8;
    // row half inside the sub-stage and 64-column block inside the sub-stage's columns
    const int h = on_extra ? ((wave - 8) >> 1) : (wave >> 2), q = on_extra ? (wave & 1) : (wave & 3);
    const bool has_extra = extra_block >= 0;
    float4_t acc[4][4];
    const int li = lane & 15, kb = lane >> 4;
    const int rrow = kb * 4 + (li >> 2);
    const int sw = rrow & 7;
    // offset of fragment nb's transposing read: the 16-byte chunk (q * 8 + nb * 2 + x) ^ (sw << 1) of the lane's row; nb * 2
    // occupies bits of its own, so fragment nb lies at tr0 ^ (nb * 32)
    const int tr0 = rrow * (on_extra ? OH_HROW_BYTES : OH_ROW_BYTES) + (((q * 8 + ((li & 3) >> 1)) ^ (sw << 1)) * 16) + (li & 1) * 8;
    const int a_base = (on_extra ? OH_HB_BYTES : OH_B_BYTES) + h * APACK_BLOCK;
    const int a_off = a_base + lane * 16, i_off = a_base + 4096 + lane * 4;
#pragma unroll
    for (int a = 0; a < 4; a++)
#pragma unroll
        for (int b = 0; b < 4; b++) acc[a][b] = (float4_t){0.f, 0.f, 0.f, 0.f};
    const int blocks_per_v = p.v / 64;
    OhRows part;
    part.init(p, wave, lane, tn, extra_half, has_extra);
    part.issue_first(p, 0, (uint32_t)__builtin_amdgcn_readfirstlane(full_block / blocks_per_v), smem_base);
    part.issue_first(p, 1, has_extra ? (uint32_t)__builtin_amdgcn_readfirstlane(extra_block / blocks_per_v) : 0u, smem_base);
    // barrier s: wait for the wave's own share of sub-stage s (the younger share, of sub-stage s + 1, may be in flight: one
    // instruction if that is an H sub-stage, two if F) and meet the others; the share of sub-stage s + 2 is issued behind
    // the first LDS reads of the interval's multiply
    auto meet = [&](int s) {
        if (s + 1 >= 2 * S) wait_vmcnt<0>();
        else if (s & 1) wait_vmcnt<2>();
        else wait_vmcnt<1>();
        __syncthreads();
    };
    auto issue = [&](int s) {
        if (s + 2 < 2 * S) part.issue_from_ring(smem, s + 2, smem_base);
    };
    const bool works = (!on_extra || has_extra) && !SPATHA_KNOB(16);
    half8_t a_cur[4];
    uint32_t i0 = 0, i1 = 0;
    // (the row pitch of a B fragment read is a template argument: one instantiation per role)
    auto frag = [&](const char* st, int off) {
        return on_extra ? read_b_fragment<OH_HROW_BYTES>(st, off) : read_b_fragment<OH_ROW_BYTES>(st, off);
    };
    // first interval of a sub-stage: operands of A (kept for the second interval) and fragments 0, 1
    auto first_half = [&](const char* st, int s) {
        if (works) {
#pragma unroll
            for (int mb = 0; mb < 4; mb++) a_cur[mb] = *(const half8_t*)(st + a_off + mb * 1024);
            i0 = *(const uint32_t*)(st + i_off);
            i1 = *(const uint32_t*)(st + i_off + 256);
            half16_t bf0 = frag(st, tr0);
            half16_t bf1 = frag(st, tr0 ^ 32);
            __builtin_amdgcn_sched_barrier(0);
            issue(s);
            __builtin_amdgcn_sched_barrier(0);
            SPATHA_MMA4(0, bf0)
            SPATHA_MMA4(1, bf1)
        } else {
            issue(s);
        }
    };
    auto second_half = [&](const char* st, int s) {
        if (works) {
            half16_t bf0 = frag(st, tr0 ^ 64);
            half16_t bf1 = frag(st, tr0 ^ 96);
            __builtin_amdgcn_sched_barrier(0);
            issue(s);
            __builtin_amdgcn_sched_barrier(0);
            SPATHA_MMA4(2, bf0)
            SPATHA_MMA4(3, bf1)
        } else {
            issue(s);
        }
    };
    if (!on_extra) {
        for (int k = 0; k < S; k++) {
            const char* st = smem + (k & 1) * OH_PAIR;
            meet(2 * k);
            first_half(st, 2 * k);
            meet(2 * k + 1);
            second_half(st, 2 * k + 1);
        }
        __syncthreads();
    } else {
        meet(0);
        issue(0);
        for (int k = 0; k < S; k++) {
            const char* st = smem + (k & 1) * OH_PAIR + OH_F_BYTES;
            meet(2 * k + 1);
            first_half(st, 2 * k + 1);
            if (k + 1 < S) meet(2 * k + 2); else __syncthreads();
            second_half(st, 2 * k + 2);
        }
    }
    __syncthreads();
    if ((on_extra && !has_extra) || SPATHA_KNOB(4)) return;
    const int64_t row0 = (int64_t)((on_extra ? extra_block : full_block) + h) * 64;
    // (an opaque copy of the lane number: what the write-out derives from it must not occupy registers during the k-loop)
    asm volatile("" : "+v"(lane));
    const int j16 = lane & 15, ib = lane >> 4;
    char* stg = smem + wave * (16 * OH_EPI_PITCH);
    const int col0 = tn * 256 + (on_extra ? extra_half * 128 : 0) + q * 64;
    if (p.fuse) fused_bias_act(acc, p.bias, row0 + ib * 16, p.act);
    if (OUT_LAYOUT == SPATHA_OUT_TRANSPOSED) {
        store_block_transposed_slab<true>(acc, stg, p.C, p.fuse ? nullptr : p.bias, row0, col0, p.rows, N, lane, true);
    } else {
        // 16-row slabs through the wave's staging buffer -> 128-byte row segments
#pragma unroll
        for (int mb = 0; mb < 4; mb++) {
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int nb = 0; nb < 4; nb++)
                    *(_Float16*)(stg + (r * 4 + ib) * OH_EPI_PITCH + (nb * 16 + j16) * 2) = (_Float16)acc[mb][nb][r];
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int it = 0; it < 2; it++) {
                const int Lr = it * 8 + (lane >> 3), ch = lane & 7;
                const int row = 16 * (Lr & 3) + 4 * mb + (Lr >> 2);
                const int col = col0 + ch * 8;
                u32x4 v = *(const u32x4*)(stg + Lr * OH_EPI_PITCH + ch * 16);
                if (col < N) store_c16(p.C + (row0 + row) * N + col, v);
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

template <int OUT_LAYOUT>
__global__ __launch_bounds__((OH_NC + OH_NP) * 64) void spmm_oh_kernel(SpmmParams p) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)LDS_PTR(char, smem);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = p.tiles_m, F = (2 * T + 2) / 3, X = T - F;          // X tiles in two column halves each
    const int tn = __builtin_amdgcn_readfirstlane((int)blockIdx.x / F), f = (int)blockIdx.x - tn * F;
    const int full_block = 2 * f;
    // the two halves of an extra tile on workgroups eight apart (same XCD) where the count allows, else on neighbours
    int extra_tile = -1, extra_half = 0;
    if (f < 2 * X) {
        if (X % 8 == 0) { extra_tile = F + (f >> 4) * 8 + (f & 7); extra_half = (f >> 3) & 1; }
        else { extra_tile = F + (f >> 1); extra_half = f & 1; }
    }
    const int extra_block = extra_tile < 0 ? -1 : 2 * extra_tile;
    if (wave < OH_NC) oh_consumer<OUT_LAYOUT>(p, smem, smem_base, wave, lane, full_block, extra_block, extra_half, tn);
    else if (wave == OH_NC) oh_producer<0>(p, smem, smem_base, lane, full_block, extra_block, extra_half, tn);
    else if (wave == OH_NC + 1) oh_producer<1>(p, smem, smem_base, lane, full_block, extra_block, extra_half, tn);
    else if (wave == OH_NC + 2) oh_producer<2>(p, smem, smem_base, lane, full_block, extra_block, extra_half, tn);
    else oh_producer<3>(p, smem, smem_base, lane, full_block, extra_block, extra_half, tn);
}

template <int OUT_LAYOUT>
hipError_t launch_oh(const SpmmParams& p, hipStream_t stream) {
    auto kern = spmm_oh_kernel<OUT_LAYOUT>;
    bool& attr_set = lds_attr_flag((const void*)kern);
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, OH_LDS);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int F = (2 * p.tiles_m + 2) / 3;
    hipLaunchKernelGGL(kern, dim3(F * p.tiles_n), dim3((OH_NC + OH_NP) * 64), OH_LDS, stream, p);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_onehalf(int variant, int out_layout, const SpmmParams& p, hipStream_t stream) {
    if (variant != SPMM_VARIANT_OH192x256) return hipErrorInvalidValue;
    if (p.v % 128 != 0 || p.rows % 128 != 0 || p.tiles_m != p.rows / 128 || p.ksplit != 1) return hipErrorInvalidValue;
    return out_layout == SPATHA_OUT_TRANSPOSED ? launch_oh<SPATHA_OUT_TRANSPOSED>(p, stream)
                                               : launch_oh<SPATHA_OUT_ROW_MAJOR>(p, stream);
}

}  // namespace spatha
