// C ABI of the library (see include/spatha.h): argument checking, plan
// management and kernel selection.  No torch types, no exceptions across the
// boundary, no exit().

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <new>
#include <vector>

#include "../../include/spatha.h"
#include "spmm_kernels.h"
#include "vnm_format.h"

#include "spatha_internal.h"

namespace {
thread_local int g_last_hip_error = 0;

inline int hip_fail(hipError_t e) {
    g_last_hip_error = (int)e;
    return SPATHA_ERR_HIP;
}

// kernels whose write-out can apply bias and activation ahead of either output layout
bool variant_has_fused_writeout(int variant) {
    using namespace spatha;
    switch (variant) {
        case SPMM_VARIANT_P128x128_S3: case SPMM_VARIANT_P64x256_S2: case SPMM_VARIANT_R64x256_S3:
        case SPMM_VARIANT_W128x128_S3: case SPMM_VARIANT_W128x256_S3: case SPMM_VARIANT_W64x256_S3:
        case SPMM_VARIANT_T128x256_S3: case SPMM_VARIANT_DS256x128_S3_C8: case SPMM_VARIANT_DSH256x128_S3_C8:
        case SPMM_VARIANT_UP512x128_S3: case SPMM_VARIANT_DU512x128_M16: case SPMM_VARIANT_WS128x128_S3:
        case SPMM_VARIANT_WS64x256_S3: case SPMM_VARIANT_OH192x256: case SPMM_VARIANT_H64x256_S2: case SPMM_VARIANT_H64x128_S3: case SPMM_VARIANT_H64x128_S2:
            return true;
        default:
            return false;
    }
}

// kernels that address B, the packed operands and the tables through buffer descriptors (32-bit offsets)
bool variant_uses_buffer_descriptors(int variant) {
    using namespace spatha;
    switch (variant) {
        case SPMM_VARIANT_128x128: case SPMM_VARIANT_64x256: case SPMM_VARIANT_P128x128_S3: case SPMM_VARIANT_P64x256_S2:
            return false;
        default:
            return true;
    }
}

bool variant_ok(const spatha_spmm_plan* plan, int N, int variant, bool fused = false) {
    using namespace spatha;
    if (variant <= 0 || variant >= SPMM_VARIANT_COUNT) return false;
    if (fused && !variant_has_fused_writeout(variant)) return false;
    const int bm = spmm_variant_bm(variant);
    if (bm == 0) return false;
    const bool half_variant = variant == SPMM_VARIANT_H64x256_S2 || variant == SPMM_VARIANT_H64x128_S3 ||
                              variant == SPMM_VARIANT_H64x128_S2 || variant == SPMM_VARIANT_DSH256x128_S3_C8;
    if (half_variant != (plan->half_tiles != 0)) return false;       // the packed operand order differs
    const uint64_t b_bytes = (uint64_t)plan->geo.cols * (uint64_t)N * 2u;
    if (variant == SPMM_VARIANT_DSH256x128_S3_C8) {
        if (plan->geo.m > 8 || plan->geo.rows % 256 != 0 || !plan->gtab) return false;
        return b_bytes < 0xE0000000ull && plan->apack_bytes < 0xE0000000ull;
    }
    if (half_variant) return plan->geo.cols <= 65535 && spmm_variant_lds(variant, plan->S) <= 160 * 1024;
    const bool unified = variant == SPMM_VARIANT_UP512x128_S3 || variant == SPMM_VARIANT_DU512x128_M16;
    if (variant == SPMM_VARIANT_DS256x128_S3_C8 || variant == SPMM_VARIANT_DS256x128_S3_PP) {
        // four 64-row blocks per tile; all 16*m dense rows of a k-step must fit one stage
        if (plan->geo.v % 64 != 0 || plan->geo.m > 8 || plan->geo.rows % 256 != 0 || !plan->gtab) return false;
    } else if (unified) {
        if (plan->geo.v % 64 != 0 || plan->geo.rows % 512 != 0 || !plan->gtab || plan->half_tiles) return false;
        if (variant == SPMM_VARIANT_DU512x128_M16 ? (plan->geo.m <= 8 || plan->geo.m > 16) : plan->geo.m > 8) return false;
        if (plan->gtab_bytes >= 0xE0000000ull) return false;
    } else if (plan->geo.v % bm != 0) {
        return false;
    }
    if (variant == SPMM_VARIANT_SKINNY && N > 64) return false;
    if ((variant == SPMM_VARIANT_WS128x128_S3 || variant == SPMM_VARIANT_WS64x256_S3) && plan->S < 2)
        return false;       // the tile hand-over to the store waves needs two k-steps per tile
    if (spmm_variant_lds(variant, plan->S) > 160 * 1024) return false;      // row table kept in LDS
    if (variant_uses_buffer_descriptors(variant) &&
        (b_bytes >= 0xE0000000ull || plan->apack_bytes >= 0xE0000000ull || plan->rowtab_bytes >= 0xE0000000ull))
        return false;
    return true;
}

// ---- Kernel choice ----------------------------------------------------------------------------------------------
// The automatic choice is a list of rules read top-down: the first rule whose class and condition hold for the shape
// and whose kernel accepts the plan (variant_ok) names the kernel.  The conditions are measured crossover points on
// MI355X (BERT-base / BERT-large / GPT-2-large / GPT-3 layer shapes, N = 2048 .. 16384, m = 4 .. 100); each rule's comment
// says what was measured.  Later rules double as the fall-backs of earlier ones.
struct Shape {
    int v, m, rows, N, S;
    int64_t cus;
    bool fused, transposed;
    // tiles of bm x bn in the output (whole row tiles only: the kernels that take a partial row tile are never chosen by count)
    int64_t tiles(int bm, int bn) const { return (int64_t)(rows / bm) * ((N + bn - 1) / bn); }
    // the last of `tiles` tiles' rounds over the CUs is at least 90 % full (a single round: 75 %)
    bool whole_rounds(int64_t t) const {
        const int64_t rounds = (t + cus - 1) / cus;
        return rounds == 1 ? t * 4 >= cus * 3 : t * 10 >= rounds * cus * 9;
    }
    // unified 512 x 128 tiles against dense-staged 256 x 128 ones by rounds of tiles over the CUs, a 512-row tile counted as
    // two and 10 % off for what it saves per tile (5120 x 1280 x 2048 at 2:8 and 2:4: 160 tiles on 256 CUs in one round, 17 and
    // 24 us, against 1.25 rounds of 320 dense-staged tiles, 20 and 32 us)
    bool unified_rounds_ahead() const {
        const int64_t r_up = (tiles(512, 128) + cus - 1) / cus, r_ds = (tiles(256, 128) + cus - 1) / cus;
        // (long k-loops, where a tile's write-out weighs less: 25 % off - 12288 x 12288 x 2048 at 64:2:8 and 2:4, 384 tiles in two
        // rounds against 768 in three, 212 / 396 against 236 / 429 us)
        return r_up * (S >= 64 ? 15 : 18) <= r_ds * 10;
    }
    // 128 x 256 tiles ahead of 128 x 128 ones: from 1024 tiles on, from 768 with two or more k-steps, from 512 with eight or
    // more; with fewer, from 192 tiles of 32 or more k-steps, and with 10 .. 31 k-steps where the rounds say so (1280 x 5120 at
    // 128:2:16 / 20 / 32: 4096 tokens, 160 tiles in one round, 18.7 / 16.5 / 13.0 against 22.0 / 18.8 / 14.1 us; 8192 tokens, 320
    // tiles in two rounds against 640 in three, 28.1 / 22.0 against 25.9 / 19.3 us at 2:20 / 2:32) (every kernel on the BERT layer shapes x N = 2048 .. 8192 x 2:10 .. 2:100;
    // 1024 x 1024 x 16384 at 128:2:16, 512 wide tiles of 4 k-steps, runs 19 % faster on 128 x 128 tiles)
    // (never for a single, half-empty column tile: GPT-3 FFN matrix at 128 tokens, 46.5 us on 128 x 128 against 61.5 us)
    bool wide() const {
        const int64_t t = tiles(128, 256);
        if (N <= 128) return false;
        if (t >= 1024 || (t >= 768 && S >= 2) || (t >= 512 && S >= 8)) return true;
        if (S >= 32) return t >= 192;
        // few tiles of 10 .. 31 k-steps: by rounds of tiles over the CUs, a 128 x 256 tile counted as 1.6 tiles of 128 x 128
        const int64_t r_wide = (t + cus - 1) / cus, r_narrow = (tiles(128, 128) + cus - 1) / cus;
        return S >= 10 && t >= 160 && r_wide * 16 <= r_narrow * 10;
    }
    // transposed output: 128 x 256 tiles from 512 tiles on, with fewer by rounds (a 128 x 256 tile counted as 1.6 of 128 x 128)
    bool wide_transposed() const {
        const int64_t t = tiles(128, 256);
        if (t >= 512) return true;
        const int64_t r_wide = (t + cus - 1) / cus, r_narrow = (tiles(128, 128) + cus - 1) / cus;
        return r_wide * 16 <= r_narrow * 10;
    }
    // 64 x 256 tiles with long k-loops: the persistent three-stage pipeline leads the per-tile one with two stages at any tile
    // count (1280 x 5120 at 64:2:10, 4096 .. 16384 tokens, 320 .. 1280 tiles: 45 / 66 / 108 against 56 / 84 / 139 us;
    // 12288 x 12288 x 512 at 64:2:16 and 64:2:10: 66 / 100 against 86 / 132 us)
    bool long_k() const { return S >= 32; }
    // More than one round of 128 x 256 tiles over the CUs and at most a round and a half: F = ceil(2T / 3) workgroups per
    // 256-column tile, each with one whole tile and a 128-column half of another, run them in ONE round of equal workgroups
    // that stay in step through k (kernel 22).  Every kernel id on 49152 / 40960 / 36864 / 34816 x 12288 (GPT-3 FFN matrix and
    // fewer rows of it; 384 .. 272 row tiles on 256 CUs) at 136 .. 256 tokens, 128:2:16, Gaussian data: 53-57 / 52 / 50 / 50 us
    // against 61-66 us for 256 tall tiles + the rest on 128 x 128 tiles in a second launch; the same rows x 1024 .. 6144
    // columns (4 .. 24 k-steps), where the 128 x 128 tiles with store waves were chosen: 1.06-1.36x ahead row-major from 8
    // k-steps on (4 k-steps: 0.94-1.06x), 1.19-1.53x transposed; 128:2:40 1.28-1.70x; 16128 x 12288 x 768 and 12288^2 x
    // 1024 (three and four column tiles) 57 us against 59-70.  Not for m <= 8 (dense staging: 1.07-1.09x at 2:8 on the long
    // k-loop only, behind at 2:4), not when the last column tile has no columns for the second half, not beyond one round of
    // such workgroups (8192 x 4096 x 1536: 41 against 27 us), and for at most four column tiles: with many of them (few row
    // tiles, a large output: 1536 x 4096 x 8192, 1280 x 5120 x 8192, 768 x 3072 x 16384, 3072 x 4096 x 3584) the 128 x 128 tiles
    // with store waves, which write a tile out under the next tile's k-loop, are level (transposed) or 3-12 % ahead (row-major).
    bool tile_and_a_half() const {
        if (m <= 8 || rows % 128 != 0 || S < 4 || (S < 8 && !transposed)) return false;
        const int64_t T = rows / 128, tn = (N + 255) / 256, F = (2 * T + 2) / 3, grid = (cus / 8) * 8;
        const int last = N - (int)(tn - 1) * 256;
        return tn <= 4 && T * tn > grid && F * tn <= grid && last > 128;
    }
    // 64 x 256 tiles: many tiles of few k-steps, m >= 32, row-major
    bool short_k_many() const { return m >= 32 && !transposed && tiles(64, 256) >= 2048 && S <= 8; }
};

enum : unsigned { V_HALF = 1u, V_128 = 2u, V_64 = 4u };       // V % 64 != 0 / V % 128 == 0 / V % 64 == 0 only

struct Rule {
    unsigned v_classes;
    int variant;
    bool (*when)(const Shape&);
};

const Rule kRules[] = {
    // few columns: streaming A is all that matters, one 64-row tile per workgroup with the k-steps split over its waves, B
    // straight from the L2 with one load per gathered row whatever N (2, 4 or 8 bytes for 16, 32 or 64 columns).  Up to 32
    // columns: 1.3-1.5x ahead of every tiled kernel on the BERT-large matrices, 31.7 us on the GPT-3 FFN matrix (5.6 TB/s;
    // 128-wide tiles 39-41).  33 .. 64 columns, V a multiple of 64: 5.7 us on 4096 x 1024 at 64:2:8 and 128:2:8 (tiled
    // kernels 6.8-7.7), 31.3 us on 12288 x 12288 at 64:2:8 (49.2), 7.4 us on 1024 x 4096 at 64:2:16 (equal); on the GPT-3 FFN
    // matrix 40.5 us, level with the 128 x 128 tiles (39.4): there the 192 registers of its four column blocks leave two
    // workgroups per CU for three tiles per CU.
    {V_HALF | V_128 | V_64, spatha::SPMM_VARIANT_SKINNY, [](const Shape& s) { return s.N <= 32; }},
    {V_128 | V_64, spatha::SPMM_VARIANT_SKINNY, [](const Shape& s) { return s.N <= 64; }},

    // -- V % 64 != 0 (1024 x 4096 x 4096 and 4096 x 1024 x 16384, m = 8 .. 32) --
    // m <= 8: the dense B stage is shared by eight 32-row blocks, the fill does not grow with the smaller V
    // (short k-loops - 8 or 10 k-steps - on 64 tiles or fewer, 1024 x 1024 up to 2048 tokens, 4096 x 1024 up to 512: the gathered
    // half-tile kernels are 9-24 % ahead; with 32 k-steps or more dense staging leads at any tile count, 1.2-3.4x on 1024 x 4096,
    // 1280 x 5120 and 12288 x 12288)
    {V_HALF, spatha::SPMM_VARIANT_DSH256x128_S3_C8, [](const Shape& s) { return s.tiles(256, 128) >= 160 || s.S >= 16; }},
    // the 256-wide tile is never behind the 128-wide one with two stages by more than 7 %, and up to 2x ahead
    {V_HALF, spatha::SPMM_VARIANT_H64x256_S2, [](const Shape& s) { return s.N > 128; }},
    // (three stages of 128 leave two waves per CU)
    {V_HALF, spatha::SPMM_VARIANT_H64x128_S2, [](const Shape&) { return true; }},
    {V_HALF, spatha::SPMM_VARIANT_H64x128_S3, [](const Shape&) { return true; }},

    // -- unified 512 x 128 tiles --
    // m <= 8, two phase groups: 3-13 % ahead of the dense-staged 256 x 128 tiles when its tiles fill whole rounds of the CUs
    // (BERT-large layer shapes at N = 16384, V = 64 and 128, m = 8 and 4: 256, 768, 1024 tiles; 3072 x 768 x 4096, 192
    // tiles: 10-12 % ahead), 10-20 % behind at 320 or 384 tiles and up to 2x behind with fewer tiles than CUs;
    // transposed output with 256 tiles of 8 k-steps measures 2-3 % behind
    {V_128 | V_64, spatha::SPMM_VARIANT_UP512x128_S3,
     [](const Shape& s) {
         const int64_t t = s.tiles(512, 128);
         // (transposed output with one or two full rounds of 8 k-steps is level with the dense-staged 256 x 128 tiles or 2-3 %
         // behind; with less than a round - 3072 x 1024 x 4096, 5120 x 1280 x 2048: 192 and 160 tiles - 11-13 % ahead)
         return s.m <= 8 && (s.whole_rounds(t) || s.unified_rounds_ahead()) &&
                (!s.transposed || t >= 2 * s.cus || s.S >= 16 || t < s.cus);
     }},
    // 8 < m <= 16, one phase group with two 64 KB stages: 7-26 % ahead of the gathered 64 x 256 tiles on the BERT-large
    // layer shapes at N = 16384 (64:2:16 and 64:2:10, both layouts); on long k-loops ahead at 1.5 rounds too (12288 x 12288
    // x 2048 at 64:2:16: 177 us against 188 us for the best gathered form).  With V % 128 == 0 the gathered 128 x 256
    // tiles share their B rows over 128 rows and are equal or up to 15 % ahead.
    {V_64, spatha::SPMM_VARIANT_DU512x128_M16,
     [](const Shape& s) {
         const int64_t t = s.tiles(512, 128);
         return s.m > 8 && (s.whole_rounds(t) || (t >= s.cus && s.S >= 32));
     }},

    // -- V % 128 == 0 --
    // transposed output, m <= 8: the kernels that write through the 8-column slab lead by 10-25 % (BERT-large layer shapes,
    // N = 16384, with bias); not on long k-loops, where the gathered 128 x 256 tile moves fewer bytes per output element
    // (GPT-3 block at 128:2:8, 96 k-steps: 6.95 ms against 8.26 ms; GPT-2-large FFN-down, 40 k-steps: dense staging 20 % ahead)
    // (m <= 5: every dense row is a gathered row or nearly so, dense staging leads at any k: 1280 x 5120 x 4096 at 2:4, 80
    // k-steps, 45 against 65 us on 128 x 128 tiles; 12288 x 12288 x 512 at 2:4 115 against 127 us on 128 x 256 tiles)
    // (from 160 tiles on, as row-major: with fewer - 1024 x 4096 x 2048 / 4096, 1280 x 5120 x 2048: 64 .. 128 tiles - the
    // gathered 128 x 128 tiles are 13-35 % ahead)
    {V_128, spatha::SPMM_VARIANT_DS256x128_S3_C8,
     [](const Shape& s) { return s.transposed && s.m <= 8 && (s.S <= 40 || s.m <= 5) && s.tiles(256, 128) >= 160; }},
    // row-major, m <= 8: dense staging leads the gathered tiles by 5-35 % as soon as its 256 x 128 tiles fill three quarters
    // of the CUs (BERT layer shapes, N = 2048 .. 16384; from 160 tiles on the GPT-2-large ones).  Up to 768 tiles the form in
    // two phase groups leads the eight-consumer form by 2-5 %; it has no fused write-out, and falls behind on long k-loops
    // (12288 x 12288 x 2048 at 64:2:8, 96 k-steps: 255 us against 239 us)
    {V_128, spatha::SPMM_VARIANT_DS256x128_S3_PP,
     [](const Shape& s) {
         const int64_t t = s.tiles(256, 128);
         return !s.transposed && !s.fused && s.m <= 8 && s.rows % 256 == 0 && t >= 160 && t <= 768 && s.S <= 32;
     }},
    {V_128, spatha::SPMM_VARIANT_DS256x128_S3_C8,
     [](const Shape& s) {
         return !s.transposed && s.m <= 8 && s.rows % 256 == 0 && s.tiles(256, 128) >= 160 && (s.S <= 64 || s.m <= 5);
     }},
    // m > 8, between one and one and a half rounds of 128 x 256 tiles: one whole tile and a column half of another per workgroup
    {V_128, spatha::SPMM_VARIANT_OH192x256, [](const Shape& s) { return s.tile_and_a_half(); }},
    // transposed output, m > 8, more than one 128-column tile: 128 x 256 tiles at any tile count (5-15 % ahead of 128 x 128 on the BERT-large and
    // GPT-2-large layer shapes, N = 4096 and 16384); 64 x 64 consumer blocks up to 16 k-steps, else the tall consumers
    // (with fewer than 512 of them only where the rounds of tiles over the CUs say so: 1024 x 4096 x 2048, 1280 x 1280 x 2048,
    // 1280 x 5120 x 2048 at 128:2:16 .. 32 - 64, 80, 80 tiles - run 24-41 % faster on 128 x 128 tiles)
    {V_128, spatha::SPMM_VARIANT_W128x256_S3,
     [](const Shape& s) { return s.transposed && s.N > 128 && s.m >= 16 && s.S <= 16 && s.wide_transposed(); }},
    {V_128, spatha::SPMM_VARIANT_T128x256_S3, [](const Shape& s) { return s.transposed && s.N > 128 && s.m > 8 && s.wide_transposed(); }},
    {V_128, spatha::SPMM_VARIANT_W128x256_S3, [](const Shape& s) { return s.transposed && s.N > 128 && s.m > 8 && s.wide_transposed(); }},
    // row-major, two or three k-steps per tile and more than two rounds of 128 x 128 tiles: the kernel with store waves (a finished tile
    // leaves while the next one's k-loop runs) leads the 128 x 256 tiles by 7-18 % and the plain 128 x 128 ones by 14-23 %
    // (4096 x 1024 x 16384 at 128:2:32, 3072 x 768 x 8192 at 128:2:40, 1024 x 1024 x 16384 at 128:2:32); with transposed output
    // it is level with the plain kernel and behind the 128 x 256 tiles
    {V_128, spatha::SPMM_VARIANT_WS128x128_S3,
     [](const Shape& s) { return !s.transposed && s.m > 8 && s.S >= 2 && s.S <= 3 && s.tiles(128, 128) > 2 * s.cus; }},
    // 128 x 256 tiles, m >= 16: the 64 x 64 consumer blocks lead the tall-consumer form by 1-13 % up to 16 k-steps per tile
    // (BERT-large, GPT-2-large layers) from 768 tiles on (fewer: the tall form is 8-10 % ahead) and trail it by 1-3 % on
    // long k-loops (GPT-3 layers)
    {V_128, spatha::SPMM_VARIANT_W128x256_S3,
     [](const Shape& s) { return s.wide() && s.m >= 16 && s.S <= 16 && s.tiles(128, 256) >= 768; }},
    {V_128, spatha::SPMM_VARIANT_T128x256_S3, [](const Shape& s) { return s.wide(); }},
    {V_128, spatha::SPMM_VARIANT_W128x256_S3, [](const Shape& s) { return s.wide(); }},
    // more than one round of 128 x 128 tiles but less than two (two full rounds: the kernel with store waves is level or up to 6 %
    // ahead), few k-steps: the same number of 64 x 256 tiles runs as one
    // round of two co-resident workgroups per CU (768 x 768 x 8192, 3072 x 768 x 2048, 1024 x 1024 x 8192, 4096 x 1024 x
    // 2048 at 128:2:10 .. 128:2:100: 5-30 % ahead)
    {V_128, spatha::SPMM_VARIANT_P64x256_S2,
     [](const Shape& s) {
         const int64_t t = s.tiles(128, 128);
         return !s.transposed && s.m > 8 && t > s.cus && t < 2 * s.cus && s.S <= 8;
     }},
    // ... and wherever the 128 x 256 tiles do not lead and every CU has a tile: 5-13 % ahead of the plain 128 x 128 kernel
    // (1024 x 1024 x 16384 at 128:2:16, 4096 x 1024 x 4096 at 128:2:20, 5120 x 1280 x 4096 at 128:2:16, 1024 x 4096 x 4096 at
    // 128:2:7 .. 128:2:40), level with it on long k-loops with many tiles; 5-7 % behind with fewer tiles than CUs, and with
    // exactly one short tile per CU (1024 x 1024 x 4096 at 128:2:40)
    {V_128, spatha::SPMM_VARIANT_WS128x128_S3,
     [](const Shape& s) {
         const int64_t t = s.tiles(128, 128);
         return !s.transposed && s.S >= 2 && t >= s.cus && (t > s.cus || s.S >= 4);
     }},
    {V_128, spatha::SPMM_VARIANT_W128x128_S3, [](const Shape&) { return true; }},
    {V_128, spatha::SPMM_VARIANT_P128x128_S3, [](const Shape&) { return true; }},
    {V_128, spatha::SPMM_VARIANT_128x128, [](const Shape&) { return true; }},

    // -- V a multiple of 64 only --
    // m <= 8: staging the dense B rows once for four 64-row blocks halves the L2 -> LDS traffic; the two forms as above
    {V_64, spatha::SPMM_VARIANT_DS256x128_S3_PP,
     [](const Shape& s) { return !s.transposed && !s.fused && s.tiles(256, 128) <= 768 && s.S <= 32; }},
    {V_64, spatha::SPMM_VARIANT_DS256x128_S3_C8, [](const Shape&) { return true; }},
    // m > 8, row-major, two or three k-steps per tile and six rounds or more of 64 x 256 tiles: the producer/consumer kernel
    // with store waves, 9-10 % ahead of the plain one and of the per-tile pipeline (4096 x 1024 x 16384 at 64:2:32, 3072 x
    // 768 x 8192 at 64:2:40); level at four rounds, behind with fewer tiles and with four k-steps or more
    {V_64, spatha::SPMM_VARIANT_WS64x256_S3,
     [](const Shape& s) {
         // (transposed output, where the store waves also add the bias: ahead from twelve rounds on only - 4096 x 1024 x 16384
         // at 64:2:32 36.3 against 39.8 us for the per-tile pipeline; at six rounds 17.0 against 15.1 us)
         return s.m > 8 && s.S >= 2 && s.S <= 3 && s.tiles(64, 256) >= (s.transposed ? 12 : 6) * s.cus;
     }},
    // m > 8, gathered 64 x 256 tiles.  32 or more k-steps per tile and many rounds: the persistent pipeline, which keeps
    // loading across tile boundaries, leads (GPT-3 layers at 64:2:16; at 64:2:32, 24 k-steps, the per-tile pipeline is
    // 10-20 % ahead); with one tile per CU or less its third stage still gives long k-loops 5-15 %
    {V_64, spatha::SPMM_VARIANT_R64x256_S3, [](const Shape& s) { return s.long_k(); }},
    {V_64, spatha::SPMM_VARIANT_W64x256_S3, [](const Shape& s) { return s.long_k(); }},
    // 16 <= m, 3072 tiles or more of few k-steps, plain row-major output: the producer/consumer kernel with the write-out
    // deferred into the next tile's steps leads the pipeline by 5-8 % (3072 / 4096 x 1024 x 16384 at 64:2:16)
    {V_64, spatha::SPMM_VARIANT_D64x256_S3,
     [](const Shape& s) {
         return !s.long_k() && !s.short_k_many() && !s.fused && !s.transposed && s.m >= 16 && s.tiles(64, 256) >= 3072 && s.S <= 8;
     }},
    // producer/consumer kernel: m >= 32 with many tiles of few k-steps, row-major, 5-10 % ahead (transposed: the pipeline
    // leads by 6-8 %); at most one tile per CU with a dozen or more k-steps, 10-17 % ahead of the per-tile pipeline
    // (768 x 3072 / 1024 x 4096 x 4096 at 64:2:10 and 64:2:20)
    {V_64, spatha::SPMM_VARIANT_W64x256_S3,
     [](const Shape& s) {
         return !s.long_k() && (s.short_k_many() || (!s.transposed && s.tiles(64, 256) <= s.cus && s.S >= 12));
     }},
    // else the per-tile pipeline with two stages (two workgroups per CU)
    {V_64, spatha::SPMM_VARIANT_P64x256_S2, [](const Shape& s) { return !s.long_k(); }},
    {V_64, spatha::SPMM_VARIANT_R64x256_S3, [](const Shape&) { return true; }},
    {V_64, spatha::SPMM_VARIANT_64x256, [](const Shape&) { return true; }},
};

int pick_variant(const spatha_spmm_plan* plan, int N, int variant, bool fused = false, int out_layout = SPATHA_OUT_ROW_MAJOR) {
    if (variant != spatha::SPMM_VARIANT_AUTO) return variant_ok(plan, N, variant, fused) ? variant : -1;
    Shape s;
    s.v = plan->geo.v; s.m = plan->geo.m; s.rows = plan->geo.rows; s.N = N; s.S = plan->S;
    s.cus = plan->cus > 0 ? plan->cus : 256;
    s.fused = fused;
    s.transposed = out_layout == SPATHA_OUT_TRANSPOSED;
    const unsigned v_class = plan->half_tiles ? V_HALF : s.v % 128 == 0 ? V_128 : s.v % 64 == 0 ? V_64 : 0u;
    for (const Rule& r : kRules)
        if ((r.v_classes & v_class) && r.when(s) && variant_ok(plan, N, r.variant, fused)) return r.variant;
    return -1;
}

// An uneven last round of 128 x 256 tiles (automatic choice only): when the tiles fill one or more rounds of the CUs and
// leave a rest of at most half a round, the rest's row tiles run as a second launch on 128 x 128 tiles - twice as many
// tiles of half the work, so that its one round keeps every CU busy (GPT-3 FFN matrix at 256 tokens: 384 tiles on 256
// CUs).  Returns the rows of that second launch (the last rows of the matrix), 0 for a single launch.
int uneven_rest_rows(const spatha_spmm_plan* plan, int N, int requested, int chosen, bool fused) {
    if (requested != spatha::SPMM_VARIANT_AUTO || plan->cus < 8) return 0;
    if (chosen != spatha::SPMM_VARIANT_T128x256_S3 && chosen != spatha::SPMM_VARIANT_W128x256_S3) return 0;
    const int grid = (plan->cus / 8) * 8;       // workgroups of the persistent kernels
    const int tiles_n = (N + 255) / 256;
    const int64_t tiles = (int64_t)(plan->geo.rows / 128) * tiles_n, rest = tiles % grid;
    if (tiles <= grid || rest == 0 || rest % tiles_n != 0) return 0;
    // (short k-loops: a second launch costs more than the half-empty round; 1280 x 5120 x 16384 at 128:2:16 / 20 / 32, 20 / 16 /
    // 10 k-steps: 52 / 46 / 36 us in one launch against 56 / 50 / 40 in two)
    if (plan->S < 32) return 0;
    const int rest_rows = (int)(rest / tiles_n) * 128;
    if ((int64_t)(rest_rows / 128) * ((N + 127) / 128) > grid) return 0;        // more than half a round: one launch
    if ((plan->geo.rows - rest_rows) % plan->geo.v != 0) return 0;
    return variant_ok(plan, N, spatha::SPMM_VARIANT_W128x128_S3, fused) ? rest_rows : 0;
}

// ---- k-split (runs that bring a workspace) ----------------------------------------------------------------------
// Few tiles with long k-loops (small rows x N, large K: the chosen kernel's tiles fill at most half of the CUs): every tile's
// k-loop is cut into `parts` parts, one workgroup each.  Parts hand their fp32 partial blocks over through the workspace; the
// part that finishes last adds them in part order and writes the block (ksplit_exchange in spmm_warpspec.hip): deterministic,
// no workgroup waits for another.
// The hand-over costs 6-9 us (three dependent trips to the memory side: partial stores, ticket, partial loads; 64 or 128 KB
// of fp32 per tile and part) and a k-step 0.3-0.6 us, so a split must save about 48 k-steps per tile and leave parts of 32:
//   1024 x 16384 x 1024 at 128:2:8   (128 tiles of 128 k-steps, 2 parts)  34.7 against 50.2 us
//   12288 x 49152 x 128 at 128:2:16  ( 96 tiles of 192 k-steps, 2 parts)  48.3 against 73.2 us
//   768 x 12288 x 2048 at 128:2:8    ( 96 tiles of  96 k-steps, 2 parts)  30.5 against 38.9 us
//   1024 x 24576 x 2048 at 128:2:16  (128 tiles of  96 k-steps, 2 parts)  31.9 against 39.3 us
//   tiles of 64 k-steps in four parts of 16: between 15 % ahead and 7 % behind (256 x 8192 x 256, 4096 x 16384 x 256): not split.
// The rest of an uneven last round as a split second launch of the same kernel (instead of smaller tiles, uneven_rest_rows)
// was measured as well and does not pay: GPT-3 FFN matrix at 256 tokens (24 saved steps) 75 against 65 us, its FFN-down matrix
// at 1024 tokens (96 saved steps) 228 against 232 us; 128 x 256 tiles hand over twice the bytes.
#ifndef SPATHA_KSPLIT_MIN_SAVED_STEPS
#define SPATHA_KSPLIT_MIN_SAVED_STEPS 48
#endif
#ifndef SPATHA_KSPLIT_MIN_PART_STEPS
#define SPATHA_KSPLIT_MIN_PART_STEPS 32
#endif

struct SplitChoice {
    int variant = 0;        // kernel of the split launch (6 or 10)
    int parts = 1;
    size_t tickets_bytes = 0, partial_bytes = 0;
    size_t bytes() const { return tickets_bytes + partial_bytes; }
};

bool split_choice(const spatha_spmm_plan* plan, int N, int requested, int chosen, bool fused, SplitChoice* out) {
    using namespace spatha;
    if (requested != SPMM_VARIANT_AUTO || plan->cus < 8 || plan->half_tiles) return false;
    int var = chosen;
    if (var == SPMM_VARIANT_WS128x128_S3) var = SPMM_VARIANT_W128x128_S3;      // the store waves have no hand-over
    // (the 128 x 256 tiles with 64 x 64 consumer blocks are chosen for short k-loops only, where a split never pays)
    if (var != SPMM_VARIANT_W128x128_S3 && var != SPMM_VARIANT_T128x256_S3) return false;
    if (!variant_ok(plan, N, var, fused)) return false;
    const int bm = spmm_variant_bm(var), bn = spmm_variant_bn(var), S = plan->S;
    const int grid = (plan->cus / 8) * 8;
    const int64_t tiles = (int64_t)(plan->geo.rows / bm) * ((N + bn - 1) / bn);
    if (tiles * 2 > grid) return false;
    // as many parts as fit one round of the CUs, at most four, S a multiple of them
    int k = (int)std::min<int64_t>(grid / tiles, 4);
    while (k > 1 && (S % k != 0 || S / k < SPATHA_KSPLIT_MIN_PART_STEPS || S - S / k < SPATHA_KSPLIT_MIN_SAVED_STEPS)) --k;
    if (k < 2) return false;
    SplitChoice c;
    c.variant = var;
    c.parts = k;
    const int blocks_per_tile = (bm / 64) * (bn / 64);
    c.tickets_bytes = (((size_t)tiles * blocks_per_tile * 4) + 255) & ~(size_t)255;
    c.partial_bytes = (size_t)tiles * c.parts * bm * bn * 4;
    *out = c;
    return true;
}
}  // namespace

namespace spatha {

int note_hip_error(hipError_t e) { return hip_fail(e); }

void plan_layout(int rows, int m, int v, int ksp, PlanLayout* out) {
    out->S = (ksp + 31) / 32;
    out->half_tiles = (v % 64 != 0);      // V = 32, 96, ...: a wave tile spans two V blocks
    out->apack_bytes = (size_t)((rows + 63) / 64) * out->S * APACK_BLOCK;    // rows % 64 == 32: V a multiple of 32 only
    out->rowtab_bytes = (size_t)(rows / v) * out->S * 64 * 4;
    out->gtab_bytes = 0;
    if ((m <= 8 && rows % 256 == 0) || (m <= 16 && rows % 512 == 0 && !out->half_tiles)) {
        // gather table of the dense-staged kernels: one entry per 64-row block, or per 32-row block when V % 64 != 0
        const int block_rows = out->half_tiles ? 32 : 64;
        out->gtab_bytes = (size_t)(rows / block_rows) * out->S * 64 * 2;
    }
}

hipError_t plan_pack(const spatha_spmm_plan* plan, const uint16_t* values_dev, const uint32_t* metadata_dev,
                     const uint32_t* columns_dev, hipStream_t stream) {
    const spatha_vnm_geometry& geo = plan->geo;
    hipError_t e = launch_pack(values_dev, metadata_dev, columns_dev, geo.rows, geo.cols, geo.m, geo.v, geo.ksp, plan->S,
                               plan->half_tiles, plan->apack, plan->rowtab, stream);
    if (e != hipSuccess) return e;
    if (plan->gtab) {
        e = launch_pack_gtab(columns_dev, geo.rows, geo.m, geo.v, geo.ksp, plan->S, plan->half_tiles ? 32 : 64, plan->gtab, stream);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

}  // namespace spatha

extern "C" {

const char* spatha_status_string(int status) {
    switch (status) {
        case SPATHA_OK: return "ok";
        case SPATHA_ERR_BAD_ARGUMENT: return "bad argument";
        case SPATHA_ERR_BAD_SHAPE: return "shape not representable in V:N:M (rows % V, V % 32, m >= 4, N % 8)";
        case SPATHA_ERR_UNSUPPORTED: return "no kernel for this configuration";
        case SPATHA_ERR_HIP: return "HIP runtime error";
        case SPATHA_ERR_NO_DEVICE: return "no HIP device";
        case SPATHA_ERR_TOO_LARGE: return "size beyond the entry point's capacity";
        case SPATHA_ERR_IO: return "file missing, truncated, not a V:N:M container, or corrupt";
        default: return "unknown status";
    }
}

int spatha_last_hip_error(void) { return g_last_hip_error; }

const char* spatha_version(void) { return "0.1.0"; }

int spatha_vnm_geometry_init(int rows, int cols, int n, int m, int v, spatha_vnm_geometry* out) {
    return spatha::geometry_init(rows, cols, n, m, v, out);
}

int spatha_vnm_random_pattern(int rows, int cols, int n, int m, int v, uint32_t* metadata, uint32_t* columns) {
    return spatha::random_pattern(rows, cols, n, m, v, metadata, columns);
}

int spatha_fill_rand_small_ints_f16(uint16_t* out, int64_t count) {
    if (!out || count < 0) return SPATHA_ERR_BAD_ARGUMENT;
    // fp16 bit patterns of -4..4
    static const uint16_t enc[9] = {0xC400, 0xC200, 0xC000, 0xBC00, 0x0000, 0x3C00, 0x4000, 0x4200, 0x4400};
    for (int64_t i = 0; i < count; i++) out[i] = enc[std::rand() % 9];
    return SPATHA_OK;
}

int spatha_benchmark_inputs_f16(int rows, int cols, int ncols_b, int n, int m, int v, uint16_t* b, uint32_t* metadata,
                                uint32_t* columns, uint16_t* values) {
    spatha_vnm_geometry geo;
    int st = spatha::geometry_init(rows, cols, n, m, v, &geo);
    if (st != SPATHA_OK) return st;
    if (!b || !metadata || !columns || !values || ncols_b <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    st = spatha_fill_rand_small_ints_f16(b, (int64_t)cols * ncols_b);
    if (st == SPATHA_OK) st = spatha::random_pattern(rows, cols, n, m, v, metadata, columns);
    if (st == SPATHA_OK) st = spatha_fill_rand_small_ints_f16(values, geo.n_values);
    return st;
}

int spatha_vnm_encode_f32(const float* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n,
                          int m, int v, float* values, uint32_t* metadata, int threads) {
    return spatha::encode_f32(dense, mask, columns, rows, cols, n, m, v, values, metadata, threads);
}
int spatha_vnm_encode_f16(const uint16_t* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols,
                          int n, int m, int v, uint16_t* values, uint32_t* metadata, int threads) {
    return spatha::encode_f16(dense, mask, columns, rows, cols, n, m, v, values, metadata, threads);
}
int spatha_vnm_decode_f32(const float* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                          int n, int m, int v, float* dense, int threads) {
    return spatha::decode_f32(values, metadata, columns, rows, cols, n, m, v, dense, threads);
}
int spatha_vnm_decode_f16(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows,
                          int cols, int n, int m, int v, uint16_t* dense, int threads) {
    return spatha::decode_f16(values, metadata, columns, rows, cols, n, m, v, dense, threads);
}
int spatha_vnm_select_columns_f32(const float* dense_abs, int rows, int cols, int n, int m, int v, int32_t* masks,
                                  int32_t* columns, int threads) {
    return spatha::select_columns_f32(dense_abs, rows, cols, n, m, v, masks, columns, threads);
}
int spatha_vnm_file_write(const char* path, int rows, int cols, int n, int m, int v, int value_bits, const void* values,
                          const uint32_t* metadata, const uint32_t* columns) {
    return spatha::file_write(path, rows, cols, n, m, v, value_bits, values, metadata, columns);
}

int spatha_vnm_file_info(const char* path, spatha_vnm_geometry* geometry, int* value_bits) {
    return spatha::file_info(path, geometry, value_bits);
}

int spatha_vnm_file_read(const char* path, void* values, uint32_t* metadata, uint32_t* columns) {
    return spatha::file_read(path, values, metadata, columns);
}

int spatha_vnm_select_columns_f32_gpu(const float* dense_abs, int rows, int cols, int n, int m, int v, int32_t* masks,
                                      int32_t* columns, int threads, int exact_ties, void* stream) {
    spatha_vnm_geometry geo;
    int st = spatha::geometry_init(rows, cols, n, m, v, &geo);
    if (st) return st;
    if (!dense_abs || !masks || !columns) return SPATHA_ERR_BAD_ARGUMENT;
    int per_block = 0;
    const int tasks = spatha::select_task_count(rows, cols, m, v, &per_block);
    std::vector<spatha::GroupTask> winners((size_t)tasks);
    if (tasks > 0) {
        if ((size_t)v * (size_t)m * sizeof(float) > 150u * 1024u) return SPATHA_ERR_TOO_LARGE;   // one V x m block per workgroup in LDS
        float* d_abs = nullptr;
        spatha::SelectWinner* d_out = nullptr;
        std::vector<spatha::SelectWinner> h_out((size_t)tasks);
        const size_t bytes = (size_t)rows * (size_t)cols * sizeof(float);
        hipStream_t s = (hipStream_t)stream;
        hipError_t e = hipMalloc((void**)&d_abs, bytes);
        if (e == hipSuccess) e = hipMalloc((void**)&d_out, (size_t)tasks * sizeof(spatha::SelectWinner));
        if (e == hipSuccess) e = hipMemcpyAsync(d_abs, dense_abs, bytes, hipMemcpyHostToDevice, s);
        if (e == hipSuccess) e = spatha::launch_select_winners(d_abs, rows, cols, m, v, d_out, s);
        if (e == hipSuccess) e = hipMemcpyAsync(h_out.data(), d_out, (size_t)tasks * sizeof(spatha::SelectWinner), hipMemcpyDeviceToHost, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
        if (d_abs) (void)hipFree(d_abs);
        if (d_out) (void)hipFree(d_out);
        if (e != hipSuccess) return hip_fail(e);
        for (int i = 0; i < tasks; i++) {
            winners[(size_t)i].any = h_out[(size_t)i].any != 0;
            for (int k = 0; k < 4; k++) winners[(size_t)i].best[k] = h_out[(size_t)i].best[k];
        }
    }
    return spatha::select_columns_with_winners(dense_abs, rows, cols, n, m, v, tasks > 0 ? winners.data() : nullptr,
                                               exact_ties != 0, masks, columns, threads);
}

int spatha_vnm_pack_meta_blob(const uint32_t* metadata, int64_t n_metadata, const uint32_t* columns,
                              int64_t n_columns, uint32_t* blob, int64_t* columns_offset_words,
                              int64_t* blob_words) {
    return spatha::pack_meta_blob(metadata, n_metadata, columns, n_columns, blob, columns_offset_words, blob_words);
}

int spatha_spmm_plan_create(int rows, int cols, int n, int m, int v, const uint16_t* values_dev,
                            const uint32_t* metadata_dev, const uint32_t* columns_dev, void* stream,
                            spatha_spmm_plan** out) {
    if (!out) return SPATHA_ERR_BAD_ARGUMENT;
    *out = nullptr;
    spatha_vnm_geometry geo;
    int st = spatha::geometry_init(rows, cols, n, m, v, &geo);
    if (st) return st;
    if (!values_dev || !metadata_dev || !columns_dev) return SPATHA_ERR_BAD_ARGUMENT;
    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev == 0) { g_last_hip_error = (int)e; return SPATHA_ERR_NO_DEVICE; }
    spatha_spmm_plan* plan = new (std::nothrow) spatha_spmm_plan();
    if (!plan) return SPATHA_ERR_BAD_ARGUMENT;
    spatha::PlanLayout lay;
    spatha::plan_layout(rows, m, v, geo.ksp, &lay);
    plan->geo = geo;
    plan->S = lay.S;
    plan->half_tiles = lay.half_tiles;
    plan->apack = nullptr; plan->rowtab = nullptr; plan->zeros = nullptr; plan->gtab = nullptr;
    plan->apack_bytes = lay.apack_bytes; plan->rowtab_bytes = lay.rowtab_bytes;
    plan->gtab_bytes = lay.gtab_bytes;
    e = hipGetDevice(&plan->device);
    if (e != hipSuccess) { delete plan; return hip_fail(e); }
    plan->cus = 0;
    if (hipDeviceGetAttribute(&plan->cus, hipDeviceAttributeMultiprocessorCount, plan->device) != hipSuccess) plan->cus = 0;
    if ((e = hipMalloc((void**)&plan->apack, lay.apack_bytes)) != hipSuccess ||
        (e = hipMalloc((void**)&plan->rowtab, lay.rowtab_bytes)) != hipSuccess ||
        (e = hipMalloc(&plan->zeros, 1024)) != hipSuccess ||
        (e = hipMemsetAsync(plan->zeros, 0, 1024, (hipStream_t)stream)) != hipSuccess ||
        (lay.gtab_bytes && (e = hipMalloc((void**)&plan->gtab, lay.gtab_bytes)) != hipSuccess) ||
        (e = spatha::plan_pack(plan, values_dev, metadata_dev, columns_dev, (hipStream_t)stream)) != hipSuccess) {
        spatha_spmm_plan_destroy(plan);
        return hip_fail(e);
    }
    // the derived copies are complete before the plan is handed out: a later run on another stream has nothing to order
    // itself against
    if ((e = hipStreamSynchronize((hipStream_t)stream)) != hipSuccess) {
        spatha_spmm_plan_destroy(plan);
        return hip_fail(e);
    }
    *out = plan;
    return SPATHA_OK;
}

int spatha_spmm_plan_destroy(spatha_spmm_plan* plan) {
    if (!plan) return SPATHA_OK;
    hipError_t first = hipSuccess, e;
    if (plan->apack && (e = hipFree(plan->apack)) != hipSuccess && first == hipSuccess) first = e;
    if (plan->rowtab && (e = hipFree(plan->rowtab)) != hipSuccess && first == hipSuccess) first = e;
    if (plan->zeros && (e = hipFree(plan->zeros)) != hipSuccess && first == hipSuccess) first = e;
    if (plan->gtab && (e = hipFree(plan->gtab)) != hipSuccess && first == hipSuccess) first = e;
    delete plan;
    return first == hipSuccess ? SPATHA_OK : hip_fail(first);
}

}  // extern "C"

int spatha::plan_run_check(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                           const uint16_t* out_dev, int out_layout, int activation, bool fused_entry, int variant,
                           int* chosen) {
    if (!plan || !B_dev || !out_dev || N <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (out_layout != SPATHA_OUT_ROW_MAJOR && out_layout != SPATHA_OUT_TRANSPOSED) return SPATHA_ERR_BAD_ARGUMENT;
    if (!fused_entry && out_layout == SPATHA_OUT_ROW_MAJOR && bias_dev) return SPATHA_ERR_BAD_ARGUMENT;
    if (activation != SPATHA_ACT_NONE && activation != SPATHA_ACT_GELU && activation != SPATHA_ACT_GELU_TANH)
        return SPATHA_ERR_BAD_ARGUMENT;
    if (N % 8 != 0) return SPATHA_ERR_BAD_SHAPE;      // 16-byte row segments of B and C
    if (((uintptr_t)B_dev & 15) || ((uintptr_t)out_dev & 15) || ((uintptr_t)bias_dev & 15)) return SPATHA_ERR_BAD_ARGUMENT;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev != plan->device) return SPATHA_ERR_BAD_ARGUMENT;   // plans live on one device
    // the bias of the transposed layout alone stays in the write-out itself
    const bool fuse = activation != SPATHA_ACT_NONE || (out_layout == SPATHA_OUT_ROW_MAJOR && bias_dev);
    const int var = pick_variant(plan, N, variant, fuse, out_layout);
    if (var < 0) return SPATHA_ERR_UNSUPPORTED;
    if (chosen) *chosen = var;
    return SPATHA_OK;
}

int spatha::plan_run(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev, uint16_t* out_dev,
                     int out_layout, int activation, bool fused_entry, int variant, void* stream, void* workspace,
                     size_t workspace_bytes) {
    int var = -1;
    const int status = plan_run_check(plan, B_dev, N, bias_dev, out_dev, out_layout, activation, fused_entry, variant, &var);
    if (status != SPATHA_OK) return status;
    const bool fuse = activation != SPATHA_ACT_NONE || (out_layout == SPATHA_OUT_ROW_MAJOR && bias_dev);
    spatha::SpmmParams p;
    p.apack = plan->apack; p.rowtab = plan->rowtab;
    p.B = B_dev; p.bias = bias_dev; p.C = out_dev; p.zeros = plan->zeros; p.gtab = plan->gtab;
    p.gtab_bytes = (uint32_t)plan->gtab_bytes;
    p.rows = plan->geo.rows; p.cols = plan->geo.cols; p.N = N; p.S = plan->S; p.v = plan->geo.v; p.m = plan->geo.m;
    const int bm = spatha::spmm_variant_bm(var), bn = spatha::spmm_variant_bn(var);
    p.tiles_m = (plan->geo.rows + bm - 1) / bm;     // (only the half-tile kernels see rows % 64 != 0: a padded last tile)
    p.tiles_n = (N + bn - 1) / bn;
    p.b_bytes = (uint32_t)((uint64_t)plan->geo.cols * (uint64_t)N * 2u);     // only read by variants that passed variant_ok
    p.apack_bytes = (uint32_t)plan->apack_bytes;
    p.rowtab_bytes = (uint32_t)plan->rowtab_bytes;
    p.fuse = fuse ? 1 : 0; p.act = activation;
    p.cus = plan->cus > 0 ? plan->cus : 256;
    p.walk_group = 1;
    if (var == spatha::SPMM_VARIANT_UP512x128_S3) {
        // Packed A larger than an XCD's L2 (plain 2:4 on a 4096-row matrix: 4.7 MB against 4 MB; it is then fetched again in
        // every round, 160 MB per launch): tile rows in groups of four, so that an XCD only
        // ever sees four of them (2.4 MB, resident) and reads twice as many tile columns of B instead.  2:4 FFN-up: 85-86
        // against 87-89 us.  Where A fits anyway (64:2:8: 2.4 MB) the default walk reads less.
        const size_t a_bytes = plan->apack_bytes + plan->gtab_bytes, four_rows = a_bytes / p.tiles_m * 4;
        if (p.tiles_m % 4 == 0 && p.tiles_m >= 8 && p.tiles_n >= 32 && a_bytes > (4u << 20) && four_rows <= (3u << 20)) p.walk_group = -4;
    }
    p.ksplit = 1; p.partial = nullptr; p.partial_bytes = 0; p.tickets = nullptr;
    p.debug = 0; p.skew = 0; p.prof = nullptr;
#ifdef SPATHA_DEV_PROFILE
    // development builds only: switch parts of a kernel off for time accounting (results are then wrong on purpose)
    { const char* d = std::getenv("SPATHA_DEBUG_KNOBS"); p.debug = d ? std::atoi(d) : 0; }
    { const char* d = std::getenv("SPATHA_SKEW"); p.skew = d ? std::atoi(d) : 0; }
    { const char* d = std::getenv("SPATHA_PROF_PTR"); if (d) p.prof = (long long*)std::strtoull(d, nullptr, 0); }
#endif
    SplitChoice sc;
    if (workspace && split_choice(plan, N, variant, var, fuse, &sc) && workspace_bytes >= sc.bytes() &&
        ((uintptr_t)workspace & 255) == 0) {
        // every tile's k-loop in parts: the walk's m-tiles are (row tile, part) pairs
        spatha::SpmmParams q = p;
        q.tiles_m = (plan->geo.rows / spatha::spmm_variant_bm(sc.variant)) * sc.parts;
        q.tiles_n = (N + spatha::spmm_variant_bn(sc.variant) - 1) / spatha::spmm_variant_bn(sc.variant);
        q.ksplit = sc.parts;
        q.tickets = (uint32_t*)workspace;       // zero: cleared once by spatha_spmm_workspace_init, put back by every completed run
        q.partial = (float*)((char*)workspace + sc.tickets_bytes);
        q.partial_bytes = (uint32_t)sc.partial_bytes;
        const hipError_t e2 = spatha::launch_spmm(sc.variant, out_layout, q, (hipStream_t)stream);
        return e2 == hipSuccess ? SPATHA_OK : hip_fail(e2);
    }
    if (const int rest_rows = uneven_rest_rows(plan, N, variant, var, fuse)) {
        const int main_rows = plan->geo.rows - rest_rows;
        spatha::SpmmParams head = p, tail = p;
        head.tiles_m = main_rows / 128;
        const size_t a_off = (size_t)(main_rows / 64) * plan->S * spatha::APACK_BLOCK;
        const size_t rt_off = (size_t)(main_rows / plan->geo.v) * plan->S * 64 * 4;
        tail.apack = (const uint16_t*)((const char*)plan->apack + a_off);
        tail.apack_bytes = (uint32_t)(plan->apack_bytes - a_off);
        tail.rowtab = (const uint32_t*)((const char*)plan->rowtab + rt_off);
        tail.rowtab_bytes = (uint32_t)(plan->rowtab_bytes - rt_off);
        if (bias_dev) tail.bias = bias_dev + main_rows;
        // (p.rows stays the full row count: these kernels use it as the row stride of the transposed layout only)
        tail.C = out_layout == SPATHA_OUT_TRANSPOSED ? out_dev + main_rows : out_dev + (size_t)main_rows * N;
        tail.tiles_m = rest_rows / 128;
        tail.tiles_n = (N + 127) / 128;
        // Which way the tail's tiles are walked decides what an XCD's workgroups (grid / 8 tiles at a time) pull into its L2
        // per round: column-first, the A operands of up to grid / 8 tile rows + few tile columns of B; row-first, all tile
        // columns of few tile rows.  GPT-3 FFN matrix at 256 tokens (0.44 MB of A per tile row, two tile columns of 3.1 MB):
        // 13.4 against 17.3 MB row-first, the second launch fetches 108 instead of 142 MB; with few tile rows and many tile
        // columns (1280 x 5120 at 8192 tokens: 2 x 128 tiles) column-first moves half as much.
        {
            const int64_t at_a_time = std::max(1, p.cus / 8);
            const double a_row = (double)plan->apack_bytes / (plan->geo.rows / 128.0), b_col = (double)plan->geo.cols * 128 * 2;
            const int64_t tm = tail.tiles_m, tn = tail.tiles_n;
            const double col_first = (double)std::min(at_a_time, tm) * a_row + (double)((at_a_time + tm - 1) / tm) * b_col;
            const double row_first = (double)((at_a_time + tn - 1) / tn) * a_row + (double)std::min(at_a_time, tn) * b_col;
            tail.walk_group = row_first < col_first ? 0 : 1;
        }
        hipError_t e2 = spatha::launch_spmm(var, out_layout, head, (hipStream_t)stream);
        if (e2 == hipSuccess) e2 = spatha::launch_spmm(spatha::SPMM_VARIANT_W128x128_S3, out_layout, tail, (hipStream_t)stream);
        return e2 == hipSuccess ? SPATHA_OK : hip_fail(e2);
    }
    hipError_t e = spatha::launch_spmm(var, out_layout, p, (hipStream_t)stream);
    return e == hipSuccess ? SPATHA_OK : hip_fail(e);
}

extern "C" {

int spatha_spmm_run(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                    uint16_t* out_dev, int out_layout, int variant, void* stream) {
    return spatha::plan_run(plan, B_dev, N, bias_dev, out_dev, out_layout, SPATHA_ACT_NONE, false, variant, stream);
}

int spatha_spmm_run_fused(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                          uint16_t* out_dev, int out_layout, int activation, int variant, void* stream) {
    return spatha::plan_run(plan, B_dev, N, bias_dev, out_dev, out_layout, activation, true, variant, stream);
}

size_t spatha_spmm_workspace_bytes(const spatha_spmm_plan* plan, int N, int out_layout, int fused) {
    if (!plan || N <= 0 || N % 8 != 0) return 0;
    const int var = pick_variant(plan, N, spatha::SPMM_VARIANT_AUTO, fused != 0, out_layout);
    SplitChoice sc;
    if (var < 0 || !split_choice(plan, N, spatha::SPMM_VARIANT_AUTO, var, fused != 0, &sc)) return 0;
    return sc.bytes();
}

int spatha_spmm_workspace_init(void* workspace_dev, size_t workspace_bytes, void* stream) {
    if (!workspace_dev || ((uintptr_t)workspace_dev & 255) || workspace_bytes % 4 != 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (workspace_bytes / 4 > 0x7fffffffull) return SPATHA_ERR_TOO_LARGE;
    const hipError_t e = spatha::launch_clear_words((uint32_t*)workspace_dev, (int)(workspace_bytes / 4), (hipStream_t)stream);
    return e == hipSuccess ? SPATHA_OK : hip_fail(e);
}

int spatha_spmm_run_ws(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev, uint16_t* out_dev,
                       int out_layout, int activation, void* workspace_dev, size_t workspace_bytes, void* stream) {
    return spatha::plan_run(plan, B_dev, N, bias_dev, out_dev, out_layout, activation, true, spatha::SPMM_VARIANT_AUTO, stream,
                            workspace_dev, workspace_bytes);
}

int spatha_spmm_num_variants(void) { return spatha::SPMM_VARIANT_COUNT; }

const char* spatha_spmm_kernel_name(const spatha_spmm_plan* plan, int N, int out_layout, int variant) {
    if (!plan) return nullptr;
    int var = pick_variant(plan, N, variant, false, out_layout);
    if (var < 0) return nullptr;
    if (uneven_rest_rows(plan, N, variant, var, false))     // two launches: the rest of an uneven last round on 128 x 128 tiles
        return var == spatha::SPMM_VARIANT_T128x256_S3 ? "smfmac16x16x64_warpspec_tall_tile128x256_3stage+rest_on_tile128x128"
                                                       : "smfmac16x16x64_warpspec_tile128x256_3stage+rest_on_tile128x128";
    return spatha::spmm_variant_name(var);
}

int spatha_spmm_time(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                     uint16_t* out_dev, int out_layout, int variant, int warmup, int iters, void* stream,
                     float* ms_per_launch) {
    if (!ms_per_launch || iters <= 0 || warmup < 0) return SPATHA_ERR_BAD_ARGUMENT;
    hipStream_t s = (hipStream_t)stream;
    for (int i = 0; i < warmup; i++) {
        int st = spatha_spmm_run(plan, B_dev, N, bias_dev, out_dev, out_layout, variant, stream);
        if (st) return st;
    }
    hipEvent_t t0, t1;
    hipError_t e;
    if ((e = hipEventCreate(&t0)) != hipSuccess) return hip_fail(e);
    if ((e = hipEventCreate(&t1)) != hipSuccess) { (void)hipEventDestroy(t0); return hip_fail(e); }
    int st = SPATHA_OK;
    e = hipEventRecord(t0, s);
    for (int i = 0; i < iters && e == hipSuccess && st == SPATHA_OK; i++)
        st = spatha_spmm_run(plan, B_dev, N, bias_dev, out_dev, out_layout, variant, stream);
    if (e == hipSuccess) e = hipEventRecord(t1, s);
    if (e == hipSuccess) e = hipEventSynchronize(t1);
    float ms = 0.f;
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, t0, t1);
    (void)hipEventDestroy(t0);
    (void)hipEventDestroy(t1);
    if (st) return st;
    if (e != hipSuccess) return hip_fail(e);
    *ms_per_launch = ms / (float)iters;
    return SPATHA_OK;
}

int spatha_spmm_tune(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                     uint16_t* out_dev, int out_layout, int warmup, int iters, void* stream, int* best_variant,
                     float* best_ms, float* auto_ms, float* ms_per_variant) {
    if (!best_variant || !best_ms) return SPATHA_ERR_BAD_ARGUMENT;
    // (a first, untimed pass of the automatic choice: argument checks, and the clocks are up when the first id is timed)
    float t_auto = 0.f;
    int st = spatha_spmm_time(plan, B_dev, N, bias_dev, out_dev, out_layout, spatha::SPMM_VARIANT_AUTO, warmup, iters, stream, &t_auto);
    if (st) return st;
    int best = spatha::SPMM_VARIANT_AUTO;
    float t_best = 0.f;
    for (int id = 1; id < spatha::SPMM_VARIANT_COUNT; id++) {
        if (ms_per_variant) ms_per_variant[id] = -1.f;
        if (!variant_ok(plan, N, id, false)) continue;
        float t = 0.f;
        st = spatha_spmm_time(plan, B_dev, N, bias_dev, out_dev, out_layout, id, warmup, iters, stream, &t);
        if (st == SPATHA_ERR_UNSUPPORTED) continue;     // (accepted by the shape checks, refused by the kernel's launcher)
        if (st) return st;
        if (ms_per_variant) ms_per_variant[id] = t;
        if (best == spatha::SPMM_VARIANT_AUTO || t < t_best) { t_best = t; best = id; }
    }
    // the automatic choice last, in the same warm state as the ids: it wins ties (it may be one of them)
    st = spatha_spmm_time(plan, B_dev, N, bias_dev, out_dev, out_layout, spatha::SPMM_VARIANT_AUTO, warmup, iters, stream, &t_auto);
    if (st) return st;
    if (auto_ms) *auto_ms = t_auto;
    if (ms_per_variant) ms_per_variant[0] = t_auto;
    if (best == spatha::SPMM_VARIANT_AUTO || t_auto <= t_best) { t_best = t_auto; best = spatha::SPMM_VARIANT_AUTO; }
    *best_variant = best;
    *best_ms = t_best;
    return SPATHA_OK;
}

int spatha_dense_gemm_f16(const uint16_t* A_dev, const uint16_t* B_dev, int rows, int cols, int N, uint16_t* C_dev,
                          void* stream) {
    if (!A_dev || !B_dev || !C_dev || rows <= 0 || cols <= 0 || N <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (N % 8 != 0 || cols % 8 != 0) return SPATHA_ERR_BAD_SHAPE;
    hipError_t e = spatha::launch_dense_gemm(A_dev, B_dev, rows, cols, N, C_dev, (hipStream_t)stream);
    return e == hipSuccess ? SPATHA_OK : hip_fail(e);
}

int spatha_transpose_f16(const uint16_t* in_dev, int rows, int cols, uint16_t* out_dev, void* stream) {
    if (!in_dev || !out_dev || rows <= 0 || cols <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (((uintptr_t)in_dev | (uintptr_t)out_dev) & 15u) return SPATHA_ERR_BAD_ARGUMENT;
    if ((rows + 63) / 64 > 65535) return SPATHA_ERR_TOO_LARGE;
    hipError_t e = spatha::launch_transpose_f16(in_dev, rows, cols, out_dev, (hipStream_t)stream);
    return e == hipSuccess ? SPATHA_OK : hip_fail(e);
}

int spatha_add_layernorm_f16(const uint16_t* x_dev, const uint16_t* residual_dev, const uint16_t* gamma_dev,
                             const uint16_t* beta_dev, float eps, int tokens, int hidden, uint16_t* out_dev, void* stream) {
    if (!x_dev || !gamma_dev || !beta_dev || !out_dev || tokens <= 0 || hidden <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (hidden % 8 != 0) return SPATHA_ERR_BAD_SHAPE;
    if (hidden > 4096) return SPATHA_ERR_UNSUPPORTED;           // a lane keeps hidden / 64 values in registers
    if (((uintptr_t)x_dev | (uintptr_t)residual_dev | (uintptr_t)gamma_dev | (uintptr_t)beta_dev | (uintptr_t)out_dev) & 15u)
        return SPATHA_ERR_BAD_ARGUMENT;
    hipError_t e = spatha::launch_add_layernorm_f16(x_dev, residual_dev, gamma_dev, beta_dev, eps, tokens, hidden, out_dev,
                                                    (hipStream_t)stream);
    return e == hipSuccess ? SPATHA_OK : hip_fail(e);
}

int spatha_add_layernorm_f16_t(const uint16_t* x_dev, const uint16_t* residual_dev, const uint16_t* gamma_dev,
                               const uint16_t* beta_dev, float eps, int tokens, int hidden, uint16_t* out_dev, uint16_t* out_t_dev,
                               void* stream) {
    if (!x_dev || !gamma_dev || !beta_dev || !out_dev || !out_t_dev || tokens <= 0 || hidden <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (hidden % 8 != 0 || tokens % 8 != 0) return SPATHA_ERR_BAD_SHAPE;       // 16-byte pieces of both layouts
    if (hidden > 4096) return SPATHA_ERR_UNSUPPORTED;
    if (((uintptr_t)x_dev | (uintptr_t)residual_dev | (uintptr_t)gamma_dev | (uintptr_t)beta_dev | (uintptr_t)out_dev |
         (uintptr_t)out_t_dev) & 15u)
        return SPATHA_ERR_BAD_ARGUMENT;
    hipError_t e = spatha::launch_add_layernorm_f16_t(x_dev, residual_dev, gamma_dev, beta_dev, eps, tokens, hidden, out_dev, out_t_dev,
                                                      (hipStream_t)stream);
    return e == hipSuccess ? SPATHA_OK : hip_fail(e);
}

}  // extern "C"
