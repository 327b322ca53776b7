// Host side of the V:N:M format: geometry, random pattern, dense->V:N:M
// encoder, V:N:M->dense decoder, magnitude column selector, device blob layout.
//
// Storage contract (identical to UDC-GAC/venom, src/format/format_sr_nm.cpp and
// end2end/grouped_nmv_tensor.py), written as closed forms.  For row r, m-column
// group g and kept slot j in {0,1}, with
//     r = 16*R16 + 4*q + 2*p + s   (q in 0..3; p, s in 0..1)
//     g = 4*t + u                  (u in 0..3)
//     b = r / V
//   values   index = R16*16*Ksp + t*128 + q*32 + u*8 + p*4 + s*2 + j
//   metadata word  = (r/32)*(Ksp/8)*16 + t*16 + ((r%32)/16)*8 + q*2 + p
//   metadata bits  = [s*16 + u*4 + j*2, +2)  -> position c in 0..3
//   column-loc     = columns[b*(Ksp/2)*4 + g*4 + c]
//   dense column   = g*m + column-loc         (ignored when >= cols)
// Everything here is integer / data-movement work and is parallel over
// independent row pairs or V-row blocks.

#include "vnm_format.h"

#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace spatha {

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

int geometry_init(int rows, int cols, int n, int m, int v, spatha_vnm_geometry* out) {
    if (!out) return SPATHA_ERR_BAD_ARGUMENT;
    if (rows <= 0 || cols <= 0 || n != 2 || m < 4 || v <= 0) return SPATHA_ERR_BAD_ARGUMENT;
    if (v % 32 != 0 || rows % v != 0) return SPATHA_ERR_BAD_SHAPE;
    int64_t groups = ceil_div(cols, m);
    int64_t ksp = ceil_div(groups * n, 16) * 16;
    out->rows = rows; out->cols = cols; out->n = n; out->m = m; out->v = v;
    out->ksp = (int32_t)ksp;
    out->n_values = (int64_t)rows * ksp;
    out->n_metadata = (int64_t)(rows / 2) * (ksp / 8);
    out->n_columns = (int64_t)(rows / v) * (ksp / n) * 4;
    return SPATHA_OK;
}

namespace {

struct SlotMap {
    int64_t ksp;
    explicit SlotMap(int64_t ksp_) : ksp(ksp_) {}
    // index of the first of the two values of (row, group)
    inline int64_t value_index(int64_t r, int64_t g) const {
        int64_t R16 = r >> 4, q = (r >> 2) & 3, p = (r >> 1) & 1, s = r & 1, t = g >> 2, u = g & 3;
        return R16 * 16 * ksp + t * 128 + q * 32 + u * 8 + p * 4 + s * 2;
    }
    inline int64_t meta_word(int64_t r, int64_t g) const {
        int64_t q = (r >> 2) & 3, p = (r >> 1) & 1, t = g >> 2;
        return (r >> 5) * (ksp >> 3) * 16 + t * 16 + ((r >> 4) & 1) * 8 + q * 2 + p;
    }
    static inline int meta_shift(int64_t r, int64_t g) { return (int)((r & 1) * 16 + (g & 3) * 4); }
};

inline void set_threads(int threads) {
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
    else omp_set_num_threads(omp_get_num_procs());
#else
    (void)threads;
#endif
}

template <class T> inline bool is_nonzero(T x);
template <> inline bool is_nonzero<float>(float x) { return x != 0.f; }
// fp16 bit pattern: +0 and -0 are the only zeros
template <> inline bool is_nonzero<uint16_t>(uint16_t x) { return (x & 0x7fffu) != 0; }

template <class T>
int encode(const T* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m, int v,
           T* values, uint32_t* metadata, int threads) {
    spatha_vnm_geometry g;
    int st = geometry_init(rows, cols, n, m, v, &g);
    if (st) return st;
    if (!dense || !columns || !values || !metadata) return SPATHA_ERR_BAD_ARGUMENT;
    const int64_t ngroups = g.ksp / 2;
    SlotMap map(g.ksp);
    for (int64_t i = 0; i < g.n_columns; i++)
        if (columns[i] >= (uint32_t)m) return SPATHA_ERR_BAD_ARGUMENT;
    set_threads(threads);
    std::atomic<int> overflow{0};
    // one task = one row pair, which owns whole metadata words
#pragma omp parallel for schedule(static)
    for (int64_t rp = 0; rp < rows / 2; rp++) {
        for (int64_t grp4 = 0; grp4 < ngroups / 4; grp4++) {
            uint32_t word = 0;
            for (int s = 0; s < 2; s++) {
                int64_t r = rp * 2 + s;
                const uint32_t* cl = columns + (r / v) * ngroups * 4;
                for (int u = 0; u < 4; u++) {
                    int64_t grp = grp4 * 4 + u;
                    T val[4];
                    uint32_t pos[4];
                    int cnt = 0;
                    uint32_t used = 0;
                    for (uint32_t c = 0; c < 4; c++) {
                        int64_t dcol = grp * m + cl[grp * 4 + c];
                        // a column offset listed twice (the reference's selector leaves the fourth
                        // offset of a 3-wide tail group at 0) names one matrix column: its first
                        // listing is the entry, later listings add nothing
                        bool repeat = false;
                        for (uint32_t e = 0; e < c; e++) repeat |= (cl[grp * 4 + e] == cl[grp * 4 + c]);
                        if (repeat && dcol < cols) continue;
                        if (dcol < cols) {
                            int64_t di = r * cols + dcol;
                            bool keep = mask ? (mask[di] != 0) : is_nonzero<T>(dense[di]);
                            if (keep) {
                                if (cnt < 4) { val[cnt] = dense[di]; pos[cnt] = c; }
                                cnt++;
                                used |= 1u << c;
                            }
                        } else if (c < 2) {
                            // a selected column beyond the matrix: explicit zero entry at position 0
                            if (cnt < 4) { val[cnt] = (T)0; pos[cnt] = 0; }
                            cnt++;
                            used |= 1u;
                        }
                    }
                    if (cnt > 2) { overflow.store(1); cnt = 2; }
                    if (cnt < 2) {
                        // fewer than n kept entries: zero-valued entries at the lowest unused
                        // positions, pair kept in ascending position order
                        for (uint32_t c = 0; c < 4 && cnt < 2; c++)
                            if (!(used & (1u << c))) { val[cnt] = (T)0; pos[cnt] = c; used |= 1u << c; cnt++; }
                        if (pos[0] > pos[1]) { std::swap(pos[0], pos[1]); std::swap(val[0], val[1]); }
                    }
                    int64_t vi = map.value_index(r, grp);
                    values[vi] = val[0];
                    values[vi + 1] = val[1];
                    word |= (pos[0] | (pos[1] << 2)) << (s * 16 + u * 4);
                }
            }
            metadata[map.meta_word(rp * 2, grp4 * 4)] = word;
        }
    }
    return overflow.load() ? SPATHA_ERR_BAD_ARGUMENT : SPATHA_OK;
}

template <class T>
int decode(const T* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols, int n, int m, int v,
           T* dense, int threads) {
    spatha_vnm_geometry g;
    int st = geometry_init(rows, cols, n, m, v, &g);
    if (st) return st;
    if (!dense || !columns || !values || !metadata) return SPATHA_ERR_BAD_ARGUMENT;
    const int64_t ngroups = g.ksp / 2;
    SlotMap map(g.ksp);
    for (int64_t i = 0; i < g.n_columns; i++)
        if (columns[i] >= (uint32_t)m) return SPATHA_ERR_BAD_ARGUMENT;
    set_threads(threads);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; r++) {
        T* out = dense + r * cols;
        std::memset(out, 0, sizeof(T) * (size_t)cols);
        const uint32_t* cl = columns + (r / v) * ngroups * 4;
        for (int64_t grp = 0; grp < ngroups; grp++) {
            uint32_t nib = (metadata[map.meta_word(r, grp)] >> SlotMap::meta_shift(r, grp)) & 0xfu;
            int64_t vi = map.value_index(r, grp);
            for (int j = 0; j < 2; j++) {
                int64_t dcol = grp * m + cl[grp * 4 + ((nib >> (2 * j)) & 3u)];
                if (dcol < cols) out[dcol] = values[vi + j];
            }
        }
    }
    return SPATHA_OK;
}

// ---------------------------------------------------------------------------
// Magnitude selector.
//
// For one (V-row block, m-column group) the winner is the first ascending
// 4-subset of columns, in lexicographic order, with the strictly largest
//     total = sum over rows (in row order) of  top1 + top2   (float32, in that order)
// and the mask marks, per row, the two largest of the winner's four entries.
// The totals do not depend on how equal magnitudes are ordered, so winners are
// found independently per (block, group).  Which of several EQUAL magnitudes a
// row keeps does depend on it: the reference sorts a permutation array that
// persists over the whole matrix (std::partial_sort on `indices`,
// grouped_nmv_tensor.py:122-123,155).  When a winner has such a tie in its
// second/third place, the permutation's history is replayed sequentially so
// that the mask matches bit for bit.
// ---------------------------------------------------------------------------
inline void top2_of(const float* v, int take, int& i1, int& i2) {
    // indices of the largest and second largest; the lower index wins ties
    i1 = 0;
    for (int i = 1; i < take; i++) if (v[i] > v[i1]) i1 = i;
    i2 = -1;
    for (int i = 0; i < take; i++) {
        if (i == i1) continue;
        if (i2 < 0 || v[i] > v[i2]) i2 = i;
    }
}

template <class Visit>
inline void for_each_subset(int width, int take, Visit&& visit) {
    int pick[4] = {0, 1, 2, 3};
    if (width < take) return;
    while (true) {
        visit(pick);
        int i = take - 1;
        while (i >= 0 && pick[i] == width - take + i) i--;
        if (i < 0) break;
        pick[i]++;
        for (int k = i + 1; k < take; k++) pick[k] = pick[k - 1] + 1;
    }
}

void find_winner(const float* base, int ld, int v_rows, GroupTask& t) {
    float best = 0.f;
    t.any = false;
    t.tie = false;
    std::fill(t.best, t.best + 4, 0);
    const int take = t.take;
    for_each_subset(t.width, take, [&](const int* pick) {
        float total = 0.f;
        for (int r = 0; r < v_rows; r++) {
            const float* row = base + (int64_t)r * ld;
            float x[4];
            for (int i = 0; i < take; i++) x[i] = row[pick[i]];
            int i1, i2;
            top2_of(x, take, i1, i2);
            total += x[i1];
            total += x[i2];
        }
        if (total > best) {
            best = total;
            t.any = true;
            for (int i = 0; i < take; i++) t.best[i] = pick[i];
        }
    });
}

// does the winner's mask depend on the permutation history (second and third largest equal in some row)?
void check_tie(const float* base, int ld, int v_rows, GroupTask& t) {
    t.tie = false;
    if (!t.any) return;
    const int take = t.take;
    for (int r = 0; r < v_rows && !t.tie; r++) {
        const float* row = base + (int64_t)r * ld;
        float x[4];
        for (int i = 0; i < take; i++) x[i] = row[t.best[i]];
        std::sort(x, x + take, [](float a, float b) { return a > b; });
        if (take > 2 && x[1] == x[2]) t.tie = true;
    }
}

}  // namespace

int encode_f32(const float* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m,
               int v, float* values, uint32_t* metadata, int threads) {
    return encode<float>(dense, mask, columns, rows, cols, n, m, v, values, metadata, threads);
}
int encode_f16(const uint16_t* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m,
               int v, uint16_t* values, uint32_t* metadata, int threads) {
    return encode<uint16_t>(dense, mask, columns, rows, cols, n, m, v, values, metadata, threads);
}
int decode_f32(const float* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols, int n,
               int m, int v, float* dense, int threads) {
    return decode<float>(values, metadata, columns, rows, cols, n, m, v, dense, threads);
}
int decode_f16(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols, int n,
               int m, int v, uint16_t* dense, int threads) {
    return decode<uint16_t>(values, metadata, columns, rows, cols, n, m, v, dense, threads);
}

int select_task_count(int rows, int cols, int m, int v, int* per_block_out) {
    const int blocks = rows / v, full = cols / m, rem = cols % m;
    const int per_block = full + ((rem >= 3) ? 1 : 0);       // a tail of three or more columns goes through the search
    if (per_block_out) *per_block_out = per_block;
    return blocks * per_block;
}

int select_columns_f32(const float* dense_abs, int rows, int cols, int n, int m, int v, int32_t* masks,
                       int32_t* columns, int threads) {
    return select_columns_with_winners(dense_abs, rows, cols, n, m, v, nullptr, true, masks, columns, threads);
}

int select_columns_with_winners(const float* dense_abs, int rows, int cols, int n, int m, int v, const GroupTask* winners,
                                bool replay_ties, int32_t* masks, int32_t* columns, int threads) {
    spatha_vnm_geometry g;
    int st = geometry_init(rows, cols, n, m, v, &g);
    if (st) return st;
    if (!dense_abs || !masks || !columns) return SPATHA_ERR_BAD_ARGUMENT;
    const int blocks = rows / v, full = cols / m, rem = cols % m;
    const int64_t cols_per_block = (int64_t)(g.ksp / n) * 4;
    const int tail = (rem >= 3) ? 1 : 0;          // tail group goes through the search
    const int per_block = full + tail;
    std::vector<GroupTask> tasks((size_t)blocks * per_block);
    set_threads(threads);

    // Phase 1: winners, independent per (block, group): searched here, or taken from the caller (the GPU search).
#pragma omp parallel for schedule(dynamic, 1) collapse(2)
    for (int b = 0; b < blocks; b++)
        for (int gi = 0; gi < per_block; gi++) {
            GroupTask& t = tasks[(size_t)b * per_block + gi];
            if (gi < full) { t.width = m; t.take = 4; }
            else { t.width = rem; t.take = (rem == 3) ? 3 : 4; }
            const float* base = dense_abs + (int64_t)b * v * cols + (int64_t)gi * m;
            if (winners) {
                const GroupTask& w = winners[(size_t)b * per_block + gi];
                t.any = w.any;
                for (int i = 0; i < 4; i++) t.best[i] = w.any ? w.best[i] : 0;
            } else {
                find_winner(base, cols, v, t);
            }
            check_tie(base, cols, v, t);
        }

    // Equal magnitudes in a winner: which of them a row keeps depends, in the reference, on a permutation that every
    // partial_sort call of the whole run has shaped.  Reproducing it means replaying the run sequentially (the cost of
    // the complete search on one thread); without the replay the lower column wins, which keeps the same magnitudes.
    bool need_replay = false;
    if (replay_ties)
        for (const GroupTask& t : tasks) need_replay |= t.tie;

    // Phase 2: masks and column offsets.  Without ties the two largest of each
    // row are unique as a set and the mask needs no history.
    auto emit = [&](int b, int gi, const GroupTask& t, const std::vector<int>* tie_mask) {
        int64_t col0 = (int64_t)gi * m;
        for (int r = 0; r < v; r++) {
            int32_t* mrow = masks + ((int64_t)b * v + r) * cols + col0;
            for (int j = 0; j < t.width; j++) mrow[j] = 0;
            if (!t.any) continue;
            if (tie_mask) {
                for (int j = 0; j < t.width; j++) mrow[j] = (*tie_mask)[(size_t)r * t.width + j];
            } else {
                const float* row = dense_abs + ((int64_t)b * v + r) * cols + col0;
                float x[4];
                for (int i = 0; i < t.take; i++) x[i] = row[t.best[i]];
                int i1, i2;
                top2_of(x, t.take, i1, i2);
                mrow[t.best[i1]] = 1;
                mrow[t.best[i2]] = 1;
            }
        }
    };
    auto emit_columns = [&](int b, int gi, const GroupTask& t, int stale3) {
        int32_t* out = columns + (int64_t)b * cols_per_block + (int64_t)gi * 4;
        if (t.take == 4) {
            for (int i = 0; i < 4; i++) out[i] = t.any ? t.best[i] : 0;
        } else {
            // width-3 tail: only three offsets are written; the fourth keeps the caller's value
            for (int i = 0; i < 3; i++) out[i] = t.any ? t.best[i] : 0;
            (void)stale3;
        }
    };

    if (!need_replay) {
#pragma omp parallel for schedule(static) collapse(2)
        for (int b = 0; b < blocks; b++)
            for (int gi = 0; gi < per_block; gi++) {
                const GroupTask& t = tasks[(size_t)b * per_block + gi];
                emit(b, gi, t, nullptr);
                emit_columns(b, gi, t, 0);
            }
    } else {
        // Replay the permutation history in the reference's visiting order: all full groups of
        // all blocks first, then the tail groups (grouped_nmv_tensor.py:125-189, :191-333).
        std::vector<float> vv(4, 0.f);
        std::vector<size_t> order(4);
        std::iota(order.begin(), order.end(), (size_t)0);
        std::vector<int> tie_mask;
        auto replay = [&](int b, int gi) {
            const GroupTask& t = tasks[(size_t)b * per_block + gi];
            const float* base = dense_abs + (int64_t)b * v * cols + (int64_t)gi * m;
            bool emitted = false;
            for_each_subset(t.width, t.take, [&](const int* pick) {
                bool is_winner = t.any && !emitted && std::equal(pick, pick + t.take, t.best);
                if (is_winner) tie_mask.assign((size_t)v * t.width, 0);
                for (int r = 0; r < v; r++) {
                    const float* row = base + (int64_t)r * cols;
                    for (int i = 0; i < t.take; i++) vv[i] = row[pick[i]];
                    std::partial_sort(order.begin(), order.begin() + n, order.end(),
                                      [&](size_t a, size_t c) { return vv[a] > vv[c]; });
                    if (is_winner)
                        for (int k = 0; k < n; k++) tie_mask[(size_t)r * t.width + pick[order[k]]] = 1;
                }
                if (is_winner) { emit(b, gi, t, &tie_mask); emitted = true; }
            });
            if (!t.any) emit(b, gi, t, nullptr);
            emit_columns(b, gi, t, 0);
        };
        for (int b = 0; b < blocks; b++)
            for (int gi = 0; gi < full; gi++) replay(b, gi);
        if (tail) {
            if (rem == 3) vv[3] = -1.f;   // the unused fourth candidate never reaches the top two
            for (int b = 0; b < blocks; b++) replay(b, full);
        }
    }

    if (rem > 0 && rem < 3) {
        // a tail narrower than three columns is kept whole
        for (int64_t r = 0; r < rows; r++)
            for (int j = cols - rem; j < cols; j++) masks[r * cols + j] = 1;
        for (int b = 0; b < blocks; b++)
            for (int i = 0; i < 4; i++) columns[(int64_t)b * cols_per_block + (int64_t)full * 4 + i] = i;
    }
    return SPATHA_OK;
}

// Random pattern from the C library's rand(), in the reference's drawing order
// (src/format/format_sr_nm.cpp:151-237): first every metadata word, walking
// 32-row blocks, then 4-group tiles, then the 16 words of a tile, then the 8
// pairs of a word; afterwards the column offsets per V-row block and group.
// Each draw permutes an array that is never reset, with the C++ library's
// classic shuffle (swap element i with element rand() % (i+1)).
namespace {
template <int LEN_MAX>
inline void shuffle_in_place(unsigned* a, int len) {
    for (int i = 1; i < len; i++) {
        int j = std::rand() % (i + 1);
        if (i != j) std::swap(a[i], a[j]);
    }
}
}  // namespace

int random_pattern(int rows, int cols, int n, int m, int v, uint32_t* metadata, uint32_t* columns) {
    spatha_vnm_geometry g;
    int st = geometry_init(rows, cols, n, m, v, &g);
    if (st) return st;
    if (!metadata || !columns) return SPATHA_ERR_BAD_ARGUMENT;
    const int64_t words_per_tile = 16;                 // 32 rows / 2 rows per word
    const int64_t tiles = g.ksp / 8;                   // 4-group tiles per row
    const int64_t full_groups = cols / m;              // groups entirely inside the matrix
    const int64_t full_tiles = full_groups / 4;        // tiles made of full groups only
    const bool has_tail_tile = (cols % m) != 0;        // the reference only then touches a partial tile
    unsigned pair[4] = {0, 1, 2, 3};
    auto draw_pair = [&]() -> uint32_t {
        shuffle_in_place<4>(pair, 4);
        std::sort(pair, pair + 2);
        return pair[0] | (pair[1] << 2);
    };
    for (int64_t rb = 0; rb < rows / 32; rb++) {
        int64_t tile = 0;
        for (; tile < full_tiles; tile++)
            for (int64_t w = 0; w < words_per_tile; w++) {
                uint32_t word = 0;
                for (int k = 0; k < 8; k++) word |= draw_pair() << (4 * k);
                metadata[rb * tiles * words_per_tile + tile * words_per_tile + w] = word;
            }
        if (has_tail_tile) {
            int64_t left = cols - 4 * (int64_t)m * full_tiles;   // dense columns not yet covered
            for (int64_t w = 0; w < words_per_tile; w++) {
                uint32_t word = 0;
                for (int s = 0; s < 2; s++) {
                    int64_t k = 0;
                    for (; k < left / m; k++) word |= draw_pair() << (4 * (k + 4 * s));
                    if (left % m > 0) word |= (0u | (1u << 2)) << (4 * (k + 4 * s));
                }
                metadata[rb * tiles * words_per_tile + tile * words_per_tile + w] = word;
            }
        }
    }
    std::vector<unsigned> quad(m);
    std::iota(quad.begin(), quad.end(), 0u);
    const int64_t cols_per_block = (int64_t)(g.ksp / n) * 4;
    for (int64_t b = 0; b < rows / v; b++) {
        int64_t grp = 0;
        for (; grp < full_groups; grp++) {
            for (int i = 1; i < m; i++) {
                int j = std::rand() % (i + 1);
                if (i != j) std::swap(quad[i], quad[j]);
            }
            std::sort(quad.begin(), quad.begin() + 4);
            for (int w = 0; w < 4; w++) columns[b * cols_per_block + grp * 4 + w] = quad[w];
        }
        if (cols % m != 0)
            for (int w = 0; w < 4; w++) columns[b * cols_per_block + grp * 4 + w] = (uint32_t)w;
    }
    return SPATHA_OK;
}

int pack_meta_blob(const uint32_t* metadata, int64_t n_metadata, const uint32_t* columns, int64_t n_columns,
                   uint32_t* blob, int64_t* columns_offset_words, int64_t* blob_words) {
    if (n_metadata < 0 || n_columns < 0) return SPATHA_ERR_BAD_ARGUMENT;
    int64_t off = ceil_div(n_metadata, 8) * 8;
    int64_t total = off + ceil_div(n_columns, 8) * 8;
    if (columns_offset_words) *columns_offset_words = off;
    if (blob_words) *blob_words = total;
    if (blob) {
        if (!metadata || !columns) return SPATHA_ERR_BAD_ARGUMENT;
        std::memset(blob, 0, sizeof(uint32_t) * (size_t)total);
        std::memcpy(blob, metadata, sizeof(uint32_t) * (size_t)n_metadata);
        std::memcpy(blob + off, columns, sizeof(uint32_t) * (size_t)n_columns);
    }
    return SPATHA_OK;
}

// ---------------------------------------------------------------------------
// On-disk container for an encoded matrix.  The reference parses --path_to_dset
// (src/util/argparse.h:123-126) but never reads a file; this format lets an
// encoded model be cached instead of re-encoded at every load.
//   bytes  0.. 3  "VNMF"            4.. 7  version (1)       8..11  value bits (16 or 32)
//         12..31  rows, cols, n, m, v (int32 each)          32..55  n_values, n_metadata, n_columns (int64)
//         56..63  FNV-1a 64 of the payload
//   payload: values, metadata words, column-loc words, in this order, little endian.
// ---------------------------------------------------------------------------
namespace {
struct FileHeader {
    char magic[4];
    uint32_t version, value_bits;
    int32_t rows, cols, n, m, v;
    int64_t n_values, n_metadata, n_columns;
    uint64_t checksum;
};
static_assert(sizeof(FileHeader) == 64, "header layout");

uint64_t fnv1a(uint64_t h, const void* data, size_t bytes) {
    const unsigned char* p = (const unsigned char*)data;
    for (size_t i = 0; i < bytes; i++) {
        h ^= p[i];
        h *= 1099511628211ull;
    }
    return h;
}
constexpr uint64_t FNV_SEED = 14695981039346656037ull;

int read_header(std::FILE* f, FileHeader& h) {
    if (std::fread(&h, sizeof(h), 1, f) != 1) return SPATHA_ERR_IO;
    if (std::memcmp(h.magic, "VNMF", 4) != 0 || h.version != 1) return SPATHA_ERR_IO;
    if (h.value_bits != 16 && h.value_bits != 32) return SPATHA_ERR_IO;
    spatha_vnm_geometry g;
    int st = geometry_init(h.rows, h.cols, h.n, h.m, h.v, &g);
    if (st != SPATHA_OK) return SPATHA_ERR_IO;
    if (g.n_values != h.n_values || g.n_metadata != h.n_metadata || g.n_columns != h.n_columns) return SPATHA_ERR_IO;
    return SPATHA_OK;
}
}  // namespace

int file_write(const char* path, int rows, int cols, int n, int m, int v, int value_bits, const void* values,
               const uint32_t* metadata, const uint32_t* columns) {
    if (!path || !values || !metadata || !columns || (value_bits != 16 && value_bits != 32)) return SPATHA_ERR_BAD_ARGUMENT;
    spatha_vnm_geometry g;
    int st = geometry_init(rows, cols, n, m, v, &g);
    if (st != SPATHA_OK) return st;
    FileHeader h;
    std::memcpy(h.magic, "VNMF", 4);
    h.version = 1;
    h.value_bits = (uint32_t)value_bits;
    h.rows = rows; h.cols = cols; h.n = n; h.m = m; h.v = v;
    h.n_values = g.n_values; h.n_metadata = g.n_metadata; h.n_columns = g.n_columns;
    const size_t vb = (size_t)g.n_values * (value_bits / 8), mb = (size_t)g.n_metadata * 4, cb = (size_t)g.n_columns * 4;
    h.checksum = fnv1a(fnv1a(fnv1a(FNV_SEED, values, vb), metadata, mb), columns, cb);
    std::FILE* f = std::fopen(path, "wb");
    if (!f) return SPATHA_ERR_IO;
    bool ok = std::fwrite(&h, sizeof(h), 1, f) == 1 && std::fwrite(values, 1, vb, f) == vb &&
              std::fwrite(metadata, 1, mb, f) == mb && std::fwrite(columns, 1, cb, f) == cb;
    ok = (std::fclose(f) == 0) && ok;
    return ok ? SPATHA_OK : SPATHA_ERR_IO;
}

int file_info(const char* path, spatha_vnm_geometry* geo, int* value_bits) {
    if (!path || !geo) return SPATHA_ERR_BAD_ARGUMENT;
    std::FILE* f = std::fopen(path, "rb");
    if (!f) return SPATHA_ERR_IO;
    FileHeader h;
    int st = read_header(f, h);
    std::fclose(f);
    if (st != SPATHA_OK) return st;
    if (value_bits) *value_bits = (int)h.value_bits;
    return geometry_init(h.rows, h.cols, h.n, h.m, h.v, geo);
}

int file_read(const char* path, void* values, uint32_t* metadata, uint32_t* columns) {
    if (!path || !values || !metadata || !columns) return SPATHA_ERR_BAD_ARGUMENT;
    std::FILE* f = std::fopen(path, "rb");
    if (!f) return SPATHA_ERR_IO;
    FileHeader h;
    int st = read_header(f, h);
    if (st != SPATHA_OK) {
        std::fclose(f);
        return st;
    }
    const size_t vb = (size_t)h.n_values * (h.value_bits / 8), mb = (size_t)h.n_metadata * 4, cb = (size_t)h.n_columns * 4;
    bool ok = std::fread(values, 1, vb, f) == vb && std::fread(metadata, 1, mb, f) == mb && std::fread(columns, 1, cb, f) == cb;
    char extra;
    ok = ok && std::fread(&extra, 1, 1, f) == 0;          // nothing may follow the payload
    std::fclose(f);
    if (!ok) return SPATHA_ERR_IO;
    if (fnv1a(fnv1a(fnv1a(FNV_SEED, values, vb), metadata, mb), columns, cb) != h.checksum) return SPATHA_ERR_IO;
    return SPATHA_OK;
}

}  // namespace spatha
