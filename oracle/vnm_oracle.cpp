// CPU oracle for the V:N:M (VENOM) format and the Spatha SpMM.
//
// THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  It restates, on the CPU, the
// algorithms of the reference (UDC-GAC/venom) that the GPU library must agree
// with.  Only the test-suite, the smoke check and the benchmark's
// "cpu_baseline" leg may load it; the shipped library never links or calls it.
//
// Every function names the reference lines it follows.  The loop nests keep the
// reference's iteration order on purpose (the encoder's behaviour for rows with
// fewer than n kept entries depends on it), while the product code uses closed
// forms; agreement between the two is therefore a real check.
//
// Pinning status (what independent evidence each function is checked against
// in tests/):
//   vo_sizes          closed forms + golden vectors written by the reference's
//                     Python host code (tests/golden)
//   vo_encode_*       golden vectors (mask driven), closed-form index maps,
//                     decode(encode(x)) == x
//   vo_decode         golden vectors, closed-form index maps
//   vo_select_columns golden vectors incl. ties, brute force on tiny inputs
//   vo_spmm_*         dense product of vo_decode(A) with B in float64 (numpy)
//   vo_random_mask    known answers for five shapes drawn from one stream,
//                     derived without this file (tests/golden/
//                     make_random_mask_kat.py: glibc's rand() and libstdc++'s
//                     random_shuffle restated in Python, the draws walked in
//                     the reference's order); that restatement of rand() is
//                     held against the C library and shuffle_rand against the
//                     real std::random_shuffle (a C++14 snippet the test builds)
//   vo_half<->float   numpy.float16 conversion on all 65536 bit patterns
//
// Build: see oracle/build.py (g++ -O2 -fopenmp -shared).

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include <numeric>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

inline int round_up(int x, int y) { return ((x + y - 1) / y) * y; }

// IEEE binary16 <-> binary32, round to nearest even, software only.
inline float half_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else {  // subnormal: renormalise
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

inline uint16_t float_to_half(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
    uint32_t absx = x & 0x7fffffffu;
    if (absx >= 0x7f800000u) {  // inf / nan
        return (uint16_t)(sign | 0x7c00u | ((absx > 0x7f800000u) ? (0x200u | ((absx >> 13) & 0x3ffu)) : 0u));
    }
    if (absx >= 0x477ff000u) {  // >= 65520 rounds to inf
        return (uint16_t)(sign | 0x7c00u);
    }
    if (absx < 0x33000001u) {  // <= 2^-25 rounds to zero (ties to even -> 0)
        return sign;
    }
    int32_t e = (int32_t)(absx >> 23) - 127;
    uint32_t man = (absx & 0x7fffffu) | 0x800000u;
    int shift;
    uint32_t base;
    if (e < -14) {  // subnormal result
        shift = 13 + (-14 - e);
        base = 0;
    } else {
        shift = 13;
        base = (uint32_t)(e + 15) << 10;
        man &= 0x7fffffu;
    }
    uint32_t q = man >> shift;
    uint32_t rem = man & ((1u << shift) - 1u);
    uint32_t halfway = 1u << (shift - 1);
    uint32_t r = base + q;
    if (rem > halfway || (rem == halfway && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}

// fp16 + fp16 with one rounding (what a hardware half-precision add or fma
// with multiplier 1 returns): the exact sum fits a double.
inline uint16_t add_half(uint16_t a, uint16_t b) {
    double x = (double)half_to_float(a) + (double)half_to_float(b);
    if (x == 0.0 || !std::isfinite(x)) return float_to_half((float)x);
    int e = std::ilogb(x);
    if (e < -14) e = -14;
    double scale = std::ldexp(1.0, e - 10);
    double q = std::nearbyint(x / scale);   // default mode: ties to even
    return float_to_half((float)(q * scale));
}

// Derived sizes, format_sr_nm.cpp:45-60.
struct Geometry {
    int rows, cols, n, m, v, brow, mbrow;
    int m_fixed = 4, bits_meta = 2, mrow_m = 2, brow_fixed = 16;
    int nelems, nelems_col;
    int cols_sp, cols_sp_pad_nm, cols_sp_pad;
    Geometry(int rows_, int cols_, int n_, int m_, int v_, int brow_, int mbrow_)
        : rows(rows_), cols(cols_), n(n_), m(m_), v(v_), brow(brow_), mbrow(mbrow_) {
        nelems = 32 / bits_meta;
        nelems_col = nelems / mrow_m;
        cols_sp = (cols / m) * n;
        cols_sp_pad_nm = (round_up(cols, m) / m) * n;
        cols_sp_pad = round_up((round_up(cols, m) / m) * n, 16);
    }
    long n_values() const { return (long)rows * cols_sp_pad; }
    long n_columns() const { return (long)(rows / v) * (cols_sp_pad / n) * m_fixed; }
    long n_metadata() const { return (long)(rows / mrow_m) * (cols_sp_pad / nelems_col); }
};

// libstdc++'s std::random_shuffle(first, last) (bits/stl_algo.h): element i is
// swapped with element rand() % (i + 1), for i = 1 .. len-1.
inline void shuffle_rand(std::vector<unsigned>& a) {
    for (size_t i = 1; i < a.size(); i++) {
        size_t j = (size_t)(std::rand() % (int)(i + 1));
        if (i != j) std::swap(a[i], a[j]);
    }
}

// Shared walk over (row, group-of-four-groups) used by encoder and decoder,
// format_sr_nm.cpp:347-351 / :441-445.  The callback gets the loop counters.
template <class F>
void walk_tiles(const Geometry& g, F&& body) {
    int bm_m = g.rows / g.v;
    int mbrow_m = g.v / g.mbrow;
    int mbrow_m2 = g.mbrow / g.brow_fixed;
    int brow_m = g.brow_fixed / g.brow;
    int mcol_kk = g.nelems / g.mrow_m / g.n;
    int mcol_k = g.cols_sp_pad / g.n / mcol_kk;
    for (int bm_i = 0; bm_i < bm_m; bm_i++)
        for (int mbrow_i = 0; mbrow_i < mbrow_m; mbrow_i++)
            for (int mbrow_i2 = 0; mbrow_i2 < mbrow_m2; mbrow_i2++)
                for (int brow_i = 0; brow_i < brow_m; brow_i++)
                    for (int mcol_i = 0; mcol_i < mcol_k; mcol_i++)
                        body(bm_i, mbrow_i, mbrow_i2, brow_i, mcol_i, mcol_kk, mcol_k);
}

template <class T, class IsKept>
void encode_impl(const Geometry& g, const T* dense, const uint32_t* columns_in, T* values_out,
                 uint32_t* meta_out, IsKept&& is_kept) {
    // Scratch that persists over the whole walk, as in format_sr_nm.cpp:437-439
    // (the reference leaves it uninitialised; zero is the only defined choice).
    // A third kept entry is written one slot further on, where the next (row, group) of the
    // walk overwrites it; the slack absorbs the one case that would leave the arrays.
    std::vector<T> vals(g.nelems + 8, (T)0);
    std::vector<uint32_t> idxs(g.nelems + 8, 0u);
    std::vector<uint32_t> cols(64, 0u);
    const int n = g.n, mrow_m = g.mrow_m, m_fixed = g.m_fixed;
    walk_tiles(g, [&](int bm_i, int mbrow_i, int mbrow_i2, int brow_i, int mcol_i, int mcol_kk, int mcol_k) {
        int col_kk = mcol_kk, col_k = mcol_k;
        for (int a = 0; a < col_kk; a++)       // :447-452
            for (int b = 0; b < m_fixed; b++)
                cols[a * m_fixed + b] = columns_in[(long)bm_i * col_k * col_kk * m_fixed + mcol_i * col_kk * m_fixed + a * m_fixed + b];
        long row_base = (long)bm_i * g.v + mbrow_i * g.mbrow + mbrow_i2 * g.brow_fixed + brow_i * g.brow;
        for (int mbrow_ii = 0; mbrow_ii < g.brow / mrow_m; mbrow_ii++) {
            for (int mcol_ii = 0; mcol_ii < mcol_kk; mcol_ii++) {      // :455-503
                for (int mbrow_iii = 0; mbrow_iii < mrow_m; mbrow_iii++) {
                    int pos = 0;
                    long row = row_base + mbrow_ii * mrow_m + mbrow_iii;
                    for (int c = 0; c < m_fixed; c++) {
                        uint32_t off = cols[mcol_ii * m_fixed + c];
                        long dcol = (long)mcol_i * g.m * mcol_kk + mcol_ii * g.m + off;
                        if (dcol < g.cols) {
                            long di = row * g.cols + dcol;
                            if (is_kept(di)) {
                                idxs[mbrow_iii * n + mcol_ii * mrow_m * n + pos] = (uint32_t)c;
                                vals[mcol_ii * mrow_m * n + mbrow_iii * n + pos] = dense[di];
                                pos++;
                            }
                        } else if (c < 2) {    // :486-499
                            idxs[mbrow_iii * n + mcol_ii * mrow_m * n + pos] = 0u;
                            vals[mcol_ii * mrow_m * n + mbrow_iii * n + pos] = (T)0;
                            pos++;
                        }
                    }
                }
            }
            uint32_t word = 0;                                         // :505-536
            for (int mbrow_iii = 0; mbrow_iii < mrow_m; mbrow_iii++)
                for (int mcol_ii = 0; mcol_ii < mcol_kk; mcol_ii++)
                    for (int j = 0; j < n; j++) {
                        long vi = (long)bm_i * g.v * g.cols_sp_pad + (long)mbrow_i * g.mbrow * g.cols_sp_pad +
                                  (long)mbrow_i2 * g.brow_fixed * g.cols_sp_pad + brow_i * g.brow * g.nelems / mrow_m +
                                  (long)mcol_i * g.brow_fixed * g.nelems / mrow_m + mbrow_ii * mrow_m * n +
                                  mcol_ii * n * g.brow + mbrow_iii * n + j;
                        values_out[vi] = vals[mcol_ii * mrow_m * n + mbrow_iii * n + j];
                        uint32_t t = idxs[mbrow_iii * n + mcol_ii * mrow_m * n + j];
                        word |= t << (mbrow_iii * (g.nelems / mrow_m) * g.bits_meta + mcol_ii * n * g.bits_meta + j * g.bits_meta);
                    }
            long wi = (long)bm_i * mcol_k * g.v / mrow_m + (long)mbrow_i * mcol_k * g.mbrow / mrow_m +
                      mbrow_i2 * g.brow_fixed / mrow_m + brow_i * g.brow / mrow_m + (long)mcol_i * g.mbrow / mrow_m + mbrow_ii;
            meta_out[wi] = word;
        }
    });
}

template <class T>
void decode_impl(const Geometry& g, const T* values, const uint32_t* meta, const uint32_t* columns_in, T* dense_out) {
    // format_sr_nm.cpp:327-417 (Python twin grouped_nmv_tensor.py:390-476).
    std::vector<uint32_t> idxs(g.nelems, 0u), cols(64, 0u);
    const int n = g.n, mrow_m = g.mrow_m, m_fixed = g.m_fixed;
    walk_tiles(g, [&](int bm_i, int mbrow_i, int mbrow_i2, int brow_i, int mcol_i, int mcol_kk, int mcol_k) {
        int col_kk = mcol_kk, col_k = mcol_k;
        for (int a = 0; a < col_kk; a++)
            for (int b = 0; b < m_fixed; b++)
                cols[a * m_fixed + b] = columns_in[(long)bm_i * col_k * col_kk * m_fixed + mcol_i * col_kk * m_fixed + a * m_fixed + b];
        long row_base = (long)bm_i * g.v + mbrow_i * g.mbrow + mbrow_i2 * g.brow_fixed + brow_i * g.brow;
        for (int mbrow_ii = 0; mbrow_ii < g.brow / mrow_m; mbrow_ii++) {
            long wi = (long)bm_i * mcol_k * g.v / mrow_m + (long)mbrow_i * mcol_k * g.mbrow / mrow_m +
                      mbrow_i2 * g.brow_fixed / mrow_m + brow_i * g.brow / mrow_m + (long)mcol_i * g.mbrow / mrow_m + mbrow_ii;
            uint32_t word = meta[wi];
            for (int mbrow_iii = 0; mbrow_iii < mrow_m; mbrow_iii++)   // :360-377
                for (int mcol_ii = 0; mcol_ii < mcol_kk; mcol_ii++)
                    for (int j = 0; j < n; j++)
                        idxs[mbrow_iii * n + mcol_ii * mrow_m * n + j] =
                            (word >> (mbrow_iii * (g.nelems / mrow_m) * g.bits_meta + mcol_ii * n * g.bits_meta + j * g.bits_meta)) & 0x3u;
            for (int mcol_ii = 0; mcol_ii < mcol_kk; mcol_ii++)        // :379-408
                for (int mbrow_iii = 0; mbrow_iii < mrow_m; mbrow_iii++)
                    for (int j = 0; j < n; j++) {
                        uint32_t off = cols[mcol_ii * m_fixed + idxs[mcol_ii * mrow_m * n + mbrow_iii * n + j]];
                        long dcol = (long)mcol_i * g.m * mcol_kk + mcol_ii * g.m + off;
                        if (dcol < g.cols) {
                            long row = row_base + mbrow_ii * mrow_m + mbrow_iii;
                            long vi = (long)bm_i * g.v * g.cols_sp_pad + (long)mbrow_i * g.mbrow * g.cols_sp_pad +
                                      (long)mbrow_i2 * g.brow_fixed * g.cols_sp_pad + brow_i * g.brow * g.nelems / mrow_m +
                                      (long)mcol_i * g.brow_fixed * g.nelems / mrow_m + mbrow_ii * mrow_m * n +
                                      mcol_ii * n * g.brow + mbrow_iii * n + j;
                            dense_out[row * g.cols + dcol] = values[vi];
                        }
                    }
        }
    });
}

// One m-wide column group of the magnitude selector: try every ascending
// subset of `width` candidate columns (4, or 3 in the remainder==3 branch),
// grouped_nmv_tensor.py:136-175, :218-252, :278-316.
struct SelectorState {
    std::vector<float> v;
    std::vector<int> vx;
    std::vector<size_t> order;  // persists across rows, quadruples, groups and blocks (:122-123)
    SelectorState() : v(4, 0.f), vx(4, 0), order(4) { std::iota(order.begin(), order.end(), 0); }
};

void select_group(SelectorState& st, const float* dense, int ld, int v_rows, int n, int ncand, int take,
                  int mask_ld, int* best_mask, int* best_cols) {
    float best = 0.f;
    std::vector<int> mask((size_t)v_rows * mask_ld);
    std::vector<int> pick(take);
    // ascending subsets in lexicographic order
    for (int i = 0; i < take; i++) pick[i] = i;
    if (ncand < take) return;
    while (true) {
        for (int i = 0; i < take; i++) st.vx[i] = pick[i];
        float total = 0.f;
        std::fill(mask.begin(), mask.end(), 0);
        for (int r = 0; r < v_rows; r++) {
            for (int i = 0; i < take; i++) st.v[i] = dense[(long)r * ld + pick[i]];
            std::partial_sort(st.order.begin(), st.order.begin() + n, st.order.end(),
                              [&](size_t a, size_t b) { return st.v[a] > st.v[b]; });
            for (int k = 0; k < n; k++) {
                total += dense[(long)r * ld + st.vx[st.order[k]]];
                mask[(size_t)r * mask_ld + st.vx[st.order[k]]] = 1;
            }
        }
        if (total > best) {
            best = total;
            std::copy(mask.begin(), mask.end(), best_mask);
            for (int i = 0; i < 4; i++) best_cols[i] = st.vx[i];
        }
        int i = take - 1;
        while (i >= 0 && pick[i] == ncand - take + i) i--;
        if (i < 0) break;
        pick[i]++;
        for (int k = i + 1; k < take; k++) pick[k] = pick[k - 1] + 1;
    }
}

}  // namespace

extern "C" {

// --- fp16 helpers ----------------------------------------------------------
void vo_half_to_float(const uint16_t* in, float* out, long count) {
    for (long i = 0; i < count; i++) out[i] = half_to_float(in[i]);
}
void vo_float_to_half(const float* in, uint16_t* out, long count) {
    for (long i = 0; i < count; i++) out[i] = float_to_half(in[i]);
}
void vo_add_half(const uint16_t* a, const uint16_t* b, uint16_t* out, long count) {
    for (long i = 0; i < count; i++) out[i] = add_half(a[i], b[i]);
}

// --- sizes: format_sr_nm.cpp:53-60, grouped_nmv_tensor.py:709-719 ---------
int vo_sizes(int rows, int cols, int n, int m, int v, long* out4) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    out4[0] = g.cols_sp_pad;
    out4[1] = g.n_values();
    out4[2] = g.n_metadata();
    out4[3] = g.n_columns();
    return 0;
}

// --- random pattern: format_sr_nm.cpp:151-237 ------------------------------
// Uses the process-wide rand() stream exactly as the reference does; call
// vo_srand(1) first to start from glibc's default state.
void vo_srand(unsigned seed) { std::srand(seed); }
int vo_rand(void) { return std::rand(); }
// one shuffle of a caller-held array, exposed so that the tests can hold it against libstdc++'s std::random_shuffle
void vo_shuffle(unsigned* a, int len) {
    std::vector<unsigned> v(a, a + len);
    shuffle_rand(v);
    std::copy(v.begin(), v.end(), a);
}

int vo_random_mask(int rows, int cols, int n, int m, int v, int mbrow, uint32_t* meta, uint32_t* columns) {
    Geometry g(rows, cols, n, m, v, 4, mbrow);
    int ncol = g.cols_sp, ncol_pad = g.cols_sp_pad_nm;
    std::vector<unsigned> arr(g.m_fixed);
    std::iota(arr.begin(), arr.end(), 0u);
    for (int i = 0; i < rows / mbrow; i++) {
        int j = 0;
        for (; j < ncol / g.nelems_col; j++) {
            for (int k = 0; k < mbrow / g.mrow_m; k++) {
                uint32_t word = 0;
                for (int grp = 0; grp < g.nelems / n; grp++) {
                    shuffle_rand(arr);
                    std::sort(arr.begin(), arr.begin() + n);
                    for (int w = 0; w < n; w++) word |= arr[w] << (grp * n * g.bits_meta + w * g.bits_meta);
                }
                meta[(long)i * mbrow / g.mrow_m * g.cols_sp_pad / g.nelems_col + (long)j * mbrow / g.mrow_m + k] = word;
            }
        }
        if (ncol_pad > ncol) {   // :179-210
            for (int k = 0; k < mbrow / g.mrow_m; k++) {
                uint32_t word = 0;
                int resto = cols - 4 * m * (ncol / g.nelems_col);
                for (int t = 0; t < g.mrow_m; t++) {
                    int grp = 0;
                    for (; grp < resto / m; grp++) {
                        shuffle_rand(arr);
                        std::sort(arr.begin(), arr.begin() + n);
                        for (int w = 0; w < n; w++) word |= arr[w] << ((grp + t * 4) * n * g.bits_meta + w * g.bits_meta);
                    }
                    if (resto % m > 0)
                        for (int w = 0; w < n; w++) word |= (uint32_t)w << ((grp + t * 4) * n * g.bits_meta + w * g.bits_meta);
                }
                meta[(long)i * mbrow / 2 * g.cols_sp_pad / 8 + (long)j * mbrow / 2 + k] = word;
            }
        }
    }
    std::vector<unsigned> arr2(m);
    std::iota(arr2.begin(), arr2.end(), 0u);
    int resto = cols - (ncol / n) * m;
    for (int i = 0; i < rows / v; i++) {   // :213-236
        int j = 0;
        for (; j < ncol / n; j++) {
            shuffle_rand(arr2);
            std::sort(arr2.begin(), arr2.begin() + g.m_fixed);
            for (int w = 0; w < g.m_fixed; w++) columns[(long)i * (g.cols_sp_pad / n) * g.m_fixed + j * g.m_fixed + w] = arr2[w];
        }
        if (resto > 0)
            for (int w = 0; w < g.m_fixed; w++) columns[(long)i * (g.cols_sp_pad / n) * g.m_fixed + j * g.m_fixed + w] = (uint32_t)w;
    }
    return 0;
}

// Values / dense-B fill of the reference benchmark: (float)(rand() % 9 - 4),
// format_sr_nm.cpp:64-68 and matrix_utils.h:90-96.
void vo_fill_rand_ints(float* out, long count) {
    for (long i = 0; i < count; i++) out[i] = (float)(std::rand() % 9 - 4);
}

// --- encoder ---------------------------------------------------------------
// mask == NULL: nonzero-driven (format_sr_nm.cpp:419-543);
// mask != NULL: mask-driven (grouped_nmv_tensor.py:529-665).
int vo_encode_f32(const float* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m,
                  int v, float* values, uint32_t* meta) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    if (mask) encode_impl<float>(g, dense, columns, values, meta, [&](long i) { return mask[i] != 0; });
    else encode_impl<float>(g, dense, columns, values, meta, [&](long i) { return dense[i] != 0.f; });
    return 0;
}
// fp16 storage (bit patterns); the kept test converts to float like static_cast<float>(val) != 0.
int vo_encode_f16(const uint16_t* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m,
                  int v, uint16_t* values, uint32_t* meta) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    if (mask) encode_impl<uint16_t>(g, dense, columns, values, meta, [&](long i) { return mask[i] != 0; });
    else encode_impl<uint16_t>(g, dense, columns, values, meta, [&](long i) { return half_to_float(dense[i]) != 0.f; });
    return 0;
}

// --- decoder ---------------------------------------------------------------
int vo_decode_f32(const float* values, const uint32_t* meta, const uint32_t* columns, int rows, int cols, int n, int m,
                  int v, float* dense) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    decode_impl<float>(g, values, meta, columns, dense);
    return 0;
}
int vo_decode_f16(const uint16_t* values, const uint32_t* meta, const uint32_t* columns, int rows, int cols, int n,
                  int m, int v, uint16_t* dense) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    decode_impl<uint16_t>(g, values, meta, columns, dense);
    return 0;
}

// --- magnitude selector: grouped_nmv_tensor.py:112-334 ---------------------
// dense_abs: |A| as fp32, row-major rows x cols.  sparse (may be NULL) is
// multiplied by the mask in place as the reference does.  masks and columns
// must be zero-initialised by the caller (:759-760).
int vo_select_columns(const float* dense_abs, float* sparse, int rows, int cols, int n, int m, int v, int32_t* masks,
                      int32_t* columns) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    int bm_m = rows / v, mcol_k = cols / m, mcol_k_p = (cols - 1) / m + 1;
    long indexes_cols = (long)(g.cols_sp_pad / n) * 4;
    SelectorState st;
    std::vector<int> best_mask, best_cols(4);
    auto run = [&](int bm_i, int mcol_i, int width, int ncand, int take, int ncols_out) {
        const float* base = dense_abs + (long)bm_i * v * cols + (long)mcol_i * m;
        best_mask.assign((size_t)v * width, 0);
        std::fill(best_cols.begin(), best_cols.end(), 0);
        select_group(st, base, cols, v, n, ncand, take, width, best_mask.data(), best_cols.data());
        for (int i = 0; i < v; i++)
            for (int j = 0; j < width; j++) {
                long di = (long)bm_i * v * cols + (long)i * cols + (long)mcol_i * m + j;
                int keep = best_mask[(size_t)i * width + j];
                masks[di] = keep;
                if (sparse) sparse[di] *= (float)keep;
            }
        for (int i = 0; i < ncols_out; i++) columns[bm_i * indexes_cols + (long)mcol_i * 4 + i] = best_cols[i];
    };
    for (int bm_i = 0; bm_i < bm_m; bm_i++)
        for (int mcol_i = 0; mcol_i < mcol_k; mcol_i++) run(bm_i, mcol_i, m, m, 4, 4);
    int rem = cols % m;
    if (rem > 0) {
        if (rem < 3) {   // :196-206
            for (int i = 0; i < rows; i++)
                for (int j = cols - rem; j < cols; j++) masks[(long)i * cols + j] = 1;
            for (int bm_i = 0; bm_i < bm_m; bm_i++)
                for (int j = 0; j < 4; j++) columns[bm_i * indexes_cols + (long)mcol_k * 4 + j] = j;
        } else if (rem == 3) {   // :207-267 (v[3] = -1 keeps slot 3 out of the top n)
            st.v[3] = -1.f;
            for (int bm_i = 0; bm_i < bm_m; bm_i++)
                for (int mcol_i = mcol_k; mcol_i < mcol_k_p; mcol_i++) run(bm_i, mcol_i, rem, rem, 3, rem);
        } else {         // :268-331
            for (int bm_i = 0; bm_i < bm_m; bm_i++)
                for (int mcol_i = mcol_k; mcol_i < mcol_k_p; mcol_i++) run(bm_i, mcol_i, rem, rem, 4, 4);
        }
    }
    return 0;
}

// --- SpMM on the compressed form -------------------------------------------
// C[r][:] += values[r, g, j] * B[g*m + columns[b, g, pos(r, g, j)]][:], the
// arithmetic meaning the reference kernel gives the format
// (blockwise_kernel.h:869-881); out-of-range B rows contribute zero.
// fp16 in, fp32 accumulate in storage order, fp16 round-to-nearest-even out
// (mma.h:557-575, :726-739).  out_layout 0: C[rows][N]; 1: C^T[N][rows] (+bias
// per row, added in fp16 after rounding, as the end-to-end kernel does,
// end2end/spatha_mod/block_sparse/spmm/blockwise_kernel.h:296-341).
int vo_spmm_f16(const uint16_t* values, const uint32_t* meta, const uint32_t* columns, int rows, int cols, int n, int m,
                int v, const uint16_t* B, int N, const uint16_t* bias, int out_layout, uint16_t* C, int threads) {
    Geometry g(rows, cols, n, m, v, 4, 32);
    const int ksp = g.cols_sp_pad, ngroups = ksp / 2;
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#endif
    std::vector<float> Bf((size_t)cols * N);
#pragma omp parallel for schedule(static)
    for (long i = 0; i < (long)cols * N; i++) Bf[i] = half_to_float(B[i]);
#pragma omp parallel
    {
        std::vector<float> acc(N);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < rows; r++) {
            std::fill(acc.begin(), acc.end(), 0.f);
            int R16 = r / 16, q = (r % 16) / 4, p = (r % 4) / 2, s = r % 2, b = r / v;
            for (int grp = 0; grp < ngroups; grp++) {
                int t = grp / 4, u = grp % 4;
                long wi = (long)(r / 32) * (ksp / 8) * 16 + (long)t * 16 + ((r % 32) / 16) * 8 + q * 2 + p;
                uint32_t word = meta[wi];
                for (int j = 0; j < 2; j++) {
                    long vi = (long)R16 * 16 * ksp + (long)t * 128 + q * 32 + u * 8 + p * 4 + s * 2 + j;
                    float a = half_to_float(values[vi]);
                    uint32_t pos = (word >> (s * 16 + u * 4 + j * 2)) & 3u;
                    long k = (long)grp * m + columns[(long)b * ngroups * 4 + (long)grp * 4 + pos];
                    if (k >= cols || a == 0.f) continue;
                    const float* brow = &Bf[(size_t)k * N];
                    for (int c = 0; c < N; c++) acc[c] += a * brow[c];
                }
            }
            for (int c = 0; c < N; c++) {
                uint16_t h = float_to_half(acc[c]);
                if (out_layout == 0) {
                    C[(long)r * N + c] = h;
                } else {
                    if (bias) h = add_half(h, bias[r]);
                    C[(long)c * rows + r] = h;
                }
            }
        }
    }
    return 0;
}

// Dense check product C = A_dense * B with fp32 accumulation and fp16 output,
// the role cuBLAS plays in the reference's --check (cublas_gemm.cpp:54-96).
int vo_dense_gemm_f16(const uint16_t* A, const uint16_t* B, int rows, int cols, int N, uint16_t* C, int threads) {
#ifdef _OPENMP
    if (threads > 0) omp_set_num_threads(threads);
#endif
    std::vector<float> Bf((size_t)cols * N);
    for (long i = 0; i < (long)cols * N; i++) Bf[i] = half_to_float(B[i]);
#pragma omp parallel
    {
        std::vector<float> acc(N);
#pragma omp for schedule(dynamic, 4)
        for (int r = 0; r < rows; r++) {
            std::fill(acc.begin(), acc.end(), 0.f);
            for (int k = 0; k < cols; k++) {
                float a = half_to_float(A[(long)r * cols + k]);
                if (a == 0.f) continue;
                const float* brow = &Bf[(size_t)k * N];
                for (int c = 0; c < N; c++) acc[c] += a * brow[c];
            }
            for (int c = 0; c < N; c++) C[(long)r * N + c] = float_to_half(acc[c]);
        }
    }
    return 0;
}

// The reference's acceptance rule: any |a - b| > 1.0 flags the run
// (benchmark_spmm.cpp:51-74).  Returns 1 on mismatch, 0 otherwise.
int vo_check_results(const uint16_t* a, const uint16_t* b, long count) {
    for (long i = 0; i < count; i++)
        if (std::fabs(half_to_float(a[i]) - half_to_float(b[i])) > 1.0f) return 1;
    return 0;
}

int vo_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

}  // extern "C"
