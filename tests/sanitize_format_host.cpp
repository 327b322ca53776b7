// Host format builder under AddressSanitizer + UndefinedBehaviorSanitizer (built and run by tests/test_sanitizers.py):
// every entry point of vnm_format.cpp on shapes that reach its edge cases (K % m != 0, padding groups, a 3-wide tail,
// zero blocks, ties, one block, V = 32 and 160, container files that are damaged).  The buffers are sized exactly as
// spatha_vnm_geometry says, so any write or read outside them is reported.  Exit status 0 = clean.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "../venom_amd/csrc/vnm_format.h"

static unsigned long long rng_state = 88172645463325252ull;
static unsigned rnd() {
    rng_state ^= rng_state << 13;
    rng_state ^= rng_state >> 7;
    rng_state ^= rng_state << 17;
    return (unsigned)(rng_state >> 11);
}

#define CHECK(cond)                                                              \
    do {                                                                         \
        if (!(cond)) {                                                           \
            std::fprintf(stderr, "line %d: %s failed\n", __LINE__, #cond);       \
            std::exit(2);                                                        \
        }                                                                        \
    } while (0)

static void one_shape(int rows, int cols, int m, int v, bool zero_block, bool ties, const std::string& tmp,
                      bool with_selector = true) {
    spatha_vnm_geometry geo;
    CHECK(spatha::geometry_init(rows, cols, 2, m, v, &geo) == SPATHA_OK);
    std::vector<float> dense((size_t)rows * cols), mag((size_t)rows * cols);
    for (size_t i = 0; i < dense.size(); i++) {
        const int q = (int)(rnd() % (ties ? 3 : 2001)) - (ties ? 1 : 1000);
        dense[i] = (float)q / (ties ? 1.0f : 256.0f);
    }
    if (zero_block)
        for (int r = 0; r < v && r < rows; r++)
            for (int c = 0; c < cols; c++) dense[(size_t)r * cols + c] = 0.f;
    for (size_t i = 0; i < dense.size(); i++) mag[i] = dense[i] < 0 ? -dense[i] : dense[i];

    // magnitude selector (with and without the replay of ties), then the mask-driven encoder and the decoder
    std::vector<int32_t> masks((size_t)rows * cols), columns((size_t)geo.n_columns);
    if (with_selector) {
    for (int threads : {1, 4}) {
        CHECK(spatha::select_columns_f32(mag.data(), rows, cols, 2, m, v, masks.data(), columns.data(), threads) == SPATHA_OK);
        CHECK(spatha::select_columns_with_winners(mag.data(), rows, cols, 2, m, v, nullptr, false, masks.data(), columns.data(),
                                                  threads) == SPATHA_OK);
    }
    std::vector<float> values((size_t)geo.n_values), back((size_t)rows * cols);
    std::vector<uint32_t> metadata((size_t)geo.n_metadata);
    CHECK(spatha::encode_f32(dense.data(), masks.data(), (const uint32_t*)columns.data(), rows, cols, 2, m, v, values.data(),
                             metadata.data(), 3) == SPATHA_OK);
    CHECK(spatha::decode_f32(values.data(), metadata.data(), (const uint32_t*)columns.data(), rows, cols, 2, m, v, back.data(),
                             3) == SPATHA_OK);
    for (size_t i = 0; i < back.size(); i++) CHECK(back[i] == (masks[i] ? dense[i] : 0.f));
    }

    // fp16 path on the benchmark's random pattern, non-zero driven encoder
    std::vector<uint32_t> meta2((size_t)geo.n_metadata), col2((size_t)geo.n_columns);
    std::srand(1);
    CHECK(spatha::random_pattern(rows, cols, 2, m, v, meta2.data(), col2.data()) == SPATHA_OK);
    std::vector<uint16_t> v16((size_t)geo.n_values), d16((size_t)rows * cols), v16b((size_t)geo.n_values);
    for (auto& x : v16) x = (uint16_t)(0x3c00 + rnd() % 64);          // small positive halfs
    CHECK(spatha::decode_f16(v16.data(), meta2.data(), col2.data(), rows, cols, 2, m, v, d16.data(), 2) == SPATHA_OK);
    std::vector<uint32_t> meta3((size_t)geo.n_metadata);
    CHECK(spatha::encode_f16(d16.data(), nullptr, col2.data(), rows, cols, 2, m, v, v16b.data(), meta3.data(), 2) == SPATHA_OK);
    std::vector<uint16_t> d16b((size_t)rows * cols);
    CHECK(spatha::decode_f16(v16b.data(), meta3.data(), col2.data(), rows, cols, 2, m, v, d16b.data(), 2) == SPATHA_OK);
    CHECK(std::memcmp(d16.data(), d16b.data(), d16.size() * 2) == 0);

    // device blob layout and the container file (whole, truncated, corrupted)
    std::vector<uint32_t> blob((size_t)geo.n_metadata + (size_t)geo.n_columns + 64);
    int64_t off = 0, words = 0;
    CHECK(spatha::pack_meta_blob(meta2.data(), geo.n_metadata, col2.data(), geo.n_columns, blob.data(), &off, &words) == SPATHA_OK);
    CHECK(words <= (int64_t)blob.size());
    const std::string path = tmp + "/m.vnm";
    CHECK(spatha::file_write(path.c_str(), rows, cols, 2, m, v, 16, v16.data(), meta2.data(), col2.data()) == SPATHA_OK);
    spatha_vnm_geometry g2;
    int bits = 0;
    CHECK(spatha::file_info(path.c_str(), &g2, &bits) == SPATHA_OK && bits == 16 && g2.n_values == geo.n_values);
    std::vector<uint16_t> vr((size_t)geo.n_values);
    std::vector<uint32_t> mr((size_t)geo.n_metadata), cr((size_t)geo.n_columns);
    CHECK(spatha::file_read(path.c_str(), vr.data(), mr.data(), cr.data()) == SPATHA_OK);
    CHECK(std::memcmp(vr.data(), v16.data(), vr.size() * 2) == 0);
    {   // flip one byte of the payload: the checksum must catch it
        FILE* f = std::fopen(path.c_str(), "r+b");
        CHECK(f != nullptr);
        std::fseek(f, 80, SEEK_SET);
        int c = std::fgetc(f);
        std::fseek(f, 80, SEEK_SET);
        std::fputc(c ^ 0x55, f);
        std::fclose(f);
        CHECK(spatha::file_read(path.c_str(), vr.data(), mr.data(), cr.data()) == SPATHA_ERR_IO);
    }
    {   // cut the file short
        FILE* f = std::fopen(path.c_str(), "wb");
        CHECK(f != nullptr);
        std::fputs("short", f);
        std::fclose(f);
        CHECK(spatha::file_info(path.c_str(), &g2, &bits) == SPATHA_ERR_IO);
    }
    std::remove(path.c_str());
}

int main(int argc, char** argv) {
    const std::string tmp = argc > 1 ? argv[1] : "/tmp";
    // bad shapes are refused before anything is touched
    spatha_vnm_geometry geo;
    CHECK(spatha::geometry_init(100, 128, 2, 8, 64, &geo) != SPATHA_OK);
    CHECK(spatha::geometry_init(128, 128, 3, 8, 64, &geo) != SPATHA_OK);
    one_shape(64, 64, 8, 64, false, false, tmp);
    one_shape(128, 100, 8, 32, false, false, tmp);      // K % m = 4
    one_shape(64, 35, 8, 32, false, true, tmp);         // 3-wide tail, ties
    one_shape(160, 200, 7, 160, true, false, tmp);      // K % m = 4, one V block, a zero block
    one_shape(256, 130, 4, 128, false, true, tmp);      // K % m = 2
    one_shape(96, 96, 32, 32, true, true, tmp);
    one_shape(64, 256, 100, 64, false, false, tmp, false);     // K % m = 56 (without the selector: C(100, 4) subsets)
    std::puts("sanitized host format builder: ok");
    return 0;
}
