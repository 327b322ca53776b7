// Host-side V:N:M format builder (C++ interface behind the C ABI of spatha.h).
#pragma once

#include <cstdint>

#include "../../include/spatha.h"

namespace spatha {

int geometry_init(int rows, int cols, int n, int m, int v, spatha_vnm_geometry* out);

int random_pattern(int rows, int cols, int n, int m, int v, uint32_t* metadata, uint32_t* columns);

int encode_f32(const float* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m,
               int v, float* values, uint32_t* metadata, int threads);
int encode_f16(const uint16_t* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n, int m,
               int v, uint16_t* values, uint32_t* metadata, int threads);
int decode_f32(const float* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols, int n,
               int m, int v, float* dense, int threads);
int decode_f16(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols, int n,
               int m, int v, uint16_t* dense, int threads);

// One (V-row block, m-column group) of the magnitude selector.
struct GroupTask {
    int width;      // candidate columns in this group (m, or cols % m in the tail)
    int take;       // subset size (4, or 3 in the tail of width 3)
    int best[4];    // winning subset (ascending); all zero when every total is 0
    bool any;       // a subset had total > 0
    bool tie;       // the winner's mask depends on the permutation history
};
// tasks of the search: (rows / v) blocks x per_block groups, block-major
int select_task_count(int rows, int cols, int m, int v, int* per_block_out);
// the selector with the winners of the search supplied by the caller (winners == nullptr: searched on the host)
// replay_ties: reproduce the reference's choice among EQUAL magnitudes (sequential replay of the whole run when any
// winner has such a tie); false: the lower column index wins
int select_columns_with_winners(const float* dense_abs, int rows, int cols, int n, int m, int v, const GroupTask* winners,
                                bool replay_ties, int32_t* masks, int32_t* columns, int threads);
int select_columns_f32(const float* dense_abs, int rows, int cols, int n, int m, int v, int32_t* masks,
                       int32_t* columns, int threads);

int file_write(const char* path, int rows, int cols, int n, int m, int v, int value_bits, const void* values,
               const uint32_t* metadata, const uint32_t* columns);
int file_info(const char* path, spatha_vnm_geometry* geo, int* value_bits);
int file_read(const char* path, void* values, uint32_t* metadata, uint32_t* columns);

int pack_meta_blob(const uint32_t* metadata, int64_t n_metadata, const uint32_t* columns, int64_t n_columns,
                   uint32_t* blob, int64_t* columns_offset_words, int64_t* blob_words);

}  // namespace spatha
