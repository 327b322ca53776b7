/*
 * spatha.h -- C ABI of the MI355X (gfx950) Spatha library: the V:N:M sparse
 * format builder and the V:N:M sparse x dense SpMM.
 *
 * Plain C: pointers, sizes and an opaque handle.  Every entry point returns a
 * spatha_status (0 = success), never exits the process and never throws.
 * Host-side format functions take host pointers; spmm functions take device
 * pointers and a HIP stream (passed as void* so that the header needs no HIP
 * include; NULL is the default stream) and are stream ordered: no hidden
 * synchronisation.  The caller owns every buffer it passes in; a handle owns
 * only the copies it derives itself.
 *
 * Each declaration names the interface of the reference (UDC-GAC/venom) that it
 * stands in for.
 */
#ifndef SPATHA_H
#define SPATHA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum spatha_status {
    SPATHA_OK = 0,
    SPATHA_ERR_BAD_ARGUMENT = 1,   /* null pointer, negative size, n != 2, ...              */
    SPATHA_ERR_BAD_SHAPE = 2,      /* rows % V, V % 32, m < 4, N alignment, ...             */
    SPATHA_ERR_UNSUPPORTED = 3,    /* valid format, but no kernel for the request          */
    SPATHA_ERR_HIP = 4,            /* a HIP runtime call failed; see spatha_last_hip_error  */
    SPATHA_ERR_NO_DEVICE = 5,      /* no HIP device visible                                 */
    SPATHA_ERR_TOO_LARGE = 6,      /* beyond a fixed capacity of the entry point            */
    SPATHA_ERR_IO = 7              /* file missing, truncated, not a V:N:M container, or corrupt */
} spatha_status;

const char* spatha_status_string(int status);
/* hipError_t of the last failing HIP call made by this library on this thread. */
int spatha_last_hip_error(void);
/* "major.minor.patch" */
const char* spatha_version(void);

/* ------------------------------------------------------------------------ *
 * Format geometry.
 * Replaces the size arithmetic of Format_sr_nm<T>::init
 * (src/format/format_sr_nm.cpp:45-60) and SrNMTensor.to_sparse_sr_nm
 * (end2end/grouped_nmv_tensor.py:709-719).
 * ------------------------------------------------------------------------ */
typedef struct spatha_vnm_geometry {
    int32_t rows, cols, n, m, v;
    int32_t ksp;          /* stored values per row: ROUND_UP(ceil(cols/m)*n, 16) */
    int64_t n_values;     /* rows * ksp                                           */
    int64_t n_metadata;   /* (rows/2) * (ksp/8) 32-bit words                      */
    int64_t n_columns;    /* (rows/v) * (ksp/n) * 4 32-bit words                  */
} spatha_vnm_geometry;

int spatha_vnm_geometry_init(int rows, int cols, int n, int m, int v, spatha_vnm_geometry* out);

/* ------------------------------------------------------------------------ *
 * Host format builder (CPU; OpenMP over V-row blocks; threads <= 0 = all).
 * ------------------------------------------------------------------------ */

/* Random V:N:M pattern drawn from the C library's rand() in the reference's
 * order, so that an un-seeded process produces the reference benchmark's
 * pattern.  Replaces Format_sr_nm<T>::random_mask
 * (src/format/format_sr_nm.cpp:151-237) and BlockwiseSpMatrix::random_mask
 * (include/spatha/block_sparse/spmm/blockwise_format.h:159-246).
 * metadata / columns must hold n_metadata / n_columns words, zero-filled. */
int spatha_vnm_random_pattern(int rows, int cols, int n, int m, int v, uint32_t* metadata, uint32_t* columns);

/* (float)(rand() % 9 - 4) fill used for A's values and for B by the reference
 * benchmark (src/format/format_sr_nm.cpp:64-68, src/util/matrix_utils.h:88-97). */
int spatha_fill_rand_small_ints_f16(uint16_t* out, int64_t count);

/* The inputs of one `benchmark_spmm --sparsity-type n-to-m` run, drawn from
 * rand() in the reference's order: the cols x ncols_b entries of B first
 * (Dataset's n:m constructor, src/dataset/dataset.cpp:70-90, fills B before it
 * initialises the format), then the pattern (src/format/format_sr_nm.cpp:62),
 * then the rows x ksp stored values of A in storage order (:64-68).
 * metadata / columns must be zero-filled (n_metadata / n_columns words). */
int spatha_benchmark_inputs_f16(int rows, int cols, int ncols_b, int n, int m, int v, uint16_t* b, uint32_t* metadata,
                                uint32_t* columns, uint16_t* values);

/* Dense -> V:N:M.  dense is row-major rows x cols; columns holds, per V-row
 * block and per m-column group, the 4 selected column offsets (ascending).
 * mask == NULL: an entry is kept when it is non-zero
 *   (Format_sr_nm<T>::to_sparse_sr_nm, src/format/format_sr_nm.cpp:419-543);
 * mask != NULL (int32 rows x cols, 0/1): an entry is kept when its mask is set
 *   (to_sparse_sr_nm / func2, end2end/grouped_nmv_tensor.py:487-675).
 * A (row, group) with fewer than n kept entries gets zero-valued entries at the
 * lowest unused positions (the reference leaves stale data there); more than n
 * kept entries is an error (SPATHA_ERR_BAD_ARGUMENT). */
int spatha_vnm_encode_f32(const float* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols, int n,
                          int m, int v, float* values, uint32_t* metadata, int threads);
int spatha_vnm_encode_f16(const uint16_t* dense, const int32_t* mask, const uint32_t* columns, int rows, int cols,
                          int n, int m, int v, uint16_t* values, uint32_t* metadata, int threads);

/* V:N:M -> dense (dense is overwritten, zeros where nothing is stored).
 * Replaces Format_sr_nm<T>::to_dense (src/format/format_sr_nm.cpp:327-417) and
 * to_dense / func3 (end2end/grouped_nmv_tensor.py:345-485). */
int spatha_vnm_decode_f32(const float* values, const uint32_t* metadata, const uint32_t* columns, int rows, int cols,
                          int n, int m, int v, float* dense, int threads);
int spatha_vnm_decode_f16(const uint16_t* values, const uint32_t* metadata, const uint32_t* columns, int rows,
                          int cols, int n, int m, int v, uint16_t* dense, int threads);

/* Magnitude selector: per V-row block and m-column group pick the 4 columns
 * that maximise the sum over rows of the n largest magnitudes; emits the 0/1
 * mask and the column offsets.  dense_abs holds |A| as fp32.  masks (rows x
 * cols) and columns (n_columns) must be zero-filled by the caller.
 * Replaces group_n_m2 / func and nm_vector_mask_sparsify
 * (end2end/grouped_nmv_tensor.py:81-343, :746-779). */
int spatha_vnm_select_columns_f32(const float* dense_abs, int rows, int cols, int n, int m, int v, int32_t* masks,
                                  int32_t* columns, int threads);

/* The same selector with its search phase (all C(m,4) column subsets of every V x m block: 35 960 at m = 32) on the
 * GPU.  All pointers are HOST memory; the call uploads |A|, runs the search on `stream`, waits for it and finishes on
 * the host (it allocates and frees device scratch).  exact_ties != 0: masks and column offsets are bit-identical to
 * spatha_vnm_select_columns_f32, i.e. to the reference; when a winning subset has two EQUAL magnitudes competing for a
 * row's second slot, that costs a sequential replay of the reference's whole run (its choice among equals depends on
 * every comparison made before).  exact_ties == 0: the lower column index wins such a tie (same magnitudes kept, no
 * replay) - the setting for converting fp16 models, where equal magnitudes are common.  Same reference functions as
 * above. */
int spatha_vnm_select_columns_f32_gpu(const float* dense_abs, int rows, int cols, int n, int m, int v, int32_t* masks,
                                      int32_t* columns, int threads, int exact_ties, void* stream);

/* Layout of the single "metadata + column-loc" device blob the reference
 * uploads: metadata words first, column-loc words at the next multiple of 8
 * words.  Replaces BlockwiseSpMatrix<T>::transform_and_sync_device
 * (include/spatha/block_sparse/spmm/blockwise_format.h:327-373) and
 * Format_sr_nm<T>::transform_and_sync_device (src/format/format_sr_nm.cpp:239-285).
 * blob may be NULL to query sizes only. */
int spatha_vnm_pack_meta_blob(const uint32_t* metadata, int64_t n_metadata, const uint32_t* columns,
                              int64_t n_columns, uint32_t* blob, int64_t* columns_offset_words,
                              int64_t* blob_words);

/* On-disk container of an encoded matrix (64-byte header: magic "VNMF", version, value width, shape,
 * array lengths, FNV-1a checksum; then values, metadata, column-loc).  The reference parses
 * --path_to_dset (src/util/argparse.h:123-126, src/benchmark_spmm.cpp) but never opens the file; these
 * three functions give the flag a meaning: an encoded matrix can be cached instead of re-encoded.
 * value_bits is 16 (fp16 values) or 32 (fp32).  spatha_vnm_file_info reports the sizes the caller has to
 * allocate before spatha_vnm_file_read; a checksum or size mismatch is SPATHA_ERR_IO. */
int spatha_vnm_file_write(const char* path, int rows, int cols, int n, int m, int v, int value_bits, const void* values,
                          const uint32_t* metadata, const uint32_t* columns);
int spatha_vnm_file_info(const char* path, spatha_vnm_geometry* geometry, int* value_bits);
int spatha_vnm_file_read(const char* path, void* values, uint32_t* metadata, uint32_t* columns);

/* ------------------------------------------------------------------------ *
 * SpMM on the GPU:  C[rows x N] = A_vnm[rows x cols] * B[cols x N],
 * fp16 operands, fp32 accumulation, fp16 result (round to nearest even).
 * ------------------------------------------------------------------------ */
typedef struct spatha_spmm_plan spatha_spmm_plan;

/* Builds a plan from the three canonical arrays, which are DEVICE pointers
 * (values fp16[n_values], metadata u32[n_metadata], columns u32[n_columns]).
 * The plan keeps derived copies laid out for the gfx950 sparse matrix
 * instructions; the canonical arrays are not referenced after the call's work
 * on `stream` has completed.  Replaces SpmmNMInitFn / SpmmBlockwiseOp::initialize
 * (include/spatha/block_sparse/spmm/blockwise_op.h:98-161, :209-223) together
 * with BlockwiseSpMatrix::init_sparse_device (blockwise_format.h:285-325). */
int spatha_spmm_plan_create(int rows, int cols, int n, int m, int v, const uint16_t* values_dev,
                            const uint32_t* metadata_dev, const uint32_t* columns_dev, void* stream,
                            spatha_spmm_plan** out);
int spatha_spmm_plan_destroy(spatha_spmm_plan* plan);

#define SPATHA_OUT_ROW_MAJOR 0   /* C[rows][N]           (benchmark path)                  */
#define SPATHA_OUT_TRANSPOSED 1  /* C^T[N][rows] + bias  (PyTorch extension path)          */

/* Runs one SpMM.  B is row-major cols x N (N contiguous), N % 8 == 0.
 * out_layout SPATHA_OUT_ROW_MAJOR writes C[rows][N]; bias must be NULL
 *   (SpmmNMExecFn, blockwise_op.h:233-238; main loop blockwise_kernel.h:739-944).
 * out_layout SPATHA_OUT_TRANSPOSED writes C^T[N][rows] and, when bias != NULL,
 *   adds bias[row] in fp16 to the rounded product (spmm_cuda,
 *   end2end/spatha_mod/block_sparse/spmm/blockwise_library.cu:294-389, fused
 *   epilogue end2end/spatha_mod/block_sparse/spmm/blockwise_kernel.h:294-343).
 * variant selects a kernel: 0 = automatic. */
int spatha_spmm_run(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                    uint16_t* out_dev, int out_layout, int variant, void* stream);

#define SPATHA_ACT_NONE 0
#define SPATHA_ACT_GELU 1        /* 0.5 x (1 + erf(x / sqrt 2))                                   */
#define SPATHA_ACT_GELU_TANH 2   /* 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))  ("gelu_new") */

/* spatha_spmm_run with the layer's elementwise tail fused into the write-out: in either layout
 *   out = act(fp16(fp16(A B) + bias[row]))
 * (bias may be NULL, act may be SPATHA_ACT_NONE; the activation is evaluated in fp32 on the fp16 sum and
 * rounded once).  The bias part is the reference's fused epilogue (blockwise_kernel.h:294-343) made available
 * to the row-major layout as well; the activation has no counterpart in the reference's kernels, whose
 * callers apply it as a separate elementwise pass over the output (the feed-forward block of the models in
 * end2end/).  Row-major output with bias lets a following spatha_spmm_run consume `out` as its B operand
 * without a transposed copy.  Kernels without the fused write-out are skipped by the automatic choice and
 * refused (SPATHA_ERR_UNSUPPORTED) when named. */
int spatha_spmm_run_fused(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                          uint16_t* out_dev, int out_layout, int activation, int variant, void* stream);

/* spatha_spmm_run_fused (automatic kernel choice) for callers that bring scratch memory: with a workspace the library may
 * split k-loops over several workgroups where tiles alone leave compute units idle: few tiles with long k-loops (small
 * rows x N and large K, the "split-K for small M*N" case: e.g. 1024 x 16384 x 1024 at 128:2:8 runs 128 tiles of 128
 * k-steps on 256 CUs, 50 us unsplit and 35 us in two parts).  The parts of a tile hand fp32 partial sums over through the
 * workspace and the part that finishes last adds them in a fixed order, so results do not depend on timing; with
 * integer-valued operands they equal spatha_spmm_run's bit for bit, otherwise they may differ from it by the rounding of
 * another summation order.  spatha_spmm_workspace_bytes names the size a call needs for N columns (0: this shape is
 * never split; the call then equals spatha_spmm_run_fused); a smaller or NULL workspace is not an error, the call just
 * does not split.  The workspace (256-byte aligned device memory) is cleared ONCE with spatha_spmm_workspace_init after it
 * has been allocated; every completed call leaves it ready for the next one, of any plan and shape (clear it again after a
 * call that failed).  It belongs to a call until the call's work on `stream` has completed: calls that overlap in time
 * need a workspace each.  Neither call allocates or synchronises.  No counterpart in the reference, whose kernels cover
 * such shapes by a search over 179 tile tuples (src/spmm/spatha_spmm.hpp:49-585). */
size_t spatha_spmm_workspace_bytes(const spatha_spmm_plan* plan, int N, int out_layout, int fused);
int spatha_spmm_workspace_init(void* workspace_dev, size_t workspace_bytes, void* stream);
int spatha_spmm_run_ws(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev, uint16_t* out_dev,
                       int out_layout, int activation, void* workspace_dev, size_t workspace_bytes, void* stream);

/* One SpMM straight from the canonical arrays, for callers that cannot allocate (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same result as
 * spatha_spmm_plan_create + spatha_spmm_run (automatic kernel choice) + spatha_spmm_plan_destroy on the same arguments,
 * but the derived copies of A that a plan would hipMalloc live in a fixed 8 MiB array in device memory that belongs to
 * the library (each GPU the library runs on holds its own copy until the process ends), and the call allocates and
 * frees nothing: it launches the pack kernels and the SpMM kernel on `stream`.  A matrix whose derived copies exceed
 * the array is refused with SPATHA_ERR_TOO_LARGE (the array holds e.g. 4096 x 1024 or 1024 x 4096 at 2:8 and
 * 4096 x 1024 at 2:4).  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (two
 * streams, two threads) race; calls ordered on one stream do not.  Every argument check and the kernel choice happen
 * before the first launch, so a refused call has not touched the array.  The first call on a device looks up the
 * array's address and sets kernel attributes, which a stream capture cannot hold: make one call outside the capture
 * (any shape that reaches the same kernel) before recording calls into a graph. */
int spatha_spmm_run_noalloc(int rows, int cols, int n, int m, int v, const uint16_t* values_dev,
                            const uint32_t* metadata_dev, const uint32_t* columns_dev, const uint16_t* B_dev, int N,
                            const uint16_t* bias_dev, uint16_t* out_dev, int out_layout, void* stream);

/* Kernel variants are numbered 1 .. spatha_spmm_num_variants() - 1; 0 selects automatically. */
int spatha_spmm_num_variants(void);

/* Name / tile shape of the kernel `variant` (or of the automatic choice for N
 * when variant == 0) would use, for logs; returns NULL if unsupported.  The
 * automatic choice may be two launches (the row tiles of an uneven last round of
 * 128 x 256 tiles on 128 x 128 tiles): the name then ends in "+rest_on_tile128x128". */
const char* spatha_spmm_kernel_name(const spatha_spmm_plan* plan, int N, int out_layout, int variant);

/* Times `iters` back-to-back launches with HIP events on `stream` after
 * `warmup` untimed ones; *ms_per_launch is the mean.  Replaces cuTime
 * (src/cuda_utils.h:61-87) as used by Spatha<T,T2>::spmm
 * (src/spmm/spatha_spmm.cpp:55-82). */
int spatha_spmm_time(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                     uint16_t* out_dev, int out_layout, int variant, int warmup, int iters, void* stream,
                     float* ms_per_launch);

/* Times the automatic choice and every kernel id that accepts this plan, N and layout (spatha_spmm_time each), and
 * reports the fastest: *best_variant (0 when nothing beats the automatic choice, which may be a form no single id gives,
 * see spatha_spmm_kernel_name), *best_ms, and *auto_ms, the automatic choice's time.  ms_per_variant, when not NULL,
 * holds spatha_spmm_num_variants() floats: [0] the automatic choice, [id] that kernel, negative where it does not apply.
 * The result of every timed kernel lands in out_dev.  For callers that would rather measure their shape than trust the
 * rule table; replaces the search over the reference's tile tuples (src/spmm/spatha_spmm.hpp:49-585, swept per shape by
 * benchmark/run_spmm_spatha.sh). */
int spatha_spmm_tune(const spatha_spmm_plan* plan, const uint16_t* B_dev, int N, const uint16_t* bias_dev,
                     uint16_t* out_dev, int out_layout, int warmup, int iters, void* stream, int* best_variant,
                     float* best_ms, float* auto_ms, float* ms_per_variant);

/* Dense fp16 GEMM C[rows x N] = A[rows x cols] * B[cols x N] (fp32 accumulate)
 * on the GPU: the dense baseline and --check product of the benchmark.
 * Replaces Cublas_gemm<half,half,float>::sgemm (src/gemm/cublas_gemm.cpp:54-96). */
int spatha_dense_gemm_f16(const uint16_t* A_dev, const uint16_t* B_dev, int rows, int cols, int N, uint16_t* C_dev,
                          void* stream);

/* out[cols x rows] = transpose of in[rows x cols], fp16, both row-major and 16-byte aligned.
 * The PyTorch layer needs the activation as [in_features, tokens] for spatha_spmm_run; this replaces the
 * `dense.contiguous()` of a transposed view in sparse_dense_mul_dispatch
 * (end2end/bert_pytorch.py:85-87, called from SrnmSpmm.forward :126-136). */
int spatha_transpose_f16(const uint16_t* in_dev, int rows, int cols, uint16_t* out_dev, void* stream);

/* out[tokens x hidden] = LayerNorm(x + residual) over the last dimension, fp16 in and out, fp32 arithmetic
 * (the sum is rounded to fp16 first, as the separate addition would; biased variance; gamma, beta of length hidden).
 * residual_dev may be NULL (plain layer norm).  hidden % 8 == 0 and hidden <= 4096 (SPATHA_ERR_UNSUPPORTED beyond);
 * all pointers 16-byte aligned; out may alias x or residual.
 * One kernel for the `LayerNorm(dropout(dense(h)) + input)` tail of the stock BertSelfOutput / BertOutput modules
 * that the reference's harness runs after its attention-output and FFN-down SpMMs (the model of
 * end2end/bert_pytorch.py:170-171; the SpMM layers it swaps in are :108-167). */
int spatha_add_layernorm_f16(const uint16_t* x_dev, const uint16_t* residual_dev, const uint16_t* gamma_dev,
                             const uint16_t* beta_dev, float eps, int tokens, int hidden, uint16_t* out_dev, void* stream);

/* spatha_add_layernorm_f16 that writes its result twice: out[tokens][hidden] as above and out_t[hidden][tokens], the
 * feature-major copy a following spatha_spmm_run takes as its B operand - the copy the reference's layer makes with
 * `x.T.contiguous()` in front of every SpMM (end2end/bert_pytorch.py:87, :130-134), here written by the kernel that
 * already holds the values.  tokens % 8 == 0 as well. */
int spatha_add_layernorm_f16_t(const uint16_t* x_dev, const uint16_t* residual_dev, const uint16_t* gamma_dev,
                               const uint16_t* beta_dev, float eps, int tokens, int hidden, uint16_t* out_dev, uint16_t* out_t_dev,
                               void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SPATHA_H */
