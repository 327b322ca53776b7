// benchmark_spmm for gfx950: the command-line driver of the V:N:M SpMM, with the flags and the
// CSV row of the reference driver (src/benchmark_spmm.cpp:157-222, src/util/argparse.h:24-233),
// calling the library only through its C ABI (include/spatha.h).
//
//   benchmark_spmm --sparsity-type n-to-m --spmm spatha --gemm cuBlas --precision half
//                  --meta-block-size 32 --block-size 4 --nn_row 2 --mm_row 8
//                  --m 1024 --k 4096 --n 4096 --d 0.5 --bm 128 --bn 64 --bk 32 --wm 32 --wn 64
//                  --wk 32 --mm 16 --mn 8 --mk 32 --nstage 2 --random --check
//
// --bm is V, as in the reference.  The other tile flags (--bn --bk --w* --m[mnk] --nstage) name
// NVIDIA tile shapes that do not exist here: they are accepted, echoed in the CSV row and
// otherwise ignored; the kernel is chosen by the library (or with --variant <id>).
// Inputs are drawn from the C library's rand() in the reference's order (B, then the pattern,
// then A's values), all small integers, so --check compares exactly representable numbers.
// stdout: one CSV row
//   spmm_code,arch,m,k,n,meta_block_sz,block_sz,nn_row,mm_row,density,bm,bn,bk,wm,wn,wk,mm,mn,mk,
//   nstage,spmm_time_ms,gemm_time_ms,speedup,error
// followed by appended columns: spmm_us,dense_equiv_tflops,pct_smfmac_peak,hbm_gbs,kernel,
//   cpu_encode_decode_s,cpu_threads,gemm_impl
// gemm_time_ms / speedup are against the vendor library's dense fp16 GEMM (hipBLASLt; the reference's column is
// against cuBLAS, src/gemm/cublas_gemm.cpp:54-96); gemm_impl says which GEMM was timed ("hipblaslt", or "in-tree"
// when the vendor library has no kernel for the shape).  --check always compares with the library's own exact
// dense product (spatha_dense_gemm_f16).

#include <hip/hip_runtime_api.h>

#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include "../../include/spatha.h"
#include "vendor_gemm.h"

namespace {

const char* kUsage =
    "\tRequired cmdline args:\n"
    "\t--sparsity-type [csr/cvs/n-to-m]   (only n-to-m is implemented)\n"
    "\t--spmm [CLASP/sputnik/spatha/cuSparseLt]   (only spatha is implemented)\n"
    "\t--gemm [cuBlas]\n"
    "\t--precision [single, half, int8]   (only half is implemented)\n"
    "\t--m [M] --k [K] --n [N] --d [density between 0~1]\n"
    "\tOptional cmdline args:\n"
    "\t--block-size [4] --meta-block-size [32] --nn_row [2] --mm_row [m] --acc_t [fp32]\n"
    "\t--bm [V] --bn --bk --wm --wn --wk --mm --mn --mk --nstage   (tile flags: only --bm is used)\n"
    "\t--variant [kernel id, 0 = automatic] --tune --random --check --path_to_dset [file]\n";

[[noreturn]] void die(const std::string& msg) {
    std::fprintf(stderr, "%s%s\n", kUsage, msg.c_str());
    std::exit(EXIT_FAILURE);
}

#define HIP_OK(call)                                                                            \
    do {                                                                                        \
        hipError_t e_ = (call);                                                                 \
        if (e_ != hipSuccess) {                                                                 \
            std::fprintf(stderr, "HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(EXIT_FAILURE);                                                            \
        }                                                                                       \
    } while (0)

#define SPATHA_OK_OR_DIE(call)                                                                  \
    do {                                                                                        \
        int s_ = (call);                                                                        \
        if (s_ != SPATHA_OK) {                                                                  \
            std::fprintf(stderr, "spatha error %d (%s) at %s:%d\n", s_, spatha_status_string(s_), __FILE__, __LINE__); \
            std::exit(EXIT_FAILURE);                                                            \
        }                                                                                       \
    } while (0)

float half_bits_to_float(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16, exp = (h >> 10) & 0x1fu, man = h & 0x3ffu, bits;
    if (exp == 0) {
        if (man == 0) bits = sign;
        else {
            int e = -1;
            do { man <<= 1; e++; } while (!(man & 0x400u));
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
        }
    } else if (exp == 31) bits = sign | 0x7f800000u | (man << 13);
    else bits = sign | ((exp + 112u) << 23) | (man << 13);
    float f;
    std::memcpy(&f, &bits, 4);
    return f;
}

}  // namespace

int main(int argc, const char** argv) {
    int m = 0, n = 0, k = 0, block_sz = 1, meta_block_sz = 0, spmm_code = -1, gemm_code = -1, acc_code = 0;
    int pattern_code = -1, precision_code = -1, bm = 0, bn = 0, bk = 0, wm = 0, wn = 0, wk = 0, mm = 0, mn = 0, mk = 0;
    int nstage = 0, nn_row = 0, mm_row = 0, variant = 0;
    bool tune = false;
    float density = 0.f;
    unsigned seed = 2022;
    bool check = false;
    std::string path_to_dset;

    auto next_int = [&](int& i) { return std::atoi(argv[++i]); };
    for (int i = 1; i < argc; ++i) {
        const std::string a = argv[i];
        const bool has_val = i != argc - 1;
        if (a == "--m" && has_val) m = next_int(i);
        else if (a == "--n" && has_val) n = next_int(i);
        else if (a == "--k" && has_val) k = next_int(i);
        else if (a == "--d" && has_val) density = (float)std::atof(argv[++i]);
        else if (a == "--block-size" && has_val) block_sz = next_int(i);
        else if (a == "--meta-block-size" && has_val) meta_block_sz = next_int(i);
        else if (a == "--nn_row" && has_val) nn_row = next_int(i);
        else if (a == "--mm_row" && has_val) mm_row = next_int(i);
        else if (a == "--bm" && has_val) bm = next_int(i);
        else if (a == "--bn" && has_val) bn = next_int(i);
        else if (a == "--bk" && has_val) bk = next_int(i);
        else if (a == "--wm" && has_val) wm = next_int(i);
        else if (a == "--wn" && has_val) wn = next_int(i);
        else if (a == "--wk" && has_val) wk = next_int(i);
        else if (a == "--mm" && has_val) mm = next_int(i);
        else if (a == "--mn" && has_val) mn = next_int(i);
        else if (a == "--mk" && has_val) mk = next_int(i);
        else if (a == "--nstage" && has_val) nstage = next_int(i);
        else if (a == "--variant" && has_val) variant = next_int(i);
        else if (a == "--tune") tune = true;
        else if (a == "--path_to_dset" && has_val) path_to_dset = argv[++i];
        else if (a == "--random") seed = (unsigned)std::chrono::system_clock::now().time_since_epoch().count();
        else if (a == "--check") check = true;
        else if (a == "--sparsity-type" && has_val) {
            const std::string v = argv[++i];
            pattern_code = v == "csr" ? 0 : v == "cvs" ? 1 : v == "n-to-m" ? 2 : -1;
        } else if (a == "--spmm" && has_val) {
            const std::string v = argv[++i];
            spmm_code = v == "CLASP" ? 0 : v == "sputnik" ? 1 : v == "spatha" ? 2 : v == "cuSparseLt" ? 3 : -1;
        } else if (a == "--gemm" && has_val) {
            const std::string v = argv[++i];
            gemm_code = v == "cuBlas" ? 0 : v == "cuBlasLt" ? 1 : -1;
        } else if (a == "--precision" && has_val) {
            const std::string v = argv[++i];
            precision_code = v == "single" ? 0 : v == "half" ? 1 : v == "int8" ? 3 : -1;
        } else if (a == "--acc_t" && has_val) {
            const std::string v = argv[++i];
            acc_code = v == "fp32" ? 0 : v == "fp16" ? 1 : -1;
        } else {
            die("unknown or incomplete argument: " + a);
        }
    }
    (void)seed;   // the reference stores the seed and never reads it; inputs depend on the shape only
    if (m == 0 || n == 0 || k == 0 || density == 0.f) die("Forget to set m,n,k,density or the path to an input file?");
    if (pattern_code != 2) die("sparsity-pattern is not given or unsupported (only n-to-m).");
    if (spmm_code != 2) die("only --spmm spatha is implemented.");
    if (gemm_code != 0) die("only --gemm cuBlas (the dense baseline of this build) is implemented.");
    if (precision_code != 1) die("only precision:half is implemented");
    if (acc_code != 0) die("accumulator type unsupported.");
    if (block_sz != 4 || meta_block_sz != 32) die("the V:N:M layout is defined for --block-size 4 --meta-block-size 32 only.");
    if (nn_row != 2 || mm_row < 4) die("--nn_row must be 2 and --mm_row >= 4.");
    if (bm <= 0) die("--bm (V) is required.");
    const int V = bm;

    spatha_vnm_geometry geo;
    int st = spatha_vnm_geometry_init(m, k, nn_row, mm_row, V, &geo);
    if (st != SPATHA_OK) die(std::string("shape not representable: ") + spatha_status_string(st));
    if (n % 8 != 0) die("--n must be a multiple of 8.");

    // ---- inputs, in the reference's drawing order: B, pattern, values
    std::vector<uint16_t> hB((size_t)k * n), hVal((size_t)geo.n_values);
    std::vector<uint32_t> hMeta((size_t)geo.n_metadata, 0u), hCols((size_t)geo.n_columns, 0u);
    SPATHA_OK_OR_DIE(spatha_benchmark_inputs_f16(m, k, n, nn_row, mm_row, V, hB.data(), hMeta.data(), hCols.data(), hVal.data()));
    // --path_to_dset (parsed and ignored by the reference, src/util/argparse.h:123-126): the encoded A is read
    // from that container when it exists (its shape must match the flags), and written there otherwise
    if (!path_to_dset.empty()) {
        spatha_vnm_geometry fg;
        int bits = 0;
        if (spatha_vnm_file_info(path_to_dset.c_str(), &fg, &bits) == SPATHA_OK) {
            if (bits != 16 || fg.rows != m || fg.cols != k || fg.n != nn_row || fg.m != mm_row || fg.v != V)
                die("--path_to_dset: the stored matrix does not match --m/--k/--nn_row/--mm_row/--bm (or is not fp16).");
            SPATHA_OK_OR_DIE(spatha_vnm_file_read(path_to_dset.c_str(), hVal.data(), hMeta.data(), hCols.data()));
        } else {
            SPATHA_OK_OR_DIE(spatha_vnm_file_write(path_to_dset.c_str(), m, k, nn_row, mm_row, V, 16, hVal.data(), hMeta.data(),
                                                   hCols.data()));
        }
    }

    // ---- host format conversion, timed: decode (the dense operand of the check) and re-encode of that dense matrix
    //      (non-zero driven, as the reference's init_from_dense does, src/format/format_sr_nm.cpp:108-149)
    const int threads = (int)std::thread::hardware_concurrency();
    std::vector<uint16_t> hDense((size_t)m * k);
    auto t0 = std::chrono::steady_clock::now();
    SPATHA_OK_OR_DIE(spatha_vnm_decode_f16(hVal.data(), hMeta.data(), hCols.data(), m, k, nn_row, mm_row, V, hDense.data(), 0));
    {
        std::vector<uint16_t> reVal((size_t)geo.n_values);
        std::vector<uint32_t> reMeta((size_t)geo.n_metadata, 0u);
        SPATHA_OK_OR_DIE(spatha_vnm_encode_f16(hDense.data(), nullptr, hCols.data(), m, k, nn_row, mm_row, V, reVal.data(),
                                               reMeta.data(), 0));
    }
    double cpu_convert_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();

    // ---- device
    uint16_t *dB, *dC, *dVal, *dDense, *dCref;
    uint32_t *dMeta, *dCols;
    // the dense baseline wants K to be a multiple of 8: zero columns of A / zero rows of B are appended for it
    // (the SpMM is given the same B buffer with its true K)
    const int kpad = (k + 7) / 8 * 8;
    if (kpad != k) {
        std::vector<uint16_t> padded((size_t)m * kpad, 0);
        for (int r = 0; r < m; r++) std::memcpy(&padded[(size_t)r * kpad], &hDense[(size_t)r * k], (size_t)k * 2);
        hDense.swap(padded);
    }
    HIP_OK(hipMalloc((void**)&dB, (size_t)kpad * n * 2));
    HIP_OK(hipMemset(dB, 0, (size_t)kpad * n * 2));
    HIP_OK(hipMalloc((void**)&dC, (size_t)m * n * 2));
    HIP_OK(hipMalloc((void**)&dCref, (size_t)m * n * 2));
    HIP_OK(hipMalloc((void**)&dVal, hVal.size() * 2));
    HIP_OK(hipMalloc((void**)&dMeta, hMeta.size() * 4));
    HIP_OK(hipMalloc((void**)&dCols, hCols.size() * 4));
    HIP_OK(hipMalloc((void**)&dDense, hDense.size() * 2));
    HIP_OK(hipMemcpy(dB, hB.data(), hB.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dVal, hVal.data(), hVal.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dMeta, hMeta.data(), hMeta.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dCols, hCols.data(), hCols.size() * 4, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dDense, hDense.data(), hDense.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemset(dC, 0, (size_t)m * n * 2));

    spatha_spmm_plan* plan = nullptr;
    st = spatha_spmm_plan_create(m, k, nn_row, mm_row, V, dVal, dMeta, dCols, nullptr, &plan);
    if (st != SPATHA_OK) {
        std::fprintf(stderr, "no kernel for this configuration: %s\n", spatha_status_string(st));
        return EXIT_FAILURE;
    }
    if (tune) {
        // --tune: every kernel id that takes the shape is timed, the fastest one runs the benchmark (times to stderr)
        std::vector<float> per((size_t)spatha_spmm_num_variants(), -1.f);
        float best_ms = 0.f, auto_ms = 0.f;
        SPATHA_OK_OR_DIE(spatha_spmm_tune(plan, dB, n, nullptr, dC, SPATHA_OUT_ROW_MAJOR, 5, 30, nullptr, &variant, &best_ms, &auto_ms,
                                          per.data()));
        for (size_t id = 0; id < per.size(); id++)
            if (per[id] >= 0.f)
                std::fprintf(stderr, "tune: id %2zu %-72s %9.2f us%s\n", id, spatha_spmm_kernel_name(plan, n, SPATHA_OUT_ROW_MAJOR, (int)id),
                             per[id] * 1e3f, (int)id == variant ? "  <- fastest" : "");
    }
    const char* kname = spatha_spmm_kernel_name(plan, n, SPATHA_OUT_ROW_MAJOR, variant);
    if (!kname) {
        std::fprintf(stderr, "kernel variant %d does not support V=%d / this shape\n", variant, V);
        return EXIT_FAILURE;
    }

    // ---- timing: 10 warm-up + 100 timed launches between two events (src/cuda_utils.h:61-87)
    float spmm_ms = 0.f;
    SPATHA_OK_OR_DIE(spatha_spmm_time(plan, dB, n, nullptr, dC, SPATHA_OUT_ROW_MAJOR, variant, 11, 100, nullptr, &spmm_ms));
    // dense baseline: the vendor GEMM, 10 warm-up + 100 timed launches like the SpMM (into a buffer of its own);
    // the exact in-tree product that --check compares with is computed afterwards
    float gemm_ms = 0.f;
    const char* gemm_impl = "hipblaslt";
    {
        hipEvent_t e0, e1;
        HIP_OK(hipEventCreate(&e0));
        HIP_OK(hipEventCreate(&e1));
        VendorGemm* vg = vendor_gemm_create(m, kpad, n);
        uint16_t* dCvendor = nullptr;
        if (vg) HIP_OK(hipMalloc((void**)&dCvendor, (size_t)m * n * 2));
        auto run_gemm = [&]() {
            if (vg) {
                if (vendor_gemm_run(vg, dDense, dB, dCvendor, nullptr) != 0) die("hipBLASLt matmul failed");
            } else {
                SPATHA_OK_OR_DIE(spatha_dense_gemm_f16(dDense, dB, m, kpad, n, dCref, nullptr));
            }
        };
        if (!vg) gemm_impl = "in-tree";
        const int reps = vg ? 100 : 20;
        for (int i = 0; i < (vg ? 10 : 3); i++) run_gemm();
        HIP_OK(hipEventRecord(e0, nullptr));
        for (int i = 0; i < reps; i++) run_gemm();
        HIP_OK(hipEventRecord(e1, nullptr));
        HIP_OK(hipEventSynchronize(e1));
        HIP_OK(hipEventElapsedTime(&gemm_ms, e0, e1));
        gemm_ms /= reps;
        vendor_gemm_destroy(vg);
        if (dCvendor) (void)hipFree(dCvendor);
        HIP_OK(hipEventDestroy(e0));
        HIP_OK(hipEventDestroy(e1));
    }
    if (check) SPATHA_OK_OR_DIE(spatha_dense_gemm_f16(dDense, dB, m, kpad, n, dCref, nullptr));

    int error = 0;
    if (check) {
        std::vector<uint16_t> hC((size_t)m * n), hRef((size_t)m * n);
        HIP_OK(hipMemcpy(hC.data(), dC, hC.size() * 2, hipMemcpyDeviceToHost));
        HIP_OK(hipMemcpy(hRef.data(), dCref, hRef.size() * 2, hipMemcpyDeviceToHost));
        for (size_t i = 0; i < hC.size(); i++) {
            const float a = half_bits_to_float(hC[i]), b = half_bits_to_float(hRef[i]);
            if (std::fabs(a - b) > 1.0f) {      // the reference's acceptance rule, benchmark_spmm.cpp:51-74
                std::fprintf(stderr, "(%zu,%zu): %g vs %g\n", i / n, i % n, a, b);
                error = 1;
                break;
            }
        }
    }

    const double t = spmm_ms * 1e-3;
    const double flops_dense = 2.0 * m * (double)k * n;
    const double flops_sparse = 2.0 * m * (double)n * 2.0 * geo.ksp;
    const double bytes = 2.0 * m * geo.ksp + 4.0 * (m / 2) * (geo.ksp / 8) + 16.0 * (m / V) * (geo.ksp / 2) + 2.0 * k * (double)n +
                         2.0 * m * (double)n;
    std::printf("%d,%s,%d,%d,%d,%d,%d,%d,%d,%g,%d,%d,%d,%d,%d,%d,%d,%d,%d,%d,%g,%g,%g,%d", spmm_code, "gfx950", m, k, n,
                meta_block_sz, block_sz, nn_row, mm_row, (double)density, bm, bn, bk, wm, wn, wk, mm, mn, mk, nstage,
                spmm_ms, gemm_ms, gemm_ms / spmm_ms, error);
    std::printf(",%.3f,%.1f,%.2f,%.1f,%s,%.4f,%d,%s\n", spmm_ms * 1e3, flops_dense / t / 1e12, 100.0 * flops_sparse / t / 5.033e15,
                bytes / t / 1e9, kname, cpu_convert_s, threads, gemm_impl);

    spatha_spmm_plan_destroy(plan);
    for (void* ptr : {(void*)dB, (void*)dC, (void*)dCref, (void*)dVal, (void*)dMeta, (void*)dCols, (void*)dDense}) (void)hipFree(ptr);
    return error ? 2 : 0;
}
