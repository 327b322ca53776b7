// PyTorch C++ extension for the operator (end2end/spatha_mod/block_sparse/api/spatha.cu:41-65 in the reference:
// `spmm(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, B_num_cols, vec_length, n, m, nnz,
// seed, mbrow, brow) -> Tensor`, bound with pybind11 under the name `spmm`).  Same argument order and meaning; the work
// itself goes through the C ABI of include/spatha.h on torch's current HIP stream.  Written against the ROCm build of
// PyTorch directly (c10/hip, ATen/hip), not passed through a source translator.
//
// The reference packs nothing per call (its kernel reads the canonical arrays); here the derived operand copies live
// in a plan, so the extension keeps a cache of plans keyed by the identity and version of the three weight tensors.
// An entry holds the tensors, so an address cannot be recycled under a stale plan.  A plan is held through a shared_ptr whose
// deleter destroys it: a launch keeps its own reference, so an eviction or clear_plan_cache() from another thread cannot
// free the plan's device buffers under a launch that is being enqueued.  An in-place update of the weights bumps the tensors'
// version: the miss that follows drops the entries of the same three addresses with an older version, so a loop that
// re-sparsifies in place keeps one plan per matrix.  A write that torch does not see (through `.data` or a raw pointer)
// leaves the version alone: call invalidate_plans(values) or clear_plan_cache() after one.

#include <torch/extension.h>

#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>

#include <list>
#include <map>
#include <memory>
#include <mutex>
#include <stdexcept>
#include <string>
#include <tuple>
#include <unordered_map>

#include "../../include/spatha.h"

namespace {

struct PlanKey {
    const void *values, *metadata, *columns;
    uint32_t v_values, v_metadata, v_columns;
    int rows, cols, n, m, v, device;
    bool operator==(const PlanKey& o) const {
        return values == o.values && metadata == o.metadata && columns == o.columns && v_values == o.v_values &&
               v_metadata == o.v_metadata && v_columns == o.v_columns && rows == o.rows && cols == o.cols && n == o.n &&
               m == o.m && v == o.v && device == o.device;
    }
};
struct PlanKeyHash {
    size_t operator()(const PlanKey& k) const {
        size_t h = std::hash<const void*>()(k.values);
        auto mix = [&h](size_t x) { h ^= x + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2); };
        mix(std::hash<const void*>()(k.metadata));
        mix(std::hash<const void*>()(k.columns));
        mix(((size_t)k.v_values << 32) ^ ((size_t)k.v_metadata << 16) ^ k.v_columns);
        mix(((size_t)k.rows << 32) ^ (size_t)k.cols);
        mix(((size_t)k.m << 40) ^ ((size_t)k.v << 20) ^ ((size_t)k.n << 8) ^ (size_t)k.device);
        return h;
    }
};
struct PlanEntry {
    PlanKey key;
    std::shared_ptr<spatha_spmm_plan> plan;
    torch::Tensor values, metadata, columns;      // kept alive for the plan's lifetime
};

constexpr size_t kMaxPlans = 1024;
std::mutex g_lock;
std::list<PlanEntry> g_lru;                                                           // most recently used first
std::unordered_map<PlanKey, std::list<PlanEntry>::iterator, PlanKeyHash> g_index;

void check(int status, const char* what) {
    if (status != SPATHA_OK)
        throw std::runtime_error(std::string(what) + ": " + spatha_status_string(status) +
                                 (status == SPATHA_ERR_HIP ? " (HIP error " + std::to_string(spatha_last_hip_error()) + ")" : ""));
}

// Scratch memory of split runs (spatha_spmm_run_ws): one zero-initialised buffer per (device, stream), grown on demand.
// Calls on one stream are ordered, so they can share it; the library leaves it clean after every completed call.
std::map<std::pair<int, hipStream_t>, torch::Tensor> g_workspaces;

torch::Tensor workspace_for(int device, hipStream_t stream, size_t bytes, const torch::TensorOptions& like) {
    std::lock_guard<std::mutex> guard(g_lock);
    torch::Tensor& ws = g_workspaces[{device, stream}];
    if (!ws.defined() || (size_t)ws.numel() < bytes) ws = torch::zeros({(int64_t)bytes}, like.dtype(torch::kUInt8));
    return ws;
}

void check_weight(const torch::Tensor& t, c10::ScalarType a, c10::ScalarType b, const char* name) {
    TORCH_CHECK(t.is_cuda(), name, " must live on the GPU");
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
    TORCH_CHECK(t.scalar_type() == a || t.scalar_type() == b, name, " has the wrong dtype");
}

uint32_t version_of(const torch::Tensor& t) { return (uint32_t)t.unsafeGetTensorImpl()->version_counter().current_version(); }

bool same_storage(const PlanKey& a, const PlanKey& b) {
    return a.values == b.values && a.metadata == b.metadata && a.columns == b.columns && a.device == b.device;
}

// (g_lock held) drops every entry for which `stale` holds; launches that still hold a reference keep their plan alive
template <class Pred>
void drop_entries(Pred stale) {
    for (auto it = g_lru.begin(); it != g_lru.end();) {
        if (stale(*it)) {
            g_index.erase(it->key);
            it = g_lru.erase(it);
        } else {
            ++it;
        }
    }
}

std::shared_ptr<spatha_spmm_plan> plan_for(const torch::Tensor& values, const torch::Tensor& metadata, const torch::Tensor& columns, int rows,
                           int cols, int n, int m, int v, hipStream_t stream) {
    PlanKey key{values.data_ptr(), metadata.data_ptr(), columns.data_ptr(), version_of(values), version_of(metadata),
                version_of(columns), rows, cols, n, m, v, (int)values.get_device()};
    std::lock_guard<std::mutex> guard(g_lock);
    auto hit = g_index.find(key);
    if (hit != g_index.end()) {
        g_lru.splice(g_lru.begin(), g_lru, hit->second);
        return hit->second->plan;
    }
    spatha_spmm_plan* raw = nullptr;
    check(spatha_spmm_plan_create(rows, cols, n, m, v, (const uint16_t*)values.data_ptr(), (const uint32_t*)metadata.data_ptr(),
                                  (const uint32_t*)columns.data_ptr(), stream, &raw),
          "spatha_spmm_plan_create");
    std::shared_ptr<spatha_spmm_plan> plan(raw, [](spatha_spmm_plan* p) { spatha_spmm_plan_destroy(p); });
    // the same three tensors at another version: the weights were rewritten in place, those plans are stale
    drop_entries([&key](const PlanEntry& e) { return same_storage(e.key, key); });
    g_lru.push_front(PlanEntry{key, plan, values, metadata, columns});
    g_index[key] = g_lru.begin();
    while (g_lru.size() > kMaxPlans) {
        g_index.erase(g_lru.back().key);
        g_lru.pop_back();
    }
    return plan;
}

torch::Tensor run(const torch::Tensor& A_metadata, const torch::Tensor& A_indices, const torch::Tensor& A_values,
                  const torch::Tensor& rhs_matrix, const c10::optional<torch::Tensor>& bias, int rows, int cols, int v, int n, int m,
                  bool transposed_out, int activation, bool fused) {
    check_weight(A_values, torch::kFloat16, torch::kFloat16, "A_values");
    check_weight(A_metadata, torch::kInt32, torch::kInt32, "A_metadata");
    check_weight(A_indices, torch::kInt32, torch::kInt32, "A_indices");
    check_weight(rhs_matrix, torch::kFloat16, torch::kFloat16, "rhs_matrix");
    TORCH_CHECK(rhs_matrix.dim() == 2 && rhs_matrix.size(0) == cols, "rhs_matrix must be [A_num_cols, tokens]");
    TORCH_CHECK(rhs_matrix.get_device() == A_values.get_device(), "operands live on different devices");
    const uint16_t* bias_ptr = nullptr;
    if (bias.has_value() && bias->defined()) {
        check_weight(*bias, torch::kFloat16, torch::kFloat16, "bias");
        TORCH_CHECK(bias->numel() == rows, "bias must have A_num_rows elements");
        bias_ptr = (const uint16_t*)bias->data_ptr();
    }
    const int tokens = (int)rhs_matrix.size(1);
    const c10::hip::HIPGuardMasqueradingAsCUDA device_guard(A_values.device());
    if (tokens % 8 != 0 && tokens > 0) {
        // The library moves rows of B and C in 16-byte pieces: a token count that is no multiple of 8 runs on a copy of
        // rhs_matrix with zero columns appended, and the result is cut back (the appended columns give bias-only rows /
        // columns, which are dropped).
        const int pad = 8 - tokens % 8;
        torch::Tensor padded = torch::constant_pad_nd(rhs_matrix, {0, pad}, 0);
        torch::Tensor full = run(A_metadata, A_indices, A_values, padded, bias, rows, cols, v, n, m, transposed_out, activation, fused);
        return transposed_out ? full.narrow(0, 0, tokens) : full.narrow(1, 0, tokens).contiguous();
    }
    hipStream_t stream = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(A_values.get_device()).stream();
    // (this reference outlives the launch calls below, whatever another thread does to the cache meanwhile)
    const std::shared_ptr<spatha_spmm_plan> plan = plan_for(A_values.detach(), A_metadata, A_indices, rows, cols, n, m, v, stream);
    torch::Tensor out = torch::empty(transposed_out ? std::vector<int64_t>{tokens, rows} : std::vector<int64_t>{rows, tokens},
                                     rhs_matrix.options());
    const int layout = transposed_out ? SPATHA_OUT_TRANSPOSED : SPATHA_OUT_ROW_MAJOR;
    // few tokens against a long k-loop: the library splits the k-loops over workgroups if it is given scratch memory
    const bool fuses = fused && (activation != SPATHA_ACT_NONE || (!transposed_out && bias_ptr));
    if (const size_t need = spatha_spmm_workspace_bytes(plan.get(), tokens, layout, fuses ? 1 : 0)) {
        torch::Tensor ws = workspace_for((int)A_values.get_device(), stream, need, rhs_matrix.options());
        check(spatha_spmm_run_ws(plan.get(), (const uint16_t*)rhs_matrix.data_ptr(), tokens, bias_ptr, (uint16_t*)out.data_ptr(), layout,
                                 fused ? activation : SPATHA_ACT_NONE, ws.data_ptr(), (size_t)ws.numel(), stream),
              "spatha_spmm_run_ws");
        return out;
    }
    if (fused)
        check(spatha_spmm_run_fused(plan.get(), (const uint16_t*)rhs_matrix.data_ptr(), tokens, bias_ptr, (uint16_t*)out.data_ptr(), layout,
                                    activation, 0, stream),
              "spatha_spmm_run_fused");
    else
        check(spatha_spmm_run(plan.get(), (const uint16_t*)rhs_matrix.data_ptr(), tokens, bias_ptr, (uint16_t*)out.data_ptr(), layout, 0,
                              stream),
              "spatha_spmm_run");
    return out;
}

// out[B_num_cols, A_num_rows] = (A_vnm @ rhs_matrix).T + bias, fp16: the reference operator.  vec_length is V and is
// honoured at run time; nnz and seed are accepted and unused, as there; mbrow / brow must be 32 / 4, the only layout the
// format defines.
torch::Tensor spmm(torch::Tensor A_metadata, torch::Tensor A_indices, torch::Tensor A_values, torch::Tensor rhs_matrix,
                   c10::optional<torch::Tensor> bias, int A_num_rows, int A_num_cols, int B_num_cols, int vec_length, int n, int m,
                   int nnz, int seed, int mbrow, int brow) {
    (void)nnz;
    (void)seed;
    TORCH_CHECK(mbrow == 32 && brow == 4, "only mbrow=32, brow=4 is defined for the V:N:M layout");
    TORCH_CHECK(rhs_matrix.dim() == 2 && rhs_matrix.size(1) == B_num_cols, "B_num_cols does not match rhs_matrix");
    return run(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, vec_length, n, m, true, SPATHA_ACT_NONE,
               false);
}

// act((A_vnm @ rhs_matrix) + bias) as [A_num_rows, tokens] (ready to be the rhs of the next spmm) or, with
// transposed_out, as [tokens, A_num_rows]; activation: 0 none, 1 GELU (erf), 2 GELU (tanh)
torch::Tensor spmm_fused(torch::Tensor A_metadata, torch::Tensor A_indices, torch::Tensor A_values, torch::Tensor rhs_matrix,
                         c10::optional<torch::Tensor> bias, int A_num_rows, int A_num_cols, int vec_length, int n, int m,
                         int activation, bool transposed_out) {
    return run(A_metadata, A_indices, A_values, rhs_matrix, bias, A_num_rows, A_num_cols, vec_length, n, m, transposed_out,
               activation, true);
}

void clear_plan_cache() {
    std::lock_guard<std::mutex> guard(g_lock);
    g_lru.clear();
    g_index.clear();
    g_workspaces.clear();
}

// Drops the plans built from this values tensor (any version): for weights changed behind torch's back.
int64_t invalidate_plans(const torch::Tensor& A_values) {
    std::lock_guard<std::mutex> guard(g_lock);
    const size_t before = g_lru.size();
    const void* ptr = A_values.data_ptr();
    drop_entries([ptr](const PlanEntry& e) { return e.key.values == ptr; });
    return (int64_t)(before - g_lru.size());
}

int64_t plan_cache_size() {
    std::lock_guard<std::mutex> guard(g_lock);
    return (int64_t)g_lru.size();
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, mod) {
    mod.def("spmm", &spmm, "V:N:M SpMM: (A_vnm @ rhs).T + bias", py::arg("A_metadata"), py::arg("A_indices"), py::arg("A_values"),
            py::arg("rhs_matrix"), py::arg("bias"), py::arg("A_num_rows"), py::arg("A_num_cols"), py::arg("B_num_cols"),
            py::arg("vec_length"), py::arg("n"), py::arg("m"), py::arg("nnz") = 0, py::arg("seed") = 0, py::arg("mbrow") = 32,
            py::arg("brow") = 4);
    mod.def("spmm_fused", &spmm_fused, "V:N:M SpMM with bias and activation in the write-out", py::arg("A_metadata"),
            py::arg("A_indices"), py::arg("A_values"), py::arg("rhs_matrix"), py::arg("bias"), py::arg("A_num_rows"),
            py::arg("A_num_cols"), py::arg("vec_length"), py::arg("n"), py::arg("m"), py::arg("activation") = 0,
            py::arg("transposed_out") = false);
    mod.def("clear_plan_cache", &clear_plan_cache, "drop every cached plan");
    mod.def("invalidate_plans", &invalidate_plans, "drop the cached plans built from this values tensor; returns how many",
            py::arg("A_values"));
    mod.def("plan_cache_size", &plan_cache_size, "number of cached plans");
}
