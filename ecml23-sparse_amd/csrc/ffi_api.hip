// extern "C" entry points of libffi_hip.so: argument checks, plan cache, dispatch.
// No arithmetic lives here.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>
#include <climits>
#include <cmath>
#include <cstring>
#include <mutex>
#include <new>
#include <vector>

namespace ffi {

Options g_options;

static thread_local int g_last_hip_error = 0;

int hip_fail(hipError_t e) {
    g_last_hip_error = (int)e;
    (void)hipGetLastError();  // clear the sticky "last error" so later calls are not blamed
    return FFI_ERR_HIP;
}

namespace {

std::mutex g_cache_mutex;
std::vector<ffi_plan*> g_cache;   // plans owned by the library, one per (device, lookup, shape)
constexpr size_t kMaxCachedPlans = 8;

// The reference narrows every size to int32 and fail-fasts otherwise (forward.cu:24-28).
int check_dims(int64_t B, int64_t N, int64_t L, int64_t K, int transposed, Dims* d) {
    if (B <= 0 || N <= 0 || L <= 0 || K <= 0) return FFI_ERR_BAD_SHAPE;
    if (B >= INT32_MAX || N >= INT32_MAX || L >= INT32_MAX || K >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    if (L * K >= INT32_MAX) return FFI_ERR_TOO_LARGE;   // flat connection positions are int32
    d->B = (int)B; d->N = (int)N; d->L = (int)L; d->K = (int)K; d->tp = transposed != 0;
    return FFI_OK;
}

int plan_alloc(int L, int K, int N, ffi_plan** out) {
    ffi_plan* p = new (std::nothrow) ffi_plan();
    if (!p) return FFI_ERR_OUT_OF_MEMORY;
    if (hipGetDevice(&p->device) != hipSuccess) { delete p; return FFI_ERR_NO_DEVICE; }
    p->L = L; p->K = K; p->N = N;
    // the plan arrays themselves are sized and allocated by plan_build
    if (plan_scratch_alloc(p) != FFI_OK) {
        plan_free(p);
        delete p;
        return FFI_ERR_OUT_OF_MEMORY;
    }
    *out = p;
    return FFI_OK;
}

// The cached plan for `lookup`, if there is one (moved to the most-recently-used end).
// Caller holds g_cache_mutex.
ffi_plan* find_cached_plan(const int32_t* lookup, const Dims& d, int dev) {
    for (size_t i = 0; i < g_cache.size(); ++i) {
        ffi_plan* p = g_cache[i];
        if (p->device == dev && p->lookup == lookup && p->L == d.L && p->K == d.K && p->N == d.N) {
            g_cache.erase(g_cache.begin() + i);
            g_cache.push_back(p);
            return p;
        }
    }
    return nullptr;
}

// Builds a plan for a lookup that has none and adds it to the cache.  Caller holds g_cache_mutex.
int create_cached_plan(const int32_t* lookup, const Dims& d, int dev, hipStream_t s, ffi_plan** out) {
    if (g_cache.size() >= kMaxCachedPlans) {
        // evict the least recently used plan of this device; its stream work must have drained
        for (size_t i = 0; i < g_cache.size(); ++i) {
            if (g_cache[i]->device == dev) {
                (void)hipDeviceSynchronize();
                plan_free(g_cache[i]);
                delete g_cache[i];
                g_cache.erase(g_cache.begin() + i);
                break;
            }
        }
    }
    ffi_plan* p = nullptr;
    FFI_TRY(plan_alloc(d.L, d.K, d.N, &p));
    p->batch_hint = d.B;
    int st = plan_build(p, lookup, s);
    if (st != FFI_OK) { plan_free(p); delete p; return st; }
    g_cache.push_back(p);
    *out = p;
    return FFI_OK;
}

// What `between` computes through the plan, for the kernels that redo it when the plan turns out to be outdated
// (all null: nothing).
struct PlannedWeightGrad {
    const float* features = nullptr;
    float* weight_grad = nullptr;
    float* bias_grad = nullptr;
};

// The library's own in-place editors of a lookup matrix (ffi_rewire_f32, ffi_arrange_connections_f32) tell the cache:
// every cached plan built from that buffer on this device is marked outdated on the host, so the next backward call
// rebuilds it before it enqueues anything (no walk of an outdated plan, no recomputing kernels, reproducible sums).
// The device-side check stays for edits the library does not see (foreign kernels writing into the buffer).
void mark_cached_plans_outdated(const int32_t* lookup) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    for (ffi_plan* p : g_cache) {
        if (p->device != dev || p->lookup == nullptr) continue;
        // (an edit anywhere inside the buffer the plan was built from counts)
        const int32_t* end = p->lookup + (size_t)p->L * (size_t)p->K;
        if (lookup >= p->lookup && lookup < end) p->edited_by_library = true;
    }
}

void drop_cached_plan(ffi_plan* p) {
    for (size_t i = 0; i < g_cache.size(); ++i)
        if (g_cache[i] == p) { g_cache.erase(g_cache.begin() + i); break; }
    (void)hipDeviceSynchronize();
    plan_free(p);
    delete p;
}

// Input gradient through the plan cache, with `between(plan)` (the weight-gradient launch, or
// nothing) enqueued ahead of it.  The host never waits in the steady state (the reference's op only
// enqueues, tfsparse/cc/kernels/backward.cu:59-64): the lookup's content is checked against the cached
// plan by a kernel that leaves its verdict on the device; the plan-driven kernels follow -- they read the
// plan, never the lookup, so they are safe whatever the lookup holds now -- and behind them kernels that
// recompute both gradients straight from the lookup if the verdict says the plan is outdated (a rewire),
// and return at once otherwise.  The host looks at the verdict of an earlier call when that has arrived
// (a poll, not a wait) and only then rebuilds the plan, which does synchronise.
template <class Between>
int input_grad_cached(const int32_t* lookup, const float* weights, const float* out_grad, float* feature_grad,
                      const Dims& d, hipStream_t s, Between between, const PlannedWeightGrad& wg = PlannedWeightGrad()) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    ffi_plan* p = find_cached_plan(lookup, d, dev);
    if (!p) {
        FFI_TRY(create_cached_plan(lookup, d, dev, s, &p));
        FFI_TRY(between(p));
        return launch_input_grad(p, weights, out_grad, feature_grad, d.B, d.tp, s);
    }
    bool seen = false, current = true;
    unsigned long long bad = 0;
    FFI_TRY(plan_guard_poll(p, &seen, &current, &bad));
    if (p->edited_by_library || (seen && !current)) {
        // the lookup changed under the plan (the calls since then were served by the recomputing kernels);
        // the build fingerprints the present content, so this call needs no check
        const int st = plan_build(p, lookup, s);
        if (st != FFI_OK) { drop_cached_plan(p); return st; }
        FFI_TRY(between(p));
        return launch_input_grad(p, weights, out_grad, feature_grad, d.B, d.tp, s);
    }
    FFI_TRY(plan_guard_enqueue(p, lookup, s));
    FFI_TRY(between(p));
    bool zeroed = false;
    FFI_TRY(launch_input_grad(p, weights, out_grad, feature_grad, d.B, d.tp, s, p->d_guard + kGuardVerdict, &zeroed));
    return launch_backward_if_outdated(p->d_guard + kGuardVerdict, wg.features, lookup, weights, out_grad, feature_grad,
                                       wg.weight_grad, wg.bias_grad, d, s, zeroed);
}

}  // namespace
}  // namespace ffi

using namespace ffi;

extern "C" {

int ffi_abi_version(void) { return 1; }
const char* ffi_target_arch(void) { return "gfx950"; }
int ffi_last_hip_error(void) { return g_last_hip_error; }

const char* ffi_status_string(int status) {
    switch (status) {
        case FFI_OK: return "ok";
        case FFI_ERR_NULL_POINTER: return "null pointer argument";
        case FFI_ERR_BAD_SHAPE: return "a dimension is <= 0 or shapes disagree";
        case FFI_ERR_TOO_LARGE: return "a size exceeds the 32-bit contract";
        case FFI_ERR_HIP: return "HIP runtime call failed";
        case FFI_ERR_OUT_OF_MEMORY: return "out of memory";
        case FFI_ERR_BAD_LOOKUP: return "lookup holds a column id outside [0, num_features)";
        case FFI_ERR_NO_DEVICE: return "no usable HIP device";
        case FFI_ERR_BAD_ARGUMENT: return "bad argument";
        default: return "unknown status";
    }
}

int ffi_forward_f32(const float* features, const int32_t* lookup, const float* weights, float* result,
                    int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                    int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !result) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    return launch_forward(features, lookup, weights, nullptr, result, d, (hipStream_t)stream);
}

int ffi_forward_bias_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                         float* result, int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                         int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !bias || !result) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    return launch_forward(features, lookup, weights, bias, result, d, (hipStream_t)stream);
}

int ffi_weight_grad_f32(const float* features, const int32_t* lookup, const float* out_grad,
                        float* weight_grad, int64_t batch, int64_t num_features, int64_t num_units,
                        int64_t fan_in, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !out_grad || !weight_grad) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    return launch_weight_grad(features, lookup, out_grad, weight_grad, nullptr, d, (hipStream_t)stream);
}

int ffi_input_grad_f32(const int32_t* lookup, const float* weights, const float* out_grad,
                       float* feature_grad, int64_t batch, int64_t num_features, int64_t num_units,
                       int64_t fan_in, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!lookup || !weights || !out_grad || !feature_grad) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    return input_grad_cached(lookup, weights, out_grad, feature_grad, d, (hipStream_t)stream, [](const ffi_plan*) { return (int)FFI_OK; });
}

int ffi_backward_f32(const float* features, const int32_t* lookup, const float* weights,
                     const float* out_grad, float* feature_grad, float* weight_grad, int64_t batch,
                     int64_t num_features, int64_t num_units, int64_t fan_in, int transposed,
                     ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !out_grad) return FFI_ERR_NULL_POINTER;
    if (!feature_grad && !weight_grad) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    hipStream_t s = (hipStream_t)stream;
    // weight gradient first, then input gradient, as backward.cpp:95-107 orders them
    auto wgrad = [&](const ffi_plan* plan) {
        return weight_grad ? launch_weight_grad(features, lookup, out_grad, weight_grad, nullptr, d, s, plan) : (int)FFI_OK;
    };
    if (!feature_grad) return wgrad(nullptr);
    PlannedWeightGrad wg;
    if (weight_grad) { wg.features = features; wg.weight_grad = weight_grad; }
    return input_grad_cached(lookup, weights, out_grad, feature_grad, d, s, wgrad, wg);
}

int ffi_backward_bias_f32(const float* features, const int32_t* lookup, const float* weights,
                          const float* out_grad, float* feature_grad, float* weight_grad, float* bias_grad,
                          int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed,
                          ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !out_grad || !weight_grad || !bias_grad) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    hipStream_t s = (hipStream_t)stream;
    // the bias gradient (column sums of out_grad) is a by-product of the weight-gradient kernel
    auto wgrad = [&](const ffi_plan* plan) { return launch_weight_grad(features, lookup, out_grad, weight_grad, bias_grad, d, s, plan); };
    if (!feature_grad) return wgrad(nullptr);
    PlannedWeightGrad wg;
    wg.features = features; wg.weight_grad = weight_grad; wg.bias_grad = bias_grad;
    return input_grad_cached(lookup, weights, out_grad, feature_grad, d, s, wgrad, wg);
}

int ffi_forward_bf16_f32(const uint16_t* features, const int32_t* lookup, const uint16_t* weights, float* result,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed,
                         ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !result) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    return launch_forward_bf16(features, lookup, weights, result, d, (hipStream_t)stream);
}

int ffi_forward_topk_bf16(const uint16_t* features, const int32_t* lookup, const uint16_t* weights, float* topk_values,
                          int32_t* topk_indices, int64_t batch, int64_t num_features, int64_t num_units,
                          int64_t fan_in, int k, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !topk_values || !topk_indices) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    return launch_forward_topk_bf16(features, lookup, weights, topk_values, topk_indices, k, d, (hipStream_t)stream);
}

int ffi_topk_f32(const float* scores, int64_t batch, int64_t num_units, int k, float* topk_values, int32_t* topk_indices,
                 ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!scores || !topk_values || !topk_indices) return FFI_ERR_NULL_POINTER;
    if (batch <= 0 || num_units <= 0) return FFI_ERR_BAD_SHAPE;
    if (batch >= INT32_MAX || num_units >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    return launch_topk_f32(scores, (int)batch, (int)num_units, k, topk_values, topk_indices, (hipStream_t)stream);
}

static int check_loss_args(const int64_t* label_indices, int64_t nnz, int loss_kind, int64_t batch, int64_t num_units) {
    if (nnz < 0) return FFI_ERR_BAD_SHAPE;
    if (nnz > 0 && !label_indices) return FFI_ERR_NULL_POINTER;
    if (nnz >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    if (loss_kind != FFI_LOSS_HINGE && loss_kind != FFI_LOSS_SQUARED_HINGE && loss_kind != FFI_LOSS_BCE) return FFI_ERR_BAD_ARGUMENT;
    if (batch <= 0 || num_units <= 0) return FFI_ERR_BAD_SHAPE;
    if (batch >= INT32_MAX || num_units >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    return FFI_OK;
}

int ffi_loss_grad_f32(const float* scores, const int64_t* label_indices, const float* label_values, int64_t nnz,
                      int loss_kind, float grad_scale, float* out_grad, float* loss_sum, uint32_t* nz_words, int64_t batch,
                      int64_t num_units, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!scores || !out_grad) return FFI_ERR_NULL_POINTER;
    FFI_TRY(check_loss_args(label_indices, nnz, loss_kind, batch, num_units));
    const LossArgs la{label_indices, label_values, (int)nnz, loss_kind, grad_scale, loss_sum, nz_words, false};
    return launch_loss_grad(la, scores, out_grad, (int)batch, (int)num_units, (hipStream_t)stream);
}

int ffi_forward_topk_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias, float* scores,
                         float* topk_values, int32_t* topk_indices, int64_t batch, int64_t num_features, int64_t num_units,
                         int64_t fan_in, int k, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !topk_values || !topk_indices) return FFI_ERR_NULL_POINTER;
    if (k < 1 || k > 8) return FFI_ERR_BAD_ARGUMENT;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    const TopkArgs tk{k, topk_values, topk_indices};
    return launch_forward_topk(features, lookup, weights, bias, scores, tk, d, (hipStream_t)stream);
}

int ffi_forward_loss_topk_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                              const int64_t* label_indices, const float* label_values, int64_t nnz, int loss_kind,
                              float grad_scale, float* scores, float* out_grad, float* loss_sum, uint32_t* nz_words,
                              float* topk_values, int32_t* topk_indices, int k, int64_t batch, int64_t num_features,
                              int64_t num_units, int64_t fan_in, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !out_grad || !topk_values || !topk_indices) return FFI_ERR_NULL_POINTER;
    if (scores == out_grad) return FFI_ERR_BAD_ARGUMENT;
    if (k < 1 || k > 8) return FFI_ERR_BAD_ARGUMENT;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    const bool skip = (loss_kind & FFI_LOSS_SKIP_ZERO_STORES) != 0;
    loss_kind &= ~FFI_LOSS_SKIP_ZERO_STORES;
    if (skip && !nz_words) return FFI_ERR_NULL_POINTER;
    FFI_TRY(check_loss_args(label_indices, nnz, loss_kind, batch, num_units));
    const LossArgs la{label_indices, label_values, (int)nnz, loss_kind, grad_scale, loss_sum, nz_words, skip};
    const TopkArgs tk{k, topk_values, topk_indices};
    return launch_forward_loss(features, lookup, weights, bias, la, scores, out_grad, &tk, d, (hipStream_t)stream);
}

int ffi_threshold_metrics_f32(const float* scores, const int64_t* label_indices, const float* label_values, int64_t nnz,
                              float threshold, double* counts, int64_t batch, int64_t num_units, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!scores || !counts) return FFI_ERR_NULL_POINTER;
    FFI_TRY(check_loss_args(label_indices, nnz, FFI_LOSS_HINGE, batch, num_units));
    return launch_threshold_metrics(scores, label_indices, label_values, (int)nnz, threshold, (int)batch, (int)num_units, counts,
                                    (hipStream_t)stream);
}

int ffi_forward_loss_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                         const int64_t* label_indices, const float* label_values, int64_t nnz, int loss_kind,
                         float grad_scale, float* scores, float* out_grad, float* loss_sum, uint32_t* nz_words,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed,
                         ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !out_grad) return FFI_ERR_NULL_POINTER;
    if (scores == out_grad) return FFI_ERR_BAD_ARGUMENT;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    const bool skip = (loss_kind & FFI_LOSS_SKIP_ZERO_STORES) != 0;
    loss_kind &= ~FFI_LOSS_SKIP_ZERO_STORES;
    if (skip && !nz_words) return FFI_ERR_NULL_POINTER;
    FFI_TRY(check_loss_args(label_indices, nnz, loss_kind, batch, num_units));
    const LossArgs la{label_indices, label_values, (int)nnz, loss_kind, grad_scale, loss_sum, nz_words, skip};
    return launch_forward_loss(features, lookup, weights, bias, la, scores, out_grad, nullptr, d, (hipStream_t)stream);
}

int ffi_backward_sparse_f32(const float* features, const int32_t* lookup, const float* weights, float* out_grad,
                            const uint32_t* nz_words, int flags, float max_density, float* feature_grad, float* weight_grad,
                            float* bias_grad, int* sparse_path_taken, int64_t batch, int64_t num_features,
                            int64_t num_units, int64_t fan_in, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !out_grad) return FFI_ERR_NULL_POINTER;
    if (!feature_grad && !weight_grad) return FFI_ERR_NULL_POINTER;
    if (bias_grad && !weight_grad) return FFI_ERR_NULL_POINTER;
    const bool grad_is_partial = (flags & FFI_SPARSE_GRAD_IS_PARTIAL) != 0;
    if (flags & ~(FFI_SPARSE_GRAD_IS_PARTIAL | FFI_SPARSE_DECIDE_FROM_PREVIOUS)) return FFI_ERR_BAD_ARGUMENT;
    if (grad_is_partial && !nz_words) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    hipStream_t s = (hipStream_t)stream;
    const unsigned* words = nullptr;
    unsigned long long set_bits = 0;
    FFI_TRY(nonzero_count(out_grad, nz_words, d.B, d.L, s, (flags & FFI_SPARSE_DECIDE_FROM_PREVIOUS) != 0, &words, &set_bits));
    const double limit = (double)(max_density > 0.f ? max_density : kSparseDefaultMaxDensity) * (double)d.B * (double)d.L;
    const bool sparse = (double)set_bits <= limit && sparse_weight_grad_fits(d.B, d.N);
    if (sparse_path_taken) *sparse_path_taken = sparse ? 1 : 0;
    // the dense kernels read all of out_grad
    if (!sparse && grad_is_partial) FFI_TRY(launch_zero_unmasked(out_grad, words, d.B, d.L, s));
    auto wgrad = [&](const ffi_plan* plan) {
        if (!weight_grad) return (int)FFI_OK;
        if (sparse) return launch_weight_grad_sparse(features, lookup, out_grad, words, weight_grad, bias_grad, nullptr, d, s);
        return launch_weight_grad(features, lookup, out_grad, weight_grad, bias_grad, d, s, plan);
    };
    if (!feature_grad) return wgrad(nullptr);
    if (sparse && sparse_input_grad_fits(d.N, d.K)) {
        FFI_TRY(wgrad(nullptr));
        return launch_input_grad_sparse(lookup, weights, out_grad, words, feature_grad, d, s);
    }
    PlannedWeightGrad wg;                                  // (the sparse weight gradient reads the lookup itself)
    if (weight_grad && !sparse) { wg.features = features; wg.weight_grad = weight_grad; wg.bias_grad = bias_grad; }
    return input_grad_cached(lookup, weights, out_grad, feature_grad, d, s, wgrad, wg);
}

int ffi_adam_step_f32(float* variable, float* m, float* v, const float* gradient, int64_t count, float learning_rate,
                      float beta_1, float beta_2, float epsilon, int64_t step, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!variable || !m || !v || !gradient) return FFI_ERR_NULL_POINTER;
    if (count <= 0) return FFI_ERR_BAD_SHAPE;
    if (step < 1) return FFI_ERR_BAD_ARGUMENT;
    return launch_adam_step(variable, m, v, gradient, (size_t)count, learning_rate, beta_1, beta_2, epsilon, (long long)step,
                            (hipStream_t)stream);
}

int ffi_backward_sparse_adam_f32(const float* features, const int32_t* lookup, float* weights, float* out_grad,
                                 const uint32_t* nz_words, int flags, float max_density, float* feature_grad,
                                 float* weight_m, float* weight_v, float* bias, float* bias_m, float* bias_v,
                                 float learning_rate, float beta_1, float beta_2, float epsilon, int64_t step,
                                 int* sparse_path_taken, int64_t batch, int64_t num_features, int64_t num_units,
                                 int64_t fan_in, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !out_grad || !weight_m || !weight_v) return FFI_ERR_NULL_POINTER;
    if (bias && (!bias_m || !bias_v)) return FFI_ERR_NULL_POINTER;
    const bool grad_is_partial = (flags & FFI_SPARSE_GRAD_IS_PARTIAL) != 0;
    if (flags & ~(FFI_SPARSE_GRAD_IS_PARTIAL | FFI_SPARSE_DECIDE_FROM_PREVIOUS)) return FFI_ERR_BAD_ARGUMENT;
    if (grad_is_partial && !nz_words) return FFI_ERR_NULL_POINTER;
    if (step < 1) return FFI_ERR_BAD_ARGUMENT;
    Dims d;
    FFI_TRY(check_dims(batch, num_features, num_units, fan_in, transposed, &d));
    hipStream_t s = (hipStream_t)stream;
    const unsigned* words = nullptr;
    unsigned long long set_bits = 0;
    FFI_TRY(nonzero_count(out_grad, nz_words, d.B, d.L, s, (flags & FFI_SPARSE_DECIDE_FROM_PREVIOUS) != 0, &words, &set_bits));
    const double limit = (double)(max_density > 0.f ? max_density : kSparseDefaultMaxDensity) * (double)d.B * (double)d.L;
    const bool sparse = (double)set_bits <= limit && sparse_weight_grad_fits(d.B, d.N);
    if (sparse_path_taken) *sparse_path_taken = sparse ? 1 : 0;
    // the gradients live in a workspace: [L*K] weight gradient (16-byte aligned end), [L] bias gradient, [L] row flags
    const size_t wcount = (size_t)d.L * d.K;
    const size_t bias_at = (wcount + 3) / 4 * 4;
    float* grads = nullptr;
    FFI_TRY(workspace_get(s, kWsGradients, (bias_at + (size_t)d.L) * sizeof(float) + (size_t)d.L, (void**)&grads));
    float* gw = grads;
    float* gb = bias ? grads + bias_at : nullptr;
    unsigned char* active = reinterpret_cast<unsigned char*>(grads + bias_at + d.L);
    if (sparse) {
        // the weight gradient of labels without a non-zero out_grad entry is neither written nor read: the Adam
        // pass takes a zero for them
        FFI_TRY(launch_weight_grad_sparse(features, lookup, out_grad, words, gw, gb, active, d, s));
        if (feature_grad) {
            if (sparse_input_grad_fits(d.N, d.K)) {
                FFI_TRY(launch_input_grad_sparse(lookup, weights, out_grad, words, feature_grad, d, s));
            } else {
                FFI_TRY(input_grad_cached(lookup, weights, out_grad, feature_grad, d, s, [](const ffi_plan*) { return (int)FFI_OK; }));
            }
        }
        FFI_TRY(launch_adam_step_rows(weights, weight_m, weight_v, gw, active, d.L, d.K, learning_rate, beta_1, beta_2, epsilon,
                                      (long long)step, s));
        if (bias) FFI_TRY(launch_adam_step(bias, bias_m, bias_v, gb, (size_t)d.L, learning_rate, beta_1, beta_2, epsilon, (long long)step, s));
        return FFI_OK;
    }
    // dense kernels: gradients into a workspace, then the Adam pass
    if (grad_is_partial) FFI_TRY(launch_zero_unmasked(out_grad, words, d.B, d.L, s));
    auto wgrad = [&](const ffi_plan* plan) { return launch_weight_grad(features, lookup, out_grad, gw, gb, d, s, plan); };
    PlannedWeightGrad wg;
    wg.features = features; wg.weight_grad = gw; wg.bias_grad = gb;
    if (feature_grad) FFI_TRY(input_grad_cached(lookup, weights, out_grad, feature_grad, d, s, wgrad, wg));
    else FFI_TRY(wgrad(nullptr));
    FFI_TRY(launch_adam_step(weights, weight_m, weight_v, gw, wcount, learning_rate, beta_1, beta_2, epsilon, (long long)step, s));
    if (bias) FFI_TRY(launch_adam_step(bias, bias_m, bias_v, gb, (size_t)d.L, learning_rate, beta_1, beta_2, epsilon, (long long)step, s));
    return FFI_OK;
}

int ffi_select_threshold_f32(const float* weights, int64_t count, int64_t k, float* threshold, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!weights || !threshold) return FFI_ERR_NULL_POINTER;
    if (count <= 0) return FFI_ERR_BAD_SHAPE;
    if (k < 0 || k > count) return FFI_ERR_BAD_ARGUMENT;
    return launch_select_threshold(weights, (size_t)count, (unsigned long long)k, threshold, (hipStream_t)stream);
}

int ffi_rewire_f32(int32_t* lookup, const float* weights, float* const* arrays, int n_arrays, int64_t count,
                   int64_t num_features, const float* threshold, uint64_t seed, int64_t* rewired_count, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!lookup || !weights || !threshold || (n_arrays > 0 && !arrays)) return FFI_ERR_NULL_POINTER;
    if (n_arrays < 0 || n_arrays > 4) return FFI_ERR_BAD_ARGUMENT;
    for (int i = 0; i < n_arrays; ++i)
        if (!arrays[i]) return FFI_ERR_NULL_POINTER;
    if (count <= 0 || num_features <= 0) return FFI_ERR_BAD_SHAPE;
    if (num_features >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    mark_cached_plans_outdated(lookup);
    return launch_rewire(lookup, weights, arrays, n_arrays, (size_t)count, (unsigned)num_features, threshold,
                         (unsigned long long)seed, (long long*)rewired_count, (hipStream_t)stream);
}

int ffi_plan_create(const int32_t* lookup, int64_t num_units, int64_t fan_in, int64_t num_features,
                    int64_t batch_hint, ffi_stream_t stream, ffi_plan** plan) {
    StreamCall call_lock((hipStream_t)stream);
    if (!lookup || !plan) return FFI_ERR_NULL_POINTER;
    *plan = nullptr;
    Dims d;
    FFI_TRY(check_dims(batch_hint > 0 ? batch_hint : 1, num_features, num_units, fan_in, 0, &d));
    ffi_plan* p = nullptr;
    FFI_TRY(plan_alloc(d.L, d.K, d.N, &p));
    p->batch_hint = batch_hint > 0 ? d.B : 0;
    int st = plan_build(p, lookup, (hipStream_t)stream);
    if (st != FFI_OK) { plan_free(p); delete p; return st; }
    *plan = p;
    return FFI_OK;
}

int ffi_plan_refresh(ffi_plan* plan, const int32_t* lookup, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!plan || !lookup) return FFI_ERR_NULL_POINTER;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    if (dev != plan->device) return FFI_ERR_BAD_ARGUMENT;
    return plan_build(plan, lookup, (hipStream_t)stream);
}

int ffi_plan_destroy(ffi_plan* plan) {
    if (!plan) return FFI_OK;
    plan_free(plan);
    delete plan;
    return FFI_OK;
}

int ffi_plan_info(const ffi_plan* plan, int64_t info[8]) {
    if (!plan || !info) return FFI_ERR_NULL_POINTER;
    info[0] = plan->tiled ? 1 : 0;
    info[1] = plan->w_in_lds ? 1 : 0;
    info[2] = plan->tile_labels;
    info[3] = plan->threads;
    info[4] = plan->tiles;
    info[5] = plan->total_rows + (plan->upper ? plan->upper->total_rows : 0);   // (both column windows of a wide input)
    info[6] = (int64_t)plan->bytes;
    info[7] = plan->idx16 != nullptr ? 1 : 0;
    return FFI_OK;
}

int ffi_input_grad_planned_f32(const ffi_plan* plan, const float* weights, const float* out_grad,
                               float* feature_grad, int64_t batch, int transposed, ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!plan || !weights || !out_grad || !feature_grad) return FFI_ERR_NULL_POINTER;
    if (batch <= 0) return FFI_ERR_BAD_SHAPE;
    if (batch >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    if (dev != plan->device) return FFI_ERR_BAD_ARGUMENT;
    return launch_input_grad(plan, weights, out_grad, feature_grad, (int)batch, transposed != 0, (hipStream_t)stream);
}

int ffi_weight_grad_planned_f32(const ffi_plan* plan, const float* features, const int32_t* lookup,
                                const float* out_grad, float* weight_grad, int64_t batch, int transposed,
                                ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!plan || !features || !lookup || !out_grad || !weight_grad) return FFI_ERR_NULL_POINTER;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    if (dev != plan->device) return FFI_ERR_BAD_ARGUMENT;
    Dims d;
    FFI_TRY(check_dims(batch, plan->N, plan->L, plan->K, transposed, &d));
    return launch_weight_grad(features, lookup, out_grad, weight_grad, nullptr, d, (hipStream_t)stream, plan);
}

int ffi_arrange_connections_f32(int32_t* lookup, float* const* arrays, int n_arrays, int64_t num_units, int64_t fan_in,
                                ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!lookup || (n_arrays > 0 && !arrays)) return FFI_ERR_NULL_POINTER;
    if (n_arrays < 0 || n_arrays > 4) return FFI_ERR_BAD_ARGUMENT;
    for (int i = 0; i < n_arrays; ++i)
        if (!arrays[i]) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(1, 1, num_units, fan_in, 0, &d));
    mark_cached_plans_outdated(lookup);
    return launch_arrange_in_place(lookup, arrays, n_arrays, d.L, d.K, (hipStream_t)stream);
}

int ffi_lookup_edited(const int32_t* lookup) {
    if (!lookup) return FFI_ERR_NULL_POINTER;
    mark_cached_plans_outdated(lookup);
    return FFI_OK;
}

int ffi_cache_clear(void) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    (void)hipDeviceSynchronize();
    for (size_t i = 0; i < g_cache.size();) {
        if (g_cache[i]->device == dev) {
            plan_free(g_cache[i]);
            delete g_cache[i];
            g_cache.erase(g_cache.begin() + i);
        } else {
            ++i;
        }
    }
    workspace_clear(dev);
    nonzero_count_forget(dev);
    return FFI_OK;
}

int ffi_set_option(const char* name, int value) {
    if (name == nullptr) return FFI_ERR_BAD_ARGUMENT;
    static const struct { const char* name; int ffi::Options::*field; int lo, hi; } table[] = {
        {"wgrad_units", &ffi::Options::wgrad_units, 0, 4},
        {"wgrad_stream", &ffi::Options::wgrad_stream, -1, 0},
        {"fwd_lane64", &ffi::Options::fwd_lane64, -1, 0},
        {"plan_weights_in_lds", &ffi::Options::plan_weights_in_lds, -1, 1},
        {"workgroups_per_cu", &ffi::Options::workgroups_per_cu, 0, 16},
        {"plan_sorted_columns", &ffi::Options::plan_sorted_columns, -1, 1},
    };
    for (const auto& t : table) {
        if (std::strcmp(name, t.name) != 0) continue;
        if (value < t.lo || value > t.hi || (t.field == &ffi::Options::wgrad_units && value != 0 && value != 3 && value != 4))
            return FFI_ERR_BAD_ARGUMENT;
        // cached plans were laid out under the old choice
        const int status = ffi_cache_clear();
        if (status != FFI_OK && status != FFI_ERR_NO_DEVICE) return status;
        ffi::g_options.*(t.field) = value;
        return FFI_OK;
    }
    return FFI_ERR_BAD_ARGUMENT;
}

size_t ffi_cache_bytes(void) {
    std::lock_guard<std::mutex> lock(g_cache_mutex);
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return 0;
    size_t total = 0;
    for (ffi_plan* p : g_cache)
        if (p->device == dev) total += p->bytes;
    return total + workspace_bytes(dev);
}

size_t ffi_workspace_bytes(int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed, int passes) {
    Dims d;
    if (check_dims(batch, num_features, num_units, fan_in, transposed, &d) != FFI_OK) return 0;
    const size_t B = (size_t)d.B, N = (size_t)d.N, L = (size_t)d.L, K = (size_t)d.K;
    const bool narrow = tile_path_fits(d.N) && d.L < (1 << 25);
    const size_t ldw = (B + 31) / 32 * 32;                         // row stride of the wide kernels' own copies
    // the batch-major copy of the features (one slot, shared by the passes and by the permuted weights below)
    size_t features_slot = 0;
    if (narrow) features_slot = d.tp ? 0 : N * B * 4;
    else features_slot = (d.tp && ldw == B) ? 0 : N * ldw * 4;
    size_t total = 0, partial_slot = 0;
    if (passes & FFI_PASS_BACKWARD) {
        const bool one_window = d.N <= 1024, two_windows = !one_window && tile_path_fits(d.N) && d.N <= 2048;
        if ((one_window || two_windows) && d.K <= 1024 && d.L < (1 << 25)) {
            // tiled plan: the geometry of ffi_plan.hip, the slot rows of a slice estimated for column ids drawn uniformly
            // (longest of 64 columns whose lengths scatter like Poisson counts around tile_labels * fan_in / num_features);
            // inputs wider than 1,024 columns have one such form per half of the columns, walked one after the other
            const size_t lower = one_window ? N : ((N + 1) / 2 + 63) / 64 * 64;
            for (int win = 0; win < (one_window ? 1 : 2); ++win) {
                const size_t cols = win == 0 ? lower : N - lower;
                const size_t threads = (cols + 63) / 64 * 64;
                bool w_in_lds = false;
                const size_t TL = (size_t)plan_tile_labels((int)cols, d.K, d.L, d.B, &w_in_lds);
                const size_t tiles = (L + TL - 1) / TL, slices = threads / 64;
                const double mu = (double)TL * (double)K / (double)N;
                // (plans that sort a tile's columns by length: a slice's rows are those of columns about equally long)
                const bool sorted = plan_sorts_columns((int)threads, (int)TL, d.K, w_in_lds, (int)tiles, d.B);
                const size_t rows = sorted ? (size_t)(mu + 0.75 * std::sqrt(mu) + 1.0) : (size_t)(mu + 2.6 * std::sqrt(mu) + 3.0);
                const size_t slots = tiles * slices * rows * 64;
                total += slots * 2 * 2 + (tiles * slices + 1) * 4 + L * 2;              // 4 bytes per slot (lab16 + pos16, or slot32), slice_off, rowpos
                if (sorted) total += tiles * threads * 2;                               // the column of each thread in each tile
                if (!w_in_lds) features_slot = std::max(features_slot, slots * 4);     // weights in slot order
                const size_t nbt = (B + 31) / 32;
                const size_t per_cu = (size_t)tiled_workgroups_per_cu((int)threads, (int)TL, d.K, w_in_lds, (int)((B + 31) / 32));
                size_t streams = std::max<size_t>(1, std::min<size_t>(tiles, per_cu * (size_t)device_cu_count() / std::max<size_t>(1, nbt)));
                const size_t tiles_per_stream = (tiles + streams - 1) / streams;        // (as the launcher evens them out)
                streams = (tiles + tiles_per_stream - 1) / tiles_per_stream;
                partial_slot = std::max(partial_slot, streams * threads * nbt * 32 * 4);
            }
            if (tile_path_fits(d.N) && d.N < (1 << kArrIdBits)) total += arranged_words((long long)(L * ((K + 31) / 32))) * 2;   // idx16
        } else {
            const size_t nblocks = (L + 65535) / 65536;
            total += L * K * 4 + (nblocks * N + 1) * 4;                                 // perm, col_ptr
            partial_slot = L * ldw * 4;                                                 // out_grad, batch-major
            if (!d.tp) features_slot = std::max(features_slot, N * B * 4);
        }
    }
    return total + features_slot + partial_slot;
}

int ffi_check_lookup(const int32_t* lookup, int64_t num_units, int64_t fan_in, int64_t num_features,
                     ffi_stream_t stream) {
    StreamCall call_lock((hipStream_t)stream);
    if (!lookup) return FFI_ERR_NULL_POINTER;
    Dims d;
    FFI_TRY(check_dims(1, num_features, num_units, fan_in, 0, &d));
    ffi_plan tmp;
    tmp.L = d.L; tmp.K = d.K; tmp.N = d.N;
    if (plan_scratch_alloc(&tmp) != FFI_OK) {
        plan_free(&tmp);
        return FFI_ERR_OUT_OF_MEMORY;
    }
    unsigned long long fp = 0, bad = 0;
    int st = plan_fingerprint(&tmp, lookup, (hipStream_t)stream, &fp, &bad);
    plan_free(&tmp);
    if (st != FFI_OK) return st;
    return bad ? FFI_ERR_BAD_LOOKUP : FFI_OK;
}

}  // extern "C"
