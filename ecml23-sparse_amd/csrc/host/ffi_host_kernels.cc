// Host (CPU) implementation of the fixed-fan-in sparse layer, for the DEVICE_CPU kernels of the TensorFlow op library
// (tf/ffi_tf_cpu_ops.cc): the reference registers CPU kernels for all four ops (tfsparse/cc/kernels/register.cpp:79-80,
// 88-89,97-98,106-107) and a drop-in must serve a CPU placement too.  Plain loops over HOST pointers with the
// semantics of tfsparse/cc/kernels/forward.cpp:9-44 and backward.cpp:8-73; rows are split over the caller's threads
// by the caller (begin / end ranges), nothing here starts a thread.  Not a fallback of the GPU entry points: those
// never run on the CPU.
#include "ffi_hip.h"

#include <cstddef>
#include <cstdint>

namespace {

struct HostDims { int64_t B, N, L, K; bool tp; };

int check(int64_t B, int64_t N, int64_t L, int64_t K) {
    if (B <= 0 || N <= 0 || L <= 0 || K <= 0) return FFI_ERR_BAD_SHAPE;
    if (B >= INT32_MAX || N >= INT32_MAX || L >= INT32_MAX || K >= INT32_MAX || L * K >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    return FFI_OK;
}

inline float feature(const float* x, const HostDims& d, int64_t b, int64_t n) { return d.tp ? x[n * d.B + b] : x[b * d.N + n]; }

}  // namespace

extern "C" {

int ffi_host_forward_f32(const float* features, const int32_t* lookup, const float* weights, float* result, int64_t batch,
                         int64_t num_features, int64_t num_units, int64_t fan_in, int transposed, int64_t unit_begin,
                         int64_t unit_end) {
    if (!features || !lookup || !weights || !result) return FFI_ERR_NULL_POINTER;
    const int st = check(batch, num_features, num_units, fan_in);
    if (st != FFI_OK) return st;
    if (unit_begin < 0 || unit_end > num_units || unit_begin > unit_end) return FFI_ERR_BAD_ARGUMENT;
    const HostDims d{batch, num_features, num_units, fan_in, transposed != 0};
    for (int64_t j = unit_begin; j < unit_end; ++j) {
        const int32_t* ids = lookup + j * d.K;
        const float* w = weights + j * d.K;
        for (int64_t k = 0; k < d.K; ++k)
            if ((uint32_t)ids[k] >= (uint64_t)d.N) return FFI_ERR_BAD_LOOKUP;
        for (int64_t b = 0; b < d.B; ++b) {
            float acc = 0.f;
            for (int64_t k = 0; k < d.K; ++k) acc += w[k] * feature(features, d, b, (uint32_t)ids[k]);
            result[b * d.L + j] = acc;
        }
    }
    return FFI_OK;
}

// weight_grad rows [unit_begin, unit_end) and feature_grad rows of the batch [batch_begin, batch_end): the two halves
// split differently over threads (backward.cpp:26-35 by units, :58-72 by batch entries), each thread owning what it writes
int ffi_host_backward_f32(const float* features, const int32_t* lookup, const float* weights, const float* out_grad,
                          float* feature_grad, float* weight_grad, int64_t batch, int64_t num_features, int64_t num_units,
                          int64_t fan_in, int transposed, int64_t unit_begin, int64_t unit_end, int64_t batch_begin,
                          int64_t batch_end) {
    if (!features || !lookup || !weights || !out_grad) return FFI_ERR_NULL_POINTER;
    const int st = check(batch, num_features, num_units, fan_in);
    if (st != FFI_OK) return st;
    if (unit_begin < 0 || unit_end > num_units || unit_begin > unit_end) return FFI_ERR_BAD_ARGUMENT;
    if (batch_begin < 0 || batch_end > batch || batch_begin > batch_end) return FFI_ERR_BAD_ARGUMENT;
    const HostDims d{batch, num_features, num_units, fan_in, transposed != 0};
    if (weight_grad != nullptr) {
        for (int64_t j = unit_begin; j < unit_end; ++j) {
            const int32_t* ids = lookup + j * d.K;
            for (int64_t k = 0; k < d.K; ++k) {
                if ((uint32_t)ids[k] >= (uint64_t)d.N) return FFI_ERR_BAD_LOOKUP;
                float acc = 0.f;
                for (int64_t b = 0; b < d.B; ++b) acc += out_grad[b * d.L + j] * feature(features, d, b, (uint32_t)ids[k]);
                weight_grad[j * d.K + k] = acc;
            }
        }
    }
    if (feature_grad != nullptr) {
        for (int64_t b = batch_begin; b < batch_end; ++b)
            for (int64_t n = 0; n < d.N; ++n) feature_grad[d.tp ? n * d.B + b : b * d.N + n] = 0.f;
        for (int64_t j = 0; j < d.L; ++j) {
            const int32_t* ids = lookup + j * d.K;
            const float* w = weights + j * d.K;
            for (int64_t k = 0; k < d.K; ++k) {
                const uint32_t n = (uint32_t)ids[k];
                if (n >= (uint64_t)d.N) return FFI_ERR_BAD_LOOKUP;
                for (int64_t b = batch_begin; b < batch_end; ++b)
                    feature_grad[d.tp ? (int64_t)n * d.B + b : b * d.N + n] += w[k] * out_grad[b * d.L + j];
            }
        }
    }
    return FFI_OK;
}

}  // extern "C"
