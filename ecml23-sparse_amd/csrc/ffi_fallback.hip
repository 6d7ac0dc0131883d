// Plain kernels that recompute both gradients straight from the lookup matrix, without any preprocessed view of it.
// They are enqueued behind the plan-driven kernels of the stateless backward entry points and run only when the
// device-side check of the lookup (ffi_plan.hip) found that the cached plan is outdated -- the one call after an
// in-place rewiring (sparse/custom_layer.py:32-43) -- and return at once otherwise.  Semantics:
// tfsparse/cc/kernels/backward.cpp:8-36 (weight gradient) and :39-73 (input gradient); the input gradient scatters
// with float atomics here, as the reference's GPU kernels do (backward.cu.h:119,139,161,182), so this one call is
// not reproducible bit for bit.  Ids outside [0, num_features) are skipped.  Narrow inputs take the weight-gradient kernel
// that reads the lookup itself and an input-gradient kernel that sorts each label tile's connections by column in LDS
// (ffi_input_grad.hip; float atomics only where the workgroups add their sums to gx).
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>

namespace ffi {
namespace {

constexpr int kFbBlock = 256;

__global__ __launch_bounds__(kFbBlock) void fallback_zero_kernel(const unsigned long long* __restrict__ verdict, float* __restrict__ p,
                                                                 size_t count) {
    if (*verdict != 0) return;
    for (size_t i = (size_t)blockIdx.x * kFbBlock + threadIdx.x; i < count; i += (size_t)gridDim.x * kFbBlock) p[i] = 0.f;
}

// one thread per connection (j,k): gw[j,k] = sum_b x[b, id] * g[b, j], b ascending; gx[b, id] += w[j,k] * g[b, j]
template <bool TP>
__global__ __launch_bounds__(kFbBlock) void fallback_backward_kernel(const unsigned long long* __restrict__ verdict,
                                                                     const float* __restrict__ x, const int32_t* __restrict__ idx,
                                                                     const float* __restrict__ w, const float* __restrict__ g,
                                                                     float* __restrict__ gx, float* __restrict__ gw,
                                                                     float* __restrict__ bias_grad, int B, int N, int L, int K) {
    if (*verdict != 0) return;
    const size_t total = (size_t)L * K;
    for (size_t p = (size_t)blockIdx.x * kFbBlock + threadIdx.x; p < total; p += (size_t)gridDim.x * kFbBlock) {
        const int j = (int)(p / K), k = (int)(p - (size_t)j * K);
        const unsigned id = (unsigned)idx[p];
        const bool ok = id < (unsigned)N;
        const float wv = w[p];
        float acc = 0.f, gsum = 0.f;
        for (int b = 0; b < B; ++b) {
            const float gv = g[(size_t)b * L + j];
            gsum += gv;
            if (ok) {
                const size_t xi = TP ? (size_t)id * B + b : (size_t)b * N + id;
                if (gw != nullptr) acc = fmaf(x[xi], gv, acc);
                if (gx != nullptr) atomicAdd(&gx[xi], wv * gv);
            }
        }
        if (gw != nullptr) gw[p] = acc;
        if (bias_grad != nullptr && k == 0) bias_grad[j] = gsum;
    }
}

}  // namespace

int launch_backward_if_outdated(const unsigned long long* verdict, const float* features, const int32_t* lookup,
                                const float* weights, const float* out_grad, float* feature_grad, float* weight_grad,
                                float* bias_grad, const Dims& d, hipStream_t s, bool feature_grad_is_zeroed) {
    const int cus = device_cu_count();
    if (feature_grad != nullptr && !feature_grad_is_zeroed) {
        hipLaunchKernelGGL(fallback_zero_kernel, dim3(cus), dim3(kFbBlock), 0, s, verdict, feature_grad, (size_t)d.B * d.N);
        FFI_HIP_TRY(hipGetLastError());
    }
    float* gw = features != nullptr ? weight_grad : nullptr;
    float* gb = features != nullptr ? bias_grad : nullptr;
    if (tile_path_fits(d.N) && d.L < (1 << 25) && input_grad_unplanned_fits(d.N, d.K)) {
        // narrow inputs: the weight gradient by the kernel that needs no plan (it returns at once unless the verdict says
        // "outdated"), the input gradient by the kernel that sorts each label tile's connections by column in LDS
        if (gw != nullptr) FFI_TRY(launch_weight_grad(features, lookup, out_grad, gw, gb, d, s, nullptr, verdict));
        if (feature_grad != nullptr) FFI_TRY(launch_input_grad_unplanned(verdict, lookup, weights, out_grad, feature_grad, d, s));
        return FFI_OK;
    }
    if (d.tp)
        hipLaunchKernelGGL(fallback_backward_kernel<true>, dim3(cus * 2), dim3(kFbBlock), 0, s, verdict, features, lookup, weights,
                           out_grad, feature_grad, gw, gb, d.B, d.N, d.L, d.K);
    else
        hipLaunchKernelGGL(fallback_backward_kernel<false>, dim3(cus * 2), dim3(kFbBlock), 0, s, verdict, features, lookup, weights,
                           out_grad, feature_grad, gw, gb, d.B, d.N, d.L, d.K);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
