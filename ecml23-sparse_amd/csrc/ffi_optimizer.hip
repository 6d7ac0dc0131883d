// Optimizer step for the layer's per-connection variables: Adam as the reference trains with
// (SparseAdam, sparse/optimizer.py:9-23, a keras.optimizers.Adam; run.py:126).  The arithmetic is the
// update_step of that Keras class:
//   alpha = lr * sqrt(1 - beta_2^t) / (1 - beta_1^t)
//   m += (g - m) * (1 - beta_1);  v += (g*g - v) * (1 - beta_2);  var -= (m * alpha) / (sqrt(v) + epsilon)
// One pass over the four arrays: 16 bytes read and 12 written per connection.
#include "ffi_internal.h"

#include <algorithm>
#include <cmath>

namespace ffi {
namespace {

constexpr int kAdamThreads = 256;

__device__ __forceinline__ void adam_one(float& var, float& m, float& v, float g, float alpha, float c1, float c2, float eps) {
    m += (g - m) * c1;
    v += (g * g - v) * c2;
    var -= (m * alpha) / (sqrtf(v) + eps);
}

__global__ __launch_bounds__(kAdamThreads) void adam_step_kernel(float* __restrict__ var, float* __restrict__ m,
                                                                 float* __restrict__ v, const float* __restrict__ g,
                                                                 size_t count, float alpha, float c1, float c2, float eps) {
    const size_t nvec = count / 4;
    for (size_t i = (size_t)blockIdx.x * kAdamThreads + threadIdx.x; i < nvec; i += (size_t)gridDim.x * kAdamThreads) {
        float4 w4 = reinterpret_cast<float4*>(var)[i], m4 = reinterpret_cast<float4*>(m)[i], v4 = reinterpret_cast<float4*>(v)[i];
        const float4 g4 = reinterpret_cast<const float4*>(g)[i];
        adam_one(w4.x, m4.x, v4.x, g4.x, alpha, c1, c2, eps);
        adam_one(w4.y, m4.y, v4.y, g4.y, alpha, c1, c2, eps);
        adam_one(w4.z, m4.z, v4.z, g4.z, alpha, c1, c2, eps);
        adam_one(w4.w, m4.w, v4.w, g4.w, alpha, c1, c2, eps);
        reinterpret_cast<float4*>(var)[i] = w4;
        reinterpret_cast<float4*>(m)[i] = m4;
        reinterpret_cast<float4*>(v)[i] = v4;
    }
    if (blockIdx.x == 0 && threadIdx.x < (count & 3)) {
        const size_t e = nvec * 4 + threadIdx.x;
        adam_one(var[e], m[e], v[e], g[e], alpha, c1, c2, eps);
    }
}

}  // namespace

int launch_adam_step(float* var, float* m, float* v, const float* g, size_t count, float lr, float beta_1, float beta_2,
                     float eps, long long step, hipStream_t s) {
    // the step-dependent factor in the variable's precision, as Keras forms it (float32 pow, sqrt and divide)
    const float b1p = std::pow(beta_1, (float)step), b2p = std::pow(beta_2, (float)step);
    const float alpha = lr * std::sqrt(1.f - b2p) / (1.f - b1p);
    const bool aligned = (((uintptr_t)var | (uintptr_t)m | (uintptr_t)v | (uintptr_t)g) % 16) == 0;
    if (!aligned) return FFI_ERR_BAD_ARGUMENT;
    const size_t nvec = count / 4;
    const int blocks = (int)std::max<size_t>(1, std::min<size_t>((nvec + kAdamThreads - 1) / kAdamThreads, (size_t)device_cu_count() * 16));
    hipLaunchKernelGGL(adam_step_kernel, dim3(blocks), dim3(kAdamThreads), 0, s, var, m, v, g, count, alpha, 1.f - beta_1,
                       1.f - beta_2, eps);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
