// Optimizer step for the layer's per-connection variables: Adam as the reference trains with
// (SparseAdam, sparse/optimizer.py:9-23, a keras.optimizers.Adam; run.py:126).  The arithmetic is the
// update_step of that Keras class:
//   alpha = lr * sqrt(1 - beta_2^t) / (1 - beta_1^t)
//   m += (g - m) * (1 - beta_1);  v += (g*g - v) * (1 - beta_2);  var -= (m * alpha) / (sqrt(v) + epsilon)
// One pass over the four arrays: 16 bytes read and 12 written per connection.
#include "ffi_internal.h"
#include "ffi_adam.h"

#include <algorithm>
#include <cmath>

namespace ffi {
namespace {

constexpr int kAdamThreads = 256;

__global__ __launch_bounds__(kAdamThreads) void adam_step_kernel(float* __restrict__ var, float* __restrict__ m,
                                                                 float* __restrict__ v, const float* __restrict__ g,
                                                                 size_t count, AdamCoefficients a) {
    const size_t nvec = count / 4;
    for (size_t i = (size_t)blockIdx.x * kAdamThreads + threadIdx.x; i < nvec; i += (size_t)gridDim.x * kAdamThreads) {
        float4 w4 = reinterpret_cast<float4*>(var)[i], m4 = reinterpret_cast<float4*>(m)[i], v4 = reinterpret_cast<float4*>(v)[i];
        const float4 g4 = reinterpret_cast<const float4*>(g)[i];
        adam_four(w4, m4, v4, g4, a);
        reinterpret_cast<float4*>(var)[i] = w4;
        reinterpret_cast<float4*>(m)[i] = m4;
        reinterpret_cast<float4*>(v)[i] = v4;
    }
    if (blockIdx.x == 0 && threadIdx.x < (count & 3)) {
        const size_t e = nvec * 4 + threadIdx.x;
        adam_one(var[e], m[e], v[e], g[e], a);
    }
}

// The same step for a [rows, row_len] variable whose gradient is stored only for the rows with active[row] != 0:
// the other rows take the step of a zero gradient without their (unwritten) gradient being read.
template <bool VEC4>
__global__ __launch_bounds__(kAdamThreads) void adam_step_rows_kernel(float* __restrict__ var, float* __restrict__ m,
                                                                      float* __restrict__ v, const float* __restrict__ g,
                                                                      const unsigned char* __restrict__ active, size_t count,
                                                                      int row_len, float inv_row_len4, AdamCoefficients a) {
    if (VEC4) {
        // row of 16-byte element i: i / (row_len / 4), in floating point with a correction step (exact for i < 2^31)
        const size_t nvec = count / 4;
        const unsigned r4 = (unsigned)row_len / 4u;
        for (size_t i = (size_t)blockIdx.x * kAdamThreads + threadIdx.x; i < nvec; i += (size_t)gridDim.x * kAdamThreads) {
            unsigned row = (unsigned)((float)i * inv_row_len4);
            const long long rem = (long long)i - (long long)row * r4;
            if (rem < 0) --row;
            else if (rem >= (long long)r4) ++row;
            float4 w4 = reinterpret_cast<float4*>(var)[i], m4 = reinterpret_cast<float4*>(m)[i], v4 = reinterpret_cast<float4*>(v)[i];
            const float4 g4 = active[row] ? reinterpret_cast<const float4*>(g)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
            adam_four(w4, m4, v4, g4, a);
            reinterpret_cast<float4*>(var)[i] = w4;
            reinterpret_cast<float4*>(m)[i] = m4;
            reinterpret_cast<float4*>(v)[i] = v4;
        }
    } else {
        for (size_t i = (size_t)blockIdx.x * kAdamThreads + threadIdx.x; i < count; i += (size_t)gridDim.x * kAdamThreads) {
            const size_t row = i / (size_t)row_len;
            adam_one(var[i], m[i], v[i], active[row] ? g[i] : 0.f, a);
        }
    }
}

}  // namespace

int launch_adam_step_rows(float* var, float* m, float* v, const float* g, const unsigned char* active, int rows, int row_len,
                          float lr, float beta_1, float beta_2, float eps, long long step, hipStream_t s) {
    const AdamCoefficients a = adam_coefficients(lr, beta_1, beta_2, eps, step);
    const size_t count = (size_t)rows * (size_t)row_len;
    const bool vec4 = row_len % 4 == 0 && (((uintptr_t)var | (uintptr_t)m | (uintptr_t)v | (uintptr_t)g) % 16) == 0;
    const size_t items = vec4 ? count / 4 : count;
    const int blocks = (int)std::max<size_t>(1, std::min<size_t>((items + kAdamThreads - 1) / kAdamThreads, (size_t)device_cu_count() * 16));
    if (vec4)
        hipLaunchKernelGGL(adam_step_rows_kernel<true>, dim3(blocks), dim3(kAdamThreads), 0, s, var, m, v, g, active, count, row_len,
                           4.f / (float)row_len, a);
    else
        hipLaunchKernelGGL(adam_step_rows_kernel<false>, dim3(blocks), dim3(kAdamThreads), 0, s, var, m, v, g, active, count, row_len,
                           0.f, a);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_adam_step(float* var, float* m, float* v, const float* g, size_t count, float lr, float beta_1, float beta_2,
                     float eps, long long step, hipStream_t s) {
    const AdamCoefficients a = adam_coefficients(lr, beta_1, beta_2, eps, step);
    const bool aligned = (((uintptr_t)var | (uintptr_t)m | (uintptr_t)v | (uintptr_t)g) % 16) == 0;
    if (!aligned) return FFI_ERR_BAD_ARGUMENT;
    const size_t nvec = count / 4;
    const int blocks = (int)std::max<size_t>(1, std::min<size_t>((nvec + kAdamThreads - 1) / kAdamThreads, (size_t)device_cu_count() * 16));
    hipLaunchKernelGGL(adam_step_kernel, dim3(blocks), dim3(kAdamThreads), 0, s, var, m, v, g, count, a);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
