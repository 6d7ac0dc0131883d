// One element of the Adam update (the update_step of keras.optimizers.Adam, which the reference's
// SparseAdam, sparse/optimizer.py:9-23, inherits):
//   m += (g - m) * (1 - beta_1);  v += (g*g - v) * (1 - beta_2);  var -= (m * alpha) / (sqrt(v) + epsilon)
// with alpha = lr * sqrt(1 - beta_2^t) / (1 - beta_1^t) formed on the host.
#ifndef FFI_ADAM_H
#define FFI_ADAM_H

#include <hip/hip_runtime.h>

#include <cmath>

namespace ffi {

struct AdamCoefficients {
    float alpha;   // lr * sqrt(1 - beta_2^t) / (1 - beta_1^t)
    float c1;      // 1 - beta_1
    float c2;      // 1 - beta_2
    float eps;
};

// in the variable's precision, as Keras forms it (float32 pow, sqrt and divide); step counts from 1
inline AdamCoefficients adam_coefficients(float lr, float beta_1, float beta_2, float eps, long long step) {
    const float b1p = std::pow(beta_1, (float)step), b2p = std::pow(beta_2, (float)step);
    return AdamCoefficients{lr * std::sqrt(1.f - b2p) / (1.f - b1p), 1.f - beta_1, 1.f - beta_2, eps};
}

__device__ __forceinline__ void adam_one(float& var, float& m, float& v, float g, const AdamCoefficients& a) {
    m += (g - m) * a.c1;
    v += (g * g - v) * a.c2;
    var -= (m * a.alpha) / (sqrtf(v) + a.eps);
}

__device__ __forceinline__ void adam_four(float4& var, float4& m, float4& v, const float4& g, const AdamCoefficients& a) {
    adam_one(var.x, m.x, v.x, g.x, a);
    adam_one(var.y, m.y, v.y, g.y, a);
    adam_one(var.z, m.z, v.z, g.z, a);
    adam_one(var.w, m.w, v.w, g.w, a);
}

}  // namespace ffi

#endif  // FFI_ADAM_H
