// Element-wise losses of the reference's sparse-label training loop and their derivatives with
// respect to the score (sparse/metrics.py:142-173): margin = (2y - 1) * s,
//   hinge          relu(1 - margin)
//   squared hinge  relu(1 - margin)^2
//   bce            max(s,0) - s*y + log1p(exp(-|s|))   (tf.nn.sigmoid_cross_entropy_with_logits)
// The derivative of relu at 0 is 0, as in TensorFlow's gradient of relu.
#ifndef FFI_LOSS_H
#define FFI_LOSS_H

#include <hip/hip_runtime.h>

#include "ffi_hip.h"

namespace ffi {

// Loss and d loss / d score of one element.  The bce branch shares one exponential between the two; its
// gradient sigmoid(s) - y is formed without cancellation for y = 0 and y = 1.  With PRECISE == false it
// uses the hardware's exp2 / log2 / reciprocal approximations (about 1e-7 absolute error on values of
// order one: for the bulk of the matrix, where results are compared relative to the largest entry);
// the few listed label positions are computed with PRECISE == true.
template <bool PRECISE = false>
__device__ __forceinline__ void cwise_loss_and_grad(int kind, float s, float y, float& loss, float& grad) {
    if (kind == FFI_LOSS_BCE) {
        const float e = PRECISE ? expf(-fabsf(s)) : __expf(-fabsf(s));                 // in (0, 1]
        const float inv = PRECISE ? 1.f / (1.f + e) : __fdividef(1.f, 1.f + e);
        loss = fmaxf(s, 0.f) - s * y + (PRECISE ? log1pf(e) : __logf(1.f + e));
        grad = (s >= 0.f ? (1.f - y) - y * e : e * (1.f - y) - y) * inv;                // sigmoid(s) - y
        return;
    }
    const float sign = 2.f * y - 1.f;
    const float r = fmaxf(1.f - sign * s, 0.f);
    if (kind == FFI_LOSS_HINGE) {
        loss = r;
        grad = r > 0.f ? -sign : 0.f;
    } else {
        loss = r * r;
        grad = -2.f * sign * r;
    }
}

__device__ __forceinline__ float cwise_loss(int kind, float s, float y) {
    float l, g;
    cwise_loss_and_grad<true>(kind, s, y, l, g);
    return l;
}

__device__ __forceinline__ float cwise_loss_grad(int kind, float s, float y) {
    float l, g;
    cwise_loss_and_grad<true>(kind, s, y, l, g);
    return g;
}

// Sum of a double over the 64 lanes of a wavefront (every lane gets the total); fixed order.
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

}  // namespace ffi

#endif  // FFI_LOSS_H
