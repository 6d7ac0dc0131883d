// Weight gradient of the fixed-fan-in sparse layer for gfx950:
//   gw[j,k] = sum_b g[b,j] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/backward.cpp:8-36 in the reference).
#include "ffi_internal.h"

namespace ffi {
namespace {

constexpr int kWgBlock = 256;

// One thread per connection (j,k); works for every shape and both feature layouts.
template <bool TP>
__global__ __launch_bounds__(kWgBlock) void wgrad_connection_lane(const float* __restrict__ x,
                                                                   const int32_t* __restrict__ idx,
                                                                   const float* __restrict__ g,
                                                                   float* __restrict__ gw, int B,
                                                                   int N, int L, int K) {
    const size_t p = (size_t)blockIdx.x * kWgBlock + threadIdx.x;
    if (p >= (size_t)L * K) return;
    const int j = (int)(p / (size_t)K);
    const uint32_t n = (uint32_t)idx[p];
    float acc = 0.f;
    for (int b = 0; b < B; ++b) {
        const float xv = TP ? x[(size_t)n * B + b] : x[(size_t)b * N + n];
        acc = fmaf(xv, g[(size_t)b * L + j], acc);
    }
    gw[p] = acc;
}

}  // namespace

int launch_weight_grad(const float* x, const int32_t* idx, const float* g, float* gw, const Dims& d,
                       hipStream_t s) {
    const size_t total = (size_t)d.L * d.K;
    dim3 grid((unsigned)((total + kWgBlock - 1) / kWgBlock));
    if (d.tp)
        hipLaunchKernelGGL(wgrad_connection_lane<true>, grid, dim3(kWgBlock), 0, s, x, idx, g, gw, d.B, d.N, d.L, d.K);
    else
        hipLaunchKernelGGL(wgrad_connection_lane<false>, grid, dim3(kWgBlock), 0, s, x, idx, g, gw, d.B, d.N, d.L, d.K);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
