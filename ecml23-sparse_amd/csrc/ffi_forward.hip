// Forward pass of the fixed-fan-in sparse layer for gfx950:
//   out[b,j] = sum_k w[j,k] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/forward.cpp:9-44 in the reference).
#include "ffi_internal.h"

namespace ffi {
namespace {

constexpr int kFwdBlock = 256;  // 4 wavefronts; lanes <-> consecutive labels
constexpr int kFwdBatch = 8;    // batch rows register-blocked per thread

// Label-per-lane kernel that works for every shape and both feature layouts.
// One thread owns label j and kFwdBatch batch rows: W/idx of the row are walked once per batch
// block, x is gathered from global memory, out[b, j..j+63] is one coalesced 256-byte store.
template <bool TP>
__global__ __launch_bounds__(kFwdBlock) void fwd_label_lane(const float* __restrict__ x,
                                                             const int32_t* __restrict__ idx,
                                                             const float* __restrict__ w,
                                                             float* __restrict__ out, int B, int N,
                                                             int L, int K) {
    const int j = blockIdx.x * kFwdBlock + threadIdx.x;
    if (j >= L) return;
    const int b0 = blockIdx.y * kFwdBatch;
    const int nb = min(kFwdBatch, B - b0);
    const int32_t* ip = idx + (size_t)j * K;
    const float* wp = w + (size_t)j * K;
    float acc[kFwdBatch];
#pragma unroll
    for (int q = 0; q < kFwdBatch; ++q) acc[q] = 0.f;
    if (nb == kFwdBatch) {
        for (int k = 0; k < K; ++k) {
            const uint32_t n = (uint32_t)ip[k];
            const float wv = wp[k];
#pragma unroll
            for (int q = 0; q < kFwdBatch; ++q) {
                const float xv = TP ? x[(size_t)n * B + (b0 + q)] : x[(size_t)(b0 + q) * N + n];
                acc[q] = fmaf(wv, xv, acc[q]);
            }
        }
    } else {
        for (int k = 0; k < K; ++k) {
            const uint32_t n = (uint32_t)ip[k];
            const float wv = wp[k];
#pragma unroll
            for (int q = 0; q < kFwdBatch; ++q) {
                if (q < nb) {
                    const float xv = TP ? x[(size_t)n * B + (b0 + q)] : x[(size_t)(b0 + q) * N + n];
                    acc[q] = fmaf(wv, xv, acc[q]);
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < kFwdBatch; ++q)
        if (q < nb) out[(size_t)(b0 + q) * L + j] = acc[q];
}

}  // namespace

int launch_forward(const float* x, const int32_t* idx, const float* w, float* out, const Dims& d,
                   hipStream_t s) {
    dim3 grid((d.L + kFwdBlock - 1) / kFwdBlock, (d.B + kFwdBatch - 1) / kFwdBatch);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    if (d.tp)
        hipLaunchKernelGGL(fwd_label_lane<true>, grid, dim3(kFwdBlock), 0, s, x, idx, w, out, d.B, d.N, d.L, d.K);
    else
        hipLaunchKernelGGL(fwd_label_lane<false>, grid, dim3(kFwdBlock), 0, s, x, idx, w, out, d.B, d.N, d.L, d.K);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
