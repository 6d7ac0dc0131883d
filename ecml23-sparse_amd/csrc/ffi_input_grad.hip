// Input gradient of the fixed-fan-in sparse layer for gfx950, atomics-free:
//   gx[b,n] = sum over (j,k) with idx[j,k]==n of w[j,k] * g[b,j]
// (semantics of tfsparse/cc/kernels/backward.cpp:39-73 in the reference).
#include "ffi_internal.h"

namespace ffi {
namespace {

constexpr int kIgBlock = 256;
constexpr int kIgBatch = 4;

// One workgroup per (column n, group of kIgBatch batch rows).  Threads stride over the column's
// entries, then a fixed-shape tree combines the partial sums, so results do not depend on timing.
template <bool TP>
__global__ __launch_bounds__(kIgBlock) void igrad_column_block(const int32_t* __restrict__ perm,
                                                                const int32_t* __restrict__ col_ptr,
                                                                const float* __restrict__ w,
                                                                const float* __restrict__ g,
                                                                float* __restrict__ gx, int B, int N,
                                                                int L, int K) {
    __shared__ float part[kIgBatch][kIgBlock / 64];
    const int n = blockIdx.x;
    const int b0 = blockIdx.y * kIgBatch;
    const int beg = col_ptr[n], end = col_ptr[n + 1];
    float acc[kIgBatch];
#pragma unroll
    for (int q = 0; q < kIgBatch; ++q) acc[q] = 0.f;
    for (int e = beg + (int)threadIdx.x; e < end; e += kIgBlock) {
        const int p = perm[e];
        const int j = p / K;
        const float wv = w[p];
#pragma unroll
        for (int q = 0; q < kIgBatch; ++q)
            if (b0 + q < B) acc[q] = fmaf(wv, g[(size_t)(b0 + q) * L + j], acc[q]);
    }
#pragma unroll
    for (int q = 0; q < kIgBatch; ++q) {
        float v = acc[q];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) v += __shfl_down(v, off);
        if ((threadIdx.x & 63) == 0) part[q][threadIdx.x >> 6] = v;
    }
    __syncthreads();
    if (threadIdx.x < kIgBatch && b0 + (int)threadIdx.x < B) {
        const int q = threadIdx.x;
        float v = part[q][0];
#pragma unroll
        for (int i = 1; i < kIgBlock / 64; ++i) v += part[q][i];
        const int b = b0 + q;
        if (TP) gx[(size_t)n * B + b] = v; else gx[(size_t)b * N + n] = v;
    }
}

}  // namespace

int launch_input_grad(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp,
                      hipStream_t s) {
    dim3 grid(p->N, (B + kIgBatch - 1) / kIgBatch);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    if (tp)
        hipLaunchKernelGGL(igrad_column_block<true>, grid, dim3(kIgBlock), 0, s, p->perm, p->col_ptr, w, g, gx, B, p->N, p->L, p->K);
    else
        hipLaunchKernelGGL(igrad_column_block<false>, grid, dim3(kIgBlock), 0, s, p->perm, p->col_ptr, w, g, gx, B, p->N, p->L, p->K);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
