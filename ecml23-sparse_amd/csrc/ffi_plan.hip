// Column-ordered view ("plan") of a lookup matrix, built on the device.
//
// The input gradient sums, for every input column n, over all connections (j,k) with
// lookup[j,k] == n.  The plan lists those connections column by column, in ascending flat position
// j*K+k inside a column, which is the order the reference's CPU kernel accumulates in
// (tfsparse/cc/kernels/backward.cpp:64-72); walking it sequentially needs no atomics.
#include "ffi_internal.h"

#include <algorithm>
#include <cstring>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

namespace ffi {
namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ unsigned long long mix64(unsigned long long v) {
    v ^= v >> 30; v *= 0xbf58476d1ce4e5b9ull;
    v ^= v >> 27; v *= 0x94d049bb133111ebull;
    v ^= v >> 31;
    return v;
}

// Order-independent 64-bit content fingerprint: sum over positions of mix(position, id), plus the
// number of ids outside [0,N).  Integer atomics only, so the value is reproducible.
__global__ __launch_bounds__(kBlock) void fingerprint_kernel(const int32_t* __restrict__ idx,
                                                              size_t total, unsigned N,
                                                              unsigned long long* __restrict__ out) {
    unsigned long long h = 0, bad = 0;
    for (size_t p = (size_t)blockIdx.x * kBlock + threadIdx.x; p < total; p += (size_t)gridDim.x * kBlock) {
        const unsigned id = (unsigned)idx[p];
        h += mix64(((unsigned long long)p << 32) ^ id ^ 0x9e3779b97f4a7c15ull);
        bad += id >= N;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        h += __shfl_down(h, off);
        bad += __shfl_down(bad, off);
    }
    if ((threadIdx.x & 63) == 0) {
        atomicAdd(&out[0], h);
        if (bad) atomicAdd(&out[1], bad);
    }
}

__global__ __launch_bounds__(kBlock) void zero_u64_kernel(unsigned long long* p, int n) {
    const int i = blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0;
}

// col_ptr[n] = first position in the sorted key array whose key is >= n (n in [0,N]).
__global__ __launch_bounds__(kBlock) void col_ptr_kernel(const unsigned* __restrict__ sorted_keys,
                                                          int total, int N, int32_t* __restrict__ col_ptr) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n > N) return;
    int lo = 0, hi = total;
    while (lo < hi) {
        const int mid = lo + ((hi - lo) >> 1);
        if (sorted_keys[mid] < (unsigned)n) lo = mid + 1; else hi = mid;
    }
    col_ptr[n] = lo;
}

int bits_for(unsigned max_value) {
    int b = 1;
    while (b < 32 && (max_value >> b) != 0) ++b;
    return b;
}

}  // namespace

int plan_fingerprint(ffi_plan* p, const int32_t* lookup, hipStream_t s, unsigned long long* out,
                     unsigned long long* bad_ids) {
    const size_t total = (size_t)p->L * p->K;
    hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(kBlock), 0, s, p->d_scratch, 2);
    const unsigned blocks = (unsigned)std::min<size_t>((total + kBlock - 1) / kBlock, 2048);
    hipLaunchKernelGGL(fingerprint_kernel, dim3(blocks), dim3(kBlock), 0, s, lookup, total, (unsigned)p->N, p->d_scratch);
    FFI_HIP_TRY(hipGetLastError());
    FFI_HIP_TRY(hipMemcpyAsync(p->h_scratch, p->d_scratch, 2 * sizeof(unsigned long long), hipMemcpyDeviceToHost, s));
    FFI_HIP_TRY(hipStreamSynchronize(s));
    *out = p->h_scratch[0];
    *bad_ids = p->h_scratch[1];
    return FFI_OK;
}

int plan_build(ffi_plan* p, const int32_t* lookup, hipStream_t s) {
    const int total = p->L * p->K;  // validated to fit int32 by the caller
    unsigned long long fp = 0, bad = 0;
    FFI_TRY(plan_fingerprint(p, lookup, s, &fp, &bad));
    if (bad != 0) return FFI_ERR_BAD_LOOKUP;

    unsigned* sorted_keys = nullptr;
    void* temp = nullptr;
    size_t temp_bytes = 0;
    const int end_bit = bits_for((unsigned)(p->N - 1));
    rocprim::counting_iterator<int32_t> positions(0);
    auto cleanup = [&]() {
        if (sorted_keys) (void)hipFree(sorted_keys);
        if (temp) (void)hipFree(temp);
    };
    hipError_t e = rocprim::radix_sort_pairs(nullptr, temp_bytes, (const unsigned*)lookup, sorted_keys, positions,
                                             p->perm, (unsigned)total, 0, end_bit, s);
    if (e != hipSuccess) return hip_fail(e);
    if (hipMalloc(&sorted_keys, (size_t)total * sizeof(unsigned)) != hipSuccess ||
        hipMalloc(&temp, temp_bytes ? temp_bytes : 4) != hipSuccess) {
        (void)hipGetLastError();
        cleanup();
        return FFI_ERR_OUT_OF_MEMORY;
    }
    e = rocprim::radix_sort_pairs(temp, temp_bytes, (const unsigned*)lookup, sorted_keys, positions, p->perm,
                                  (unsigned)total, 0, end_bit, s);
    if (e != hipSuccess) { cleanup(); return hip_fail(e); }
    hipLaunchKernelGGL(col_ptr_kernel, dim3((p->N + 1 + kBlock - 1) / kBlock), dim3(kBlock), 0, s, sorted_keys, total,
                       p->N, p->col_ptr);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    cleanup();
    if (e != hipSuccess) return hip_fail(e);
    p->lookup = lookup;
    p->fingerprint = fp;
    return FFI_OK;
}

void plan_free(ffi_plan* p) {
    if (!p) return;
    if (p->perm) (void)hipFree(p->perm);
    if (p->col_ptr) (void)hipFree(p->col_ptr);
    if (p->d_scratch) (void)hipFree(p->d_scratch);
    if (p->h_scratch) (void)hipHostFree(p->h_scratch);
    p->perm = nullptr; p->col_ptr = nullptr; p->d_scratch = nullptr; p->h_scratch = nullptr;
    p->bytes = 0;
}

}  // namespace ffi
