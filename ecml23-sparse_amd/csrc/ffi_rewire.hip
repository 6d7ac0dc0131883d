// Rewiring support (sparse/layer.py:60-86, sparse/custom_layer.py:20-43): pick the connections whose
// magnitude is below a threshold, give them new random sources, clear optimizer state there.
//
//   threshold selection  the k-th smallest |w| (FixedFractionSelector: tf.nn.top_k(-|w|, k), last value) by a
//                        three-pass radix select over the 31-bit patterns of |w| (11 + 11 + 9 bits): each pass
//                        histograms one digit of the values that match the digits found so far
//                        (select_hist_kernel), a one-block kernel picks the bin that holds the k-th value
//                        (select_pick_kernel).  Integer atomics only: the result does not depend on their order.
//   rewire_kernel        every position p with |w[p]| < threshold: lookup[p] = a source drawn uniformly from
//                        [0, num_features) by a counter-based generator keyed on (seed, p); arrays[i][p] = 0.
#include "ffi_internal.h"

#include <algorithm>

namespace ffi {
namespace {

constexpr int kSelThreads = 256;
constexpr int kSelBins = 2048;

struct SelectState {
    unsigned prefix;              // digits found so far (the high bits of the answer)
    unsigned long long k;         // rank still to find among the values matching the prefix (1-based)
};

__device__ __forceinline__ unsigned magnitude_bits(float v) { return __float_as_uint(v) & 0x7fffffffu; }

// hist[bin] += number of values whose bits above (shift + nbits) equal state->prefix and whose digit is bin
__global__ __launch_bounds__(kSelThreads) void select_hist_kernel(const float* __restrict__ w, size_t count, int shift, int nbits,
                                                                   const SelectState* __restrict__ state,
                                                                   unsigned* __restrict__ hist) {
    __shared__ unsigned local[kSelBins];
    for (int i = threadIdx.x; i < kSelBins; i += kSelThreads) local[i] = 0;
    __syncthreads();
    const unsigned prefix = state->prefix;
    const int above = shift + nbits;                       // 31 in the first pass: nothing to match
    const unsigned mask = (1u << nbits) - 1u;
    for (size_t i = (size_t)blockIdx.x * kSelThreads + threadIdx.x; i < count; i += (size_t)gridDim.x * kSelThreads) {
        const unsigned key = magnitude_bits(w[i]);
        if (above >= 31 || (key >> above) == prefix) atomicAdd(&local[(key >> shift) & mask], 1u);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kSelBins; i += kSelThreads)
        if (local[i]) atomicAdd(&hist[i], local[i]);
}

// One block: the bin in which the cumulative count reaches state->k; appends it to the prefix, reduces k by the
// count of the bins below it, clears the histogram for the next pass.
__global__ __launch_bounds__(kSelThreads) void select_pick_kernel(unsigned* __restrict__ hist, int nbits, SelectState* __restrict__ state,
                                                                   int last, float* __restrict__ threshold) {
    __shared__ unsigned long long cum[kSelBins];
    const int bins = 1 << nbits;
    for (int i = threadIdx.x; i < kSelBins; i += kSelThreads) cum[i] = i < bins ? hist[i] : 0;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long below = 0;
        const unsigned long long k = state->k;
        int pick = bins - 1;
        for (int i = 0; i < bins; ++i) {
            if (below + cum[i] >= k) { pick = i; break; }
            below += cum[i];
        }
        state->prefix = (state->prefix << nbits) | (unsigned)pick;
        state->k = k - below;
        if (last) *threshold = __uint_as_float(state->prefix);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < kSelBins; i += kSelThreads) hist[i] = 0;
}

__global__ void select_init_kernel(SelectState* state, unsigned* hist, unsigned long long k, float* threshold) {
    for (int i = threadIdx.x; i < kSelBins; i += blockDim.x) hist[i] = 0;
    if (threadIdx.x == 0) {
        state->prefix = 0;
        state->k = k;
        if (k == 0) *threshold = 0.f;            // nothing is below 0 in magnitude: an empty selection
    }
}

// splitmix64 finaliser over (seed, position): a counter-based generator, so the draw of a position does not
// depend on how the launch is shaped
__device__ __forceinline__ unsigned long long mix64(unsigned long long z) {
    z += 0x9e3779b97f4a7c15ull;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

struct ArrayList {
    float* p[4];
};

__global__ __launch_bounds__(kSelThreads) void rewire_kernel(int32_t* __restrict__ lookup, const float* __restrict__ w,
                                                              ArrayList arrays, int n_arrays, size_t count,
                                                              unsigned num_features, const float* __restrict__ threshold,
                                                              unsigned long long seed, unsigned long long* __restrict__ block_counts) {
    __shared__ unsigned red[kSelThreads / 64];
    const float thr = *threshold;
    unsigned changed = 0;
    for (size_t i = (size_t)blockIdx.x * kSelThreads + threadIdx.x; i < count; i += (size_t)gridDim.x * kSelThreads) {
        if (fabsf(w[i]) < thr) {
            const unsigned long long r = mix64(seed ^ mix64((unsigned long long)i));
            lookup[i] = (int32_t)__umul64hi(r, (unsigned long long)num_features);     // uniform in [0, num_features)
            for (int a = 0; a < n_arrays; ++a) arrays.p[a][i] = 0.f;
            ++changed;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) changed += __shfl_xor(changed, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = changed;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long t = 0;
        for (int i = 0; i < kSelThreads / 64; ++i) t += red[i];
        block_counts[blockIdx.x] = t;
    }
}

__global__ __launch_bounds__(64) void rewire_count_kernel(const unsigned long long* __restrict__ block_counts, int n,
                                                          long long* __restrict__ out) {
    unsigned long long t = 0;
    for (int i = threadIdx.x; i < n; i += 64) t += block_counts[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
    if (threadIdx.x == 0) *out = (long long)t;
}

int stream_blocks(size_t count) {
    return (int)std::max<size_t>(1, std::min<size_t>((count + kSelThreads - 1) / kSelThreads, (size_t)device_cu_count() * 8));
}

}  // namespace

int launch_select_threshold(const float* w, size_t count, unsigned long long k, float* threshold, hipStream_t s) {
    unsigned char* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsRewire, 256 + kSelBins * sizeof(unsigned), (void**)&ws));
    SelectState* state = reinterpret_cast<SelectState*>(ws);
    unsigned* hist = reinterpret_cast<unsigned*>(ws + 256);
    hipLaunchKernelGGL(select_init_kernel, dim3(1), dim3(kSelThreads), 0, s, state, hist, k, threshold);
    if (k > 0) {
        const int blocks = stream_blocks(count);
        const int shifts[3] = {20, 9, 0}, bits[3] = {11, 11, 9};
        for (int pass = 0; pass < 3; ++pass) {
            hipLaunchKernelGGL(select_hist_kernel, dim3(blocks), dim3(kSelThreads), 0, s, w, count, shifts[pass], bits[pass], state, hist);
            hipLaunchKernelGGL(select_pick_kernel, dim3(1), dim3(kSelThreads), 0, s, hist, bits[pass], state, pass == 2 ? 1 : 0, threshold);
        }
    }
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_rewire(int32_t* lookup, const float* w, float* const* arrays, int n_arrays, size_t count, unsigned num_features,
                  const float* threshold, unsigned long long seed, long long* rewired, hipStream_t s) {
    ArrayList list{};
    for (int i = 0; i < n_arrays; ++i) list.p[i] = arrays[i];
    const int blocks = stream_blocks(count);
    unsigned long long* block_counts = nullptr;
    FFI_TRY(workspace_get(s, kWsRewire, 256 + std::max<size_t>(kSelBins * sizeof(unsigned), (size_t)blocks * sizeof(unsigned long long)),
                          (void**)&block_counts));
    block_counts = reinterpret_cast<unsigned long long*>(reinterpret_cast<unsigned char*>(block_counts) + 256);
    hipLaunchKernelGGL(rewire_kernel, dim3(blocks), dim3(kSelThreads), 0, s, lookup, w, list, n_arrays, count, num_features, threshold,
                       seed, block_counts);
    if (rewired != nullptr) hipLaunchKernelGGL(rewire_count_kernel, dim3(1), dim3(64), 0, s, block_counts, blocks, rewired);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
