// Loss gradient with respect to the scores of the layer: the producer of out_grad
// (SparseLossBase.call, sparse/metrics.py:136-139, over dense_sparse_cwise_op, sparse/utils.py:11-17).
//
//   loss_dense_kernel      every (b,j) as a negative: g = scale * dloss(s, 0), loss partial sums
//   loss_gather_kernel     saves the scores of the listed label positions (needed when out_grad
//                          overwrites the scores in place)
//   loss_positive_kernel   the listed label positions: g and the loss correction loss(s,y) - loss(s,0);
//                          takes s from the saved scores or the score matrix, or recomputes it from the
//                          label's row of lookup / weights when the scores were never written
//   loss_finish_kernel     sums the partial sums and the corrections in a fixed order
#include "ffi_internal.h"
#include "ffi_loss.h"

#include <algorithm>

namespace ffi {
namespace {

constexpr int kLossThreads = 256;
constexpr int kLossVecPerThread = 4;    // float4 loads in flight per thread and round

__global__ __launch_bounds__(kLossThreads) void loss_dense_kernel(const float* scores, float* g, size_t total, float scale,
                                                                  int kind, double* __restrict__ partial) {
    // `scores` and `g` may be the same buffer: every element is read before it is written, by the same thread
    // 16-byte accesses when both buffers allow them; whatever is left goes element by element
    const bool vec = (((uintptr_t)scores | (uintptr_t)g) & 15) == 0;
    const size_t nvec = vec ? total / 4 : 0;
    const size_t stride = (size_t)gridDim.x * kLossThreads;
    float lsum = 0.f;
    for (size_t v0 = (size_t)blockIdx.x * kLossThreads + threadIdx.x; v0 < nvec; v0 += stride * kLossVecPerThread) {
        float4 s[kLossVecPerThread];
#pragma unroll
        for (int i = 0; i < kLossVecPerThread; ++i) {
            const size_t v = v0 + (size_t)i * stride;
            s[i] = v < nvec ? reinterpret_cast<const float4*>(scores)[v] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int i = 0; i < kLossVecPerThread; ++i) {
            const size_t v = v0 + (size_t)i * stride;
            if (v < nvec) {
                float4 l, o;
                cwise_loss_and_grad(kind, s[i].x, 0.f, l.x, o.x);
                cwise_loss_and_grad(kind, s[i].y, 0.f, l.y, o.y);
                cwise_loss_and_grad(kind, s[i].z, 0.f, l.z, o.z);
                cwise_loss_and_grad(kind, s[i].w, 0.f, l.w, o.w);
                lsum += (l.x + l.y) + (l.z + l.w);
                o.x *= scale; o.y *= scale; o.z *= scale; o.w *= scale;
                reinterpret_cast<float4*>(g)[v] = o;
            }
        }
    }
    for (size_t e = nvec * 4 + (size_t)blockIdx.x * kLossThreads + threadIdx.x; e < total; e += stride) {
        float l, d;
        cwise_loss_and_grad(kind, scores[e], 0.f, l, d);
        lsum += l;
        g[e] = scale * d;
    }
    const double w = wave_sum((double)lsum);
    if ((threadIdx.x & 63) == 0) partial[blockIdx.x * (kLossThreads / 64) + (threadIdx.x >> 6)] = w;
}

__global__ __launch_bounds__(kLossThreads) void loss_gather_kernel(const int64_t* __restrict__ label_indices, int nnz,
                                                                   const float* __restrict__ scores, int B, int L,
                                                                   float* __restrict__ saved) {
    const int p = blockIdx.x * kLossThreads + threadIdx.x;
    if (p >= nnz) return;
    const int64_t b = label_indices[2 * (size_t)p], j = label_indices[2 * (size_t)p + 1];
    saved[p] = (b >= 0 && b < B && j >= 0 && j < L) ? scores[(size_t)b * L + j] : 0.f;
}

// One wavefront per listed label position.  x is addressed as x[b * xsb + n * xsn] (either layout).
__global__ __launch_bounds__(kLossThreads) void loss_positive_kernel(
    const int64_t* __restrict__ label_indices, const float* __restrict__ label_values, int nnz,
    const float* __restrict__ saved, const float* __restrict__ scores, const float* __restrict__ x, size_t xsb, size_t xsn,
    const int32_t* __restrict__ idx, const float* __restrict__ w, const float* __restrict__ bias, float* __restrict__ g,
    float scale, int kind, int B, int N, int L, int K, double* __restrict__ corr, unsigned* __restrict__ nz_words) {
    const int lane = threadIdx.x & 63;
    const int p = blockIdx.x * (kLossThreads / 64) + (threadIdx.x >> 6);
    if (p >= nnz) return;
    const int64_t b = label_indices[2 * (size_t)p], j = label_indices[2 * (size_t)p + 1];
    double c = 0.0;
    if (b >= 0 && b < B && j >= 0 && j < L) {
        float s;
        if (saved != nullptr) {
            s = saved[p];
        } else if (scores != nullptr) {
            s = scores[(size_t)b * L + j];
        } else {
            // the score was never written: recompute it from the label's row, lane <-> connection
            // (a different summation order than the forward kernel's, the same value up to rounding)
            float part = 0.f;
            for (int k = lane; k < K; k += 64) {
                const unsigned id = (unsigned)idx[(size_t)j * K + k];
                part = fmaf(w[(size_t)j * K + k], x[(size_t)b * xsb + (size_t)(id < (unsigned)N ? id : 0u) * xsn], part);
            }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
            s = part;
            if (bias != nullptr) s += bias[j];
        }
        const float y = label_values ? label_values[p] : 1.f;
        const float gv = scale * cwise_loss_grad(kind, s, y);
        // minus what the bulk pass charged this position as a negative (the same arithmetic as there)
        float l0, g0;
        cwise_loss_and_grad<false>(kind, s, 0.f, l0, g0);
        c = (double)cwise_loss(kind, s, y) - (double)l0;
        if (lane == 0) {
            g[(size_t)b * L + j] = gv;
            // the bulk pass set this position's mask bit from its gradient as a negative; a set bit over a zero is harmless
            if (nz_words != nullptr && gv != 0.f) atomicOr(&nz_words[(size_t)(b >> 5) * L + j], 1u << (b & 31));
        }
    }
    if (lane == 0) corr[p] = c;
}

constexpr int kFinishThreads = 1024;

__global__ __launch_bounds__(kFinishThreads) void loss_finish_kernel(const double* __restrict__ partial, int npartial,
                                                                     const double* __restrict__ corr, int ncorr,
                                                                     float* __restrict__ loss_sum) {
    __shared__ double red[kFinishThreads / 64];
    double a = 0.0;
    for (int i = threadIdx.x; i < npartial; i += kFinishThreads) a += partial[i];
    for (int i = threadIdx.x; i < ncorr; i += kFinishThreads) a += corr[i];
    a = wave_sum(a);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = a;
    __syncthreads();
    if (threadIdx.x == 0) {
        double t = 0.0;
        for (int i = 0; i < kFinishThreads / 64; ++i) t += red[i];
        *loss_sum = (float)t;
    }
}

// ---- thresholded precision / recall counts (SparsePrecision, SparseRecall: sparse/metrics.py:73-129) ----------
// per wavefront: how many scores exceed the threshold
__global__ __launch_bounds__(kLossThreads) void threshold_count_kernel(const float* __restrict__ scores, size_t total,
                                                                       float threshold, unsigned long long* __restrict__ partial) {
    const size_t nvec = (((uintptr_t)scores) & 15) == 0 ? total / 4 : 0;
    const size_t stride = (size_t)gridDim.x * kLossThreads;
    unsigned c = 0;
    for (size_t v0 = (size_t)blockIdx.x * kLossThreads + threadIdx.x; v0 < nvec; v0 += stride * kLossVecPerThread) {
        float4 s[kLossVecPerThread];
#pragma unroll
        for (int i = 0; i < kLossVecPerThread; ++i) {
            const size_t v = v0 + (size_t)i * stride;
            s[i] = v < nvec ? reinterpret_cast<const float4*>(scores)[v] : make_float4(threshold, threshold, threshold, threshold);
        }
#pragma unroll
        for (int i = 0; i < kLossVecPerThread; ++i)
            c += (s[i].x > threshold) + (s[i].y > threshold) + (s[i].z > threshold) + (s[i].w > threshold);
    }
    for (size_t e = nvec * 4 + (size_t)blockIdx.x * kLossThreads + threadIdx.x; e < total; e += stride) c += scores[e] > threshold;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
    if ((threadIdx.x & 63) == 0) partial[blockIdx.x * (kLossThreads / 64) + (threadIdx.x >> 6)] = c;
}

// per listed label position: value * [score > threshold] and value
__global__ __launch_bounds__(kLossThreads) void threshold_labels_kernel(const int64_t* __restrict__ label_indices,
                                                                        const float* __restrict__ label_values, int nnz,
                                                                        const float* __restrict__ scores, float threshold, int B,
                                                                        int L, double* __restrict__ hit, double* __restrict__ val) {
    const int p = blockIdx.x * kLossThreads + threadIdx.x;
    if (p >= nnz) return;
    const int64_t b = label_indices[2 * (size_t)p], j = label_indices[2 * (size_t)p + 1];
    double h = 0.0, v = 0.0;
    if (b >= 0 && b < B && j >= 0 && j < L) {
        v = label_values ? (double)label_values[p] : 1.0;
        h = scores[(size_t)b * L + j] > threshold ? v : 0.0;
    }
    hit[p] = h;
    val[p] = v;
}

// out[0] = number of scores above the threshold, out[1] = sum of label values at such positions, out[2] = sum of label values
__global__ __launch_bounds__(kFinishThreads) void threshold_finish_kernel(const unsigned long long* __restrict__ partial, int npartial,
                                                                          const double* __restrict__ hit, const double* __restrict__ val,
                                                                          int nnz, double* __restrict__ out) {
    __shared__ double red[3][kFinishThreads / 64];
    double a = 0.0, h = 0.0, v = 0.0;
    for (int i = threadIdx.x; i < npartial; i += kFinishThreads) a += (double)partial[i];
    for (int i = threadIdx.x; i < nnz; i += kFinishThreads) { h += hit[i]; v += val[i]; }
    a = wave_sum(a); h = wave_sum(h); v = wave_sum(v);
    if ((threadIdx.x & 63) == 0) { red[0][threadIdx.x >> 6] = a; red[1][threadIdx.x >> 6] = h; red[2][threadIdx.x >> 6] = v; }
    __syncthreads();
    if (threadIdx.x < 3) {
        double t = 0.0;
        for (int i = 0; i < kFinishThreads / 64; ++i) t += red[threadIdx.x][i];
        out[threadIdx.x] = t;
    }
}

}  // namespace

int launch_threshold_metrics(const float* scores, const int64_t* indices, const float* values, int nnz, float threshold, int B,
                             int L, double* out, hipStream_t s) {
    const size_t total = (size_t)B * (size_t)L;
    const size_t per_block = (size_t)kLossThreads * kLossVecPerThread * 4;
    const int blocks = (int)std::max<size_t>(1, std::min<size_t>((total + per_block - 1) / per_block, (size_t)device_cu_count() * 16));
    const int npartial = blocks * (kLossThreads / 64);
    unsigned char* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsLoss, ((size_t)npartial + 2 * (size_t)nnz + 2) * sizeof(double), (void**)&ws));
    unsigned long long* partial = reinterpret_cast<unsigned long long*>(ws);
    double* hit = reinterpret_cast<double*>(ws) + npartial;
    double* val = hit + nnz;
    hipLaunchKernelGGL(threshold_count_kernel, dim3(blocks), dim3(kLossThreads), 0, s, scores, total, threshold, partial);
    if (nnz > 0)
        hipLaunchKernelGGL(threshold_labels_kernel, dim3((nnz + kLossThreads - 1) / kLossThreads), dim3(kLossThreads), 0, s, indices,
                           values, nnz, scores, threshold, B, L, hit, val);
    hipLaunchKernelGGL(threshold_finish_kernel, dim3(1), dim3(kFinishThreads), 0, s, partial, npartial, hit, val, nnz, out);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int loss_partial_buffer(hipStream_t s, int npartial, int nnz, double** partial, double** corr, float** saved) {
    double* buf = nullptr;
    FFI_TRY(workspace_get(s, kWsLoss, ((size_t)npartial + 2 * (size_t)nnz + 2) * sizeof(double), (void**)&buf));
    *partial = buf;
    *corr = buf + npartial;
    if (saved) *saved = reinterpret_cast<float*>(buf + npartial + nnz);
    return FFI_OK;
}

int launch_loss_positives(const LossArgs& la, const float* saved, const float* scores, const float* x, const int32_t* idx, const float* w,
                          const float* bias, float* g, const Dims& d, const double* partial, int npartial, double* corr,
                          hipStream_t s) {
    if (la.nnz > 0) {
        const size_t xsb = d.tp ? 1 : (size_t)d.N, xsn = d.tp ? (size_t)d.B : 1;
        hipLaunchKernelGGL(loss_positive_kernel, dim3((la.nnz + kLossThreads / 64 - 1) / (kLossThreads / 64)), dim3(kLossThreads), 0, s,
                           la.indices, la.values, la.nnz, saved, scores, x, xsb, xsn, idx, w, bias, g, la.scale, la.kind, d.B, d.N,
                           d.L, d.K, corr, la.nz_words);
        FFI_HIP_TRY(hipGetLastError());
    }
    if (la.loss_sum != nullptr) {
        hipLaunchKernelGGL(loss_finish_kernel, dim3(1), dim3(kFinishThreads), 0, s, partial, npartial, corr, la.nnz, la.loss_sum);
        FFI_HIP_TRY(hipGetLastError());
    }
    return FFI_OK;
}

int launch_loss_grad(const LossArgs& la, const float* scores, float* g, int B, int L, hipStream_t s) {
    const size_t total = (size_t)B * (size_t)L;
    const size_t per_block = (size_t)kLossThreads * kLossVecPerThread * 4;
    const int blocks = (int)std::max<size_t>(1, std::min<size_t>((total + per_block - 1) / per_block, (size_t)device_cu_count() * 16));
    const int npartial = blocks * (kLossThreads / 64);
    double *partial = nullptr, *corr = nullptr;
    float* saved = nullptr;
    FFI_TRY(loss_partial_buffer(s, npartial, la.nnz, &partial, &corr, &saved));
    // when g overwrites the scores in place, the scores of the listed positions are put aside first
    const bool in_place = scores == g;
    if (in_place && la.nnz > 0) {
        hipLaunchKernelGGL(loss_gather_kernel, dim3((la.nnz + kLossThreads - 1) / kLossThreads), dim3(kLossThreads), 0, s,
                           la.indices, la.nnz, scores, B, L, saved);
        FFI_HIP_TRY(hipGetLastError());
    }
    hipLaunchKernelGGL(loss_dense_kernel, dim3(blocks), dim3(kLossThreads), 0, s, scores, g, total, la.scale, la.kind, partial);
    FFI_HIP_TRY(hipGetLastError());
    // masks of the non-zero gradients, if asked for: a scan of the finished gradient (the listed positions included)
    LossArgs la_pos = la;
    la_pos.nz_words = nullptr;
    Dims d{B, 1, L, 1, false};
    FFI_TRY(launch_loss_positives(la_pos, in_place ? saved : nullptr, scores, nullptr, nullptr, nullptr, nullptr, g, d, partial, npartial, corr, s));
    if (la.nz_words != nullptr) FFI_TRY(launch_nonzero_scan(g, la.nz_words, B, L, s));
    return FFI_OK;
}

}  // namespace ffi
