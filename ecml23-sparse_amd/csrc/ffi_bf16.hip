// Inference variant of the fixed-fan-in sparse layer for gfx950: bf16 features and weights, fp32
// accumulation, optional fused top-k per sample.  No counterpart in the reference (its ops are
// registered for float only, tfsparse/cc/kernels/register.cpp:79-109; top-k exists there only as
// tf.nn.top_k inside a Keras metric, sparse/metrics.py:19).
//
// Same scheme as the wide fp32 forward kernel: features are used as xT[N][Bp] (bf16, batch padded to
// a multiple of 8), lanes run along the batch with eight bf16 entries (one 16-byte load) per lane,
// the column id / weight of the current connection are wave-uniform scalars.  With top-k fused the
// [B,L] score matrix is never written: every lane keeps the eight best (score, label) pairs of each
// of its eight samples in registers, wavefronts write their lists, a last kernel merges them.
// Ties go to the lower label index.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>

namespace ffi {
namespace {

constexpr int kBfThreads = 256;            // 4 wavefronts
constexpr int kBfBatch = 512;              // batch entries per pass: 8 per lane
constexpr int kBfLabels = 32;              // labels per workgroup step when scores are written out
constexpr int kBfStride = kBfBatch + 1;
constexpr int kBfInflight = 4;             // connections whose 16-byte gathers a wavefront has in flight
constexpr int kTopMax = 8;                 // list length kept per sample (k <= 8)

__device__ __forceinline__ float bf16_lo(unsigned u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(unsigned u) { return __uint_as_float(u & 0xffff0000u); }

// dst[n][b] (bf16, row stride Bp, zero padded) from src [B,N] or [N,B] bf16
template <bool TP>
__global__ __launch_bounds__(256) void bf16_to_padded_t_kernel(const unsigned short* __restrict__ src,
                                                               unsigned short* __restrict__ dst, int B, int N, int Bp) {
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= (size_t)N * Bp) return;
    const int n = (int)(t / Bp), b = (int)(t % Bp);
    unsigned short v = 0;
    if (b < B) v = TP ? src[(size_t)n * B + b] : src[(size_t)b * N + n];
    dst[t] = v;
}

// eight scores of one label for the lane's eight samples
__device__ __forceinline__ void bf16_label_scores(const buffer_rsrc xr, unsigned lane_off, unsigned row_bytes,
                                                  const int32_t* __restrict__ irow, const unsigned short* __restrict__ wrow,
                                                  int K, int lane, float (&acc)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[i] = 0.f;
    for (int k0 = 0; k0 < K; k0 += 64) {
        const int kn = min(64, K - k0);
        const unsigned iv = (lane < kn) ? (unsigned)irow[k0 + lane] : 0u;
        const float wv = (lane < kn) ? bf16_lo((unsigned)wrow[k0 + lane]) : 0.f;
        int k = 0;
        for (; k + kBfInflight <= kn; k += kBfInflight) {
            uint4 x[kBfInflight];
            float ws[kBfInflight];
#pragma unroll
            for (int u = 0; u < kBfInflight; ++u) {
                const unsigned n = (unsigned)__builtin_amdgcn_readlane((int)iv, k + u);
                ws[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), k + u));
                x[u] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(xr, lane_off, n * row_bytes, 0));
            }
#pragma unroll
            for (int u = 0; u < kBfInflight; ++u) {
                acc[0] = fmaf(ws[u], bf16_lo(x[u].x), acc[0]); acc[1] = fmaf(ws[u], bf16_hi(x[u].x), acc[1]);
                acc[2] = fmaf(ws[u], bf16_lo(x[u].y), acc[2]); acc[3] = fmaf(ws[u], bf16_hi(x[u].y), acc[3]);
                acc[4] = fmaf(ws[u], bf16_lo(x[u].z), acc[4]); acc[5] = fmaf(ws[u], bf16_hi(x[u].z), acc[5]);
                acc[6] = fmaf(ws[u], bf16_lo(x[u].w), acc[6]); acc[7] = fmaf(ws[u], bf16_hi(x[u].w), acc[7]);
            }
        }
        for (; k < kn; ++k) {
            const unsigned n = (unsigned)__builtin_amdgcn_readlane((int)iv, k);
            const float wk = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), k));
            const uint4 x = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(xr, lane_off, n * row_bytes, 0));
            acc[0] = fmaf(wk, bf16_lo(x.x), acc[0]); acc[1] = fmaf(wk, bf16_hi(x.x), acc[1]);
            acc[2] = fmaf(wk, bf16_lo(x.y), acc[2]); acc[3] = fmaf(wk, bf16_hi(x.y), acc[3]);
            acc[4] = fmaf(wk, bf16_lo(x.z), acc[4]); acc[5] = fmaf(wk, bf16_hi(x.z), acc[5]);
            acc[6] = fmaf(wk, bf16_lo(x.w), acc[6]); acc[7] = fmaf(wk, bf16_hi(x.w), acc[7]);
        }
    }
}

// scores written out: grid (label blocks of 32, batch passes of 512)
__global__ __launch_bounds__(kBfThreads) void fwd_bf16_scores_kernel(const unsigned short* __restrict__ xT,
                                                                     const int32_t* __restrict__ idx,
                                                                     const unsigned short* __restrict__ w,
                                                                     float* __restrict__ out, int B, int Bp, int N, int L,
                                                                     int K) {
    extern __shared__ float tile[];                           // [32 labels][513]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j0 = blockIdx.x * kBfLabels;
    const int bc0 = blockIdx.y * kBfBatch;
    const buffer_rsrc xr = make_rsrc(xT, (size_t)N * (size_t)Bp * 2);
    const unsigned lane_off = (unsigned)(bc0 + 8 * lane) * 2u;
    const unsigned row_bytes = (unsigned)Bp * 2u;
    for (int q = 0; q < kBfLabels / 4; ++q) {
        const int jl = wave * (kBfLabels / 4) + q;
        const int j = j0 + jl;
        float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (j < L) bf16_label_scores(xr, lane_off, row_bytes, idx + (size_t)j * K, w + (size_t)j * K, K, lane, acc);
#pragma unroll
        for (int i = 0; i < 8; ++i) tile[jl * kBfStride + 8 * lane + i] = acc[i];
    }
    __syncthreads();
    const int jl = threadIdx.x & 31;
    if (j0 + jl < L) {
        for (int bb = threadIdx.x >> 5; bb < kBfBatch; bb += kBfThreads / 32) {
            const int b = bc0 + bb;
            if (b < B) out[(size_t)b * L + j0 + jl] = tile[jl * kBfStride + bb];
        }
    }
}

// Keeps `vals` sorted descending; v enters behind every element that is >= v (so among equal scores
// the earlier, i.e. lower, label stays ahead).
__device__ __forceinline__ void topk_insert(float (&vals)[kTopMax], int (&ids)[kTopMax], float v, int id) {
    float nv[kTopMax];
    int ni[kTopMax];
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) {
        const bool keep = vals[s] >= v;                          // element s stays where it is
        const bool prev_keep = (s == 0) ? true : (vals[s - 1] >= v);
        nv[s] = keep ? vals[s] : (prev_keep ? v : vals[s - 1]);
        ni[s] = keep ? ids[s] : (prev_keep ? id : ids[s - 1]);
    }
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) { vals[s] = nv[s]; ids[s] = ni[s]; }
}

// fused top-k: grid (label splits, batch passes).  Wavefront w of split s walks labels
// begin+w, begin+w+4, ... in ascending order and writes one list of 8 per sample:
// part[(b * nlists + s*4 + w) * 8 ..].
__global__ __launch_bounds__(kBfThreads) void fwd_bf16_topk_kernel(const unsigned short* __restrict__ xT,
                                                                   const int32_t* __restrict__ idx,
                                                                   const unsigned short* __restrict__ w,
                                                                   float* __restrict__ part_val, int* __restrict__ part_idx,
                                                                   int B, int Bp, int N, int L, int K, int labels_per_split,
                                                                   int nlists) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int bc0 = blockIdx.y * kBfBatch;
    const int begin = blockIdx.x * labels_per_split, end = min(begin + labels_per_split, L);
    const buffer_rsrc xr = make_rsrc(xT, (size_t)N * (size_t)Bp * 2);
    const unsigned lane_off = (unsigned)(bc0 + 8 * lane) * 2u;
    const unsigned row_bytes = (unsigned)Bp * 2u;
    float vals[8][kTopMax];
    int ids[8][kTopMax];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int s = 0; s < kTopMax; ++s) { vals[i][s] = -__builtin_inff(); ids[i][s] = -1; }
    for (int j = begin + wave; j < end; j += kBfThreads / 64) {
        float acc[8];
        bf16_label_scores(xr, lane_off, row_bytes, idx + (size_t)j * K, w + (size_t)j * K, K, lane, acc);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (acc[i] > vals[i][kTopMax - 1]) topk_insert(vals[i], ids[i], acc[i], j);
    }
    const int list = blockIdx.x * (kBfThreads / 64) + wave;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int b = bc0 + 8 * lane + i;
        if (b < B) {
            float* pv = part_val + ((size_t)b * nlists + list) * kTopMax;
            int* pi = part_idx + ((size_t)b * nlists + list) * kTopMax;
#pragma unroll
            for (int s = 0; s < kTopMax; ++s) { pv[s] = vals[i][s]; pi[s] = ids[i][s]; }
        }
    }
}

// (score descending, label ascending) order
__device__ __forceinline__ bool better(float v, int id, float w, int wid) { return v > w || (v == w && id < wid); }

__device__ __forceinline__ void topk_insert_ordered(float (&vals)[kTopMax], int (&ids)[kTopMax], float v, int id) {
    float nv[kTopMax];
    int ni[kTopMax];
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) {
        const bool keep = !better(v, id, vals[s], ids[s]);
        const bool prev_keep = (s == 0) ? true : !better(v, id, vals[s - 1], ids[s - 1]);
        nv[s] = keep ? vals[s] : (prev_keep ? v : vals[s - 1]);
        ni[s] = keep ? ids[s] : (prev_keep ? id : ids[s - 1]);
    }
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) { vals[s] = nv[s]; ids[s] = ni[s]; }
}

// One wavefront per sample merges its `nlists` lists of 8 (empty slots have label -1): every lane
// reduces a strided share of the candidates to a sorted list of its own; then k rounds in which the
// best head among the 64 lane lists (found with shuffles) is emitted and popped.
__global__ __launch_bounds__(64) void topk_merge_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx,
                                                        int B, int nlists, int k, float* __restrict__ values,
                                                        int* __restrict__ indices) {
    const int b = blockIdx.x;
    const int lane = threadIdx.x;
    float vals[kTopMax];
    int ids[kTopMax];
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) { vals[s] = -__builtin_inff(); ids[s] = 0x7fffffff; }
    const float* pv = part_val + (size_t)b * nlists * kTopMax;
    const int* pi = part_idx + (size_t)b * nlists * kTopMax;
    const int total = nlists * kTopMax;
    for (int c0 = lane; c0 < total; c0 += 64 * 8) {           // eight candidates per lane in flight
        float v8[8];
        int i8[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int c = min(c0 + 64 * u, total - 1);    // clamped, not predicated: the loads issue back to back
            i8[u] = c0 + 64 * u < total ? pi[c] : -1;
            v8[u] = pv[c];
        }
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (i8[u] >= 0 && better(v8[u], i8[u], vals[kTopMax - 1], ids[kTopMax - 1])) topk_insert_ordered(vals, ids, v8[u], i8[u]);
    }
    for (int s = 0; s < k; ++s) {
        // the best head of all lanes (empty lists carry (-inf, 0x7fffffff) and lose every comparison)
        float bv = vals[0];
        int bi = ids[0];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
        }
        if (lane == 0) {
            values[(size_t)b * k + s] = bv;
            indices[(size_t)b * k + s] = bi != 0x7fffffff ? bi : -1;
        }
        // the lane that owned it moves its list up (labels are unique, so exactly one lane matches a real winner)
        if (bi != 0x7fffffff && ids[0] == bi && vals[0] == bv) {
#pragma unroll
            for (int t = 0; t + 1 < kTopMax; ++t) { vals[t] = vals[t + 1]; ids[t] = ids[t + 1]; }
            vals[kTopMax - 1] = -__builtin_inff();
            ids[kTopMax - 1] = 0x7fffffff;
        }
    }
}

// Wave-level selection: the 64 lanes hold sorted lists of 8; kTopMax rounds in which the best head (found with
// shuffles) is taken by lane `round` and popped by its owner.  Afterwards lane s < 8 holds the s-th best in out_*.
__device__ __forceinline__ void wave_topk(float (&vals)[kTopMax], int (&ids)[kTopMax], float& out_v, int& out_i) {
    const int lane = threadIdx.x & 63;
    out_v = -__builtin_inff();
    out_i = 0x7fffffff;
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) {
        float bv = vals[0];
        int bi = ids[0];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            const float ov = __shfl_xor(bv, off, 64);
            const int oi = __shfl_xor(bi, off, 64);
            if (better(ov, oi, bv, bi)) { bv = ov; bi = oi; }
        }
        if (lane == s) { out_v = bv; out_i = bi; }
        if (bi != 0x7fffffff && ids[0] == bi && vals[0] == bv) {
#pragma unroll
            for (int t = 0; t + 1 < kTopMax; ++t) { vals[t] = vals[t + 1]; ids[t] = ids[t + 1]; }
            vals[kTopMax - 1] = -__builtin_inff();
            ids[kTopMax - 1] = 0x7fffffff;
        }
    }
}

// top-8 lists of a score matrix scores[B,L]: grid (splits, B); each thread scans a strided share of the split
// (coalesced, eight scores in flight), each wavefront then reduces its 64 lists to one: 4 lists per split.
__global__ __launch_bounds__(256) void topk_scan_kernel(const float* __restrict__ scores, int L, int labels_per_split,
                                                        float* __restrict__ part_val, int* __restrict__ part_idx, int nlists) {
    const int b = blockIdx.y;
    const int begin = blockIdx.x * labels_per_split, end = min(begin + labels_per_split, L);
    float vals[kTopMax];
    int ids[kTopMax];
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) { vals[s] = -__builtin_inff(); ids[s] = 0x7fffffff; }
    const float* row = scores + (size_t)b * L;
    for (int j0 = begin + (int)threadIdx.x; j0 < end; j0 += 256 * 8) {      // eight scores per thread in flight
        float v8[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int j = j0 + 256 * u;
            v8[u] = row[min(j, end - 1)];                 // clamped, not predicated: the eight loads issue back to back
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int j = j0 + 256 * u;
            // (ascending labels per thread, so `>` keeps the lower label among equal scores; -inf scores still enter
            // an empty slot through the label comparison)
            if (j < end && better(v8[u], j, vals[kTopMax - 1], ids[kTopMax - 1])) topk_insert_ordered(vals, ids, v8[u], j);
        }
    }
    float ov;
    int oi;
    wave_topk(vals, ids, ov, oi);
    const int lane = threadIdx.x & 63;
    if (lane < kTopMax) {
        const int list = blockIdx.x * 4 + (threadIdx.x >> 6);
        part_val[((size_t)b * nlists + list) * kTopMax + lane] = ov;
        part_idx[((size_t)b * nlists + list) * kTopMax + lane] = oi != 0x7fffffff ? oi : -1;
    }
}

int prepare_bf16_features(const unsigned short* features, int B, int N, bool tp, hipStream_t s, const unsigned short** xT,
                          int* Bp_out) {
    const int Bp = (B + 7) / 8 * 8;
    *Bp_out = Bp;
    if (tp && Bp == B && ((uintptr_t)features % 16 == 0)) { *xT = features; return FFI_OK; }
    unsigned short* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)N * Bp * 2, (void**)&ws));
    const size_t total = (size_t)N * Bp;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    if (tp) hipLaunchKernelGGL(bf16_to_padded_t_kernel<true>, dim3(blocks), dim3(256), 0, s, features, ws, B, N, Bp);
    else hipLaunchKernelGGL(bf16_to_padded_t_kernel<false>, dim3(blocks), dim3(256), 0, s, features, ws, B, N, Bp);
    FFI_HIP_TRY(hipGetLastError());
    *xT = ws;
    return FFI_OK;
}

}  // namespace

int launch_forward_bf16(const unsigned short* features, const int32_t* idx, const unsigned short* w, float* out,
                        const Dims& d, hipStream_t s) {
    const unsigned short* xT = nullptr;
    int Bp = 0;
    if ((long long)d.N * ((d.B + 7) / 8 * 8) * 2 >= (1ll << 32)) return FFI_ERR_TOO_LARGE;
    FFI_TRY(prepare_bf16_features(features, d.B, d.N, d.tp, s, &xT, &Bp));
    dim3 grid((d.L + kBfLabels - 1) / kBfLabels, (d.B + kBfBatch - 1) / kBfBatch);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    const size_t lds = (size_t)kBfLabels * kBfStride * sizeof(float);
    FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_bf16_scores_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL(fwd_bf16_scores_kernel, grid, dim3(kBfThreads), lds, s, xT, idx, w, out, d.B, Bp, d.N, d.L, d.K);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_forward_topk_bf16(const unsigned short* features, const int32_t* idx, const unsigned short* w, float* values,
                             int32_t* indices, int k, const Dims& d, hipStream_t s) {
    if (k < 1 || k > kTopMax) return FFI_ERR_BAD_ARGUMENT;
    const unsigned short* xT = nullptr;
    int Bp = 0;
    if ((long long)d.N * ((d.B + 7) / 8 * 8) * 2 >= (1ll << 32)) return FFI_ERR_TOO_LARGE;
    FFI_TRY(prepare_bf16_features(features, d.B, d.N, d.tp, s, &xT, &Bp));
    const int passes = (d.B + kBfBatch - 1) / kBfBatch;
    if (passes > 65535) return FFI_ERR_TOO_LARGE;
    int splits = std::max(1, std::min((d.L + 63) / 64, 2 * device_cu_count() / passes));
    const int per = (d.L + splits - 1) / splits;
    splits = (d.L + per - 1) / per;
    const int nlists = splits * (kBfThreads / 64);
    char* part = nullptr;
    const size_t list_bytes = (size_t)d.B * nlists * kTopMax * 4;
    FFI_TRY(workspace_get(s, kWsPartials, 2 * list_bytes, (void**)&part));
    float* pv = (float*)part;
    int* pi = (int*)(part + list_bytes);
    hipLaunchKernelGGL(fwd_bf16_topk_kernel, dim3(splits, passes), dim3(kBfThreads), 0, s, xT, idx, w, pv, pi, d.B, Bp, d.N,
                       d.L, d.K, per, nlists);
    hipLaunchKernelGGL(topk_merge_kernel, dim3(d.B), dim3(64), 0, s, pv, pi, d.B, nlists, k, values, indices);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_topk_merge(const float* part_val, const int* part_idx, int B, int nlists, int k, float* values, int32_t* indices,
                      hipStream_t s) {
    if (k < 1 || k > kTopMax) return FFI_ERR_BAD_ARGUMENT;
    hipLaunchKernelGGL(topk_merge_kernel, dim3(B), dim3(64), 0, s, part_val, part_idx, B, nlists, k, values, indices);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

namespace {

__global__ __launch_bounds__(256) void topk_init_kernel(int* __restrict__ count, int B, int* __restrict__ cand_idx, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < (size_t)B) count[i] = 0;
    for (size_t e = i; e < n; e += (size_t)gridDim.x * 256) cand_idx[e] = -1;
}

// A sample whose candidates did not fit its list (thousands of labels tied at the top: an all-zero feature row under a
// constant bias, say) is answered the slow way, still on the device and without a host wait: one workgroup scans the
// sample's whole row -- the stored scores, or, where the forward pass stored none, scores recomputed with that pass's own
// order of additions (k ascending, bias last) -- every thread keeping the best eight of its share, then the lists are
// merged under the same (score, lower label) order.  Workgroups of samples whose list was complete return at once.
__global__ __launch_bounds__(256) void topk_overflow_rows_kernel(const int* __restrict__ count, int cap, int k, const float* __restrict__ scores,
                                                                 const float* __restrict__ xT, const int32_t* __restrict__ idx,
                                                                 const float* __restrict__ w, const float* __restrict__ bias, int B, int N,
                                                                 int L, int K, float* __restrict__ values, int* __restrict__ indices) {
    const int b = blockIdx.x;
    if (count[b] <= cap) return;
    float vals[kTopMax];
    int ids[kTopMax];
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) { vals[s] = -__builtin_inff(); ids[s] = 0x7fffffff; }
    for (int j = threadIdx.x; j < L; j += 256) {          // ascending labels per thread: ties keep the lower label
        float v;
        if (scores != nullptr) {
            v = scores[(size_t)b * L + j];
        } else {
            v = 0.f;
            for (int c = 0; c < K; ++c) {
                const unsigned id = (unsigned)idx[(size_t)j * K + c];
                v = fmaf(w[(size_t)j * K + c], xT[(size_t)(id < (unsigned)N ? id : 0u) * B + b], v);
            }
            if (bias != nullptr) v += bias[j];
        }
        if (better(v, j, vals[kTopMax - 1], ids[kTopMax - 1])) topk_insert_ordered(vals, ids, v, j);
    }
    float ov;
    int oi;
    wave_topk(vals, ids, ov, oi);
    __shared__ float lv[4][kTopMax];
    __shared__ int li[4][kTopMax];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < kTopMax) { lv[wave][lane] = ov; li[wave][lane] = oi; }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int s = 0; s < kTopMax; ++s) {
        vals[s] = lane < 4 ? lv[lane][s] : -__builtin_inff();
        ids[s] = lane < 4 ? li[lane][s] : 0x7fffffff;
    }
    wave_topk(vals, ids, ov, oi);
    if (lane < k) {
        values[(size_t)b * k + lane] = ov;
        indices[(size_t)b * k + lane] = oi != 0x7fffffff ? oi : -1;
    }
}

// sample[b][i] = scores[b][(i * L) / S]: evenly spaced labels whose k-th best score is a threshold that at least k
// labels of the row reach
__global__ __launch_bounds__(256) void topk_sample_kernel(const float* __restrict__ scores, int L, int S, float* __restrict__ sample) {
    const int b = blockIdx.y;
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < S) sample[(size_t)b * S + i] = scores[(size_t)b * L + (int)(((long long)i * L) / S)];
}

// Every score at or above its row's threshold goes to the row's candidate list.  Such scores are a tiny share of the
// row, so the scan is a plain stream: eight loads in flight per thread, one wave-wide test, the appends on the side.
__global__ __launch_bounds__(256) void topk_filter_kernel(const float* __restrict__ scores, int L, int labels_per_split,
                                                          const float* __restrict__ tau, int tau_stride, int* __restrict__ count,
                                                          float* __restrict__ cand_val, int* __restrict__ cand_idx, int cap) {
    constexpr int kPark = 1024;                       // hits a workgroup parks in LDS before it appends them to the row's list
    __shared__ int park_count;
    __shared__ float park_val[kPark];
    __shared__ int park_idx[kPark];
    const int b = blockIdx.y;
    const int begin = blockIdx.x * labels_per_split, end = min(begin + labels_per_split, L);
    const float t = tau[(size_t)b * tau_stride];
    const float* row = scores + (size_t)b * L;
    if (threadIdx.x == 0) park_count = 0;
    __syncthreads();
    for (int j0 = begin + (int)threadIdx.x; j0 < end; j0 += 256 * 8) {
        float v8[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v8[u] = row[min(j0 + 256 * u, end - 1)];
        bool hit = false;
#pragma unroll
        for (int u = 0; u < 8; ++u) hit |= (j0 + 256 * u < end) && v8[u] >= t;
        if (__ballot(hit)) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int j = j0 + 256 * u;
                if (j < end && v8[u] >= t) {
                    const int p = atomicAdd(&park_count, 1);          // an LDS counter: no round trip to memory
                    if (p < kPark) {
                        park_val[p] = v8[u];
                        park_idx[p] = j;
                    } else {
                        const int slot = atomicAdd(&count[b], 1);
                        if (slot < cap) {
                            cand_val[(size_t)b * cap + slot] = v8[u];
                            cand_idx[(size_t)b * cap + slot] = j;
                        }
                    }
                }
            }
        }
    }
    __syncthreads();
    const int n = min(park_count, kPark);
    __shared__ int first_slot;
    if (threadIdx.x == 0) first_slot = n ? atomicAdd(&count[b], n) : 0;      // one reservation for the whole workgroup
    __syncthreads();
    for (int e = threadIdx.x; e < n; e += 256) {
        const int slot = first_slot + e;
        if (slot < cap) {
            cand_val[(size_t)b * cap + slot] = park_val[e];
            cand_idx[(size_t)b * cap + slot] = park_idx[e];
        }
    }
}

// the old way, for rows too short to be worth a threshold: every thread keeps a list, the wavefronts reduce them
int topk_by_lists(const float* scores, int B, int L, int k, float* values, int32_t* indices, hipStream_t s) {
    // enough workgroups to fill the GPU (8 per CU), each with at least 2048 scores to scan
    int splits = std::max(1, std::min((L + 2047) / 2048, (8 * device_cu_count() + B - 1) / std::max(1, B)));
    const int per = (L + splits - 1) / splits;
    splits = (L + per - 1) / per;
    const int nlists = splits * 4;
    char* part = nullptr;
    const size_t list_bytes = (size_t)B * nlists * kTopMax * 4;
    FFI_TRY(workspace_get(s, kWsPartials, 2 * list_bytes, (void**)&part));
    float* pv = (float*)part;
    int* pi = (int*)(part + list_bytes);
    hipLaunchKernelGGL(topk_scan_kernel, dim3(splits, B), dim3(256), 0, s, scores, L, per, pv, pi, nlists);
    hipLaunchKernelGGL(topk_merge_kernel, dim3(B), dim3(64), 0, s, pv, pi, B, nlists, k, values, indices);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

constexpr int kTopkRowSample = 4096;

}  // namespace

int launch_topk_candidates_init(int* count, int* cand_idx, int B, int cap, hipStream_t s) {
    hipLaunchKernelGGL(topk_init_kernel, dim3(1024), dim3(256), 0, s, count, B, cand_idx, (size_t)B * cap);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_topk_candidates_select(const float* cand_val, const int* cand_idx, const int* count, int B, int cap, int k,
                                  float* values, int32_t* indices, hipStream_t s, const TopkRowSource& src) {
    FFI_TRY(launch_topk_merge(cand_val, cand_idx, B, cap / 8, k, values, indices, s));
    hipLaunchKernelGGL(topk_overflow_rows_kernel, dim3(B), dim3(256), 0, s, count, cap, k, src.scores, src.xT, src.idx, src.w, src.bias,
                       B, src.N, src.L, src.K, values, indices);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_topk_f32(const float* scores, int B, int L, int k, float* values, int32_t* indices, hipStream_t s) {
    if (k < 1 || k > kTopMax) return FFI_ERR_BAD_ARGUMENT;
    if (B > 65535) return FFI_ERR_TOO_LARGE;
    if (L <= 16 * kTopkRowSample) return topk_by_lists(scores, B, L, k, values, indices, s);
    // Long rows: a sample of every row fixes a threshold that k of its labels reach (the k-th best of the sample), one
    // streaming pass collects the few scores at or above it, and the k best of those are the answer.  Exact; a row
    // with more than kTopkCap scores at or above its threshold (thousands of ties) is scanned whole by one workgroup.
    const int S = kTopkRowSample;
    const size_t cand = (size_t)B * kTopkCap;
    unsigned char* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsTopk, ((size_t)B * S + 2 * (size_t)B * kTopMax + (size_t)B + 2 * cand) * 4, (void**)&ws));
    float* sample = reinterpret_cast<float*>(ws);
    float* tau_val = sample + (size_t)B * S;
    int* tau_idx = reinterpret_cast<int*>(tau_val + (size_t)B * kTopMax);
    int* count = tau_idx + (size_t)B * kTopMax;
    float* cand_val = reinterpret_cast<float*>(count + B);
    int* cand_idx = reinterpret_cast<int*>(cand_val + cand);
    hipLaunchKernelGGL(topk_sample_kernel, dim3((S + 255) / 256, B), dim3(256), 0, s, scores, L, S, sample);
    FFI_HIP_TRY(hipGetLastError());
    FFI_TRY(topk_by_lists(sample, B, S, k, tau_val, tau_idx, s));
    FFI_TRY(launch_topk_candidates_init(count, cand_idx, B, kTopkCap, s));
    int splits = std::max(1, std::min((L + 2047) / 2048, (8 * device_cu_count() + B - 1) / std::max(1, B)));
    const int per = (L + splits - 1) / splits;
    splits = (L + per - 1) / per;
    hipLaunchKernelGGL(topk_filter_kernel, dim3(splits, B), dim3(256), 0, s, scores, L, per, tau_val + (k - 1), k, count, cand_val,
                       cand_idx, kTopkCap);
    FFI_HIP_TRY(hipGetLastError());
    TopkRowSource src;
    src.scores = scores; src.L = L;
    return launch_topk_candidates_select(cand_val, cand_idx, count, B, kTopkCap, k, values, indices, s, src);
}

}  // namespace ffi
