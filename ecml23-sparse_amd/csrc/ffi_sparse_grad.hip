// Backward pass for an out_grad that is mostly exact zeros (a hinge loss late in training: every
// satisfied margin has gradient 0).  The reference's GPU kernels skip such entries one by one
// (`if(out == 0) continue`, tfsparse/cc/kernels/backward.cu.h:73,94,131,151); here the zero pattern is
// made explicit once, as bit masks, and the kernels walk the set bits only:
//
//   words[t][j]      bit i set  <=>  out_grad[32 t + i, j] may be non-zero          (per label: weight gradient)
//   bits[b][j / 64]  bit j % 64 set  <=>  the same for sample b                      (per sample: input gradient)
//
//   nz_scan_kernel          words from out_grad
//   nz_count_kernel, nz_count_finish_kernel   the number of set bits (two steps, no atomics)
//   nz_transpose_kernel     bits from words
//   wgrad_sparse_kernel     lane <-> label: every lane walks the set bits of its own label and keeps 32 sums
//                           (one chunk of connections) in registers; labels with many set bits are done by
//                           the whole wavefront afterwards, lane <-> connection; rows of labels without a
//                           set bit come out as zeros
//   igrad_sparse_kernel     one workgroup per (sample, label segment): every lane takes labels from its own word of
//                           the sample's bit row and adds g * w of the label's connections into per-wavefront
//                           accumulators gx[n] in LDS (LDS float adds issued in a fixed order)
//   igrad_sparse_reduce_kernel  sums the segments in ascending order into feature_grad
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>
#include <mutex>
#include <vector>

namespace ffi {
namespace {

constexpr int kScanThreads = 256;
constexpr int kCountBlocks = 1024;

__global__ __launch_bounds__(kScanThreads) void nz_scan_kernel(const float* __restrict__ g, unsigned* __restrict__ words,
                                                               int B, int L) {
    // two labels per thread (j and j + kScanThreads): 64 independent loads in flight
    const int j0 = blockIdx.x * (2 * kScanThreads) + threadIdx.x;
    const int t = blockIdx.y;
    const int rows = min(32, B - 32 * t);
    const float* tile = g + (size_t)(32 * t) * L;
    float v[2][32];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int j = min(j0 + h * kScanThreads, L - 1);
#pragma unroll
        for (int i = 0; i < 32; ++i) v[h][i] = i < rows ? tile[(size_t)i * L + j] : 0.f;
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int j = j0 + h * kScanThreads;
        unsigned m = 0;
#pragma unroll
        for (int i = 0; i < 32; ++i) m |= (v[h][i] != 0.f ? 1u : 0u) << i;
        if (j < L) words[(size_t)t * L + j] = m;
    }
}

// g[32 t + i, j] = 0 wherever bit i of words[t][j] is clear (thread <-> label, rows written 256 bytes per wavefront).
__global__ __launch_bounds__(kScanThreads) void nz_zero_unmasked_kernel(float* __restrict__ g, const unsigned* __restrict__ words,
                                                                        int B, int L) {
    const int j = blockIdx.x * kScanThreads + threadIdx.x;
    const int t = blockIdx.y;
    if (j >= L) return;
    const int rows = min(32, B - 32 * t);
    const unsigned m = words[(size_t)t * L + j];
    float* col = g + (size_t)(32 * t) * L + j;
#pragma unroll
    for (int i = 0; i < 32; ++i)
        if (i < rows && !((m >> i) & 1u)) col[(size_t)i * L] = 0.f;
}

__global__ __launch_bounds__(kScanThreads) void nz_count_kernel(const unsigned* __restrict__ words, size_t n,
                                                                unsigned long long* __restrict__ block_counts) {
    __shared__ unsigned red[kScanThreads / 64];
    unsigned c = 0;
    for (size_t i = (size_t)blockIdx.x * kScanThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kScanThreads)
        c += __popc(words[i]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = c;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long t = 0;
        for (int i = 0; i < kScanThreads / 64; ++i) t += red[i];
        block_counts[blockIdx.x] = t;
    }
}

__global__ __launch_bounds__(64) void nz_count_finish_kernel(const unsigned long long* __restrict__ block_counts, int n,
                                                             unsigned long long* __restrict__ host_count) {
    unsigned long long t = 0;
    for (int i = threadIdx.x; i < n; i += 64) t += block_counts[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
    if (threadIdx.x == 0) *host_count = t;              // pinned host memory: the host reads it after the stream has drained
}

// One wavefront per (batch tile t, block of 64 labels): bits[32 t + i][blk] = ballot of bit i.
__global__ __launch_bounds__(kScanThreads) void nz_transpose_kernel(const unsigned* __restrict__ words,
                                                                    unsigned long long* __restrict__ bits, int B, int L,
                                                                    int nwords) {
    const int lane = threadIdx.x & 63;
    const int blk = blockIdx.x * (kScanThreads / 64) + (threadIdx.x >> 6);
    const int t = blockIdx.y;
    if (blk >= nwords) return;
    const int j = blk * 64 + lane;
    const unsigned m = j < L ? words[(size_t)t * L + j] : 0u;
    unsigned long long mine = 0;
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const unsigned long long bl = __ballot((m >> i) & 1u);
        if (lane == i) mine = bl;
    }
    const int b = 32 * t + lane;
    if (lane < 32 && b < B) bits[(size_t)b * nwords + blk] = mine;
}

constexpr int kHeavyBits = 12;     // labels with more set bits than this are left to the whole wavefront

// x is addressed as x[b * xsb + n * xsn] (either layout; byte strides), through a buffer resource with 32-bit
// offsets: batch * num_features * 4 < 2^32, checked by the launcher.
// ZERO_FILL == true: rows of labels without a set bit are written as zeros.
// ZERO_FILL == false: those rows are left alone and active[j] (one byte per label) says which rows were written:
// for a consumer that does not want to read 4 * K bytes of zeros per idle label.
template <bool VEC4, bool ZERO_FILL>
__global__ __launch_bounds__(256, 4) void wgrad_sparse_kernel(const float* __restrict__ x, unsigned xsb, unsigned xsn,
                                                              const int32_t* __restrict__ idx, const float* __restrict__ g,
                                                              const unsigned* __restrict__ words, float* __restrict__ gw,
                                                              float* __restrict__ bias_grad,
                                                              unsigned char* __restrict__ active, int B, int N, int L,
                                                              int K, int nbt) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int nwaves = gridDim.x * 4;
    const int nblk = (L + 63) / 64;
    const unsigned tail = (B & 31) ? (1u << (B & 31)) - 1u : 0xffffffffu;   // bits past the batch are ignored
    const buffer_rsrc xr = make_rsrc(x, (size_t)B * (size_t)N * sizeof(float));
    for (int blk = wave; blk < nblk; blk += nwaves) {
        const int base = blk * 64;
        const int rows = min(64, L - base);
        const int j = base + min(lane, rows - 1);
        const bool mine = lane < rows;
        int cnt = 0;
        for (int t = 0; t < nbt; ++t) {
            unsigned m = words[(size_t)t * L + j];
            if (t == nbt - 1) m &= tail;
            cnt += __popc(m);
        }
        const bool heavy = cnt > kHeavyBits;
        const bool light = mine && !heavy;
        if (ZERO_FILL) {
            // rows of labels without a set bit: zeros, written by the whole wavefront (the block's rows are contiguous
            // in gw).  The row of 16-byte element e is e / (K/4), formed in floating point (exact here: e + 0.5 is at
            // least 0.5 / (K/4) away from a multiple).
            const unsigned long long zero_rows = __ballot(mine && cnt == 0);
            float* blockrows = gw + (size_t)base * K;
            if (VEC4) {
                const int k4 = K / 4;
                const float inv_k4 = 1.f / (float)k4;
                for (int e = lane; e < rows * k4; e += 64)
                    if ((zero_rows >> (int)(((float)e + 0.5f) * inv_k4)) & 1ull)
                        reinterpret_cast<float4*>(blockrows)[e] = make_float4(0.f, 0.f, 0.f, 0.f);
            } else {
                for (int e = lane; e < rows * K; e += 64)
                    if ((zero_rows >> (e / K)) & 1ull) blockrows[e] = 0.f;
            }
        } else if (mine) {
            active[j] = cnt != 0;
        }
        // ---- every lane its own label ----
        float gsum = 0.f;
        for (int k0 = 0; k0 < K; k0 += 32) {
            unsigned ids[32];
            if (light && cnt) {
                if (VEC4 && k0 + 32 <= K) {
#pragma unroll
                    for (int q = 0; q < 8; ++q) {
                        const int4 v = *reinterpret_cast<const int4*>(idx + (size_t)j * K + k0 + 4 * q);
                        ids[4 * q] = (unsigned)v.x; ids[4 * q + 1] = (unsigned)v.y; ids[4 * q + 2] = (unsigned)v.z; ids[4 * q + 3] = (unsigned)v.w;
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < 32; ++k) ids[k] = k0 + k < K ? (unsigned)idx[(size_t)j * K + k0 + k] : 0u;
                }
                // column ids -> byte offsets of the columns in x
#pragma unroll
                for (int k = 0; k < 32; ++k) ids[k] = (ids[k] < (unsigned)N ? ids[k] : 0u) * xsn;
            } else {
#pragma unroll
                for (int k = 0; k < 32; ++k) ids[k] = 0u;
            }
            float acc[32];
#pragma unroll
            for (int k = 0; k < 32; ++k) acc[k] = 0.f;
            // the label's mask words, eight batch tiles at a time in registers; every step each lane takes the
            // next set bit of its own label (g and the 32 gathered x values are requested together)
            for (int tb = 0; tb < nbt; tb += 8) {
                unsigned mw[8];
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const int t = tb + u;
                    mw[u] = (light && cnt && t < nbt) ? words[(size_t)t * L + j] : 0u;
                    if (t == nbt - 1) mw[u] &= tail;
                }
                for (;;) {
                    int usel = -1;
                    unsigned msel = 0;
#pragma unroll
                    for (int u = 7; u >= 0; --u)
                        if (mw[u]) { usel = u; msel = mw[u]; }
                    if (!__ballot(usel >= 0)) break;
                    if (usel >= 0) {
                        const int b = 32 * (tb + usel) + __ffs((int)msel) - 1;
#pragma unroll
                        for (int u = 0; u < 8; ++u)
                            if (u == usel) mw[u] = msel & (msel - 1);
                        const float gv = g[(size_t)b * L + j];
                        const unsigned xrow = (unsigned)b * xsb;
                        // 16 gathers in flight at a time
#pragma unroll
                        for (int h = 0; h < 2; ++h) {
                            float xv[16];
#pragma unroll
                            for (int k = 0; k < 16; ++k) xv[k] = buffer_load_f32(xr, ids[16 * h + k] + xrow, 0);
#pragma unroll
                            for (int k = 0; k < 16; ++k) acc[16 * h + k] = fmaf(gv, xv[k], acc[16 * h + k]);
                        }
                        if (k0 == 0) gsum += gv;
                    }
                }
            }
            if (light && cnt) {
                float* orow = gw + (size_t)j * K + k0;
                if (VEC4 && k0 + 32 <= K) {
#pragma unroll
                    for (int q = 0; q < 8; ++q)
                        *reinterpret_cast<float4*>(orow + 4 * q) = make_float4(acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
                } else {
#pragma unroll
                    for (int k = 0; k < 32; ++k)
                        if (k0 + k < K) orow[k] = acc[k];
                }
            }
        }
        if (bias_grad != nullptr && light) bias_grad[j] = gsum;
        // ---- labels with many set bits: the whole wavefront on one label, lane <-> connection ----
        unsigned long long todo = __ballot(mine && heavy);
        while (todo) {
            const int r = __builtin_amdgcn_readfirstlane(__ffsll((long long)todo) - 1);
            todo &= todo - 1;
            const int jh = base + r;
            float hsum = 0.f;
            for (int k0 = 0; k0 < K; k0 += 64) {
                const int k = k0 + lane;
                const unsigned id = k < K ? (unsigned)idx[(size_t)jh * K + k] : 0u;
                const unsigned xcol = (id < (unsigned)N ? id : 0u) * xsn;
                float acc = 0.f;
                hsum = 0.f;
                for (int t = 0; t < nbt; ++t) {
                    unsigned m = __builtin_amdgcn_readfirstlane(words[(size_t)t * L + jh]);
                    if (t == nbt - 1) m &= tail;
                    // up to four set bits per step, their loads in flight together
                    while (m) {
                        int bb[4];
                        float gv[4], xv[4];
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            bb[u] = m ? 32 * t + __ffs((int)m) - 1 : -1;
                            m &= m ? m - 1 : 0u;
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            const int b = bb[u] < 0 ? 0 : bb[u];
                            gv[u] = bb[u] < 0 ? 0.f : g[(size_t)b * L + jh];
                            xv[u] = buffer_load_f32(xr, xcol, (unsigned)b * xsb);
                        }
#pragma unroll
                        for (int u = 0; u < 4; ++u) {
                            acc = fmaf(gv[u], xv[u], acc);
                            hsum += gv[u];
                        }
                    }
                }
                if (k < K) gw[(size_t)jh * K + k] = acc;
            }
            if (bias_grad != nullptr && lane == 0) bias_grad[jh] = hsum;
        }
    }
}

constexpr int kSgThreads = 512;
constexpr int kSgWaves = kSgThreads / 64;

// One workgroup per (sample, label segment).  Every wavefront walks its own share of the sample's bit row, 64 words
// (4096 labels) at a time, one word per lane; at every step each lane with a bit left takes its next label, loads
// that label's row of idx / w (a 32-connection chunk at a time) and adds g * w into the wavefront's own
// accumulators gx[n] in LDS.  No barriers inside the walk; the order of the adds is fixed by the lane
// assignment.  The wavefronts' accumulators are summed in ascending order at the end.
template <bool VEC4>
__global__ __launch_bounds__(kSgThreads) void igrad_sparse_kernel(const unsigned long long* __restrict__ bits, int nwords,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w, const float* __restrict__ g,
                                                                  float* __restrict__ partial, int B, int N, int L, int K,
                                                                  int S, int words_per_seg) {
    extern __shared__ __align__(16) unsigned char sg_lds[];
    float* acc = reinterpret_cast<float*>(sg_lds);                                        // [kSgWaves][N]
    const int b = blockIdx.x / S, seg = blockIdx.x % S;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < kSgWaves * N; i += kSgThreads) acc[i] = 0.f;
    __syncthreads();
    const int w_begin = seg * words_per_seg;
    const int w_end = min(w_begin + words_per_seg, nwords);
    const unsigned long long* row = bits + (size_t)b * nwords;
    const float* grow = g + (size_t)b * L;
    float* myacc = acc + (size_t)wv * N;
    for (int w0 = w_begin + wv * 64; w0 < w_end; w0 += kSgWaves * 64) {
        const int wi = w0 + lane;
        unsigned long long m = wi < w_end ? row[wi] : 0ull;
        while (__ballot(m != 0)) {
            if (m) {
                const int j = wi * 64 + __ffsll((long long)m) - 1;
                m &= m - 1;
                const float gv = grow[j];
                const size_t at = (size_t)j * K;
                for (int k0 = 0; k0 < K; k0 += 32) {
                    unsigned n[32];
                    float wk[32];
                    if (VEC4 && k0 + 32 <= K) {
#pragma unroll
                        for (int q = 0; q < 8; ++q) {
                            const int4 v = *reinterpret_cast<const int4*>(idx + at + k0 + 4 * q);
                            const float4 f = *reinterpret_cast<const float4*>(w + at + k0 + 4 * q);
                            n[4 * q] = (unsigned)v.x; n[4 * q + 1] = (unsigned)v.y; n[4 * q + 2] = (unsigned)v.z; n[4 * q + 3] = (unsigned)v.w;
                            wk[4 * q] = f.x; wk[4 * q + 1] = f.y; wk[4 * q + 2] = f.z; wk[4 * q + 3] = f.w;
                        }
                    } else {
#pragma unroll
                        for (int k = 0; k < 32; ++k) {
                            const bool in = k0 + k < K;
                            n[k] = in ? (unsigned)idx[at + k0 + k] : 0xffffffffu;
                            wk[k] = in ? w[at + k0 + k] : 0.f;
                        }
                    }
#pragma unroll
                    for (int k = 0; k < 32; ++k)
                        if (n[k] < (unsigned)N) atomicAdd(&myacc[n[k]], gv * wk[k]);
                }
            }
        }
    }
    __syncthreads();
    float* out = partial + ((size_t)seg * B + b) * N;
    for (int n = threadIdx.x; n < N; n += kSgThreads) {
        float t = acc[n];
#pragma unroll
        for (int i = 1; i < kSgWaves; ++i) t += acc[(size_t)i * N + n];
        out[n] = t;
    }
}

__global__ __launch_bounds__(256) void igrad_sparse_reduce_kernel(const float* __restrict__ partial, int S, int B, int N,
                                                                  float* __restrict__ gx, int tp) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (size_t)B * N) return;
    float t = 0.f;
    for (int s = 0; s < S; ++s) t += partial[(size_t)s * B * N + i];
    const int b = (int)(i / N), n = (int)(i - (size_t)b * N);
    gx[tp ? (size_t)n * B + b : i] = t;
}

// Pinned words the set-bit counts are written to by the count kernel, one per (device, stream), together with
// the shape of the call that wrote it: a later call on the same stream may decide from it without waiting.
struct CountSlot {
    int device;
    hipStream_t stream;
    unsigned long long* host;    // hipHostMalloc'ed, written by nz_count_finish_kernel
    int B, L;                    // shape of the last call (0: none yet)
};
std::mutex g_count_mutex;
std::vector<CountSlot> g_count_slots;

}  // namespace

int launch_nonzero_scan(const float* g, unsigned* words, int B, int L, hipStream_t s) {
    const int nbt = (B + 31) / 32;
    hipLaunchKernelGGL(nz_scan_kernel, dim3((L + 2 * kScanThreads - 1) / (2 * kScanThreads), nbt), dim3(kScanThreads), 0, s, g, words, B, L);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_zero_unmasked(float* g, const unsigned* words, int B, int L, hipStream_t s) {
    const int nbt = (B + 31) / 32;
    hipLaunchKernelGGL(nz_zero_unmasked_kernel, dim3((L + kScanThreads - 1) / kScanThreads, nbt), dim3(kScanThreads), 0, s, g, words,
                       B, L);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int nonzero_count(const float* g, const unsigned* given_words, int B, int L, hipStream_t s, bool lagged,
                  const unsigned** words_out, unsigned long long* count_out) {
    const int nbt = (B + 31) / 32;
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) return FFI_ERR_NO_DEVICE;
    const size_t head = (size_t)kCountBlocks * sizeof(unsigned long long);           // block counts
    const size_t words_bytes = (size_t)nbt * L * sizeof(unsigned);
    unsigned char* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsNonzero, head + (given_words ? 0 : words_bytes), (void**)&ws));
    unsigned long long* block_counts = reinterpret_cast<unsigned long long*>(ws);
    const unsigned* words = given_words;
    if (!given_words) {
        unsigned* scanned = reinterpret_cast<unsigned*>(ws + head);
        FFI_TRY(launch_nonzero_scan(g, scanned, B, L, s));
        words = scanned;
    }
    *words_out = words;
    std::lock_guard<std::mutex> lock(g_count_mutex);
    CountSlot* slot = nullptr;
    for (CountSlot& c : g_count_slots)
        if (c.device == dev && c.stream == s) slot = &c;
    if (!slot) {
        CountSlot c{dev, s, nullptr, 0, 0};
        if (hipHostMalloc((void**)&c.host, 64) != hipSuccess) { (void)hipGetLastError(); return FFI_ERR_OUT_OF_MEMORY; }
        *c.host = 0;
        g_count_slots.push_back(c);
        slot = &g_count_slots.back();
    }
    // the count of an earlier call of the same shape on this stream, read before this call's kernels can overwrite it
    const bool use_previous = lagged && slot->B == B && slot->L == L;
    const unsigned long long previous = *reinterpret_cast<volatile unsigned long long*>(slot->host);
    hipLaunchKernelGGL(nz_count_kernel, dim3(kCountBlocks), dim3(kScanThreads), 0, s, words, (size_t)nbt * L, block_counts);
    hipLaunchKernelGGL(nz_count_finish_kernel, dim3(1), dim3(64), 0, s, block_counts, kCountBlocks, slot->host);
    FFI_HIP_TRY(hipGetLastError());
    if (use_previous) {
        *count_out = previous;
        return FFI_OK;
    }
    FFI_HIP_TRY(hipStreamSynchronize(s));
    *count_out = *reinterpret_cast<volatile unsigned long long*>(slot->host);
    slot->B = B;
    slot->L = L;
    return FFI_OK;
}

void nonzero_count_forget(int device) {
    std::lock_guard<std::mutex> lock(g_count_mutex);
    for (CountSlot& c : g_count_slots)
        if (c.device == device) { c.B = 0; c.L = 0; }
}

int launch_weight_grad_sparse(const float* x, const int32_t* idx, const float* g, const unsigned* words, float* gw,
                              float* bias_grad, unsigned char* active, const Dims& d, hipStream_t s) {
    const int nbt = (d.B + 31) / 32;
    const int nblk = (d.L + 63) / 64;
    const int blocks = std::max(1, std::min((nblk + 3) / 4, device_cu_count() * 8));
    // byte strides of x along the batch and along the features
    const unsigned xsb = (d.tp ? 1u : (unsigned)d.N) * 4u, xsn = (d.tp ? (unsigned)d.B : 1u) * 4u;
    const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)gw | (uintptr_t)idx) % 16 == 0);
#define FFI_LAUNCH_WS(V, Z)                                                                                                  \
    hipLaunchKernelGGL((wgrad_sparse_kernel<V, Z>), dim3(blocks), dim3(256), 0, s, x, xsb, xsn, idx, g, words, gw, bias_grad, active, \
                       d.B, d.N, d.L, d.K, nbt)
    if (active == nullptr) { if (vec4) FFI_LAUNCH_WS(true, true); else FFI_LAUNCH_WS(false, true); }
    else                   { if (vec4) FFI_LAUNCH_WS(true, false); else FFI_LAUNCH_WS(false, false); }
#undef FFI_LAUNCH_WS
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

bool sparse_weight_grad_fits(int B, int N) { return (unsigned long long)B * (unsigned long long)N < (1ull << 30); }

bool sparse_input_grad_fits(int N, int K) { return N <= kSparseMaxFeatures && K <= 65535; }

int launch_input_grad_sparse(const int32_t* idx, const float* w, const float* g, const unsigned* words, float* gx,
                             const Dims& d, hipStream_t s) {
    const int nbt = (d.B + 31) / 32;
    const int nwords = (d.L + 63) / 64;
    // label segments per sample: enough workgroups to fill the GPU, each with at least one round of words
    int S = std::max(1, (4 * device_cu_count() + d.B - 1) / d.B);
    S = std::max(1, std::min(S, (nwords + kSgWaves * 64 - 1) / (kSgWaves * 64)));
    const int words_per_seg = (nwords + S - 1) / S;
    S = (nwords + words_per_seg - 1) / words_per_seg;
    const size_t bits_bytes = (size_t)d.B * nwords * sizeof(unsigned long long);
    const size_t partial_bytes = (size_t)S * d.B * d.N * sizeof(float);
    unsigned char* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsPartials, bits_bytes + partial_bytes, (void**)&ws));
    unsigned long long* bits = reinterpret_cast<unsigned long long*>(ws);
    float* partial = reinterpret_cast<float*>(ws + bits_bytes);
    hipLaunchKernelGGL(nz_transpose_kernel, dim3((nwords + 3) / 4, nbt), dim3(kScanThreads), 0, s, words, bits, d.B, d.L, nwords);
    FFI_HIP_TRY(hipGetLastError());
    const size_t lds = (size_t)kSgWaves * d.N * sizeof(float);
    const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)w | (uintptr_t)idx) % 16 == 0);
    if (vec4) {
        FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_sparse_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(igrad_sparse_kernel<true>, dim3(d.B * S), dim3(kSgThreads), lds, s, bits, nwords, idx, w, g, partial, d.B,
                           d.N, d.L, d.K, S, words_per_seg);
    } else {
        FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_sparse_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(igrad_sparse_kernel<false>, dim3(d.B * S), dim3(kSgThreads), lds, s, bits, nwords, idx, w, g, partial, d.B,
                           d.N, d.L, d.K, S, words_per_seg);
    }
    FFI_HIP_TRY(hipGetLastError());
    const size_t total = (size_t)d.B * d.N;
    hipLaunchKernelGGL(igrad_sparse_reduce_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, partial, S, d.B, d.N,
                       gx, d.tp ? 1 : 0);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
