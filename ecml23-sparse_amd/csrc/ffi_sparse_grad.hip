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
//   wgrad_sparse_kernel     a wavefront lists the labels of its block that have a set bit, then lane <-> listed
//                           label: every lane walks the set bits of its own label and keeps 32 sums (one chunk of
//                           connections) in registers; labels with many set bits are done by the whole wavefront
//                           afterwards, lane <-> connection; rows of labels without a set bit come out as zeros
//   igrad_sparse_kernel     one workgroup per (sample, label segment): a wavefront lists the set bits of a chunk of
//                           the sample's bit row, every lane takes listed labels and adds g * w of the label's
//                           connections into per-wavefront accumulators gx[n] in LDS (LDS float adds issued in a
//                           fixed order)
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
    const size_t stride = (size_t)gridDim.x * kScanThreads;
    size_t i = (size_t)blockIdx.x * kScanThreads + threadIdx.x;
    for (; i + 3 * stride < n; i += 4 * stride) {       // four loads in flight
        const unsigned a0 = words[i], a1 = words[i + stride], a2 = words[i + 2 * stride], a3 = words[i + 3 * stride];
        c += __popc(a0) + __popc(a1) + __popc(a2) + __popc(a3);
    }
    for (; i < n; i += stride) c += __popc(words[i]);
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

__global__ __launch_bounds__(kCountBlocks) void nz_count_finish_kernel(const unsigned long long* __restrict__ block_counts, int n,
                                                                       unsigned long long* __restrict__ host_count) {
    __shared__ unsigned long long red[kCountBlocks / 64];
    unsigned long long t = (int)threadIdx.x < n ? block_counts[threadIdx.x] : 0ull;       // n <= kCountBlocks
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = t;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long all = 0;
        for (int i = 0; i < kCountBlocks / 64; ++i) all += red[i];
        *host_count = all;                              // pinned host memory: the host reads it after the stream has drained
    }
}

// One wavefront per (batch tile t, kTransposeBlocks blocks of 64 labels): bits[32 t + i][blk] = bit i of the block's 64
// words.  Each half of the wavefront transposes its 32 x 32 bit matrix in five exchange steps between lanes (blocks of
// 16, 8, 4, 2, 1 swapped across the diagonal); lane i < 32 then holds sample i's bits of labels 0..31 and lane 32 + i those
// of labels 32..63.  The words of all blocks are requested before the first is used.
constexpr int kTransposeBlocks = 16;
__global__ __launch_bounds__(kScanThreads) void nz_transpose_kernel(const unsigned* __restrict__ words,
                                                                    unsigned long long* __restrict__ bits, int B, int L,
                                                                    int nwords) {
    __shared__ unsigned long long staged[kScanThreads / 64][32][kTransposeBlocks + 1];   // per wavefront: [sample][block]
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int blk0 = (blockIdx.x * (kScanThreads / 64) + wv) * kTransposeBlocks;
    const int t = blockIdx.y;
    if (blk0 >= nwords) return;
    unsigned m[kTransposeBlocks];
#pragma unroll
    for (int q = 0; q < kTransposeBlocks; ++q) {
        const int j = (blk0 + q) * 64 + lane;
        m[q] = words[(size_t)t * L + min(j, L - 1)];
        if (j >= L) m[q] = 0u;
    }
#pragma unroll
    for (int q = 0; q < kTransposeBlocks; ++q) {
        unsigned v = m[q];
#pragma unroll
        for (int step = 0; step < 5; ++step) {
            const int sh = 16 >> step;
            const unsigned low = step == 0 ? 0x0000ffffu : step == 1 ? 0x00ff00ffu : step == 2 ? 0x0f0f0f0fu
                               : step == 3 ? 0x33333333u : 0x55555555u;
            const unsigned other = (unsigned)__shfl_xor((int)v, sh, 64);
            v = (lane & sh) ? ((v & ~low) | ((other & ~low) >> sh)) : ((v & low) | ((other & low) << sh));
        }
        const unsigned upper = (unsigned)__shfl_xor((int)v, 32, 64);
        if (lane < 32) staged[wv][lane][q] = (unsigned long long)v | ((unsigned long long)upper << 32);
    }
    __builtin_amdgcn_wave_barrier();            // (LDS operations of a wavefront complete in order)
    // a sample's kTransposeBlocks words are neighbours in its bit row: 128-byte pieces, four samples per store
    const int q = lane & (kTransposeBlocks - 1);
#pragma unroll
    for (int r = 0; r < 32 / (64 / kTransposeBlocks); ++r) {
        const int i = r * (64 / kTransposeBlocks) + lane / kTransposeBlocks;
        const int b = 32 * t + i;
        if (b < B && blk0 + q < nwords) bits[(size_t)b * nwords + blk0 + q] = staged[wv][i][q];
    }
}

constexpr int kHeavyBits = 12;     // labels with more set bits than this are left to the whole wavefront

// x is addressed as x[b * xsb + n * xsn] (either layout; byte strides), through a buffer resource with 32-bit
// offsets: batch * num_features * 4 < 2^32, checked by the launcher.
// ZERO_FILL == true: rows of labels without a set bit are written as zeros.
// ZERO_FILL == false: those rows are left alone and active[j] (one byte per label) says which rows were written:
// for a consumer that does not want to read 4 * K bytes of zeros per idle label.
constexpr int kWsLabelsPerLane = 4;
constexpr int kWsBlock = 64 * kWsLabelsPerLane;      // labels a wavefront looks at in one go

template <bool VEC4, bool ZERO_FILL>
__global__ __launch_bounds__(256, 4) void wgrad_sparse_kernel(const float* __restrict__ x, unsigned xsb, unsigned xsn,
                                                              const int32_t* __restrict__ idx, const float* __restrict__ g,
                                                              const unsigned* __restrict__ words, float* __restrict__ gw,
                                                              float* __restrict__ bias_grad,
                                                              unsigned char* __restrict__ active, int B, int N, int L,
                                                              int K, int nbt) {
    // per wavefront: the labels of its block that have a set bit, as (set bits << 8) | offset in the block.  Most labels
    // have none when the gradient is sparse; the lanes then work on the compacted list, not on 64 neighbouring labels of
    // which a few are busy.
    __shared__ unsigned active_list[4][kWsBlock];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int wave = blockIdx.x * 4 + wv;
    const int nwaves = gridDim.x * 4;
    const int nblk = (L + kWsBlock - 1) / kWsBlock;
    const unsigned tail = (B & 31) ? (1u << (B & 31)) - 1u : 0xffffffffu;   // bits past the batch are ignored
    const buffer_rsrc xr = make_rsrc(x, (size_t)B * (size_t)N * sizeof(float));
    unsigned* mylist = active_list[wv];
    for (int blk = wave; blk < nblk; blk += nwaves) {
        const int block_base = blk * kWsBlock;
        int cnts[kWsLabelsPerLane];
#pragma unroll
        for (int q = 0; q < kWsLabelsPerLane; ++q) cnts[q] = 0;
        for (int t = 0; t < nbt; ++t) {
#pragma unroll
            for (int q = 0; q < kWsLabelsPerLane; ++q) {
                unsigned m = words[(size_t)t * L + min(block_base + q * 64 + lane, L - 1)];
                if (t == nbt - 1) m &= tail;
                cnts[q] += __popc(m);
            }
        }
        int total = 0;
#pragma unroll
        for (int q = 0; q < kWsLabelsPerLane; ++q) {
            const int base = block_base + q * 64;
            if (base >= L) break;                                   // wave-uniform
            const int rows = min(64, L - base);
            const bool mine = lane < rows;
            const int cnt = cnts[q];
            if (ZERO_FILL) {
                // rows of labels without a set bit: zeros, written by the whole wavefront (the rows of 64 neighbouring
                // labels are contiguous in gw).  The row of 16-byte element e is e / (K/4), formed in floating point
                // (exact here: e + 0.5 is at least 0.5 / (K/4) away from a multiple).
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
                active[base + lane] = cnt != 0;
            }
            if (bias_grad != nullptr && mine && cnt == 0) bias_grad[base + lane] = 0.f;
            const bool busy = mine && cnt > 0;
            const unsigned long long bal = __ballot(busy);
            if (busy) mylist[total + __popcll(bal & ((1ull << lane) - 1ull))] = ((unsigned)cnt << 8) | (unsigned)(q * 64 + lane);
            total += __popcll(bal);
        }
        __builtin_amdgcn_wave_barrier();        // (LDS operations of a wavefront complete in order)
        for (int e0 = 0; e0 < total; e0 += 64) {
        const bool mine = e0 + lane < total;
        const unsigned entry = mylist[min(e0 + lane, total - 1)];
        const int j = block_base + (int)(entry & 255u);
        const int cnt = (int)(entry >> 8);
        const bool heavy = cnt > kHeavyBits;
        const bool light = mine && !heavy;
        // ---- every lane its own label ----
        float gsum = 0.f;
        for (int k0 = 0; k0 < K; k0 += 32) {
            unsigned ids[32];
            if (light) {
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
                    mw[u] = (light && t < nbt) ? words[(size_t)t * L + j] : 0u;
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
            if (light) {
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
            const int jh = __builtin_amdgcn_readlane(j, r);
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
}

constexpr int kSgThreads = 512;
constexpr int kSgWaves = kSgThreads / 64;

constexpr int kSgWordsPerLane = 8;
constexpr int kSgChunk = 64 * kSgWordsPerLane;      // words of a bit row a wavefront takes in one go: 32,768 labels
constexpr int kSgList = 512;                        // set bits of a chunk that a wavefront can list

// One workgroup per (sample, label segment).  A wavefront takes its share of the sample's bit row in chunks of
// kSgChunk words, lists the labels of the chunk's set bits in LDS (when the gradient is sparse most words are empty:
// the lanes then work on the list, not each on its own word), and every lane adds g * w of its label's connections
// (a 32-connection chunk at a time) into the wavefront's own accumulators gx[n] in LDS.  A chunk with more set
// bits than the list holds is walked word by word instead.  No barriers inside the walk; the order of the adds is
// fixed by the lane assignment.  The wavefronts' accumulators are summed in ascending order at the end.
template <bool VEC4>
__global__ __launch_bounds__(kSgThreads) void igrad_sparse_kernel(const unsigned long long* __restrict__ bits, int nwords,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w, const float* __restrict__ g,
                                                                  float* __restrict__ partial, int B, int N, int L, int K,
                                                                  int S, int words_per_seg) {
    extern __shared__ __align__(16) unsigned char sg_lds[];
    float* acc = reinterpret_cast<float*>(sg_lds);                                        // [kSgWaves][N]
    int* lists = reinterpret_cast<int*>(acc + (size_t)kSgWaves * N);                      // [kSgWaves][kSgList]
    const int b = blockIdx.x / S, seg = blockIdx.x % S;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int i = threadIdx.x; i < kSgWaves * N; i += kSgThreads) acc[i] = 0.f;
    __syncthreads();
    const int w_begin = seg * words_per_seg;
    const int w_end = min(w_begin + words_per_seg, nwords);
    const unsigned long long* row = bits + (size_t)b * nwords;
    const float* grow = g + (size_t)b * L;
    float* myacc = acc + (size_t)wv * N;
    int* mylist = lists + wv * kSgList;
    // g[b, j] times the weights of label j, added at the label's columns
    auto add_label = [&](int j) {
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
    };
    for (int c0 = w_begin + wv * kSgChunk; c0 < w_end; c0 += kSgWaves * kSgChunk) {
        unsigned long long m[kSgWordsPerLane];
        int mine = 0;
#pragma unroll
        for (int q = 0; q < kSgWordsPerLane; ++q) {
            const int wi = c0 + q * 64 + lane;
            m[q] = wi < w_end ? row[wi] : 0ull;
            mine += __popcll(m[q]);
        }
        int upto = mine;                                   // inclusive prefix sum over the lanes
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int t = __shfl_up(upto, off, 64);
            if (lane >= off) upto += t;
        }
        const int total = __builtin_amdgcn_readlane(upto, 63);
        if (total == 0) continue;
        if (total <= kSgList) {
            int at = upto - mine;
#pragma unroll
            for (int q = 0; q < kSgWordsPerLane; ++q) {
                unsigned long long mm = m[q];
                const int j0 = (c0 + q * 64 + lane) * 64;
                while (mm) {
                    mylist[at++] = j0 + __ffsll((long long)mm) - 1;
                    mm &= mm - 1;
                }
            }
            __builtin_amdgcn_wave_barrier();    // (LDS operations of a wavefront complete in order)
            for (int e = lane; e < total; e += 64) add_label(mylist[e]);
            __builtin_amdgcn_wave_barrier();
        } else {
#pragma unroll 1
            for (int q = 0; q < kSgWordsPerLane; ++q) {
                unsigned long long mm = m[q];
                const int j0 = (c0 + q * 64 + lane) * 64;
                while (__ballot(mm != 0)) {
                    if (mm) {
                        const int j = j0 + __ffsll((long long)mm) - 1;
                        mm &= mm - 1;
                        add_label(j);
                    }
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
    hipLaunchKernelGGL(nz_count_finish_kernel, dim3(1), dim3(kCountBlocks), 0, s, block_counts, kCountBlocks, slot->host);
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
    const int nblk = (d.L + kWsBlock - 1) / kWsBlock;
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
    // label segments per sample: a chunk of words for every wavefront of a workgroup, more segments only as far as
    // the GPU would otherwise not be filled (a segment costs a set of LDS accumulators to clear and to sum)
    const int chunks = (nwords + kSgChunk - 1) / kSgChunk;
    const int s_full = (chunks + kSgWaves - 1) / kSgWaves;
    const int s_fill = (2 * device_cu_count() + d.B - 1) / d.B;
    int S = std::max(1, std::max(s_full, std::min(s_fill, chunks)));
    const int words_per_seg = (nwords + S - 1) / S;
    S = (nwords + words_per_seg - 1) / words_per_seg;
    const size_t bits_bytes = (size_t)d.B * nwords * sizeof(unsigned long long);
    const size_t partial_bytes = (size_t)S * d.B * d.N * sizeof(float);
    unsigned char* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsPartials, bits_bytes + partial_bytes, (void**)&ws));
    unsigned long long* bits = reinterpret_cast<unsigned long long*>(ws);
    float* partial = reinterpret_cast<float*>(ws + bits_bytes);
    hipLaunchKernelGGL(nz_transpose_kernel, dim3((nwords + 4 * kTransposeBlocks - 1) / (4 * kTransposeBlocks), nbt), dim3(kScanThreads), 0, s, words, bits, d.B, d.L, nwords);
    FFI_HIP_TRY(hipGetLastError());
    const size_t lds = (size_t)kSgWaves * d.N * sizeof(float) + (size_t)kSgWaves * kSgList * sizeof(int);
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
