// Column-ordered view ("plan") of a lookup matrix, built on the device.
//
// The input gradient sums, for every input column n, over all connections (j,k) with
// lookup[j,k] == n.  The plan lists those connections column by column so that they can be walked
// sequentially, without atomics, in an order that never changes from run to run.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>
#include <cstring>
#include <functional>

#include <rocprim/device/device_radix_sort.hpp>
#include <rocprim/iterator/counting_iterator.hpp>

namespace ffi {
namespace {

constexpr int kBlock = 256;
constexpr int kFingerprintBlocks = 1024;                 // workgroups of the fingerprint kernel (at most)
constexpr int kScratchWords = 8 + 2 * kFingerprintBlocks;  // plan scratch: 8 words for the build, then fingerprint partial sums

__device__ __forceinline__ unsigned mix32(unsigned v) {
    v ^= v >> 16; v *= 0x7feb352du;
    v ^= v >> 15; v *= 0x846ca68bu;
    v ^= v >> 16;
    return v;
}

// Order-independent 64-bit content fingerprint: sum over positions p of mix(id_p + p * odd), plus
// the number of ids outside [0,N).  Every workgroup writes its own pair of partial sums (no atomics:
// thousands of adds to one address serialise); the host adds them up.  Four ids per load when the
// array allows it.
__global__ __launch_bounds__(kBlock) void fingerprint_kernel(const int32_t* __restrict__ idx,
                                                              size_t total, unsigned N,
                                                              unsigned long long* __restrict__ out) {
    unsigned long long h = 0;
    unsigned bad = 0;
    const size_t stride = (size_t)gridDim.x * kBlock;
    const size_t tid = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const bool vec = ((uintptr_t)idx & 15) == 0;
    const size_t nvec = vec ? total / 4 : 0;
    const int4* idx4 = reinterpret_cast<const int4*>(idx);
#pragma unroll 4
    for (size_t q = tid; q < nvec; q += stride) {
        const int4 v = idx4[q];
        const unsigned p = (unsigned)(q * 4);
        h += mix32((unsigned)v.x + p * 0x9e3779b1u);
        h += mix32((unsigned)v.y + (p + 1) * 0x9e3779b1u);
        h += mix32((unsigned)v.z + (p + 2) * 0x9e3779b1u);
        h += mix32((unsigned)v.w + (p + 3) * 0x9e3779b1u);
        bad += ((unsigned)v.x >= N) + ((unsigned)v.y >= N) + ((unsigned)v.z >= N) + ((unsigned)v.w >= N);
    }
    for (size_t p = nvec * 4 + tid; p < total; p += stride) {
        const unsigned id = (unsigned)idx[p];
        h += mix32(id + (unsigned)p * 0x9e3779b1u);
        bad += id >= N;
    }
    unsigned long long b64 = bad;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        h += __shfl_down(h, off);
        b64 += __shfl_down(b64, off);
    }
    __shared__ unsigned long long part[2][kBlock / 64];
    if ((threadIdx.x & 63) == 0) { part[0][threadIdx.x >> 6] = h; part[1][threadIdx.x >> 6] = b64; }
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long hs = 0, bs = 0;
#pragma unroll
        for (int i = 0; i < kBlock / 64; ++i) { hs += part[0][i]; bs += part[1][i]; }
        out[2 * blockIdx.x] = hs;
        out[2 * blockIdx.x + 1] = bs;
    }
}

// The same fingerprint, checked on the device.  Workgroups leave their pairs of sums in guard[8 + 2 * block ..]
// (plain stores) and take a ticket from guard[2], the only atomic: a few hundred adds to one address, not
// thousands (those serialise and were measured to triple the kernel's time).  The workgroup that draws the last
// ticket adds the pairs up (integer adds: the total does not depend on the order), compares with guard[3], leaves
// the verdict in guard[4] (1 = content unchanged and every id in range), the sums in guard[5] / guard[6], and
// clears the ticket counter for the next check.
constexpr int kGuardBlock = 1024;
constexpr int kGuardBlocks = 256;                         // workgroups of the guard kernel (at most)
constexpr int kGuardWords = 8 + 2 * kGuardBlocks;
__global__ __launch_bounds__(kGuardBlock) void fingerprint_guard_kernel(const int32_t* __restrict__ idx, size_t total, unsigned N,
                                                                         unsigned long long* __restrict__ guard,
                                                                         unsigned long long* __restrict__ host_mirror,
                                                                         unsigned long long seq) {
    unsigned long long h = 0;
    unsigned bad = 0;
    const size_t stride = (size_t)gridDim.x * kGuardBlock;
    const size_t tid = (size_t)blockIdx.x * kGuardBlock + threadIdx.x;
    const bool vec = ((uintptr_t)idx & 15) == 0;
    const size_t nvec = vec ? total / 4 : 0;
    const int4* idx4 = reinterpret_cast<const int4*>(idx);
#pragma unroll 4
    for (size_t q = tid; q < nvec; q += stride) {
        const int4 v = idx4[q];
        const unsigned p = (unsigned)(q * 4);
        h += mix32((unsigned)v.x + p * 0x9e3779b1u);
        h += mix32((unsigned)v.y + (p + 1) * 0x9e3779b1u);
        h += mix32((unsigned)v.z + (p + 2) * 0x9e3779b1u);
        h += mix32((unsigned)v.w + (p + 3) * 0x9e3779b1u);
        bad += ((unsigned)v.x >= N) + ((unsigned)v.y >= N) + ((unsigned)v.z >= N) + ((unsigned)v.w >= N);
    }
    for (size_t p = nvec * 4 + tid; p < total; p += stride) {
        const unsigned id = (unsigned)idx[p];
        h += mix32(id + (unsigned)p * 0x9e3779b1u);
        bad += id >= N;
    }
    unsigned long long b64 = bad;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        h += __shfl_down(h, off);
        b64 += __shfl_down(b64, off);
    }
    __shared__ unsigned long long part[2][kGuardBlock / 64];
    __shared__ bool last;
    if ((threadIdx.x & 63) == 0) { part[0][threadIdx.x >> 6] = h; part[1][threadIdx.x >> 6] = b64; }
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long hs = 0, bs = 0;
#pragma unroll
        for (int i = 0; i < kGuardBlock / 64; ++i) { hs += part[0][i]; bs += part[1][i]; }
        // Published with atomic exchanges whose results are waited for, then the ticket: a read-modify-write at
        // device scope is carried out where all XCDs see it, and its returned value says that it has been.  (A
        // fence here would first write back every dirty line of this XCD's L2 -- the scores the forward kernel has
        // just stored among them -- which was measured to cost a third of the kernel's time.)
        const unsigned long long o1 = __hip_atomic_exchange(&guard[8 + 2 * blockIdx.x], hs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned long long o2 = __hip_atomic_exchange(&guard[9 + 2 * blockIdx.x], bs, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned long long one = 1ull;
        asm volatile("" : "+v"(one) : "v"(o1), "v"(o2));       // the ticket is not drawn before both exchanges have returned
        last = __hip_atomic_fetch_add(&guard[2], one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == (unsigned long long)gridDim.x - 1;
    }
    __syncthreads();
    if (!last) return;
    // the last workgroup adds the pairs of all workgroups: one load per thread, all in flight together (a loop of
    // dependent loads per lane costs a memory round trip per step)
    static_assert(kGuardBlocks <= kGuardBlock, "one thread per pair");
    unsigned long long hs = 0, bs = 0;
    if (threadIdx.x < gridDim.x) {
        hs = __hip_atomic_fetch_add(&guard[8 + 2 * threadIdx.x], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        bs = __hip_atomic_fetch_add(&guard[9 + 2 * threadIdx.x], 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        hs += __shfl_down(hs, off);
        bs += __shfl_down(bs, off);
    }
    __syncthreads();                                       // (thread 0 has read part[] above)
    if ((threadIdx.x & 63) == 0) { part[0][threadIdx.x >> 6] = hs; part[1][threadIdx.x >> 6] = bs; }
    __syncthreads();
    if (threadIdx.x == 0) {
        hs = 0; bs = 0;
#pragma unroll
        for (int i = 0; i < kGuardBlock / 64; ++i) { hs += part[0][i]; bs += part[1][i]; }
        const unsigned long long verdict = (hs == guard[3] && bs == 0) ? 1ull : 0ull;
        guard[5] = hs;
        guard[6] = bs;
        guard[4] = verdict;
        guard[2] = 0;
        // For the host, one word in pinned host memory: (number of this check << 2) | (verdict << 1) | (bad ids seen).
        // The host polls that word; neither a copy command nor an event is enqueued behind the kernel (an event
        // record between two kernels was measured to open a 6-us gap in front of the second).
        __hip_atomic_store(host_mirror, (seq << 2) | (verdict << 1) | (bs != 0 ? 1ull : 0ull), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// ---- tiled form ---------------------------------------------------------------------------------

// Order of a column's slots inside a tile.  The kernel that walks the plan reads, per slot, the
// 128-byte LDS row of the slot's label; rows of even labels sit in one half of the LDS banks, rows
// of odd labels in the other, and the LDS serves 16 lanes per clock only if 8 of them read each
// half.  So the lanes whose id has bit 3 clear walk their column as even, odd, even, ... labels
// and the lanes with bit 3 set as odd, even, odd, ...: slot 2t holds the t-th label of the lane's
// first parity, slot 2t+1 the t-th label of the other parity, holes are padding slots that point
// at an all-zero row of the right parity.  Inside a parity class positions ascend.
__device__ __forceinline__ unsigned parity_first(unsigned thread) { return (thread >> 3) & 1u; }       // parity walked at even slots
__device__ __forceinline__ unsigned column_slots(unsigned thread, unsigned even, unsigned odd) {
    const unsigned first = parity_first(thread) ? odd : even, second = parity_first(thread) ? even : odd;
    return max(first ? 2u * first - 1u : 0u, 2u * second);
}

// Which LDS row of the walking kernel's tile each label is staged into (rowpos[j], inside the label's tile).
// The bank half a row lies in is the parity of its row number, and a column is walked fastest when its labels
// split evenly between the halves (see above: every hole costs a slot).  The label's own parity would split a
// column's labels like coin flips (about sqrt(n) excess); here the labels of a tile are taken in ascending order
// and each goes to the half that the columns it feeds have used less so far (weighted sum over its connections
// of even-count minus odd-count of the column), which keeps the columns that matter close to an even split.
// Rows of a half are handed out in ascending order, at most `cap` per half.  One workgroup per tile; the tile's
// column ids are staged in LDS, one wavefront then decides label after label (lane <-> connection).
// (`col_lo`: the plan covers the columns [col_lo, col_lo + ncols) only; connections into other columns are left out)
// (`all_columns_count`: plans that hand the columns to threads by length -- there every column is about as long as the
// longest of its slice, so every column's balance weighs the same)
__global__ __launch_bounds__(256) void tile_color_kernel(const int32_t* __restrict__ idx, int L, int K, int tile_labels, int cap,
                                                         int ncols, unsigned short* __restrict__ rowpos, int col_lo,
                                                         int all_columns_count) {
    extern __shared__ int color_lds[];
    // (entry `ncols` of both: where connections into columns outside the window go -- weight 0, so they never count)
    int* imb = color_lds;                                                        // [ncols + 1] even minus odd labels per column
    // The tile's column ids, three 10-bit ids per word, a label's ids in W = ceil(K / 3) words of its own, and the weights as
    // 16-bit numbers: with 16-bit ids and 32-bit weights a tile of 582 labels x fan-in 32 took 44 KB of LDS, three workgroups per
    // CU and two rounds for 1,152 tiles; now 31 KB, five workgroups per CU, all tiles at once (the work of a tile is one
    // wavefront's sequential loop).
    const int W = (K + 2) / 3;
    unsigned* ids3 = reinterpret_cast<unsigned*>(color_lds + ncols + 1);         // [tile_labels * W]
    unsigned short* wt = reinterpret_cast<unsigned short*>(ids3 + (size_t)tile_labels * W);   // [ncols + 1] weight of the column's balance (at most 256)
    const int t = blockIdx.x;
    const int j0 = t * tile_labels;
    const int nl = min(tile_labels, L - j0);
    const int* src = idx + (size_t)j0 * K;
    const unsigned outside = (unsigned)min(ncols, 1023);                          // (windows are at most 640 columns wide; a single window has no ids outside)
    for (int i = threadIdx.x; i <= ncols; i += 256) { imb[i] = 0; wt[i] = 0; }
    __syncthreads();
    for (int wi = threadIdx.x; wi < nl * W; wi += 256) {
        const int jl = wi / W, k0 = 3 * (wi - jl * W);
        unsigned word = 0;
#pragma unroll
        for (int i = 0; i < 3; ++i) {
            unsigned c = outside;
            if (k0 + i < K) {
                const unsigned v = (unsigned)(src[jl * K + k0 + i] - col_lo);
                if (v < (unsigned)ncols) { c = v; atomicAdd(&imb[v], 1); }       // column lengths first (in imb: the LDS adds whole words)
            } else {
                c = (unsigned)min(ncols, 1023);                                  // (behind the label's last id: never read)
            }
            word |= c << (10 * i);
        }
        ids3[wi] = word;
    }
    __syncthreads();
    // Only the longest columns of a slice (64 columns, one wavefront of the walking kernel) set its number of slot
    // rows, so their balance counts most: weight = 256 * (length / longest of the slice)^8.
    for (int c = threadIdx.x; c < ncols; c += 256) {
        const int len = imb[c];
        imb[c] = 0;
        int longest = len;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) longest = max(longest, __shfl_xor(longest, off, 64));
        float r = longest > 0 ? (float)len / (float)longest : 0.f;
        r *= r; r *= r; r *= r;
        wt[c] = (unsigned short)(all_columns_count ? (len > 0 ? 256 : 0) : (int)(256.f * r));
    }
    __syncthreads();
    if (threadIdx.x >= 64) return;
    const int lane = threadIdx.x;
    unsigned char* half = reinterpret_cast<unsigned char*>(wt + ncols + 2);      // [tile_labels] the half each label goes to
    // column of connection k of label jl
    auto id_of = [&](int jl, int k) {
        const int q = (k * 43691) >> 17;                                         // k / 3 for k < 2^15
        return (int)((ids3[jl * W + q] >> (10 * (k - 3 * q))) & 1023u);
    };
    int placed[2] = {0, 0};
    for (int jl = 0; jl < nl; ++jl) {
        int sum = 0;
        for (int k = lane; k < K; k += 64) { const int c = id_of(jl, k); sum += wt[c] * imb[c]; }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        int color = sum > 0 ? 1 : (sum < 0 ? 0 : (placed[1] < placed[0] ? 1 : 0));
        if (placed[color] >= cap) color ^= 1;
        const int delta = color ? -1 : 1;
        for (int k = lane; k < K; k += 64) atomicAdd(&imb[id_of(jl, k)], delta);   // a column may occur twice in a label
        if (lane == 0) half[jl] = (unsigned char)color;
        ++placed[color];
    }
    // Second sweep: every label is taken out and put back into the half its columns now ask for -- the first sweep placed
    // the early labels knowing nothing of the later ones.  (Measured on uniformly drawn ids, 586-label tiles of fan-in 32
    // over 768 columns: slot rows 1.528 -> 1.514 per connection, where columns of unconstrained order would need 1.490.)
    for (int jl = 0; jl < nl; ++jl) {
        const int old = half[jl];                         // (written by lane 0 above; LDS accesses of a wavefront are in order)
        const int back = old ? 1 : -1;
        for (int k = lane; k < K; k += 64) atomicAdd(&imb[id_of(jl, k)], back);
        int sum = 0;
        for (int k = lane; k < K; k += 64) { const int c = id_of(jl, k); sum += wt[c] * imb[c]; }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
        int color = sum > 0 ? 1 : (sum < 0 ? 0 : old);
        if (color != old && placed[color] >= cap) color = old;
        const int delta = color ? -1 : 1;
        for (int k = lane; k < K; k += 64) atomicAdd(&imb[id_of(jl, k)], delta);
        if (color != old) { --placed[old]; ++placed[color]; if (lane == 0) half[jl] = (unsigned char)color; }
    }
    // rows of a half are handed out in ascending label order
    if (lane == 0) {
        int next[2] = {0, 0};
        for (int jl = 0; jl < nl; ++jl) {
            const int color = half[jl];
            rowpos[j0 + jl] = (unsigned short)(2 * next[color] + color);
            ++next[color];
        }
    }
}

// Which column each thread of the walking kernel takes in each tile (plans with `colperm`).  A wavefront walks as many
// slot rows as the longest of its 64 columns needs, so with thread t <-> column t every slice pays for its longest
// column (about 1.5 slot rows per connection for ids drawn uniformly); here the tile's columns are sorted by the slots
// they need (stable: equal columns stay in index order), cut into blocks of 64 about equally long columns, and the
// blocks dealt to the wavefronts so that the wavefronts of a SIMD (wave, wave + 4, wave + 8, ...) have about the same
// rows in total: longest block first, each to the SIMD with the least so far that still has a wavefront free.
// One workgroup per tile, one thread per column (columns up to the workgroup size exist for this purpose: the ones
// beyond the input's width have no connections).  Also stores the slot rows of each slice, as tile_count_kernel does
// for plans without the permutation.  LDS: counts [2][threads], keys [threads].
__global__ void tile_perm_kernel(const int32_t* __restrict__ idx, const unsigned short* __restrict__ rowpos, int L, int K,
                                 int tile_labels, int col_lo, unsigned short* __restrict__ colperm, unsigned* __restrict__ slice_len) {
    extern __shared__ __align__(16) unsigned perm_lds[];
    unsigned* cnt = perm_lds;                  // [2][threads]: labels in even rows, labels in odd rows
    const int t = blockIdx.x, nthreads = blockDim.x, nslices = nthreads >> 6;
    unsigned* key = cnt + 2 * nthreads;        // [threads]
    __shared__ unsigned short wave_of_block[16];
    __shared__ unsigned slice_rows[16];
    if (threadIdx.x < 16) slice_rows[threadIdx.x] = 0u;
    cnt[threadIdx.x] = 0;
    cnt[nthreads + threadIdx.x] = 0;
    __syncthreads();
    const int j0 = t * tile_labels;
    const int nl = min(tile_labels, L - j0);
    const int* src = idx + (size_t)j0 * K;
    const int total = nl * K;
    for (int e = threadIdx.x; e < total; e += nthreads) {
        const unsigned c = (unsigned)(src[e] - col_lo);
        if (c < (unsigned)nthreads) atomicAdd(&cnt[(rowpos[j0 + e / K] & 1u) * nthreads + c], 1u);
    }
    __syncthreads();
    // (the slots a column needs depend by one on the lane it gets; the larger of the two)
    const unsigned mine = 2u * max(cnt[threadIdx.x], cnt[nthreads + threadIdx.x]);
    key[threadIdx.x] = mine;
    __syncthreads();
    // place among the columns in descending order of the key: columns with a larger key, and equal ones before this one
    unsigned place = 0;
    for (int c0 = 0; c0 < nthreads; c0 += 4) {
        const uint4 k4 = *reinterpret_cast<const uint4*>(key + c0);       // (the same address in every lane: one broadcast read)
        place += (k4.x > mine || (k4.x == mine && c0 + 0 < (int)threadIdx.x)) ? 1u : 0u;
        place += (k4.y > mine || (k4.y == mine && c0 + 1 < (int)threadIdx.x)) ? 1u : 0u;
        place += (k4.z > mine || (k4.z == mine && c0 + 2 < (int)threadIdx.x)) ? 1u : 0u;
        place += (k4.w > mine || (k4.w == mine && c0 + 3 < (int)threadIdx.x)) ? 1u : 0u;
    }
    __syncthreads();
    // key[] now by place: the first of each block of 64 is the block's longest column
    key[place] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned sum[4] = {0u, 0u, 0u, 0u};
        int used[4] = {0, 0, 0, 0};
        for (int b = 0; b < nslices; ++b) {
            int best = -1;
            for (int q = 0; q < 4; ++q) {
                if (q + 4 * used[q] >= nslices) continue;                 // no wavefront left on that SIMD
                if (best < 0 || sum[q] < sum[best]) best = q;
            }
            wave_of_block[b] = (unsigned short)(best + 4 * used[best]);
            sum[best] += (used[best] == 0 ? 3u : 1u) * key[b * 64];      // (a SIMD's longest wavefront ends up walking alone)
            ++used[best];
        }
    }
    __syncthreads();
    const unsigned thread = wave_of_block[place >> 6] * 64u + (place & 63u);
    colperm[(size_t)t * nthreads + thread] = (unsigned short)threadIdx.x;
    // the slot rows of each slice: those of its longest column, now that every column knows its lane
    atomicMax(&slice_rows[thread >> 6], column_slots(thread, cnt[threadIdx.x], cnt[nthreads + threadIdx.x]));
    __syncthreads();
    if ((int)threadIdx.x < nslices) slice_len[(size_t)t * nslices + threadIdx.x] = slice_rows[threadIdx.x];
}

// One workgroup per label tile, one thread per column.  Counts the tile's connections per column
// and bank half of the label's row (integer LDS atomics: order-independent), stores the slot count of the
// longest column of each slice.
__global__ void tile_count_kernel(const int32_t* __restrict__ idx, const unsigned short* __restrict__ rowpos, int L, int K,
                                  int tile_labels, unsigned* __restrict__ slice_len, int col_lo) {
    extern __shared__ unsigned cnt[];          // [2][threads]: labels in even rows, labels in odd rows
    const int t = blockIdx.x, nthreads = blockDim.x;
    cnt[threadIdx.x] = 0;
    cnt[nthreads + threadIdx.x] = 0;
    __syncthreads();
    const int j0 = t * tile_labels;
    const int nl = min(tile_labels, L - j0);
    const int* src = idx + (size_t)j0 * K;
    const int total = nl * K;
    for (int e = threadIdx.x; e < total; e += nthreads) {
        const unsigned c = (unsigned)(src[e] - col_lo);
        if (c < (unsigned)nthreads) atomicAdd(&cnt[(rowpos[j0 + e / K] & 1u) * nthreads + c], 1u);
    }
    __syncthreads();
    const unsigned even = cnt[threadIdx.x], odd = cnt[nthreads + threadIdx.x];
    unsigned c = column_slots(threadIdx.x, even, odd);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c = max(c, (unsigned)__shfl_xor((int)c, off));
    if ((threadIdx.x & 63) == 0) slice_len[(size_t)t * (nthreads >> 6) + (threadIdx.x >> 6)] = c;
}

// Exclusive prefix sum of n values into off[0..n] by one workgroup (n is a few thousand).
__global__ __launch_bounds__(1024) void slice_scan_kernel(const unsigned* __restrict__ len, unsigned* __restrict__ off,
                                                           int n, unsigned long long* __restrict__ total_out) {
    __shared__ unsigned long long part[1024];
    const int per = (n + 1023) / 1024;
    const int b = threadIdx.x * per, e = min(b + per, n);
    unsigned long long sum = 0;
    for (int i = b; i < e; ++i) sum += len[i];
    part[threadIdx.x] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned long long run = 0;
        for (int i = 0; i < 1024; ++i) { const unsigned long long v = part[i]; part[i] = run; run += v; }
        *total_out = run;
    }
    __syncthreads();
    unsigned long long run = part[threadIdx.x];
    for (int i = b; i < e; ++i) { off[i] = (unsigned)run; run += len[i]; }
    if (threadIdx.x == 1023) off[n] = (unsigned)(part[1023] + sum);
}

// One workgroup per label tile, one thread per column n.  The tile's column ids pass through LDS
// in chunks; every thread scans them in flat-position order and places the ones equal to its
// column (see column_slots for the order), so the result is deterministic without any sort.
// Per slot: lab16 = LDS row of the label (rowpos), pos16 = position inside the tile's rows of lookup; the
// slots a column leaves empty up to the slice's length become padding: pos16 = pad_pos (kPadPos; in plans whose walking
// kernel keeps the tile's weights in LDS, tile_labels * K: the position of a zero word behind them), lab16 =
// zero_row + parity (all-zero rows).
constexpr int kFillChunk = 8192;
// With `slot32` (plans whose walking kernel keeps the tile's weights in LDS) the two go into one word per slot,
// (position << 17) | (LDS row << 7): one load per slot, the row's byte offset already in place.
__global__ void tile_fill_kernel(const int32_t* __restrict__ idx, const unsigned short* __restrict__ rowpos, int L, int K,
                                 int tile_labels, int zero_row, const unsigned* __restrict__ slice_off,
                                 unsigned short* __restrict__ lab16, unsigned short* __restrict__ pos16, unsigned pad_pos,
                                 unsigned* __restrict__ slot32, int col_lo, const unsigned short* __restrict__ colperm) {
    __shared__ __align__(16) int keys[kFillChunk];
    __shared__ unsigned short rows_of[kPlanTileLabels];     // LDS row of each label of the tile
    const int t = blockIdx.x, nthreads = blockDim.x;
    const int j0 = t * tile_labels;
    const int nl = min(tile_labels, L - j0);
    const int* src = idx + (size_t)j0 * K;
    const int total = nl * K;
    const int mine = (colperm != nullptr ? (int)colperm[(size_t)blockIdx.x * blockDim.x + threadIdx.x] : (int)threadIdx.x) + col_lo;
    const size_t sl = (size_t)t * (nthreads >> 6) + (threadIdx.x >> 6);
    const size_t row0 = slice_off[sl];
    const unsigned rows = slice_off[sl + 1] - slice_off[sl];
    const size_t at = row0 * 64 + (threadIdx.x & 63);
    auto put = [&](size_t r, unsigned lab, unsigned pos) {
        if (slot32 != nullptr) slot32[at + r * 64] = (pos << 17) | (lab << 7);
        else { lab16[at + r * 64] = (unsigned short)lab; pos16[at + r * 64] = (unsigned short)pos; }
    };
    const unsigned first = parity_first(threadIdx.x);
    for (int i = threadIdx.x; i < nl; i += nthreads) rows_of[i] = rowpos[j0 + i];
    // padding everywhere first; the thread's own slots are then overwritten (same thread: ordered)
    for (unsigned r = 0; r < rows; ++r) {
        put(r, (unsigned)zero_row + ((r & 1u) ^ first), pad_pos);
    }
    unsigned seen[2] = {0u, 0u};  // labels of each parity placed so far
    int label = 0, kk = 0;        // label and connection slot of the entry under the cursor
    for (int c0 = 0; c0 < total; c0 += kFillChunk) {
        const int n = min(kFillChunk, total - c0);
        __syncthreads();
        for (int e = threadIdx.x; e < n; e += nthreads) keys[e] = src[c0 + e];
        __syncthreads();
        for (int e = 0; e < n; ++e) {
            if (keys[e] == mine) {
                const unsigned row = rows_of[label];
                const unsigned par = row & 1u;
                const unsigned t2 = par ? seen[1]++ : seen[0]++;
                const unsigned slot = 2u * t2 + (par ^ first);
                put(slot, row, (unsigned)(c0 + e));
            }
            if (++kk == K) { kk = 0; ++label; }
        }
    }
}

// The same placement without the all-pairs scan, for tiles whose column ids, a bitmap [column][label of the tile]
// and its prefix counts fit in LDS together (every tile of a narrow layer at the fan-ins the weights-in-LDS form
// takes).  Every connection sets the bit of (its column, its label) -- integer OR, order-independent; every column's
// thread then counts, word by word of its bitmap row, the labels in even and in odd LDS rows before that word; and
// every connection finds its own slot from those counts and the bits below its own (its rank among the column's
// connections of the same bank half in ascending flat position: the order tile_fill_kernel produces), so the slots
// are written by threads <-> connections, not by a column's thread scanning for them.  Padding goes to the slots no
// connection takes (a column's thread knows them from its two totals).  A label that lists one column twice sets one
// bit for two connections: such a tile is placed by its columns' threads instead (see below), several times slower.
// Measured at 670,091 labels x fan-in 32 over 768 columns: 6.2 ms -> 0.19 ms without such labels, 1.3 ms with some in every tile.
__global__ void tile_fill_bitmap_kernel(const int32_t* __restrict__ idx, const unsigned short* __restrict__ rowpos, int L, int K,
                                        int tile_labels, int zero_row, const unsigned* __restrict__ slice_off,
                                        unsigned short* __restrict__ lab16, unsigned short* __restrict__ pos16, unsigned pad_pos,
                                        unsigned* __restrict__ slot32, int words, int col_lo,
                                        const unsigned short* __restrict__ colperm) {
    extern __shared__ __align__(16) unsigned fill_lds[];
    const int t = blockIdx.x, nthreads = blockDim.x;
    unsigned* bm = fill_lds;                                                   // [nthreads][words] (words odd: no bank conflicts)
    unsigned* pm = bm + (size_t)nthreads * words;                              // [words] labels staged in odd LDS rows
    unsigned short* pre = reinterpret_cast<unsigned short*>(pm + words);       // [nthreads][words + 1][2] labels before word w, even / odd rows
    unsigned short* rows_of = pre + (size_t)nthreads * (words + 1) * 2;        // [tile_labels]
    unsigned short* ids = rows_of + ((tile_labels + 1) & ~1);                  // [tile_labels * K]
    unsigned short* thread_of = ids + (((size_t)tile_labels * K + 1) & ~(size_t)1);   // [nthreads] the thread that walks each column
    __shared__ unsigned duplicate;
    // (bitmap and prefix counts are kept per column; slices, lanes and slot parities belong to threads)
    const unsigned mycol = colperm != nullptr ? colperm[(size_t)blockIdx.x * blockDim.x + threadIdx.x] : threadIdx.x;
    thread_of[mycol] = (unsigned short)threadIdx.x;
    const int j0 = t * tile_labels;
    const int nl = min(tile_labels, L - j0);
    const int* src = idx + (size_t)j0 * K;
    const int total = nl * K;
    const int nslices = nthreads >> 6;
    if (threadIdx.x == 0) duplicate = 0u;
    for (int i = threadIdx.x; i < nthreads * words; i += nthreads) bm[i] = 0u;
    for (int i = threadIdx.x; i < words; i += nthreads) pm[i] = 0u;
    for (int i = threadIdx.x; i < nl; i += nthreads) rows_of[i] = rowpos[j0 + i];
    for (int e = threadIdx.x; e < total; e += nthreads) {
        const unsigned c = (unsigned)(src[e] - col_lo);                       // (columns outside the plan's window: never matched)
        ids[e] = c < (unsigned)nthreads ? (unsigned short)c : (unsigned short)0xffffu;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nl; i += nthreads)
        if (rows_of[i] & 1u) atomicOr(&pm[i >> 5], 1u << (i & 31));
    {
        // (label of entry e without a division per entry: the thread's entries are nthreads apart)
        int l = (int)threadIdx.x / K, k = (int)threadIdx.x - l * K;
        const int dl = nthreads / K, dk = nthreads - dl * K;
        for (int e = threadIdx.x; e < total; e += nthreads) {
            const unsigned c = ids[e];
            if (c < (unsigned)nthreads) {
                const unsigned bit = 1u << (l & 31);
                if (atomicOr(&bm[(size_t)c * words + (l >> 5)], bit) & bit) duplicate = 1u;
            }
            l += dl; k += dk;
            if (k >= K) { k -= K; ++l; }
        }
    }
    __syncthreads();
    if (duplicate) {
        // (uniform) a label lists a column twice -- rewiring draws such labels all the time -- and the bitmap has one bit
        // for the two connections: here the column's thread walks its bitmap row in ascending label order and scans each
        // label found for the matching connections, which yields every connection, in ascending flat position
        const unsigned mine = mycol;
        const size_t sl = (size_t)t * nslices + (threadIdx.x >> 6);
        const size_t row0 = slice_off[sl];
        const unsigned rows = slice_off[sl + 1] - slice_off[sl];
        const size_t at = row0 * 64 + (threadIdx.x & 63);
        auto put = [&](size_t r, unsigned lab, unsigned pos) {
            if (slot32 != nullptr) slot32[at + r * 64] = (pos << 17) | (lab << 7);
            else { lab16[at + r * 64] = (unsigned short)lab; pos16[at + r * 64] = (unsigned short)pos; }
        };
        const unsigned first = parity_first(threadIdx.x);
        // padding everywhere first; the thread's own slots are then overwritten (same thread: ordered)
        for (unsigned r = 0; r < rows; ++r) put(r, (unsigned)zero_row + ((r & 1u) ^ first), pad_pos);
        unsigned seen[2] = {0u, 0u};
        const unsigned* my = bm + (size_t)mine * words;
        for (int wd = 0; wd < words; ++wd) {
            unsigned bits = my[wd];
            while (bits) {
                const unsigned b = (unsigned)__builtin_ctz(bits);
                bits &= bits - 1u;
                const unsigned l = 32u * (unsigned)wd + b;
                const unsigned row = rows_of[l];
                const unsigned par = row & 1u;
                const unsigned short* lrow = ids + (size_t)l * K;
                auto found = [&](int k) {
                    const unsigned t2 = par ? seen[1]++ : seen[0]++;
                    put(2u * t2 + (par ^ first), row, l * (unsigned)K + (unsigned)k);
                };
                if ((K & 7) == 0 && ((size_t)lrow & 3) == 0) {
                    // eight ids per step, as four words whose halves are compared with the column at once: a half is
                    // equal where (x ^ pattern) has a zero half (the classic "has a zero byte" test, for 16-bit lanes)
                    const unsigned* lrow2 = reinterpret_cast<const unsigned*>(lrow);
                    const unsigned pattern = mine * 0x00010001u;
                    for (int k = 0; k < K; k += 8) {
                        unsigned x[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) x[i] = lrow2[(k >> 1) + i] ^ pattern;
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            if (((x[i] - 0x00010001u) & ~x[i] & 0x80008000u) != 0u) {
                                if ((x[i] & 0xffffu) == 0u) found(k + 2 * i);
                                if ((x[i] >> 16) == 0u) found(k + 2 * i + 1);
                            }
                        }
                    }
                } else {
                    for (int k = 0; k < K; ++k)
                        if (lrow[k] == mine) found(k);
                }
            }
        }
        return;
    }
    // per column: labels in even / odd rows before each word; then the column's padding slots
    {
        const unsigned mine = mycol;
        const unsigned* my = bm + (size_t)mine * words;
        unsigned short* mp = pre + (size_t)mine * (words + 1) * 2;
        unsigned ev = 0, od = 0;
        for (int wd = 0; wd < words; ++wd) {
            mp[2 * wd] = (unsigned short)ev; mp[2 * wd + 1] = (unsigned short)od;
            const unsigned b = my[wd], o = pm[wd];
            ev += __builtin_popcount(b & ~o); od += __builtin_popcount(b & o);
        }
        const size_t sl = (size_t)t * nslices + (threadIdx.x >> 6);
        const size_t row0 = slice_off[sl];
        const unsigned rows = slice_off[sl + 1] - slice_off[sl];
        const size_t at = row0 * 64 + (threadIdx.x & 63);
        const unsigned first = parity_first(threadIdx.x);
        const unsigned cnt[2] = {ev, od};
        for (unsigned r = 0; r < rows; ++r) {
            const unsigned par = (r & 1u) ^ first;          // bank half this slot belongs to
            if ((r >> 1) >= cnt[par]) {
                const unsigned lab = (unsigned)zero_row + par;
                if (slot32 != nullptr) slot32[at + (size_t)r * 64] = (pad_pos << 17) | (lab << 7);
                else { lab16[at + (size_t)r * 64] = (unsigned short)lab; pos16[at + (size_t)r * 64] = (unsigned short)pad_pos; }
            }
        }
    }
    __syncthreads();
    // per connection: its slot
    {
        int l = (int)threadIdx.x / K, k = (int)threadIdx.x - l * K;
        const int dl = nthreads / K, dk = nthreads - dl * K;
        for (int e = threadIdx.x; e < total; e += nthreads) {
            const unsigned c = ids[e];
            if (c < (unsigned)nthreads) {
                const unsigned row = rows_of[l];
                const unsigned par = row & 1u;
                const int wd = l >> 5;
                const unsigned o = pm[wd];
                const unsigned same = bm[(size_t)c * words + wd] & (par ? o : ~o) & ((1u << (l & 31)) - 1u);
                const unsigned rank = pre[((size_t)c * (words + 1) + wd) * 2 + par] + __builtin_popcount(same);
                const unsigned thr = thread_of[c];
                const unsigned slot = 2u * rank + (par ^ parity_first(thr));
                const size_t at = (size_t)slice_off[(size_t)t * nslices + (thr >> 6)] * 64 + (thr & 63u) + (size_t)slot * 64;
                if (slot32 != nullptr) slot32[at] = ((unsigned)e << 17) | (row << 7);
                else { lab16[at] = (unsigned short)row; pos16[at] = (unsigned short)e; }
            }
            l += dl; k += dk;
            if (k >= K) { k -= K; ++l; }
        }
    }
}

// LDS the bitmap form needs, and may have
constexpr size_t kFillLdsLimit = 160 * 1024 - 64;
inline size_t tile_fill_bitmap_lds(int threads, int tile_labels, int K, int* words_out) {
    const int words = ((tile_labels + 31) / 32) | 1;
    *words_out = words;
    return (size_t)threads * words * sizeof(unsigned) + (size_t)words * sizeof(unsigned) +
           (size_t)threads * (words + 1) * 2 * sizeof(unsigned short) + (size_t)((tile_labels + 1) & ~1) * sizeof(unsigned short) +
           (((size_t)tile_labels * K + 1) & ~(size_t)1) * sizeof(unsigned short) + (size_t)threads * sizeof(unsigned short);
}

// ---- blocked global form ------------------------------------------------------------------------

// col_ptr[n] = first position in the sorted key array whose key is >= n (n in [0,N]; N = number of keys).
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

// Detaches the arrays from the plan.  keep == true (a rebuild follows): their buffers go to the spare list.
void free_spares(ffi_plan* p);
void free_arrays(ffi_plan* p, bool keep = false) {
    if (p->upper != nullptr) {
        // (the second column window's arrays: freed, never kept -- inputs that wide are rare and their plans small)
        free_arrays(p->upper, false);
        free_spares(p->upper);
        delete p->upper;
        p->upper = nullptr;
    }
    p->col_lo = 0; p->col_n = 0;
    for (const ffi_plan::Buffer& b : p->owned) {
        if (keep) p->spare.push_back(b);
        else (void)hipFree(b.ptr);
    }
    p->owned.clear();
    p->rowpos = nullptr;
    p->perm = nullptr; p->col_ptr = nullptr; p->slice_off = nullptr; p->lab16 = nullptr; p->pos16 = nullptr; p->slot32 = nullptr; p->idx16 = nullptr; p->colperm = nullptr;
    p->tiled = false; p->w_in_lds = false; p->total_rows = 0; p->bytes = 0;
}

void free_spares(ffi_plan* p) {
    for (const ffi_plan::Buffer& b : p->spare) (void)hipFree(b.ptr);
    p->spare.clear();
}

// A buffer of `count` elements for one of the plan's arrays: a spare one that fits (and is not more than half as
// large again), else a new allocation with 3 % of headroom, so that the next rebuild's slightly different sizes fit.
template <class T>
bool dev_alloc(ffi_plan* p, T** ptr, size_t count) {
    const size_t need = std::max<size_t>(count, 1) * sizeof(T);
    size_t best = p->spare.size();
    for (size_t i = 0; i < p->spare.size(); ++i)
        if (p->spare[i].bytes >= need && p->spare[i].bytes <= need + need / 2 + 4096 &&
            (best == p->spare.size() || p->spare[i].bytes < p->spare[best].bytes)) best = i;
    if (best != p->spare.size()) {
        *ptr = static_cast<T*>(p->spare[best].ptr);
        p->owned.push_back(p->spare[best]);
        p->spare.erase(p->spare.begin() + best);
        return true;
    }
    const size_t bytes = need + need / 32 + 256;
    void* raw = nullptr;
    if (hipMalloc(&raw, bytes) != hipSuccess) {
        (void)hipGetLastError();
        *ptr = nullptr;
        return false;
    }
    *ptr = static_cast<T*>(raw);
    p->owned.push_back({raw, bytes});
    return true;
}

// Returns a buffer obtained from dev_alloc to the spare list (temporaries of the build).
void dev_release(ffi_plan* p, void* ptr) {
    for (size_t i = 0; i < p->owned.size(); ++i)
        if (p->owned[i].ptr == ptr) {
            p->spare.push_back(p->owned[i]);
            p->owned.erase(p->owned.begin() + i);
            return;
        }
}

}  // namespace

// Labels per tile of the tiled form, and whether the walking kernel keeps the tile's weights in LDS (then the tiles
// are smaller).
int plan_tile_labels(int N, int K, int L, int batch_hint, bool* weights_in_lds) {
    const int threads = ((N + 63) / 64) * 64;
    int TL = std::min((std::min(std::min(kPlanTileLabels, L), threads > 768 ? threads : 2 * threads) + 1) & ~1,
                      (int)((kPadPos - 1) / (unsigned)K) & ~1);
    // Tiles whose weights fit in LDS beside the tile of out_grad: the walking kernel then reads each slot's weight
    // through the slot's word, and the weights need not be brought into slot order first (no permutation kernel, no slot-ordered
    // copy of the weights in memory).
    // Measured (gx pass, 0.2-0.67 M labels, fan-in 8...128, 64...1024 columns), against permutation + walk with the
    // tiles and workgroups per CU that suit each form (tiled_workgroups_per_cu): with up to four batch tiles the form is
    // 5-60 % faster (most where the fan-in exceeds 32); with five to eight batch
    // tiles the tile's weights are staged that many times per tile: at fan-in 32 and below still -1...-8 % with 512 or 768 columns; with 576 to 768
    // columns -5...-13 % at every fan-in from 40 to 128 (one workgroup per CU either way); but +12 % at fan-in
    // 64 / 512 columns against the two-workgroup slot-ordered form, which also wins at 320-448 columns; with sixteen
    // batch tiles -7...+6 %: not taken.
    // The tile: as many labels as fit the LDS with their weights, one label per thread to stage; a thread carries
    // 8 x 16 bytes of the tile's weights in registers across the barrier, what exceeds that is copied behind it.
    // A slot's position inside the tile's weights has 15 bits (the zero word that padding slots read included).
    bool w_in_lds = false;
    const int nbt_hint = (batch_hint + 31) / 32;
    // Measured again once a tile's columns were sorted by length (which the form gets at 384 columns and more): 576 to 768
    // columns at 12 and 16 batch tiles, fan-in 32 and 64: -2...-6 % against the slot-ordered form, so workgroups of more than
    // 512 threads take the form at any batch size.  And at 256 columns and fewer, where several workgroups share a CU in
    // either form (670,091 labels): fan-in 16 -9...-20 % up to eight batch tiles; fan-in 32 -15...-36 % at one and two
    // batch tiles, equal at three, at four -21 % with 192 columns but +8 % with 256 (+16 % at fan-in 64), and +14...+30 %
    // at five to eight batch tiles (128 and 256 columns): from fan-in 32 on the slot-ordered form takes over there.
    const bool by_shape = threads > 512 ? true
                        : threads <= 256 ? (K < 32 ? nbt_hint <= 8 : (nbt_hint <= 3 || (nbt_hint == 4 && threads < 256)))
                                         : (nbt_hint <= 4 || (nbt_hint <= 8 && K <= 32 && threads == 512));
    const bool wanted = batch_hint > 0 && g_options.plan_weights_in_lds >= 0 && (g_options.plan_weights_in_lds > 0 || by_shape);   // (unknown batch size: the form for large batches)
    if (wanted && threads <= 768) {
        int tw = std::min(TL, threads & ~1);
        // (workgroups of at most 256 threads share a CU when there are batch tiles to overlap: tiled_workgroups_per_cu)
        const size_t budget = (threads <= 256 && nbt_hint >= 2) ? kPlanLdsBudget / (size_t)(768 / threads) : kPlanLdsBudget;
        while (tw >= 64 && tiled_lds_bytes(tw, K, true) > budget) tw -= 2;
        while (tw >= 64 && (long long)tw * K >= 32768) tw -= 2;
        // a tile the bitmap fill has the LDS for (its bitmaps grow by whole words of 32 labels) builds five times faster
        // than one it has not; take the next smaller such tile where that costs at most a twentieth of the tile
        int words = 0;
        if (tw >= 64 && tile_fill_bitmap_lds(threads, tw, K, &words) > kFillLdsLimit) {
            const int fits = tw & ~31;
            if (fits >= 64 && fits * 20 >= tw * 19 && tile_fill_bitmap_lds(threads, fits, K, &words) <= kFillLdsLimit) tw = fits;
        }
        // Tiles per workgroup come in whole numbers: the walking kernel runs cus / batch tiles label streams of
        // ceil(tiles / streams) tiles each, and the largest tile can leave the last stream nearly empty, or whole CUs
        // without a stream (670,091 labels in 608-label tiles: 62 streams of 18 tiles on 64 CUs' worth of workgroups).
        // The tile shrinks to what fills every stream with that same number of tiles (582 labels there: 64 x 18); a
        // smaller tile pads a little more per connection, which costs less than the idle streams.  (Workgroups that share
        // a CU are left alone: there the streams outnumber the CUs.)
        if (tw >= 64 && (threads > 256 || nbt_hint < 2)) {
            const long long streams = std::max(1, device_cu_count() / std::max(1, nbt_hint));
            const long long tiles = ((long long)L + tw - 1) / tw;
            if (tiles > streams) {
                const long long per_stream = (tiles + streams - 1) / streams;
                int even = (int)(((long long)L + streams * per_stream - 1) / (streams * per_stream));
                even = (even + 1) & ~1;
                if (even >= 64 && even <= tw && even * 10 >= tw * 9) tw = even;
            }
        }
        if (tw >= 64) { TL = tw; w_in_lds = true; }
    }
    // the forms with weights in slot order, workgroups of at most 512 threads: one label per thread, so that two or more
    // workgroups share a CU (see tiled_workgroups_per_cu)
    if (!w_in_lds && threads <= 512) TL = std::min(TL, std::max(2, threads & ~1));
    *weights_in_lds = w_in_lds;
    return TL;
}

namespace {

// Builds the tiled form.  Returns FFI_OK with p->tiled == false if the padded size would exceed
// three times the connection count (heavily skewed column usage): the caller then builds the
// global form instead.
// (`after_row_assignment`, may be empty: called once the kernel that assigns the labels' LDS rows is enqueued -- it takes
// nearly all of every CU's LDS for itself, and work for another stream enqueued behind it starts when it ends instead of
// halving the number of its workgroups that fit)
int build_tiled(ffi_plan* p, const int32_t* lookup, hipStream_t s, const std::function<int()>& after_row_assignment = {}) {
    const int cols = p->col_n ? p->col_n : p->N;           // the columns this plan's tiled form covers, from col_lo on
    const int threads = ((cols + 63) / 64) * 64;
    // every thread of the kernel that walks the plan stages at most two labels of a tile (one when
    // the workgroup is larger than 768 threads and registers are scarcer)
    // (even, so that label parity inside a tile is the parity of the LDS row)
    // and small enough for the positions inside a tile to fit 16 bits
    bool w_in_lds = false;
    const int TL = plan_tile_labels(cols, p->K, p->L, p->batch_hint, &w_in_lds);
    const int slices = threads / 64;
    const int tiles = (p->L + TL - 1) / TL;
    const size_t nslices = (size_t)tiles * slices;
    // (the walking kernel hands its sums from the tile's thread to the column's own thread through LDS: built for the
    // weights-in-LDS form, whose workgroup has the registers for both sets of sums)
    // Measured (input gradient, weights-in-LDS form, sorted against thread t <-> column t): 768 columns x fan-in 32, batch 128:
    // 1.517 -> 1.150 slot rows per connection, 251 -> 239 us; batch 64: 151 -> 141; fan-in 16: 178 -> 170; fan-in 64 (300,000
    // labels): 207 -> 190; 512 columns: 261 -> 251; 640 columns, batch 256: 226 -> 215; no gain at 256 columns and fewer (few
    // slices to sort into, several workgroups per CU), and a loss where a workgroup walks a single tile (131,072 labels, batch
    // 32: 35.4 -> 36.5 us): there the order of the columns stays.
    const bool sorted_columns = plan_sorts_columns(threads, TL, p->K, w_in_lds, tiles, p->batch_hint);
    p->colperm = nullptr;
    unsigned* slice_len = nullptr;
    if (!dev_alloc(p, &p->slice_off, nslices + 1) || !dev_alloc(p, &slice_len, nslices)) return FFI_ERR_OUT_OF_MEMORY;
    // rows per bank half: half the tile plus some room for the balancing, within the LDS the walking kernel can have
    const int cap = tiled_rows_per_half(TL);
    if (!dev_alloc(p, &p->rowpos, (size_t)p->L)) return FFI_ERR_OUT_OF_MEMORY;
    {
        const size_t lds = ((size_t)threads + 1) * sizeof(int) + (size_t)TL * ((p->K + 2) / 3) * sizeof(unsigned) + ((size_t)threads + 2) * sizeof(unsigned short) + (size_t)TL;
        hipError_t ea = hipFuncSetAttribute((const void*)tile_color_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (ea != hipSuccess) return hip_fail(ea);
        hipLaunchKernelGGL(tile_color_kernel, dim3(tiles), dim3(256), lds, s, lookup, p->L, p->K, TL, cap, threads, p->rowpos, p->col_lo,
                           sorted_columns ? 1 : 0);
    }
    if (after_row_assignment) {
        const int st = after_row_assignment();
        if (st != FFI_OK) return st;
    }
    if (sorted_columns) {
        if (!dev_alloc(p, &p->colperm, (size_t)tiles * threads)) return FFI_ERR_OUT_OF_MEMORY;
        hipLaunchKernelGGL(tile_perm_kernel, dim3(tiles), dim3(threads), 3 * threads * sizeof(unsigned), s, lookup, p->rowpos, p->L, p->K, TL,
                           p->col_lo, p->colperm, slice_len);
    } else {
        hipLaunchKernelGGL(tile_count_kernel, dim3(tiles), dim3(threads), 2 * threads * sizeof(unsigned), s, lookup, p->rowpos, p->L,
                           p->K, TL, slice_len, p->col_lo);
    }
    hipLaunchKernelGGL(slice_scan_kernel, dim3(1), dim3(1024), 0, s, slice_len, p->slice_off, (int)nslices,
                       p->d_scratch + 2);
    hipError_t e = hipGetLastError();
    if (e == hipSuccess) e = hipMemcpyAsync(p->h_scratch + 2, p->d_scratch + 2, sizeof(unsigned long long), hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    dev_release(p, slice_len);
    if (e != hipSuccess) return hip_fail(e);
    const unsigned long long rows = p->h_scratch[2];
    const unsigned long long connections = (unsigned long long)p->L * p->K;
    // too skewed (a window of the columns may have two slots per connection of the layer: how many of them fall into
    // it is not counted), or beyond what the walking kernel's 32-bit buffer offsets reach (256 bytes per row)
    const unsigned long long allowed = p->col_n ? 2ull : 3ull;
    if (rows * 64ull > allowed * connections + 64ull * nslices || rows >= (1ull << 24)) return FFI_OK;
    if (w_in_lds) {
        if (!dev_alloc(p, &p->slot32, (size_t)rows * 64)) return FFI_ERR_OUT_OF_MEMORY;
    } else if (!dev_alloc(p, &p->lab16, (size_t)rows * 64) || !dev_alloc(p, &p->pos16, (size_t)rows * 64)) {
        return FFI_ERR_OUT_OF_MEMORY;
    }
    {
        int words = 0;
        const size_t fill_lds = tile_fill_bitmap_lds(threads, TL, p->K, &words);
        const unsigned pad_pos = w_in_lds ? (unsigned)TL * (unsigned)p->K : kPadPos;
        if (fill_lds <= kFillLdsLimit) {
            hipError_t ea = hipFuncSetAttribute((const void*)tile_fill_bitmap_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)fill_lds);
            if (ea != hipSuccess) return hip_fail(ea);
            hipLaunchKernelGGL(tile_fill_bitmap_kernel, dim3(tiles), dim3(threads), fill_lds, s, lookup, p->rowpos, p->L, p->K, TL, 2 * cap,
                               p->slice_off, p->lab16, p->pos16, pad_pos, p->slot32, words, p->col_lo, p->colperm);
        } else {
            hipLaunchKernelGGL(tile_fill_kernel, dim3(tiles), dim3(threads), 0, s, lookup, p->rowpos, p->L, p->K, TL, 2 * cap, p->slice_off,
                               p->lab16, p->pos16, pad_pos, p->slot32, p->col_lo, p->colperm);
        }
    }
    e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e != hipSuccess) return hip_fail(e);
    p->tiled = true;
    p->w_in_lds = w_in_lds;
    p->tile_labels = TL; p->threads = threads; p->slices = slices; p->tiles = tiles; p->zero_row = 2 * cap;
    p->total_rows = (long long)rows;
    p->bytes += (size_t)rows * 64 * 2 * sizeof(unsigned short) + (nslices + 1) * sizeof(unsigned) + (size_t)p->L * sizeof(unsigned short) +
                (p->colperm ? (size_t)tiles * threads * sizeof(unsigned short) : 0);
    return FFI_OK;
}

// key[p] = (label block of p) * N + column id of p
__global__ __launch_bounds__(kBlock) void block_key_kernel(const int32_t* __restrict__ idx, int total, int K, int N,
                                                           int block_labels, unsigned* __restrict__ key) {
    const int p = blockIdx.x * kBlock + threadIdx.x;
    if (p >= total) return;
    const int j = p / K;
    key[p] = (unsigned)(j / block_labels) * (unsigned)N + (unsigned)idx[p];
}

constexpr int kPlanBlockLabels = 65536;

int build_global(ffi_plan* p, const int32_t* lookup, hipStream_t s) {
    const int total = p->L * p->K;  // validated to fit int32 by the caller
    const int nblocks = (p->L + kPlanBlockLabels - 1) / kPlanBlockLabels;
    const long long nkeys = (long long)nblocks * p->N;
    if (nkeys >= (1ll << 31)) return FFI_ERR_TOO_LARGE;
    if (!dev_alloc(p, &p->perm, (size_t)total) || !dev_alloc(p, &p->col_ptr, (size_t)nkeys + 1)) return FFI_ERR_OUT_OF_MEMORY;
    unsigned* keys = nullptr;
    unsigned* sorted_keys = nullptr;
    void* temp = nullptr;
    size_t temp_bytes = 0;
    const int end_bit = bits_for((unsigned)(nkeys - 1));
    rocprim::counting_iterator<int32_t> positions(0);
    auto cleanup = [&]() {
        if (keys) (void)hipFree(keys);
        if (sorted_keys) (void)hipFree(sorted_keys);
        if (temp) (void)hipFree(temp);
    };
    // stable LSD radix sort of ((block, column), flat position): positions stay ascending inside a column
    hipError_t e = rocprim::radix_sort_pairs(nullptr, temp_bytes, keys, sorted_keys, positions, p->perm, (unsigned)total, 0,
                                             end_bit, s);
    if (e != hipSuccess) return hip_fail(e);
    if (hipMalloc(&keys, (size_t)total * sizeof(unsigned)) != hipSuccess ||
        hipMalloc(&sorted_keys, (size_t)total * sizeof(unsigned)) != hipSuccess ||
        hipMalloc(&temp, temp_bytes ? temp_bytes : 4) != hipSuccess) {
        (void)hipGetLastError();
        cleanup();
        return FFI_ERR_OUT_OF_MEMORY;
    }
    hipLaunchKernelGGL(block_key_kernel, dim3((total + kBlock - 1) / kBlock), dim3(kBlock), 0, s, lookup, total, p->K, p->N,
                       kPlanBlockLabels, keys);
    e = rocprim::radix_sort_pairs(temp, temp_bytes, keys, sorted_keys, positions, p->perm, (unsigned)total, 0, end_bit, s);
    if (e != hipSuccess) { cleanup(); return hip_fail(e); }
    hipLaunchKernelGGL(col_ptr_kernel, dim3((unsigned)((nkeys + 1 + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, sorted_keys,
                       total, (int)nkeys, p->col_ptr);
    e = hipGetLastError();
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    cleanup();
    if (e != hipSuccess) return hip_fail(e);
    p->block_labels = kPlanBlockLabels;
    p->nblocks = nblocks;
    p->bytes += (size_t)total * sizeof(int32_t) + ((size_t)nkeys + 1) * sizeof(int32_t);
    return FFI_OK;
}

// ---- arranged column ids for the weight gradient ------------------------------------------------
// The weight-gradient kernel reads, per connection, the 128-byte LDS row of the connection's
// column: even columns sit in one half of the LDS banks, odd columns in the other, and the LDS
// serves 16 lanes per clock only if 8 of them read each half.  Lanes l and l+8 work on labels j and
// j+8, so if the labels with bit 3 clear take their connections as even, odd, even, ... columns and
// the others as odd, even, odd, ..., the two lanes always read opposite halves (as far as a label's
// even and odd columns pair up; what is left over comes last).  One thread per (label, chunk of 32
// connections); entry i of a unit = (connection inside the chunk << 11) | column id; units are
// numbered chunk-major (u = chunk * L + label) so that consecutive lanes work on consecutive labels, and stored in
// blocks of 64 (arranged_quarter_offset).
// A wavefront takes 64 consecutive units (one block of the stored layout): their ids pass through LDS so that both
// the loads (128 contiguous bytes of a row per half wavefront) and the stores (the block's 4 KB in one piece) are
// coalesced; a thread per unit would read its row with a stride of a whole row between lanes (measured at
// 670,091 labels x fan-in 32: 0.95 ms, against 0.1 ms this way).
__global__ __launch_bounds__(kBlock) void arrange_units_kernel(const int32_t* __restrict__ idx, int L, int K, int nchunks,
                                                                unsigned short* __restrict__ out) {
    __shared__ int in[kBlock / 64][64][33];
    __shared__ __align__(16) unsigned short outb[kBlock / 64][2048];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const long long total = (long long)L * nchunks;
    const long long u0 = ((long long)blockIdx.x * (kBlock / 64) + wave) * 64;
    if (u0 >= total) return;                              // (whole wavefronts; no workgroup barrier below)
    // (chunk and label of the wavefront's first unit by one division; the units behind it by stepping)
    const int c0 = (int)(u0 / L), j0 = (int)(u0 - (long long)c0 * L);
    {
        const int k = lane & 31;
#pragma unroll 4
        for (int r = 0; r < 32; ++r) {
            const int q = 2 * r + (lane >> 5);
            int c = c0, j = j0 + q;
            while (j >= L) { j -= L; ++c; }
            int v = -1;
            if (c < nchunks && c * 32 + k < K) v = idx[(size_t)j * K + c * 32 + k];
            in[wave][q][k] = v;
        }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    {
        const long long u = u0 + lane;
        const int* row = in[wave][lane];
        unsigned short* ob = outb[wave];
        auto dst = [&](unsigned pos) -> unsigned short& { return ob[(pos >> 3) * 512 + (unsigned)lane * 8 + (pos & 7u)]; };
        int kn = 0;
        if (u < total) {
            int c = c0, j = j0 + lane;
            while (j >= L) { j -= L; ++c; }
            kn = min(32, K - c * 32);
            const unsigned role = ((unsigned)j >> 3) & 1u;        // parity taken at even positions
            unsigned nfirst = 0;
            for (int k = 0; k < kn; ++k) nfirst += (((unsigned)row[k] & 1u) == role) ? 1u : 0u;
            const unsigned m = min(nfirst, (unsigned)kn - nfirst);
            unsigned tf = 0, ts = 0;
            for (int k = 0; k < kn; ++k) {
                const unsigned id = (unsigned)row[k];
                const bool first = (id & 1u) == role;
                const unsigned t = first ? tf++ : ts++;
                const unsigned pos = t < m ? 2u * t + (first ? 0u : 1u) : 2u * m + (t - m);
                dst(pos) = (unsigned short)(((unsigned)k << kArrIdBits) | id);
            }
        }
        // a chunk the fan-in does not fill (and the units behind the last one, which pad the array to whole blocks): the
        // rest points at connection 31, which such a chunk never stores
        for (int k = kn; k < 32; ++k) dst((unsigned)k) = (unsigned short)(31u << kArrIdBits);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    uint4* o4 = reinterpret_cast<uint4*>(out + (size_t)(u0 >> 6) * 2048);
    const uint4* b4 = reinterpret_cast<const uint4*>(outb[wave]);
#pragma unroll
    for (int i = 0; i < 4; ++i) o4[i * 64 + lane] = b4[i * 64 + lane];
}

// The same reordering applied in place to the lookup matrix itself and to up to four float
// matrices of its shape (weights, optimizer state): one thread per (label, chunk of 32).
struct ArrangeArrays { float* a[4]; };
__global__ __launch_bounds__(kBlock) void arrange_in_place_kernel(int32_t* __restrict__ idx, ArrangeArrays arr, int L, int K,
                                                                   int nchunks) {
    const long long u = (long long)blockIdx.x * kBlock + threadIdx.x;
    if (u >= (long long)L * nchunks) return;
    const int c = (int)(u / L), j = (int)(u - (long long)c * L);
    const int k0 = c * 32, kn = min(32, K - k0);
    int32_t* row = idx + (size_t)j * K + k0;
    const unsigned role = ((unsigned)j >> 3) & 1u;
    int32_t ids[32];
    unsigned char pos[32];
    unsigned nfirst = 0;
    for (int k = 0; k < kn; ++k) { ids[k] = row[k]; nfirst += (((unsigned)ids[k] & 1u) == role) ? 1u : 0u; }
    const unsigned m = min(nfirst, (unsigned)kn - nfirst);
    unsigned tf = 0, ts = 0;
    for (int k = 0; k < kn; ++k) {
        const bool first = ((unsigned)ids[k] & 1u) == role;
        const unsigned t = first ? tf++ : ts++;
        pos[k] = (unsigned char)(t < m ? 2u * t + (first ? 0u : 1u) : 2u * m + (t - m));
    }
    for (int k = 0; k < kn; ++k) row[pos[k]] = ids[k];
    for (int a = 0; a < 4; ++a) {
        if (arr.a[a] == nullptr) continue;
        float* frow = arr.a[a] + (size_t)j * K + k0;
        float v[32];
        for (int k = 0; k < kn; ++k) v[k] = frow[k];
        for (int k = 0; k < kn; ++k) frow[pos[k]] = v[k];
    }
}

}  // namespace

int launch_arrange_in_place(int32_t* lookup, float* const* arrays, int n_arrays, int L, int K, hipStream_t s) {
    ArrangeArrays arr{{nullptr, nullptr, nullptr, nullptr}};
    for (int i = 0; i < n_arrays && i < 4; ++i) arr.a[i] = arrays[i];
    const int nchunks = (K + 31) / 32;
    const long long units = (long long)L * nchunks;
    hipLaunchKernelGGL(arrange_in_place_kernel, dim3((unsigned)((units + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, lookup, arr,
                       L, K, nchunks);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

namespace {

int build_arranged(ffi_plan* p, const int32_t* lookup, hipStream_t s) {
    const int nchunks = (p->K + 31) / 32;
    const long long units = (long long)p->L * nchunks;
    if (!dev_alloc(p, &p->idx16, arranged_words(units))) return FFI_ERR_OUT_OF_MEMORY;
    hipLaunchKernelGGL(arrange_units_kernel, dim3((unsigned)((units + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, lookup,
                       p->L, p->K, nchunks, p->idx16);
    FFI_HIP_TRY(hipGetLastError());
    p->bytes += arranged_words(units) * sizeof(unsigned short);
    return FFI_OK;
}

}  // namespace

// device/pinned scratch words and the fingerprint event of a plan
int plan_scratch_alloc(ffi_plan* p) {
    const bool ok = hipMalloc(&p->d_scratch, kScratchWords * sizeof(unsigned long long)) == hipSuccess &&
                    hipHostMalloc(&p->h_scratch, kScratchWords * sizeof(unsigned long long)) == hipSuccess &&
                    hipEventCreateWithFlags(&p->fp_done, hipEventDisableTiming) == hipSuccess &&
                    hipMemset(p->d_scratch, 0, kScratchWords * sizeof(unsigned long long)) == hipSuccess &&
                    hipMalloc(&p->d_guard, kGuardWords * sizeof(unsigned long long)) == hipSuccess &&
                    hipHostMalloc(&p->h_guard, 8 * sizeof(unsigned long long)) == hipSuccess &&
                    hipMemset(p->d_guard, 0, kGuardWords * sizeof(unsigned long long)) == hipSuccess;
    if (!ok) {
        (void)hipGetLastError();
        return FFI_ERR_OUT_OF_MEMORY;
    }
    std::memset(p->h_guard, 0, 8 * sizeof(unsigned long long));      // check number 0: nothing has finished yet
    return FFI_OK;
}

int plan_fingerprint_begin(ffi_plan* p, const int32_t* lookup, hipStream_t s) {
    const size_t total = (size_t)p->L * p->K;
    const unsigned blocks = (unsigned)std::min<size_t>((total / 4 + kBlock - 1) / kBlock + 1, kFingerprintBlocks);
    // words 0..7 of the scratch arrays belong to the plan build; the workgroups' partial sums follow
    unsigned long long* partials = p->d_scratch + 8;
    hipLaunchKernelGGL(fingerprint_kernel, dim3(blocks), dim3(kBlock), 0, s, lookup, total, (unsigned)p->N, partials);
    FFI_HIP_TRY(hipGetLastError());
    FFI_HIP_TRY(hipMemcpyAsync(p->h_scratch + 8, partials, 2 * (size_t)blocks * sizeof(unsigned long long), hipMemcpyDeviceToHost, s));
    FFI_HIP_TRY(hipEventRecord(p->fp_done, s));
    p->fp_blocks = (int)blocks;
    return FFI_OK;
}

int plan_fingerprint_end(ffi_plan* p, unsigned long long* out, unsigned long long* bad_ids) {
    FFI_HIP_TRY(hipEventSynchronize(p->fp_done));
    unsigned long long h = 0, bad = 0;
    for (int i = 0; i < p->fp_blocks; ++i) {
        h += p->h_scratch[8 + 2 * i];
        bad += p->h_scratch[8 + 2 * i + 1];
    }
    *out = h;
    *bad_ids = bad;
    return FFI_OK;
}

int plan_fingerprint(ffi_plan* p, const int32_t* lookup, hipStream_t s, unsigned long long* out,
                     unsigned long long* bad_ids) {
    FFI_TRY(plan_fingerprint_begin(p, lookup, s));
    return plan_fingerprint_end(p, out, bad_ids);
}

namespace {
int plan_build_arrays(ffi_plan* p, const int32_t* lookup, hipStream_t s, unsigned long long* fp_out);
}

// On failure the plan is left without arrays and without a lookup: it matches no cache key and
// launch_input_grad refuses it.
int plan_build(ffi_plan* p, const int32_t* lookup, hipStream_t s) {
    unsigned long long fp = 0;
    const int st = plan_build_arrays(p, lookup, s, &fp);
    if (st != FFI_OK) {
        free_arrays(p);
        p->lookup = nullptr;
        p->fingerprint = ~0ull;
        return st;
    }
    p->lookup = lookup;
    p->fingerprint = fp;
    // what the device-side check compares with; the build has synchronised, no check of this plan is in flight
    const unsigned long long guard_init[8] = {0, 0, 0, fp, 1, fp, 0, 0};
    FFI_HIP_TRY(hipMemcpy(p->d_guard, guard_init, sizeof(guard_init), hipMemcpyHostToDevice));
    // checks enqueued before this build (all finished: the build synchronises) are of no interest any more
    p->guard_seen = p->guard_seq;
    p->guard_stale = false;
    p->edited_by_library = false;
    return FFI_OK;
}

namespace {
int plan_build_arrays(ffi_plan* p, const int32_t* lookup, hipStream_t s, unsigned long long* fp_out) {
    unsigned long long fp = 0, bad = 0;
    FFI_TRY(plan_fingerprint(p, lookup, s, &fp, &bad));
    if (bad != 0) return FFI_ERR_BAD_LOOKUP;   // also keeps the build kernels' LDS counters in range
    // a rebuild replaces the arrays: whatever still reads the old ones must have drained
    if (!p->owned.empty()) FFI_HIP_TRY(hipDeviceSynchronize());
    free_arrays(p, true);                      // (their buffers serve the new arrays where they fit)
    // The arranged ids of the weight gradient depend on the lookup alone: their kernel runs on a helper stream beside
    // the kernels of the tiled form (of which the longest runs one wavefront per tile and leaves the memory system idle).
    // (ids < 2^11 and an [N][32] fp32 tile in LDS: the shapes the narrow weight-gradient kernel takes)
    const bool arranged = tile_path_fits(p->N) && p->N < (1 << kArrIdBits);
    bool helper_busy = false;
    if (arranged) {
        if (p->helper_stream == nullptr) {
            if (hipStreamCreateWithFlags(&p->helper_stream, hipStreamNonBlocking) != hipSuccess ||
                hipEventCreateWithFlags(&p->helper_event, hipEventDisableTiming) != hipSuccess) {
                (void)hipGetLastError();
                if (p->helper_stream) { (void)hipStreamDestroy(p->helper_stream); p->helper_stream = nullptr; }
            }
        }
    }
    // (enqueued from inside the tiled build, behind the row-assignment kernel, where there is a tiled build)
    bool arranged_enqueued = !arranged;
    auto enqueue_arranged = [&]() -> int {
        if (arranged_enqueued) return FFI_OK;
        arranged_enqueued = true;
        hipStream_t hs = p->helper_stream ? p->helper_stream : s;
        // (the fingerprint above has synchronised `s`: the lookup is final, the helper needs no further ordering)
        if (hs != s) helper_busy = true;
        return build_arranged(p, lookup, hs);
    };
    auto join = [&]() -> int {
        if (helper_busy) { helper_busy = false; FFI_HIP_TRY(hipStreamSynchronize(p->helper_stream)); }
        return FFI_OK;
    };
    // tiled form: one thread per column (N <= 1024), tiles of at least 62 labels with positions in 16 bits
    // (and 32 rows of out_grad within 32-bit byte offsets, as the kernels' buffer loads need)
    if (p->N <= 1024 && p->K <= 1024 && p->L < (1 << 25)) {
        int st = build_tiled(p, lookup, s, enqueue_arranged);
        if (st != FFI_OK) { (void)join(); free_arrays(p); return st; }
    } else if (tile_path_fits(p->N) && p->N <= 2048 && p->K <= 1024 && p->L < (1 << 25)) {
        // 1,025 to 1,216 columns: the LDS tile of the other two passes holds them, a workgroup of one thread per column
        // does not.  Two tiled forms, one per half of the columns; each walk stages the tile's out_grad itself, which costs
        // far less than the cache-bound global form (measured at 1,216 columns, c2's other dimensions: 1.58 ms).
        const int lower = ((p->N + 1) / 2 + 63) / 64 * 64;
        p->col_lo = 0; p->col_n = lower;
        int st = build_tiled(p, lookup, s, enqueue_arranged);
        if (st == FFI_OK && p->tiled) {
            ffi_plan* u = new (std::nothrow) ffi_plan();
            if (u == nullptr) st = FFI_ERR_OUT_OF_MEMORY;
            else {
                u->device = p->device; u->L = p->L; u->K = p->K; u->N = p->N; u->batch_hint = p->batch_hint;
                u->col_lo = lower; u->col_n = p->N - lower;
                u->d_scratch = p->d_scratch; u->h_scratch = p->h_scratch;      // (borrowed for the build; never freed through `u`)
                p->upper = u;
                st = build_tiled(u, lookup, s);
                u->d_scratch = nullptr; u->h_scratch = nullptr;
                if (st == FFI_OK && u->tiled) p->bytes += u->bytes;
            }
        }
        if (st != FFI_OK) { (void)join(); free_arrays(p); return st; }
        if (!p->tiled || !p->upper || !p->upper->tiled) {
            // too skewed for the tiled form in one of the halves: both go, the global form serves all columns
            ffi_plan* u = p->upper;
            p->upper = nullptr;
            if (u) { free_arrays(u, false); free_spares(u); delete u; }
            p->tiled = false;
            p->col_lo = 0; p->col_n = 0;
        }
    }
    {
        const int st = enqueue_arranged();         // (no tiled build took place, or it ended before its row assignment)
        if (st != FFI_OK) { (void)join(); free_arrays(p); return st; }
    }
    if (!p->tiled) {
        // (the tiled form's arrays, if any were made, go back to the spare list; the arranged ids stay)
        for (void* q : {(void*)p->slice_off, (void*)p->rowpos, (void*)p->lab16, (void*)p->pos16, (void*)p->slot32, (void*)p->colperm})
            if (q) dev_release(p, q);
        p->slice_off = nullptr; p->rowpos = nullptr; p->lab16 = nullptr; p->pos16 = nullptr; p->slot32 = nullptr; p->colperm = nullptr;
        const size_t arranged_bytes = p->idx16 ? arranged_words((long long)p->L * ((p->K + 31) / 32)) * sizeof(unsigned short) : 0;
        p->bytes = 0;
        int st = build_global(p, lookup, s);
        if (st != FFI_OK) { (void)join(); free_arrays(p); return st; }
        p->bytes += arranged_bytes;
    }
    {
        const int st = join();
        if (st != FFI_OK) { free_arrays(p); return st; }
    }
    free_spares(p);                            // what this build did not reuse
    *fp_out = fp;
    return FFI_OK;
}
}  // namespace

int plan_guard_enqueue(ffi_plan* p, const int32_t* lookup, hipStream_t s) {
    // A check of this plan that may still be running on another stream shares the accumulators: the two must not
    // overlap.  The other stream's handle may be gone by now (its owner may have destroyed it), so it is not touched:
    // the host waits for the device.  Only a lookup used from two streams in turn pays this, once per switch.
    if (p->guard_seq != p->guard_seen && p->guard_stream != s) {
        FFI_HIP_TRY(hipDeviceSynchronize());
        bool seen = false, current = true;
        unsigned long long bad = 0;
        (void)plan_guard_poll(p, &seen, &current, &bad);          // (the result stays with the next check if it was bad)
        if (seen && !current) p->guard_stale = true;
    }
    const size_t total = (size_t)p->L * p->K;
    const unsigned blocks = (unsigned)std::min<size_t>((total / 4 + kGuardBlock - 1) / kGuardBlock + 1, kGuardBlocks);
    unsigned long long* mirror = nullptr;
    FFI_HIP_TRY(hipHostGetDevicePointer((void**)&mirror, p->h_guard, 0));
    hipLaunchKernelGGL(fingerprint_guard_kernel, dim3(blocks), dim3(kGuardBlock), 0, s, lookup, total, (unsigned)p->N, p->d_guard, mirror,
                       p->guard_seq + 1);
    FFI_HIP_TRY(hipGetLastError());
    p->guard_seq += 1;
    p->guard_stream = s;
    return FFI_OK;
}

int plan_guard_poll(ffi_plan* p, bool* seen, bool* current, unsigned long long* bad_ids) {
    *seen = false;
    if (p->guard_stale) {                                  // an outdated verdict met while switching streams
        p->guard_stale = false;
        *seen = true; *current = false; *bad_ids = 0;
        return FFI_OK;
    }
    if (p->guard_seq == p->guard_seen) return FFI_OK;
    // the last check that has finished (checks of a plan finish in the order they were enqueued)
    const unsigned long long word = __atomic_load_n(p->h_guard, __ATOMIC_ACQUIRE);
    const unsigned long long done = word >> 2;
    if (done <= p->guard_seen || done > p->guard_seq) return FFI_OK;        // nothing new (or a word of before the last build)
    p->guard_seen = done;
    *seen = true;
    *current = ((word >> 1) & 1ull) != 0;
    *bad_ids = word & 1ull;
    return FFI_OK;
}

void plan_free(ffi_plan* p) {
    if (!p) return;
    free_arrays(p);
    free_spares(p);
    if (p->helper_stream) { (void)hipStreamSynchronize(p->helper_stream); (void)hipStreamDestroy(p->helper_stream); p->helper_stream = nullptr; }
    if (p->helper_event) { (void)hipEventDestroy(p->helper_event); p->helper_event = nullptr; }
    if (p->d_scratch) (void)hipFree(p->d_scratch);
    if (p->h_scratch) (void)hipHostFree(p->h_scratch);
    if (p->fp_done) (void)hipEventDestroy(p->fp_done);
    if (p->d_guard) (void)hipFree(p->d_guard);
    if (p->h_guard) (void)hipHostFree(p->h_guard);
    p->d_scratch = nullptr; p->h_scratch = nullptr; p->fp_done = nullptr;
    p->d_guard = nullptr; p->h_guard = nullptr; p->guard_seq = 0; p->guard_seen = 0; p->guard_stale = false;
}

}  // namespace ffi
