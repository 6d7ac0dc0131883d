// Forward pass of the fixed-fan-in sparse layer for gfx950:
//   out[b,j] = sum_k w[j,k] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/forward.cpp:9-44 in the reference).
//
//   fwd_lane32_kernel  narrow inputs (a [N][32] fp32 tile of x fits in LDS): every multiply-add
//                      takes its x operand from LDS; the LDS delivers 128 bytes per clock per CU,
//                      which bounds the kernel (4 bytes per multiply-add), so the layout is chosen
//                      to keep the gathers free of bank conflicts and the instruction count low.
// Other shapes go to the wide-input kernel (ffi_wide.hip).
#include "ffi_internal.h"
#include "ffi_lds_tile.h"
#include "ffi_loss.h"

#include <algorithm>
#include <climits>
#include <mutex>

namespace ffi {
namespace {

// ------------------------------------------------------------------------------------------------
// Narrow-input kernel: xs[n][c] = x[b0+c, n] for the workgroup's 32 batch rows sits in LDS (one row =
// 128 bytes); thread <-> label, 32 accumulators (one per batch row of the tile), W and idx of the
// label in registers.  Workgroups that walk the same labels for different batch tiles sit on one
// XCD, so W/idx rows fetched by one are L2 hits for the others.  Each lane reads whole 128-byte rows of xs with
// the chunk order skewed by its lane id; the accumulators are brought back to natural batch order
// before the stores, which are then full 256-byte rows of out per wavefront.
// ------------------------------------------------------------------------------------------------
// `base` is a raw LDS address: (address of the tile + (lane & 7) * 16) + row * 128.  The tile is 128-byte aligned, so the
// chunk bits can be flipped with XOR after the add: one add and seven XORs per row instead of an add per read.
typedef float lds_v4f __attribute__((ext_vector_type(4)));
typedef const lds_v4f __attribute__((address_space(3)))* lds_v4f_ptr;
template <int C>
__device__ __forceinline__ void fwd_lane_step(unsigned base, float wv, float (&acc)[32]) {
    const lds_v4f v = *(lds_v4f_ptr)(size_t)(skew_addr<C>(base));
    acc[4 * C + 0] = fmaf(wv, v.x, acc[4 * C + 0]);
    acc[4 * C + 1] = fmaf(wv, v.y, acc[4 * C + 1]);
    acc[4 * C + 2] = fmaf(wv, v.z, acc[4 * C + 2]);
    acc[4 * C + 3] = fmaf(wv, v.w, acc[4 * C + 3]);
}

// One connection of the lane's label: the eight 16-byte reads of row `rb` (chunk order skewed per lane) and their 32
// multiply-adds, in a pinned order -- two reads in flight; a read's registers are refilled as soon as its four values
// are used, under the multiply-adds of the other read.  Left to itself the scheduler finds this order or one that
// waits for each read in turn (13 % slower over the whole kernel), depending on code far away from here.
__device__ __forceinline__ void fwd_lane_connection(unsigned rb, float wv, float (&acc)[32]) {
    lds_v4f a = *(lds_v4f_ptr)(size_t)rb;
    lds_v4f b = *(lds_v4f_ptr)(size_t)(rb ^ 16u);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        acc[8 * p + 0] = fmaf(wv, a.x, acc[8 * p + 0]);
        acc[8 * p + 4] = fmaf(wv, b.x, acc[8 * p + 4]);
        acc[8 * p + 1] = fmaf(wv, a.y, acc[8 * p + 1]);
        acc[8 * p + 2] = fmaf(wv, a.z, acc[8 * p + 2]);
        acc[8 * p + 3] = fmaf(wv, a.w, acc[8 * p + 3]);
        acc[8 * p + 5] = fmaf(wv, b.y, acc[8 * p + 5]);
        __builtin_amdgcn_sched_barrier(0);
        if (p < 3) a = *(lds_v4f_ptr)(size_t)(rb ^ (unsigned)(32 * p + 32));
        __builtin_amdgcn_sched_barrier(0);
        acc[8 * p + 6] = fmaf(wv, b.z, acc[8 * p + 6]);
        acc[8 * p + 7] = fmaf(wv, b.w, acc[8 * p + 7]);
        __builtin_amdgcn_sched_barrier(0);
        if (p < 3) b = *(lds_v4f_ptr)(size_t)(rb ^ (unsigned)(32 * p + 48));
        __builtin_amdgcn_sched_barrier(0);
    }
}

// What the kernel does with a finished score s (after the bias):
//   kEpiScores       out = s
//   kEpiLossGrad     out = scale * dloss(s, 0)/ds, the loss gradient of a position that is not a listed label
//                    (listed positions are patched afterwards), and the loss(s, 0) summed per wavefront
//   kEpiLossGradAndScores  both: scores to `out`, gradients to `gout`
//   kEpiNone         nothing is stored (only the top-k candidates below are wanted)
//   kEpiLossGradSkewed  kEpiLossGrad for launches that do not store gradients that are exactly zero (nearly nothing is
//                    stored then): the accumulators stay in the lane's skewed register order (register q holds batch
//                    entry q ^ 4 (lane & 7)), the 96 conditional moves back to natural order are left out, the few stores
//                    address their rows per lane and only the mask's bits are put in order
enum FwdEpilogue { kEpiScores = 0, kEpiLossGrad = 1, kEpiLossGradAndScores = 2, kEpiNone = 3, kEpiLossGradSkewed = 4 };

constexpr int kTopkPark = 24;           // candidates per (workgroup, batch row) parked in LDS: 32 x 24 x 8 bytes = 6 KB

// Per-sample top-k without the score matrix (TOPK): tau[b] is a score that at least k labels of sample b are
// known to reach (the k-th best of a sample of the labels, found beforehand), so the k best scores are among
// those >= tau[b]; every such (label, score) is appended to the sample's candidate list, a few hundred to a
// few thousand entries out of all labels, and a small kernel selects the k best afterwards.
struct FwdTopk {
    const float* tau;     // tau[b * tau_stride]
    int tau_stride;
    int* count;           // [B] candidates appended so far (may run past cap: the list is then incomplete)
    float* cand_val;      // [B][cap]
    int* cand_idx;        // [B][cap]
    int cap;
};

struct FwdLoss {
    float* gout;        // [B,L] gradients (kEpiLossGradAndScores), else unused
    double* partial;    // [gridDim.x * wavefronts per workgroup] loss sums
    unsigned* words;    // [ceil(B/32)][L] masks of the non-zero gradients to fill in, or null
    float scale;
    int kind;
    int skip_zero_stores;   // != 0: gradients that are exactly zero are not stored (needs words)
};

// Scores of one label for the 32 samples of a batch tile -> scaled loss gradients (in place), the sum of the
// losses of the first `nrows` samples, and the mask of the non-zero gradients among them.
template <int KIND>
__device__ __forceinline__ void loss_epilogue(float (&acc)[32], bool all_rows, unsigned valid_bits, float scale, float& loss,
                                              unsigned& mask) {
    // `all_rows` (workgroup-uniform): the batch tile is full; else bit q of `valid_bits` says whether register q belongs
    // to a sample of the batch (rows past it count for nothing)
    float l = 0.f;
    unsigned m = 0;
    if (all_rows) {
#pragma unroll
        for (int b = 0; b < 32; ++b) {
            float lb, gb;
            cwise_loss_and_grad(KIND, acc[b], 0.f, lb, gb);
            l += lb;
            m |= (gb != 0.f ? 1u : 0u) << b;
            acc[b] = scale * gb;
        }
    } else {
#pragma unroll
        for (int b = 0; b < 32; ++b) {
            float lb, gb;
            cwise_loss_and_grad(KIND, acc[b], 0.f, lb, gb);
            const bool in = (valid_bits >> b) & 1u;
            l += in ? lb : 0.f;
            m |= (in && gb != 0.f ? 1u : 0u) << b;
            acc[b] = scale * gb;
        }
    }
    loss = l;
    mask = m;
}

// VEC: how a label's column ids and weights are loaded.  0: one by one (any fan-in, any alignment); 1: by 16-byte quads
// (fan-in a multiple of four, 16-byte aligned arrays), a partly filled last chunk one by one; 2: by quads, for a fan-in
// below one chunk of 32 (a build of its own: the same code inside the general loop costs the full chunks 25 %).
template <int VEC, int EPI, bool TOPK>
__global__ __launch_bounds__(kTileThreads) void fwd_lane32_kernel(const float* __restrict__ xT,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w,
                                                                  const float* __restrict__ bias,
                                                                  float* __restrict__ out, int B, int N,
                                                                  int L, int K, int nbt, int labels_per_stream,
                                                                  FwdLoss fl, FwdTopk ft) {
    extern __shared__ __align__(128) float xs[];
    __shared__ __align__(16) float tau_s[kTileBatch];
    __shared__ int local_count[kTileBatch];      // candidates parked per batch row (may run past kTopkPark)
    __shared__ int local_base[kTileBatch];
    int2* local_cand = reinterpret_cast<int2*>(xs + (size_t)N * kTileBatch);      // behind the tile (TOPK launches only)
    const int u = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int bt = u % nbt, stream = u / nbt;
    const int b0 = bt * kTileBatch;
    stage_rows32<kTileThreads, 8>(xs, xT, N, B, b0);       // (eight loads in flight per thread: the tile arrives in one round trip at 768 rows)
    if (TOPK && threadIdx.x < kTileBatch) local_count[threadIdx.x] = 0;
    if (TOPK && threadIdx.x < kTileBatch)          // rows past the batch never qualify
        tau_s[threadIdx.x] = b0 + (int)threadIdx.x < B ? ft.tau[(size_t)(b0 + threadIdx.x) * ft.tau_stride] : __builtin_inff();
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const unsigned skewbase = (unsigned)(size_t)(__attribute__((address_space(3))) float*)xs + (unsigned)(lane & 7) * 16u;
    const int l_begin = stream * labels_per_stream;
    const int l_end = min(l_begin + labels_per_stream, L);
    const int nchunks = (K + 31) / 32;
    // rows of out for this batch tile, reached through a scalar row offset plus the lane's label
    const int nrows = min(kTileBatch, B - b0);
    float* obase = out + (size_t)b0 * (size_t)L;
    const buffer_rsrc orsrc = make_rsrc(obase, (size_t)nrows * (size_t)L * sizeof(float));
    buffer_rsrc grsrc = orsrc;
    if (EPI == kEpiLossGradAndScores) grsrc = make_rsrc(fl.gout + (size_t)b0 * (size_t)L, (size_t)nrows * (size_t)L * sizeof(float));
    float lsum = 0.f;

    constexpr bool VEC4 = VEC >= 1;
    constexpr bool SHORT = VEC == 2;
    constexpr bool SKEW = EPI == kEpiLossGradSkewed;
    constexpr bool LOSS = EPI == kEpiLossGrad || EPI == kEpiLossGradAndScores || SKEW;
    static_assert(!(SKEW && TOPK), "the top-k tests need the natural order");
    // registers (in the order the epilogue sees them) that belong to samples of the batch
    const unsigned rows_valid = nrows >= kTileBatch ? 0xffffffffu : (1u << nrows) - 1u;
    const unsigned regs_valid = SKEW ? xor_permute_bits(rows_valid, lane & 7) : rows_valid;

    for (int base = l_begin; base < l_end; base += kTileThreads) {
        if (base + (int)(threadIdx.x & ~63u) >= l_end) break;     // nothing left for this wavefront
        const int j = base + (int)threadIdx.x;
        const bool valid = j < l_end;
        const int jj = valid ? j : l_end - 1;
        const int32_t* irow = idx + (size_t)jj * K;
        const float* wrow = w + (size_t)jj * K;
        float acc[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] = 0.f;
        for (int ch = 0; ch < nchunks; ++ch) {
            const int k0 = ch * 32;
            const bool full = VEC4 && !SHORT && k0 + 32 <= K;
            unsigned idp[16];
            float wv[32];
            if (SHORT) {
                // the one, partly filled chunk: the quads behind its end re-read its first quad, so that the loads stay
                // unconditional; their connections are skipped below
                const int quads = K >> 2;
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const int at = 4 * (q < quads ? q : 0);
                    const int4 v = *reinterpret_cast<const int4*>(irow + at);
                    idp[2 * q + 0] = (unsigned)v.x | ((unsigned)v.y << 16);
                    idp[2 * q + 1] = (unsigned)v.z | ((unsigned)v.w << 16);
                    const float4 f = *reinterpret_cast<const float4*>(wrow + at);
                    wv[4 * q] = f.x; wv[4 * q + 1] = f.y; wv[4 * q + 2] = f.z; wv[4 * q + 3] = f.w;
                }
            } else if (full) {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const int4 v = *reinterpret_cast<const int4*>(irow + k0 + 4 * q);
                    idp[2 * q + 0] = (unsigned)v.x | ((unsigned)v.y << 16);
                    idp[2 * q + 1] = (unsigned)v.z | ((unsigned)v.w << 16);
                    const float4 f = *reinterpret_cast<const float4*>(wrow + k0 + 4 * q);
                    wv[4 * q] = f.x; wv[4 * q + 1] = f.y; wv[4 * q + 2] = f.z; wv[4 * q + 3] = f.w;
                }
            } else {
#pragma unroll
                for (int q = 0; q < 16; ++q) {
                    const unsigned a = (k0 + 2 * q < K) ? (unsigned)irow[k0 + 2 * q] : 0u;
                    const unsigned b = (k0 + 2 * q + 1 < K) ? (unsigned)irow[k0 + 2 * q + 1] : 0u;
                    idp[q] = a | (b << 16);
                }
#pragma unroll
                for (int k = 0; k < 32; ++k) wv[k] = (k0 + k < K) ? wrow[k0 + k] : 0.f;
            }
            const int kn = min(32, K - k0);
#pragma unroll
            for (int k = 0; k < 32; ++k) {
                if (full || k < kn) {
                    const unsigned id = (k & 1) ? (idp[k >> 1] >> 16) : (idp[k >> 1] & 0xffffu);
                    const unsigned rb = (id << 7) + skewbase;
                    fwd_lane_connection(rb, wv[k], acc);
                }
            }
        }
        if (!SKEW) xor_permute_groups(acc, lane & 7);      // back to natural batch order
        if (bias != nullptr) {                             // added after the sum, as a separate bias_add would
            const float bj = bias[jj];
#pragma unroll
            for (int i = 0; i < 32; ++i) acc[i] += bj;
        }
        if (TOPK) {
            // Scores that reach their sample's threshold are rare (about one in a thousand), but a wavefront holds 2048 of
            // them: the tests are wave-uniform and hierarchical (four groups of eight batch rows, then the rows of a group
            // that has a hit), so that a row without a hit costs one compare.
            float tv[32];
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                const float4 t4 = *reinterpret_cast<const float4*>(tau_s + 4 * c);
                tv[4 * c] = t4.x; tv[4 * c + 1] = t4.y; tv[4 * c + 2] = t4.z; tv[4 * c + 3] = t4.w;
            }
#pragma unroll
            for (int grp = 0; grp < 4; ++grp) {
                bool hit = false;
#pragma unroll
                for (int b = 8 * grp; b < 8 * grp + 8; ++b) hit |= acc[b] >= tv[b];
                hit &= valid;
                if (__ballot(hit)) {
#pragma unroll
                    for (int b = 8 * grp; b < 8 * grp + 8; ++b) {
                        const bool h = valid && acc[b] >= tv[b];
                        if (__ballot(h)) {
                            if (h) {
                                // parked in the workgroup's LDS segment of the sample (an LDS counter answers in a few dozen
                                // clocks, a global one in microseconds); a full segment sends the entry to memory directly
                                const int lslot = atomicAdd(&local_count[b], 1);
                                if (lslot < kTopkPark) {
                                    local_cand[b * kTopkPark + lslot] = make_int2(j, __float_as_int(acc[b]));
                                } else {
                                    const int slot = atomicAdd(&ft.count[b0 + b], 1);
                                    if (slot < ft.cap) {
                                        ft.cand_val[(size_t)(b0 + b) * ft.cap + slot] = acc[b];
                                        ft.cand_idx[(size_t)(b0 + b) * ft.cap + slot] = j;
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
        const unsigned lane_off = (unsigned)j * 4u;
        const unsigned stride = (unsigned)L * 4u;
        if ((EPI == kEpiScores || EPI == kEpiLossGradAndScores) && valid) {
#pragma unroll
            for (int b = 0; b < 32; ++b)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[b]), orsrc, lane_off, (unsigned)b * stride, 0);
        }
        if (LOSS) {
            float l = 0.f;
            unsigned m = 0;
            const bool all_rows = nrows >= kTileBatch;
            // the loss kind is the same for the whole launch: one straight-line epilogue per kind
            if (fl.kind == FFI_LOSS_SQUARED_HINGE) loss_epilogue<FFI_LOSS_SQUARED_HINGE>(acc, all_rows, regs_valid, fl.scale, l, m);
            else if (fl.kind == FFI_LOSS_HINGE) loss_epilogue<FFI_LOSS_HINGE>(acc, all_rows, regs_valid, fl.scale, l, m);
            else loss_epilogue<FFI_LOSS_BCE>(acc, all_rows, regs_valid, fl.scale, l, m);
            if (valid) {
                lsum += l;
                if (SKEW) {
                    // register q is the gradient of batch entry q ^ r4: its row of out_grad is the lane's own
                    unsigned r4 = (unsigned)(lane & 7) << 2;
                    asm volatile("" : "+v"(r4));           // keeps the 32 row offsets from being hoisted out of the label loop
#pragma unroll
                    for (int q = 0; q < 32; ++q)
                        if ((m >> q) & 1u)
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[q]), orsrc,
                                                                  lane_off + ((unsigned)q ^ r4) * stride, 0u, 0);
                    m = xor_permute_bits(m, lane & 7);
                } else if (fl.skip_zero_stores) {
#pragma unroll
                    for (int b = 0; b < 32; ++b)
                        if ((m >> b) & 1u)
                            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[b]), EPI == kEpiLossGrad ? orsrc : grsrc, lane_off, (unsigned)b * stride, 0);
                } else {
#pragma unroll
                    for (int b = 0; b < 32; ++b)
                        __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[b]), EPI == kEpiLossGrad ? orsrc : grsrc, lane_off, (unsigned)b * stride, 0);
                }
                if (fl.words != nullptr) fl.words[(size_t)bt * L + j] = m;
            }
        }
    }
    if (TOPK) {
        // the parked candidates go to their samples' lists: one reservation per (workgroup, sample)
        __syncthreads();
        if (threadIdx.x < kTileBatch) {
            const int n = min(local_count[threadIdx.x], kTopkPark);
            local_base[threadIdx.x] = n ? atomicAdd(&ft.count[b0 + threadIdx.x], n) : 0;
        }
        __syncthreads();
        for (int e = threadIdx.x; e < kTileBatch * kTopkPark; e += kTileThreads) {
            const int b = e / kTopkPark, i = e % kTopkPark;
            if (i < min(local_count[b], kTopkPark)) {
                const int2 c = local_cand[e];
                const int slot = local_base[b] + i;
                if (slot < ft.cap) {
                    ft.cand_val[(size_t)(b0 + b) * ft.cap + slot] = __int_as_float(c.y);
                    ft.cand_idx[(size_t)(b0 + b) * ft.cap + slot] = c.x;
                }
            }
        }
    }
    if (LOSS) {
        const double t = wave_sum((double)lsum);
        if (lane == 0) fl.partial[(size_t)blockIdx.x * (kTileThreads / 64) + (threadIdx.x >> 6)] = t;
    }
}

// ------------------------------------------------------------------------------------------------
// The same kernel over batch tiles of 64 for inputs narrow enough that an [N][64] fp32 tile of x fits in LDS
// (N <= kLane64MaxN): a row is 256 bytes and covers all 64 banks, so with the chunk order skewed by (lane & 15)
// the 32 lanes the LDS serves together hit every bank exactly twice whatever rows they read (128-byte rows sit in
// one half of the banks and the random parities of the rows cost about 1.7x), and W/idx are read once per 64
// batch rows instead of once per 32.  Plain scores only.
// ------------------------------------------------------------------------------------------------
constexpr int kLane64Batch = 64;
constexpr int kLane64MaxN = 608;        // 152 KB of LDS

template <int THREADS>
__device__ __forceinline__ void stage_rows64(float* __restrict__ xs, const float* __restrict__ src, int rows, int ld, int c0) {
    const bool vec = (ld % 4 == 0) && (c0 + kLane64Batch <= ld) && (((uintptr_t)src & 15) == 0);
    if (vec) {
        // thread -> (row, 16-byte chunk): 16 threads per row, all of a thread's loads before its first LDS write
        constexpr int kRowsPerIter = THREADS / 16;
        constexpr int kInFlight = 4;
        const int q = threadIdx.x & 15;
        const float* p = src + c0 + 4 * q;
        for (int r0 = threadIdx.x >> 4; r0 < rows; r0 += kRowsPerIter * kInFlight) {
            float4 v[kInFlight];
#pragma unroll
            for (int i = 0; i < kInFlight; ++i) {
                const int r = r0 + i * kRowsPerIter;
                v[i] = make_float4(0.f, 0.f, 0.f, 0.f);
                if (r < rows) v[i] = *reinterpret_cast<const float4*>(p + (size_t)r * ld);
            }
#pragma unroll
            for (int i = 0; i < kInFlight; ++i) {
                const int r = r0 + i * kRowsPerIter;
                if (r < rows) *reinterpret_cast<float4*>(xs + r * kLane64Batch + 4 * q) = v[i];
            }
        }
    } else {
        const int c = threadIdx.x & 63;
        const bool in = c0 + c < ld;
        const float* p = src + c0 + c;
        for (int r = threadIdx.x >> 6; r < rows; r += THREADS / 64)
            xs[r * kLane64Batch + c] = in ? p[(size_t)r * ld] : 0.f;
    }
}

// base = address of the row + (lane & 15) * 16 (the tile is 256-byte aligned: the chunk bits are flipped with XOR)
template <int C>
__device__ __forceinline__ void fwd_lane64_step(unsigned base, float wv, float (&acc)[64]) {
    const lds_v4f v = *(lds_v4f_ptr)(size_t)(C == 0 ? base : (base ^ (unsigned)(C * 16)));
    acc[4 * C + 0] = fmaf(wv, v.x, acc[4 * C + 0]);
    acc[4 * C + 1] = fmaf(wv, v.y, acc[4 * C + 1]);
    acc[4 * C + 2] = fmaf(wv, v.z, acc[4 * C + 2]);
    acc[4 * C + 3] = fmaf(wv, v.w, acc[4 * C + 3]);
}

// v[4c+i] <-> v[4(c ^ r)+i] for r in [0,16): its own inverse; four stages of conditional swaps.
__device__ __forceinline__ void xor_permute_groups64(float (&v)[64], int r) {
    const bool b8 = r & 8, b4 = r & 4, b2 = r & 2, b1 = r & 1;
#pragma unroll
    for (int e = 0; e < 64; ++e)
        if (!(e & 32)) cond_swap(b8, v[e], v[e + 32]);
#pragma unroll
    for (int e = 0; e < 64; ++e)
        if (!(e & 16)) cond_swap(b4, v[e], v[e + 16]);
#pragma unroll
    for (int e = 0; e < 64; ++e)
        if (!(e & 8)) cond_swap(b2, v[e], v[e + 8]);
#pragma unroll
    for (int e = 0; e < 64; ++e)
        if (!(e & 4)) cond_swap(b1, v[e], v[e + 4]);
}

template <bool VEC4>
__global__ __launch_bounds__(kTileThreads) void fwd_lane64_kernel(const float* __restrict__ xT, const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w, const float* __restrict__ bias,
                                                                  float* __restrict__ out, int B, int N, int L, int K, int nbt,
                                                                  int labels_per_stream) {
    extern __shared__ __align__(256) float xs[];
    const int u = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int bt = u % nbt, stream = u / nbt;
    const int b0 = bt * kLane64Batch;
    stage_rows64<kTileThreads>(xs, xT, N, B, b0);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const unsigned skewbase = (unsigned)(size_t)(__attribute__((address_space(3))) float*)xs + (unsigned)(lane & 15) * 16u;
    const int l_begin = stream * labels_per_stream;
    const int l_end = min(l_begin + labels_per_stream, L);
    // rows of out for this batch tile, reached through a scalar row offset plus the lane's label; rows past the batch
    // lie beyond the resource's size and their stores are dropped
    const int nrows = min(kLane64Batch, B - b0);
    const buffer_rsrc orsrc = make_rsrc(out + (size_t)b0 * (size_t)L, (size_t)nrows * (size_t)L * sizeof(float));
    for (int base = l_begin; base < l_end; base += kTileThreads) {
        if (base + (int)(threadIdx.x & ~63u) >= l_end) break;     // nothing left for this wavefront
        const int j = base + (int)threadIdx.x;
        const bool valid = j < l_end;
        const int jj = valid ? j : l_end - 1;
        const int32_t* irow = idx + (size_t)jj * K;
        const float* wrow = w + (size_t)jj * K;
        float acc[64];
#pragma unroll
        for (int i = 0; i < 64; ++i) acc[i] = 0.f;
        for (int k0 = 0; k0 < K; k0 += 16) {
            const bool full = VEC4 && k0 + 16 <= K;
            unsigned idp[8];
            float wv[16];
            if (full) {
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int4 v = *reinterpret_cast<const int4*>(irow + k0 + 4 * q);
                    idp[2 * q + 0] = (unsigned)v.x | ((unsigned)v.y << 16);
                    idp[2 * q + 1] = (unsigned)v.z | ((unsigned)v.w << 16);
                    const float4 f = *reinterpret_cast<const float4*>(wrow + k0 + 4 * q);
                    wv[4 * q] = f.x; wv[4 * q + 1] = f.y; wv[4 * q + 2] = f.z; wv[4 * q + 3] = f.w;
                }
            } else {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const unsigned a = (k0 + 2 * q < K) ? (unsigned)irow[k0 + 2 * q] : 0u;
                    const unsigned b = (k0 + 2 * q + 1 < K) ? (unsigned)irow[k0 + 2 * q + 1] : 0u;
                    idp[q] = a | (b << 16);
                }
#pragma unroll
                for (int k = 0; k < 16; ++k) wv[k] = (k0 + k < K) ? wrow[k0 + k] : 0.f;
            }
            const int kn = min(16, K - k0);
#pragma unroll
            for (int k = 0; k < 16; ++k) {
                if (full || k < kn) {
                    const unsigned id = (k & 1) ? (idp[k >> 1] >> 16) : (idp[k >> 1] & 0xffffu);
                    const unsigned rb = (id << 8) + skewbase;
                    fwd_lane64_step<0>(rb, wv[k], acc); fwd_lane64_step<1>(rb, wv[k], acc);
                    fwd_lane64_step<2>(rb, wv[k], acc); fwd_lane64_step<3>(rb, wv[k], acc);
                    fwd_lane64_step<4>(rb, wv[k], acc); fwd_lane64_step<5>(rb, wv[k], acc);
                    fwd_lane64_step<6>(rb, wv[k], acc); fwd_lane64_step<7>(rb, wv[k], acc);
                    fwd_lane64_step<8>(rb, wv[k], acc); fwd_lane64_step<9>(rb, wv[k], acc);
                    fwd_lane64_step<10>(rb, wv[k], acc); fwd_lane64_step<11>(rb, wv[k], acc);
                    fwd_lane64_step<12>(rb, wv[k], acc); fwd_lane64_step<13>(rb, wv[k], acc);
                    fwd_lane64_step<14>(rb, wv[k], acc); fwd_lane64_step<15>(rb, wv[k], acc);
                }
            }
        }
        xor_permute_groups64(acc, lane & 15);              // back to natural batch order
        if (bias != nullptr) {                             // added after the sum, as a separate bias_add would
            const float bj = bias[jj];
#pragma unroll
            for (int i = 0; i < 64; ++i) acc[i] += bj;
        }
        if (valid) {
            const unsigned lane_off = (unsigned)j * 4u;
            const unsigned stride = (unsigned)L * 4u;
#pragma unroll
            for (int b = 0; b < 64; ++b)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[b]), orsrc, lane_off, (unsigned)b * stride, 0);
        }
    }
}

template <bool VEC4>
int launch_lane64(const float* xT, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d, hipStream_t s) {
    const int cus = device_cu_count();
    const int nbt = (d.B + kLane64Batch - 1) / kLane64Batch;
    int streams = std::max(1, cus / nbt);
    const int per_stream = (d.L + streams - 1) / streams;
    streams = (d.L + per_stream - 1) / per_stream;
    const size_t lds = (size_t)d.N * kLane64Batch * sizeof(float);
    FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_lane64_kernel<VEC4>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((fwd_lane64_kernel<VEC4>), dim3(streams * nbt), dim3(kTileThreads), lds, s, xT, idx, w, bias, out, d.B, d.N,
                       d.L, d.K, nbt, per_stream);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

// (64 rows of out of a batch tile are reached through 32-bit byte offsets)
// Where the tile of 64 samples fits, and where it pays.  Measured against the 32-sample kernel at 501,070 labels, 256-608
// columns: +2...+10 % from 192 samples up at every fan-in, -3...-14 % at 64-160 samples with a fan-in up to 40; +5...+12 %
// from 128 samples up with a fan-in of 64 or more; +20...+37 % at fan-in 48 at every batch size (a last chunk of 16
// connections is a full chunk here, and loaded one by one there).
bool lane64_fits(const Dims& d) {
    if (d.N > kLane64MaxN || d.B <= kTileBatch || d.L >= (1 << 24) || g_options.fwd_lane64 < 0) return false;
    return d.B >= 192 || (d.K >= 64 && d.B >= 128) || (d.K > 32 && d.K % 32 != 0 && d.K % 16 == 0);
}

}  // namespace

namespace {

constexpr int kTopkSample = 4096;      // labels whose scores set the per-sample thresholds

// scores of every (L / S)-th label for all samples: sample_scores[b][i] (the thresholds' raw material)
__global__ __launch_bounds__(256) void fwd_sample_kernel(const float* __restrict__ xT, const int32_t* __restrict__ idx,
                                                         const float* __restrict__ w, const float* __restrict__ bias, int B, int N,
                                                         int L, int K, int S, float* __restrict__ sample_scores) {
    const int i = blockIdx.x;
    const int j = (int)(((long long)i * L) / S);
    const int32_t* irow = idx + (size_t)j * K;
    const float* wrow = w + (size_t)j * K;
    for (int b = threadIdx.x; b < B; b += 256) {
        float acc = 0.f, mag = 0.f;
        for (int k = 0; k < K; ++k) {
            const unsigned id = (unsigned)irow[k];
            const float xv = xT[(size_t)(id < (unsigned)N ? id : 0u) * B + b];
            acc = fmaf(wrow[k], xv, acc);
            mag = fmaf(fabsf(wrow[k]), fabsf(xv), mag);
        }
        if (bias != nullptr) { acc += bias[j]; mag += fabsf(bias[j]); }
        // The main kernel sums the same products in another order; its score of this label differs from `acc` by at
        // most a few rounding errors of the largest partial sum (K * 2^-24 * mag).  The threshold must not exceed the
        // main kernel's value, so the sampled score is lowered by a bound on that difference.
        sample_scores[(size_t)b * S + i] = acc - (float)(K + 2) * 1.2e-7f * mag;
    }
}

template <int VEC, int EPI, bool TOPK>
int launch_lane32(const float* xT, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d, int nbt,
                  int per_stream, int blocks, size_t lds, const FwdLoss& fl, const FwdTopk& ft, hipStream_t s) {
    FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_lane32_kernel<VEC, EPI, TOPK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((fwd_lane32_kernel<VEC, EPI, TOPK>), dim3(blocks), dim3(kTileThreads), lds, s, xT, idx, w, bias, out, d.B, d.N,
                       d.L, d.K, nbt, per_stream, fl, ft);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

template <int EPI>
int launch_lane32_any(bool vec4, bool topk, const float* xT, const int32_t* idx, const float* w, const float* bias, float* out,
                      const Dims& d, int nbt, int per_stream, int blocks, size_t lds, const FwdLoss& fl, const FwdTopk& ft,
                      hipStream_t s) {
    // (see fwd_lane32_kernel: 2 = quads, fan-in below one chunk)
    // Rows that are not 16-byte aligned (a fan-in that is no multiple of four, or unaligned arrays) still take build 1
    // when they hold a full chunk: its 16-byte loads are per-lane gathers of 4-byte-aligned addresses, which the
    // memory system serves, and only the last, partly filled chunk is loaded one by one (fan-in 33: 412 -> 215 us, fan-in 63: 1.10 -> 0.58 ms).
    const int vec = vec4 ? (d.K < 32 ? 2 : 1) : ((((uintptr_t)w | (uintptr_t)idx) % 4 == 0 && d.K >= 32) ? 1 : 0);
#define FFI_LANE32(VEC, E, T) launch_lane32<VEC, E, T>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, ft, s)
    if constexpr (EPI != kEpiLossGradSkewed) {              // (that epilogue has no top-k form)
        if (topk) return vec == 2 ? FFI_LANE32(2, EPI, true) : vec == 1 ? FFI_LANE32(1, EPI, true) : FFI_LANE32(0, EPI, true);
    }
    if (EPI == kEpiNone) return FFI_OK;                     // nothing to compute
    constexpr int E = EPI == kEpiNone ? kEpiScores : EPI;
    return vec == 2 ? FFI_LANE32(2, E, false) : vec == 1 ? FFI_LANE32(1, E, false) : FFI_LANE32(0, E, false);
#undef FFI_LANE32
}

// Narrow-input forward pass with the given epilogue; `la` is needed for the loss epilogues only, `tk` (may be
// null) asks for the per-sample top-k without the score matrix.
// `xt_scratch` (may be null): room for N * B floats that takes the place of the library workspace for the
// batch-major copy of [B,N] features.
int forward_tiles(const float* x, const int32_t* idx, const float* w, const float* bias, float* out, float* gout, int epi,
                  const LossArgs* la, const TopkArgs* tk, const Dims& d, hipStream_t s, float* xt_scratch = nullptr) {
    const float* xT = x;
    if (!d.tp) {
        float* ws = xt_scratch;
        if (ws == nullptr) FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)d.N * d.B * sizeof(float), (void**)&ws));
        FFI_TRY(launch_transpose(x, ws, d.B, d.N, s));   // [B,N] -> [N,B]
        xT = ws;
    }
    const size_t lds = tile_lds_bytes(d.N);
    const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)w | (uintptr_t)idx) % 16 == 0);
    if (epi == kEpiScores && tk == nullptr && lane64_fits(d)) {
        // (16-byte loads for the full chunks of 16 also where rows are only 4-byte aligned: see launch_lane32_any)
        const bool quads = vec4 || ((((uintptr_t)w | (uintptr_t)idx) % 4 == 0) && d.K >= 16);
        return quads ? launch_lane64<true>(xT, idx, w, bias, out, d, s) : launch_lane64<false>(xT, idx, w, bias, out, d, s);
    }
    const int cus = device_cu_count();
    const int nbt = (d.B + kTileBatch - 1) / kTileBatch;
    int streams = std::max(1, cus / nbt);
    const int per_stream = (d.L + streams - 1) / streams;
    streams = (d.L + per_stream - 1) / per_stream;
    const int blocks = streams * nbt;
    FwdLoss fl{gout, nullptr, nullptr, 0.f, 0, 0};
    FwdTopk ft{};
    const bool topk = tk != nullptr;
    int* count = nullptr;
    size_t lds_topk = lds;
    if (topk) {
        // thresholds: the k-th best score of every sample among kTopkSample evenly spaced labels
        const int S = std::min(kTopkSample, d.L);
        const size_t cand = (size_t)d.B * kTopkCap;
        unsigned char* ws = nullptr;
        const size_t bytes = ((size_t)d.B * S + 2 * (size_t)d.B * 8 + (size_t)d.B + 2 * cand) * 4;
        FFI_TRY(workspace_get(s, kWsTopk, bytes, (void**)&ws));
        float* sample_scores = reinterpret_cast<float*>(ws);
        float* tau_val = sample_scores + (size_t)d.B * S;
        int* tau_idx = reinterpret_cast<int*>(tau_val + (size_t)d.B * 8);
        count = tau_idx + (size_t)d.B * 8;
        float* cand_val = reinterpret_cast<float*>(count + d.B);
        int* cand_idx = reinterpret_cast<int*>(cand_val + cand);
        hipLaunchKernelGGL(fwd_sample_kernel, dim3(S), dim3(256), 0, s, xT, idx, w, bias, d.B, d.N, d.L, d.K, S, sample_scores);
        FFI_HIP_TRY(hipGetLastError());
        FFI_TRY(launch_topk_f32(sample_scores, d.B, S, tk->k, tau_val, tau_idx, s));
        FFI_TRY(launch_topk_candidates_init(count, cand_idx, d.B, kTopkCap, s));
        // LDS behind the tile of x holds the workgroup's candidates until the end of the kernel
        ft = FwdTopk{tau_val + (tk->k - 1), tk->k, count, cand_val, cand_idx, kTopkCap};
        lds_topk = lds + (size_t)kTileBatch * kTopkPark * sizeof(int2);
    }
    int npartial = 0;
    double* corr = nullptr;
    if (epi == kEpiLossGrad || epi == kEpiLossGradAndScores) {
        npartial = blocks * (kTileThreads / 64);
        FFI_TRY(loss_partial_buffer(s, npartial, la->nnz, &fl.partial, &corr, nullptr));
        fl.scale = la->scale;
        fl.kind = la->kind;
        fl.words = la->nz_words;
        fl.skip_zero_stores = la->skip_zero_stores ? 1 : 0;
    }
    if (epi == kEpiScores) FFI_TRY(launch_lane32_any<kEpiScores>(vec4, topk, xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds_topk, fl, ft, s));
    else if (epi == kEpiLossGrad && !topk && fl.skip_zero_stores)
        FFI_TRY(launch_lane32_any<kEpiLossGradSkewed>(vec4, false, xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds_topk, fl, ft, s));
    else if (epi == kEpiLossGrad) FFI_TRY(launch_lane32_any<kEpiLossGrad>(vec4, topk, xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds_topk, fl, ft, s));
    else if (epi == kEpiLossGradAndScores) FFI_TRY(launch_lane32_any<kEpiLossGradAndScores>(vec4, topk, xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds_topk, fl, ft, s));
    else FFI_TRY(launch_lane32_any<kEpiNone>(vec4, topk, xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds_topk, fl, ft, s));
    if (topk) {
        // (a sample with more candidates than its list holds: its row once more, from the score matrix if there is one)
        TopkRowSource src;
        if (epi == kEpiScores || epi == kEpiLossGradAndScores) src.scores = out;
        src.xT = xT; src.idx = idx; src.w = w; src.bias = bias; src.N = d.N; src.L = d.L; src.K = d.K;
        FFI_TRY(launch_topk_candidates_select(ft.cand_val, ft.cand_idx, count, d.B, kTopkCap, tk->k, tk->values, tk->indices, s, src));
    }
    if (epi != kEpiLossGrad && epi != kEpiLossGradAndScores) return FFI_OK;
    // the listed label positions: from the score matrix when it was written, else recomputed from x ([N,B] here)
    Dims dt = d;
    dt.tp = true;
    float* g = epi == kEpiLossGrad ? out : gout;
    return launch_loss_positives(*la, nullptr, epi == kEpiLossGrad ? nullptr : out, xT, idx, w, bias, g, dt, fl.partial, npartial,
                                 corr, s);
}

}  // namespace

int launch_forward(const float* x, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d,
                   hipStream_t s) {
    // (the kernel reaches the 32 rows of out of a batch tile through 32-bit byte offsets)
    if (tile_path_fits(d.N) && d.L < (1 << 25)) return forward_tiles(x, idx, w, bias, out, nullptr, kEpiScores, nullptr, nullptr, d, s);
    return launch_forward_wide(x, idx, w, bias, out, d, s);
}

int launch_forward_loss(const float* x, const int32_t* idx, const float* w, const float* bias, const LossArgs& la,
                        float* scores, float* g, const TopkArgs* tk, const Dims& d, hipStream_t s) {
    if (tile_path_fits(d.N) && d.L < (1 << 25)) {
        if (scores == nullptr) return forward_tiles(x, idx, w, bias, g, nullptr, kEpiLossGrad, &la, tk, d, s);
        return forward_tiles(x, idx, w, bias, scores, g, kEpiLossGradAndScores, &la, tk, d, s);
    }
    // wide inputs: scores by the wide kernel (into g itself when the caller wants no scores), top-k from them, then
    // the loss gradient as a pass of its own
    float* sc = scores ? scores : g;
    FFI_TRY(launch_forward_wide(x, idx, w, bias, sc, d, s));
    if (tk != nullptr) FFI_TRY(launch_topk_f32(sc, d.B, d.L, tk->k, tk->values, tk->indices, s));
    return launch_loss_grad(la, sc, g, d.B, d.L, s);
}

int launch_forward_topk(const float* x, const int32_t* idx, const float* w, const float* bias, float* scores, const TopkArgs& tk,
                        const Dims& d, hipStream_t s) {
    if (tile_path_fits(d.N) && d.L < (1 << 25))
        return forward_tiles(x, idx, w, bias, scores, nullptr, scores ? kEpiScores : kEpiNone, nullptr, &tk, d, s);
    // wide inputs: the score matrix (the caller's, or a workspace), then its top-k
    float* sc = scores;
    if (sc == nullptr) FFI_TRY(workspace_get(s, kWsScores, (size_t)d.B * d.L * sizeof(float), (void**)&sc));
    FFI_TRY(launch_forward_wide(x, idx, w, bias, sc, d, s));
    return launch_topk_f32(sc, d.B, d.L, tk.k, tk.values, tk.indices, s);
}

// ---- forward pass for callers that cannot allocate ------------------------------------------------
// The only device memory the narrow forward pass needs beyond its inputs and outputs is the [N][B]
// copy of [B,N] features.  Here it lives in a fixed array inside the library's code object (one copy
// per GPU, held until the process ends) instead of a workspace from hipMalloc.
namespace {

constexpr size_t kNoAllocFloats = (size_t)1 << 20;             // 4 MiB: batch * num_features may not exceed this
static __device__ __align__(256) float scratch[kNoAllocFloats];

constexpr int kNoAllocMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kNoAllocMaxDevices] = {nullptr};           // device address of `scratch` on each GPU

// The address of this GPU's copy of `scratch` (looked up once per device, with that device current).
int scratch_address(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return FFI_ERR_NO_DEVICE; }
    if (dev < 0 || dev >= kNoAllocMaxDevices) return FFI_ERR_NO_DEVICE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        float* ptr = nullptr;
        FFI_HIP_TRY(hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch)));
        if (ptr == nullptr) return FFI_ERR_HIP;
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return FFI_OK;
}

}  // namespace
}  // namespace ffi

extern "C" int ffi_forward_noalloc_f32(const float* features, const int32_t* lookup, const float* weights, float* result,
                                       int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed,
                                       ffi_stream_t stream) {
    using namespace ffi;
    StreamCall call_lock((hipStream_t)stream);
    if (!features || !lookup || !weights || !result) return FFI_ERR_NULL_POINTER;
    if (batch <= 0 || num_features <= 0 || num_units <= 0 || fan_in <= 0) return FFI_ERR_BAD_SHAPE;
    if (batch >= INT32_MAX || num_features >= INT32_MAX || num_units >= INT32_MAX || fan_in >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    if (num_units * fan_in >= INT32_MAX) return FFI_ERR_TOO_LARGE;
    // only the shapes of the narrow kernel, which needs nothing but the fixed array
    if (!tile_path_fits((int)num_features) || num_units >= (1 << 25)) return FFI_ERR_TOO_LARGE;
    if ((uint64_t)batch * (uint64_t)num_features > kNoAllocFloats) return FFI_ERR_TOO_LARGE;
    const Dims d{(int)batch, (int)num_features, (int)num_units, (int)fan_in, transposed != 0};
    float* xt = nullptr;
    if (!d.tp) FFI_TRY(scratch_address(&xt));
    return forward_tiles(features, lookup, weights, nullptr, result, nullptr, kEpiScores, nullptr, nullptr, d, (hipStream_t)stream, xt);
}
