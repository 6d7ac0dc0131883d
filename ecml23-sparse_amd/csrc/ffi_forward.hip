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
template <int C>
__device__ __forceinline__ void fwd_lane_step(const char* __restrict__ xs_bytes, unsigned base, float wv, float (&acc)[32]) {
    const float4 v = *reinterpret_cast<const float4*>(xs_bytes + skew_addr<C>(base));
    acc[4 * C + 0] = fmaf(wv, v.x, acc[4 * C + 0]);
    acc[4 * C + 1] = fmaf(wv, v.y, acc[4 * C + 1]);
    acc[4 * C + 2] = fmaf(wv, v.z, acc[4 * C + 2]);
    acc[4 * C + 3] = fmaf(wv, v.w, acc[4 * C + 3]);
}

// What the kernel does with a finished score s (after the bias):
//   kEpiScores       out = s
//   kEpiLossGrad     out = scale * dloss(s, 0)/ds, the loss gradient of a position that is not a listed label
//                    (listed positions are patched afterwards), and the loss(s, 0) summed per wavefront
//   kEpiLossGradAndScores  both: scores to `out`, gradients to `gout`
enum FwdEpilogue { kEpiScores = 0, kEpiLossGrad = 1, kEpiLossGradAndScores = 2 };

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
__device__ __forceinline__ void loss_epilogue(float (&acc)[32], int nrows, float scale, float& loss, unsigned& mask) {
    float l = 0.f;
    unsigned m = 0;
    if (nrows == 32) {
#pragma unroll
        for (int b = 0; b < 32; ++b) {
            float lb, gb;
            cwise_loss_and_grad(KIND, acc[b], 0.f, lb, gb);
            l += lb;
            m |= (gb != 0.f ? 1u : 0u) << b;
            acc[b] = scale * gb;
        }
    } else {                               // last batch tile: rows past the batch count for nothing
#pragma unroll
        for (int b = 0; b < 32; ++b) {
            float lb, gb;
            cwise_loss_and_grad(KIND, acc[b], 0.f, lb, gb);
            l += b < nrows ? lb : 0.f;
            m |= (b < nrows && gb != 0.f ? 1u : 0u) << b;
            acc[b] = scale * gb;
        }
    }
    loss = l;
    mask = m;
}

template <bool VEC4, int EPI>
__global__ __launch_bounds__(kTileThreads) void fwd_lane32_kernel(const float* __restrict__ xT,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w,
                                                                  const float* __restrict__ bias,
                                                                  float* __restrict__ out, int B, int N,
                                                                  int L, int K, int nbt, int labels_per_stream,
                                                                  FwdLoss fl) {
    extern __shared__ __align__(16) float xs[];
    const char* xs_bytes = reinterpret_cast<const char*>(xs);
    const int u = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int bt = u % nbt, stream = u / nbt;
    const int b0 = bt * kTileBatch;
    stage_rows32<kTileThreads>(xs, xT, N, B, b0);
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const unsigned skew = (unsigned)(lane & 7) * 16u;
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
            const bool full = VEC4 && k0 + 32 <= K;
            unsigned idp[16];
            float wv[32];
            if (full) {
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
                    const unsigned rb = (id << 7) | skew;
                    fwd_lane_step<0>(xs_bytes, rb, wv[k], acc); fwd_lane_step<1>(xs_bytes, rb, wv[k], acc);
                    fwd_lane_step<2>(xs_bytes, rb, wv[k], acc); fwd_lane_step<3>(xs_bytes, rb, wv[k], acc);
                    fwd_lane_step<4>(xs_bytes, rb, wv[k], acc); fwd_lane_step<5>(xs_bytes, rb, wv[k], acc);
                    fwd_lane_step<6>(xs_bytes, rb, wv[k], acc); fwd_lane_step<7>(xs_bytes, rb, wv[k], acc);
                }
            }
        }
        xor_permute_groups(acc, lane & 7);                 // back to natural batch order
        if (bias != nullptr) {                             // added after the sum, as a separate bias_add would
            const float bj = bias[jj];
#pragma unroll
            for (int i = 0; i < 32; ++i) acc[i] += bj;
        }
        const unsigned lane_off = (unsigned)j * 4u;
        const unsigned stride = (unsigned)L * 4u;
        if (EPI != kEpiLossGrad && valid) {
#pragma unroll
            for (int b = 0; b < 32; ++b)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[b]), orsrc, lane_off, (unsigned)b * stride, 0);
        }
        if (EPI != kEpiScores) {
            float l = 0.f;
            unsigned m = 0;
            // the loss kind is the same for the whole launch: one straight-line epilogue per kind
            if (fl.kind == FFI_LOSS_SQUARED_HINGE) loss_epilogue<FFI_LOSS_SQUARED_HINGE>(acc, nrows, fl.scale, l, m);
            else if (fl.kind == FFI_LOSS_HINGE) loss_epilogue<FFI_LOSS_HINGE>(acc, nrows, fl.scale, l, m);
            else loss_epilogue<FFI_LOSS_BCE>(acc, nrows, fl.scale, l, m);
            if (valid) {
                lsum += l;
                if (fl.skip_zero_stores) {
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
    if (EPI != kEpiScores) {
        const double t = wave_sum((double)lsum);
        if (lane == 0) fl.partial[(size_t)blockIdx.x * (kTileThreads / 64) + (threadIdx.x >> 6)] = t;
    }
}

}  // namespace

namespace {

template <bool VEC4, int EPI>
int launch_lane32(const float* xT, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d, int nbt,
                  int per_stream, int blocks, size_t lds, const FwdLoss& fl, hipStream_t s) {
    FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_lane32_kernel<VEC4, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    hipLaunchKernelGGL((fwd_lane32_kernel<VEC4, EPI>), dim3(blocks), dim3(kTileThreads), lds, s, xT, idx, w, bias, out, d.B, d.N,
                       d.L, d.K, nbt, per_stream, fl);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

// Narrow-input forward pass with the given epilogue; `la` is needed for the loss epilogues only.
int forward_tiles(const float* x, const int32_t* idx, const float* w, const float* bias, float* out, float* gout, int epi,
                  const LossArgs* la, const Dims& d, hipStream_t s) {
    const float* xT = x;
    if (!d.tp) {
        float* ws = nullptr;
        FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)d.N * d.B * sizeof(float), (void**)&ws));
        FFI_TRY(launch_transpose(x, ws, d.B, d.N, s));   // [B,N] -> [N,B]
        xT = ws;
    }
    const size_t lds = tile_lds_bytes(d.N);
    const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)w | (uintptr_t)idx) % 16 == 0);
    const int cus = device_cu_count();
    const int nbt = (d.B + kTileBatch - 1) / kTileBatch;
    int streams = std::max(1, cus / nbt);
    const int per_stream = (d.L + streams - 1) / streams;
    streams = (d.L + per_stream - 1) / per_stream;
    const int blocks = streams * nbt;
    FwdLoss fl{gout, nullptr, nullptr, 0.f, 0, 0};
    if (epi == kEpiScores)
        return vec4 ? launch_lane32<true, kEpiScores>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, s)
                    : launch_lane32<false, kEpiScores>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, s);
    const int npartial = blocks * (kTileThreads / 64);
    double* corr = nullptr;
    FFI_TRY(loss_partial_buffer(s, npartial, la->nnz, &fl.partial, &corr, nullptr));
    fl.scale = la->scale;
    fl.kind = la->kind;
    fl.words = la->nz_words;
    fl.skip_zero_stores = la->skip_zero_stores ? 1 : 0;
    if (epi == kEpiLossGrad) {
        FFI_TRY(vec4 ? (launch_lane32<true, kEpiLossGrad>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, s))
                     : (launch_lane32<false, kEpiLossGrad>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, s)));
    } else {
        FFI_TRY(vec4 ? (launch_lane32<true, kEpiLossGradAndScores>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, s))
                     : (launch_lane32<false, kEpiLossGradAndScores>(xT, idx, w, bias, out, d, nbt, per_stream, blocks, lds, fl, s)));
    }
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
    if (tile_path_fits(d.N) && d.L < (1 << 25)) return forward_tiles(x, idx, w, bias, out, nullptr, kEpiScores, nullptr, d, s);
    return launch_forward_wide(x, idx, w, bias, out, d, s);
}

int launch_forward_loss(const float* x, const int32_t* idx, const float* w, const float* bias, const LossArgs& la,
                        float* scores, float* g, const Dims& d, hipStream_t s) {
    if (tile_path_fits(d.N) && d.L < (1 << 25)) {
        if (scores == nullptr) return forward_tiles(x, idx, w, bias, g, nullptr, kEpiLossGrad, &la, d, s);
        return forward_tiles(x, idx, w, bias, scores, g, kEpiLossGradAndScores, &la, d, s);
    }
    // wide inputs: scores by the wide kernel (into g itself when the caller wants no scores), then the
    // loss gradient as a pass of its own
    float* sc = scores ? scores : g;
    FFI_TRY(launch_forward_wide(x, idx, w, bias, sc, d, s));
    return launch_loss_grad(la, sc, g, d.B, d.L, s);
}

}  // namespace ffi
