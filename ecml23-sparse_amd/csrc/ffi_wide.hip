// Wide-input kernels of the fixed-fan-in sparse layer for gfx950 (any shape; used when a
// [N][32] tile of x does not fit in LDS).
//
// With tens of thousands of input columns neither x nor out_grad can live in LDS, so the gathered
// operand comes through the cache hierarchy instead.  Everything is arranged so that one gather is
// one contiguous row: features are used as xT[N][B] and out_grad (for the input gradient) as
// gT[L][B], lanes run along the batch, and the column id / weight of the current connection are
// wave-uniform scalars.  The kernels are bound by cache (L2 / last-level) bandwidth: every
// connection moves B*4 bytes.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>

namespace ffi {
namespace {

constexpr int kWideThreads = 256;   // 4 wavefronts per workgroup
constexpr int kWideLabels = 64;     // labels per workgroup: 16 per wavefront
constexpr int kWideBatch = 128;     // batch entries per pass: each lane owns b and b+64
constexpr int kWideInflight = 8;      // connections whose gathers a wavefront has in flight
constexpr int kWideStride = kWideBatch + 1;   // LDS row stride in floats (odd: conflict-free both ways)

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

// ---- forward ------------------------------------------------------------------------------------
// grid (label blocks, batch passes).  A wavefront walks 16 labels one after the other; per
// connection it loads one 512-byte piece of row idx[j,k] of xT and does two multiply-adds per lane.
// Results go through LDS so that out is written in 256-byte rows.
// TWO == false (batch <= 64): lanes own one batch entry each, the loads and multiply-adds of the second half are left out.
template <bool TWO>
__global__ __launch_bounds__(kWideThreads) void fwd_wide_kernel(const float* __restrict__ xT,
                                                                const int32_t* __restrict__ idx,
                                                                const float* __restrict__ w,
                                                                const float* __restrict__ bias, float* __restrict__ out,
                                                                int B, int N, int L, int K, int ldb) {
    __shared__ float tile[kWideLabels * kWideStride];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j0 = blockIdx.x * kWideLabels;
    const int bc0 = blockIdx.y * kWideBatch;
    const buffer_rsrc xr = make_rsrc(xT, (size_t)N * (size_t)ldb * sizeof(float));
    const unsigned lane_off0 = (unsigned)(bc0 + lane) * 4u, lane_off1 = lane_off0 + 256u;
    const unsigned row_bytes = (unsigned)ldb * 4u;
    for (int q = 0; q < kWideLabels / 4; ++q) {
        const int jl = wave * (kWideLabels / 4) + q;
        const int j = j0 + jl;
        float acc0 = 0.f, acc1 = 0.f;
        if (j < L) {                                            // wave-uniform
            const int32_t* irow = idx + (size_t)j * K;
            const float* wrow = w + (size_t)j * K;
            for (int k0 = 0; k0 < K; k0 += 64) {
                const int kn = min(64, K - k0);
                // one connection per lane, handed out below as wave-uniform scalars
                const unsigned iv = (lane < kn) ? (unsigned)irow[k0 + lane] : 0u;
                const float wv = (lane < kn) ? wrow[k0 + lane] : 0.f;
                int k = 0;
                for (; k + kWideInflight <= kn; k += kWideInflight) {
                    float x0[kWideInflight], x1[kWideInflight], ws[kWideInflight];
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        const unsigned n = (unsigned)__builtin_amdgcn_readlane((int)iv, k + u);
                        ws[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), k + u));
                        x0[u] = buffer_load_f32(xr, lane_off0, n * row_bytes);
                        x1[u] = TWO ? buffer_load_f32(xr, lane_off1, n * row_bytes) : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        acc0 = fmaf(ws[u], x0[u], acc0);
                        if (TWO) acc1 = fmaf(ws[u], x1[u], acc1);
                    }
                }
                if (k < kn) {
                    // the last, partly filled group, its gathers in flight together like the others: connections behind
                    // the end repeat the last one and are left out of the sum (one gather at a time cost 40 % at fan-in 12)
                    float x0[kWideInflight], x1[kWideInflight], ws[kWideInflight];
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        const int kk = min(k + u, kn - 1);
                        const unsigned n = (unsigned)__builtin_amdgcn_readlane((int)iv, kk);
                        const float wk = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), kk));
                        ws[u] = wk;
                        x0[u] = buffer_load_f32(xr, lane_off0, n * row_bytes);
                        x1[u] = TWO ? buffer_load_f32(xr, lane_off1, n * row_bytes) : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        if (k + u < kn) {                       // wave-uniform
                            acc0 = fmaf(ws[u], x0[u], acc0);
                            if (TWO) acc1 = fmaf(ws[u], x1[u], acc1);
                        }
                    }
                }
            }
        }
        tile[jl * kWideStride + lane] = acc0;
        tile[jl * kWideStride + 64 + lane] = acc1;
    }
    __syncthreads();
    // out[b, j0 .. j0+63]: one wavefront writes one 256-byte row per step
    const int jl = threadIdx.x & 63;
    if (j0 + jl < L) {
        const bool has_bias = bias != nullptr;
        const float bj = has_bias ? bias[j0 + jl] : 0.f;
        for (int bb = threadIdx.x >> 6; bb < (TWO ? kWideBatch : kWideBatch / 2); bb += kWideThreads / 64) {
            const int b = bc0 + bb;
            const float v = tile[jl * kWideStride + bb];
            if (b < B) out[(size_t)b * L + j0 + jl] = has_bias ? v + bj : v;
        }
    }
}

// ---- weight gradient ----------------------------------------------------------------------------
// grid (label blocks).  Per batch pass the workgroup brings g[b, j0..j0+63] into LDS (coalesced
// along labels), then every wavefront handles 16 labels: per connection one 512-byte piece of the
// xT row times the label's out_grad, summed over the lanes, accumulated over the batch passes in
// LDS by a single lane (fixed order: reproducible).
template <bool TWO>
__global__ __launch_bounds__(kWideThreads) void wgrad_wide_kernel(const float* __restrict__ xT,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ g, float* __restrict__ gw,
                                                                  float* __restrict__ bias_grad, int B, int N, int L,
                                                                  int K, int ldb) {
    extern __shared__ float smem[];
    float* gt = smem;                                   // [64 labels][129]
    float* res = smem + kWideLabels * kWideStride;      // [64 labels][K]
    float* bres = res + kWideLabels * K;                // [64 labels] column sums of out_grad
    if (threadIdx.x < kWideLabels) bres[threadIdx.x] = 0.f;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j0 = blockIdx.x * kWideLabels;
    const buffer_rsrc xr = make_rsrc(xT, (size_t)N * (size_t)ldb * sizeof(float));
    const unsigned row_bytes = (unsigned)ldb * 4u;
    for (int t = threadIdx.x; t < kWideLabels * K; t += kWideThreads) res[t] = 0.f;
    for (int bc0 = 0; bc0 < B; bc0 += kWideBatch) {
        __syncthreads();
        {
            const int jl = threadIdx.x & 63;
            const bool in = j0 + jl < L;
            for (int bb = threadIdx.x >> 6; bb < (TWO ? kWideBatch : kWideBatch / 2); bb += kWideThreads / 64) {
                const int b = bc0 + bb;
                gt[jl * kWideStride + bb] = (in && b < B) ? g[(size_t)b * L + j0 + jl] : 0.f;
            }
        }
        __syncthreads();
        const unsigned lane_off0 = (unsigned)(bc0 + lane) * 4u, lane_off1 = lane_off0 + 256u;
        // lanes past the end of the batch would read the next row of xT: their out_grad is zero, but
        // keep their x operand finite too
        const bool in0 = bc0 + lane < B, in1 = bc0 + 64 + lane < B;
        for (int q = 0; q < kWideLabels / 4; ++q) {
            const int jl = wave * (kWideLabels / 4) + q;
            const int j = j0 + jl;
            if (j >= L) break;                                  // wave-uniform
            const float g0 = gt[jl * kWideStride + lane], g1 = TWO ? gt[jl * kWideStride + 64 + lane] : 0.f;
            if (bias_grad != nullptr) {                         // wave-uniform
                const float gs = wave_sum(g0 + g1);
                if (lane == 0) bres[jl] += gs;
            }
            const int32_t* irow = idx + (size_t)j * K;
            for (int k0 = 0; k0 < K; k0 += 64) {
                const int kn = min(64, K - k0);
                const unsigned iv = (lane < kn) ? (unsigned)irow[k0 + lane] : 0u;
                float mine = 0.f;                               // lane k collects connection k0+k
                int k = 0;
                for (; k + kWideInflight <= kn; k += kWideInflight) {
                    float x0[kWideInflight], x1[kWideInflight];
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        const unsigned n = (unsigned)__builtin_amdgcn_readlane((int)iv, k + u);
                        x0[u] = buffer_load_f32(xr, lane_off0, n * row_bytes);
                        x1[u] = TWO ? buffer_load_f32(xr, lane_off1, n * row_bytes) : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        const float p = TWO ? fmaf(in1 ? x1[u] : 0.f, g1, (in0 ? x0[u] : 0.f) * g0) : (in0 ? x0[u] : 0.f) * g0;
                        const float s = wave_sum(p);
                        if (lane == k + u) mine = s;
                    }
                }
                if (k < kn) {
                    // (the last, partly filled group: gathers in flight together, the connections behind the end repeat
                    // the last one and are not kept)
                    float x0[kWideInflight], x1[kWideInflight];
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        const unsigned n = (unsigned)__builtin_amdgcn_readlane((int)iv, min(k + u, kn - 1));
                        x0[u] = buffer_load_f32(xr, lane_off0, n * row_bytes);
                        x1[u] = TWO ? buffer_load_f32(xr, lane_off1, n * row_bytes) : 0.f;
                    }
#pragma unroll
                    for (int u = 0; u < kWideInflight; ++u) {
                        if (k + u < kn) {                       // wave-uniform
                            const float p = TWO ? fmaf(in1 ? x1[u] : 0.f, g1, (in0 ? x0[u] : 0.f) * g0) : (in0 ? x0[u] : 0.f) * g0;
                            const float s = wave_sum(p);
                            if (lane == k + u) mine = s;
                        }
                    }
                }
                if (lane < kn) res[jl * K + k0 + lane] += mine;
            }
        }
    }
    __syncthreads();
    for (int t = threadIdx.x; t < kWideLabels * K; t += kWideThreads) {
        const int jl = t / K;
        if (j0 + jl < L) gw[(size_t)j0 * K + t] = res[t];
    }
    if (bias_grad != nullptr && threadIdx.x < kWideLabels && j0 + (int)threadIdx.x < L) bias_grad[j0 + threadIdx.x] = bres[threadIdx.x];
}

// ---- input gradient -----------------------------------------------------------------------------
// One wavefront per (column n, batch pass).  The plan lists the connections of a column, grouped by
// label block and in ascending position; the wavefront walks them in that order (64 at a time: one
// per lane, then handed out as scalars), gathering one 512-byte piece of row j of gT per
// connection.  No atomics, fixed order: reproducible.  Label blocks bound the part of gT that is
// live at any time, so the gathers are served by the last-level cache.
template <bool TWO>
__global__ __launch_bounds__(kWideThreads) void igrad_wide_kernel(const int32_t* __restrict__ perm,
                                                                  const int32_t* __restrict__ col_ptr,
                                                                  const float* __restrict__ w,
                                                                  const float* __restrict__ gT, float* __restrict__ gxT,
                                                                  int B, int N, int L, int K, int nblocks,
                                                                  unsigned kdiv_mul, unsigned kdiv_shift, int ldb) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = blockIdx.x * (kWideThreads / 64) + wave;
    if (n >= N) return;                                         // wave-uniform
    const int bc0 = blockIdx.y * kWideBatch;
    const buffer_rsrc gr = make_rsrc(gT, (size_t)L * (size_t)ldb * sizeof(float));
    const unsigned lane_off0 = (unsigned)(bc0 + lane) * 4u, lane_off1 = lane_off0 + 256u;
    float acc0 = 0.f, acc1 = 0.f;
    for (int blk = 0; blk < nblocks; ++blk) {
        const int beg = col_ptr[(size_t)blk * N + n], end = col_ptr[(size_t)blk * N + n + 1];
        for (int e0 = beg; e0 < end; e0 += 64) {
            const int cnt = min(64, end - e0);
            int p = 0;
            float wv = 0.f;
            if (lane < cnt) { p = perm[e0 + lane]; wv = w[p]; }
            // label of the connection: p / K by multiply-high and shift (exact for p < 2^31)
            const unsigned jv = kdiv_mul ? (__umulhi((unsigned)p, kdiv_mul) >> kdiv_shift) : (unsigned)p;
            int i = 0;
            for (; i + kWideInflight <= cnt; i += kWideInflight) {
                float a[kWideInflight], b[kWideInflight], ws[kWideInflight];
#pragma unroll
                for (int u = 0; u < kWideInflight; ++u) {
                    const unsigned j = (unsigned)__builtin_amdgcn_readlane((int)jv, i + u);
                    ws[u] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), i + u));
                    // rows of gT are ldb*4 bytes; L*ldb*4 < 2^32 is checked by the launcher
                    a[u] = buffer_load_f32(gr, lane_off0, j * (unsigned)ldb * 4u);
                    b[u] = TWO ? buffer_load_f32(gr, lane_off1, j * (unsigned)ldb * 4u) : 0.f;
                }
#pragma unroll
                for (int u = 0; u < kWideInflight; ++u) {
                    acc0 = fmaf(ws[u], a[u], acc0);
                    if (TWO) acc1 = fmaf(ws[u], b[u], acc1);
                }
            }
            if (i < cnt) {
                // (the last, partly filled group: in flight together, what lies behind the end is left out of the sum)
                float a[kWideInflight], b[kWideInflight], ws[kWideInflight];
#pragma unroll
                for (int u = 0; u < kWideInflight; ++u) {
                    const int ii = min(i + u, cnt - 1);
                    const unsigned j = (unsigned)__builtin_amdgcn_readlane((int)jv, ii);
                    const float wk = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wv), ii));
                    ws[u] = wk;
                    a[u] = buffer_load_f32(gr, lane_off0, j * (unsigned)ldb * 4u);
                    b[u] = TWO ? buffer_load_f32(gr, lane_off1, j * (unsigned)ldb * 4u) : 0.f;
                }
#pragma unroll
                for (int u = 0; u < kWideInflight; ++u) {
                    if (i + u < cnt) {                          // wave-uniform
                        acc0 = fmaf(ws[u], a[u], acc0);
                        if (TWO) acc1 = fmaf(ws[u], b[u], acc1);
                    }
                }
            }
        }
    }
    if (bc0 + lane < B) gxT[(size_t)n * B + bc0 + lane] = acc0;
    if (TWO && bc0 + 64 + lane < B) gxT[(size_t)n * B + bc0 + 64 + lane] = acc1;
}

// floor(p / d) for 0 <= p < 2^31 as (p * mul) >> (32 + shift)
void magic_divisor(unsigned d, unsigned* mul, unsigned* shift) {
    if (d == 1) { *mul = 0; *shift = 0; return; }               // mul == 0 means: quotient = p
    unsigned s = 0;
    while ((1ull << s) < d) ++s;                                   // s = ceil(log2 d)
    const unsigned long long m = ((1ull << (32 + s - 1)) + d - 1) / d;   // fits 32 bits, error < 2^-31
    *mul = (unsigned)m;
    *shift = s - 1;
}

}  // namespace

// Row stride (in floats) of the library's own [rows][batch] copies: a multiple of 32, so that rows start on 128-byte
// lines and a gathered row piece touches as few lines as it can.
int wide_row_stride(int B) { return (B + 31) / 32 * 32; }

bool wide_offsets_fit(long long rows, long long B) { return rows * wide_row_stride((int)B) * 4 < (1ll << 32); }

namespace {

// xT[N][ldb] for the wide kernels: the caller's [N,B] buffer itself when its rows are aligned already, else a copy.
int wide_features(const float* x, const Dims& d, hipStream_t s, const float** xT, int* ldb) {
    const int ld = wide_row_stride(d.B);
    if (d.tp && ld == d.B) { *xT = x; *ldb = d.B; return FFI_OK; }
    float* ws = nullptr;
    FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)d.N * ld * sizeof(float), (void**)&ws));
    if (d.tp) {
        FFI_HIP_TRY(hipMemcpy2DAsync(ws, (size_t)ld * sizeof(float), x, (size_t)d.B * sizeof(float), (size_t)d.B * sizeof(float),
                                     (size_t)d.N, hipMemcpyDeviceToDevice, s));
    } else {
        FFI_TRY(launch_transpose(x, ws, d.B, d.N, s, d.N, ld));     // [B,N] -> [N,ld]
    }
    *xT = ws;
    *ldb = ld;
    return FFI_OK;
}

}  // namespace

int launch_forward_wide(const float* x, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d,
                        hipStream_t s) {
    if (!wide_offsets_fit(d.N, d.B)) return FFI_ERR_TOO_LARGE;
    const float* xT = nullptr;
    int ldb = 0;
    FFI_TRY(wide_features(x, d, s, &xT, &ldb));
    dim3 grid((d.L + kWideLabels - 1) / kWideLabels, (d.B + kWideBatch - 1) / kWideBatch);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    if (d.B > 64) hipLaunchKernelGGL(fwd_wide_kernel<true>, grid, dim3(kWideThreads), 0, s, xT, idx, w, bias, out, d.B, d.N, d.L, d.K, ldb);
    else hipLaunchKernelGGL(fwd_wide_kernel<false>, grid, dim3(kWideThreads), 0, s, xT, idx, w, bias, out, d.B, d.N, d.L, d.K, ldb);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_weight_grad_wide(const float* x, const int32_t* idx, const float* g, float* gw, float* bias_grad, const Dims& d,
                            hipStream_t s) {
    if (!wide_offsets_fit(d.N, d.B)) return FFI_ERR_TOO_LARGE;
    const size_t lds = ((size_t)kWideLabels * kWideStride + (size_t)kWideLabels * d.K + kWideLabels) * sizeof(float);
    if (lds > 150 * 1024) return FFI_ERR_TOO_LARGE;               // fan-in beyond ~450
    const float* xT = nullptr;
    int ldb = 0;
    FFI_TRY(wide_features(x, d, s, &xT, &ldb));
    const dim3 grid((d.L + kWideLabels - 1) / kWideLabels);
    if (d.B > 64) {
        FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_wide_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(wgrad_wide_kernel<true>, grid, dim3(kWideThreads), lds, s, xT, idx, g, gw, bias_grad, d.B, d.N, d.L, d.K, ldb);
    } else {
        FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_wide_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        hipLaunchKernelGGL(wgrad_wide_kernel<false>, grid, dim3(kWideThreads), lds, s, xT, idx, g, gw, bias_grad, d.B, d.N, d.L, d.K, ldb);
    }
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

int launch_input_grad_wide(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp, hipStream_t s) {
    if (!wide_offsets_fit(p->L, B)) return FFI_ERR_TOO_LARGE;
    const int ldb = wide_row_stride(B);
    float* gT = nullptr;
    FFI_TRY(workspace_get(s, kWsPartials, (size_t)p->L * ldb * sizeof(float), (void**)&gT));
    FFI_TRY(launch_transpose(g, gT, B, p->L, s, p->L, ldb));      // [B,L] -> [L,ldb]
    float* gxT = gx;
    if (!tp) FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)p->N * B * sizeof(float), (void**)&gxT));
    unsigned mul = 0, shift = 0;
    magic_divisor((unsigned)p->K, &mul, &shift);
    dim3 grid((p->N + kWideThreads / 64 - 1) / (kWideThreads / 64), (B + kWideBatch - 1) / kWideBatch);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    if (B > 64)
        hipLaunchKernelGGL(igrad_wide_kernel<true>, grid, dim3(kWideThreads), 0, s, p->perm, p->col_ptr, w, gT, gxT, B, p->N, p->L,
                           p->K, p->nblocks, mul, shift, ldb);
    else
        hipLaunchKernelGGL(igrad_wide_kernel<false>, grid, dim3(kWideThreads), 0, s, p->perm, p->col_ptr, w, gT, gxT, B, p->N,
                           p->L, p->K, p->nblocks, mul, shift, ldb);
    FFI_HIP_TRY(hipGetLastError());
    if (!tp) FFI_TRY(launch_transpose(gxT, gx, p->N, B, s));      // [N,B] -> [B,N]
    return FFI_OK;
}

}  // namespace ffi
