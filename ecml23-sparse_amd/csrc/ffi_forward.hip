// Forward pass of the fixed-fan-in sparse layer for gfx950:
//   out[b,j] = sum_k w[j,k] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/forward.cpp:9-44 in the reference).
//
// Two kernels:
//   fwd_rows32_kernel  narrow inputs (a [N][32] fp32 tile of x fits in LDS): every multiply-add
//                      takes its x operand from LDS, which makes LDS read bandwidth (128 B/clk/CU)
//                      the binding resource, so the layout is chosen for conflict-free reads.
//   fwd_label_lane     any shape; x gathered from global memory.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>
#include <cstdlib>

namespace ffi {
namespace {

// ------------------------------------------------------------------------------------------------
// Narrow-input kernel.
//
// LDS holds xs[n][c] = x[b0+c, n] for the workgroup's 32 batch rows: one row is 128 bytes, i.e.
// exactly one pass over the 32 LDS banks.  Eight consecutive lanes own one label and read one
// whole row with a single ds_read_b128 each (lane s takes batch entries 4s..4s+3), so every group
// of eight lanes touches all 32 banks exactly once: no bank conflicts whatever the column ids are.
// A wavefront therefore works on 8 labels at a time and each lane keeps 4 accumulators.
//
// W and idx rows are read with fully coalesced 16-byte global loads: inside each quad, lane q
// keeps connections 8q..8q+7 of the current 32-connection chunk, and the value needed at step k
// is taken from its owner with a quad_perm DPP operand (both quads of a label hold a copy).
// ------------------------------------------------------------------------------------------------
// The 32 connections of a chunk are handled as four octets.  The eight row reads of an octet are
// issued back to back, and the reads of the next octet go out before the multiply-adds of the
// current one, so every wavefront keeps 8-16 LDS requests in flight (with one or two, the LDS
// pipe idles on latency).
template <int Q, bool FULL>
__device__ __forceinline__ void fwd_reads(const char* __restrict__ xs_bytes, const unsigned (&o8)[8], unsigned myoff,
                                          int kvalid, float4 (&xv)[8]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (FULL || (Q * 8 + i) < kvalid) {
            const unsigned a = quad_bcast<Q>(o8[i]) + myoff;
            xv[i] = *reinterpret_cast<const float4*>(xs_bytes + a);
        }
    }
}

template <int Q, bool FULL>
__device__ __forceinline__ void fwd_fmas(const float (&w8)[8], int kvalid, const float4 (&xv)[8], float (&acc)[4]) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (FULL || (Q * 8 + i) < kvalid) {
            const float wk = quad_bcast<Q>(w8[i]);
            acc[0] = fmaf(wk, xv[i].x, acc[0]);
            acc[1] = fmaf(wk, xv[i].y, acc[1]);
            acc[2] = fmaf(wk, xv[i].z, acc[2]);
            acc[3] = fmaf(wk, xv[i].w, acc[3]);
        }
    }
}

template <bool FULL>
__device__ __forceinline__ void fwd_chunk(const char* __restrict__ xs_bytes, const float (&w8)[8],
                                          const unsigned (&o8)[8], unsigned myoff, int kvalid,
                                          float (&acc)[4]) {
    float4 xa[8], xb[8];
    fwd_reads<0, FULL>(xs_bytes, o8, myoff, kvalid, xa);
    fwd_reads<1, FULL>(xs_bytes, o8, myoff, kvalid, xb);
    __builtin_amdgcn_sched_barrier(0);
    fwd_fmas<0, FULL>(w8, kvalid, xa, acc);
    __builtin_amdgcn_sched_barrier(0);
    fwd_reads<2, FULL>(xs_bytes, o8, myoff, kvalid, xa);
    __builtin_amdgcn_sched_barrier(0);
    fwd_fmas<1, FULL>(w8, kvalid, xb, acc);
    __builtin_amdgcn_sched_barrier(0);
    fwd_reads<3, FULL>(xs_bytes, o8, myoff, kvalid, xb);
    __builtin_amdgcn_sched_barrier(0);
    fwd_fmas<2, FULL>(w8, kvalid, xa, acc);
    fwd_fmas<3, FULL>(w8, kvalid, xb, acc);
}

template <bool VEC4>
__global__ __launch_bounds__(kTileThreads) void fwd_rows32_kernel(const float* __restrict__ xT,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w,
                                                                  float* __restrict__ out, int B, int N,
                                                                  int L, int K, int nbt,
                                                                  int groups_per_stream) {
    extern __shared__ __align__(16) float xs[];
    const int u = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int bt = u % nbt, stream = u / nbt;
    const int b0 = bt * kTileBatch;
    stage_rows32<kTileThreads>(xs, xT, N, B, b0);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 3, s = lane & 7, sq = lane & 3;
    const unsigned myoff = (unsigned)s * 16u;
    const char* xs_bytes = reinterpret_cast<const char*>(xs);
    const int total_groups = (L + kLabelsPerWave - 1) / kLabelsPerWave;
    const int g_begin = stream * groups_per_stream;
    const int g_end = min(g_begin + groups_per_stream, total_groups);
    const int nfull = K / 32, ktail = K - nfull * 32;

    // Software pipeline over (label group, 32-connection chunk) steps: the W/idx registers of the
    // next step are requested before the current step's multiply-adds, so global-load latency
    // hides behind LDS work.
    const int nchunks = nfull + (ktail ? 1 : 0);
    const int stride = kTileThreads / 64;
    int grp = g_begin + wave, ch = 0;
    float w8[8];
    unsigned o8[8];
    auto row_of = [&](int gidx) -> size_t {
        const int j = gidx * kLabelsPerWave + g;
        return (size_t)(j < L ? j : L - 1) * K;            // keep every lane's loads in bounds
    };
    auto issue = [&](int gidx, int c, float (&wd)[8], unsigned (&od)[8]) {
        const size_t row = row_of(gidx);
        if (c < nfull) load_chunk8<VEC4, true>(w + row, idx + row, c * 32 + sq * 8, K, wd, od);
        else load_chunk8<VEC4, false>(w + row, idx + row, c * 32 + sq * 8, K, wd, od);
    };
    if (grp < g_end) issue(grp, 0, w8, o8);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    while (grp < g_end) {
        int ngrp = grp, nch = ch + 1;
        if (nch == nchunks) { nch = 0; ngrp = grp + stride; }
        float w8n[8];
        unsigned o8n[8];
        const bool more = ngrp < g_end;
#ifdef FFI_EXP_NOLOAD
        if (more) { for (int i = 0; i < 8; ++i) { w8n[i] = w8[i] * 1.0001f; o8n[i] = (o8[i] + 128u * 7u) % (128u * (unsigned)N); } }
#else
        if (more) issue(ngrp, nch, w8n, o8n);
#endif
        if (ch < nfull) fwd_chunk<true>(xs_bytes, w8, o8, myoff, 32, acc);
        else fwd_chunk<false>(xs_bytes, w8, o8, myoff, ktail, acc);
        if (ch == nchunks - 1) {
            const int j = grp * kLabelsPerWave + g;
            if (j < L) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    const int b = b0 + 4 * s + c;
#ifdef FFI_EXP_NOSTORE
                    if (b < B && acc[c] == 12345.678f) out[(size_t)b * L + j] = acc[c];
#else
                    if (b < B) out[(size_t)b * L + j] = acc[c];
#endif
                }
            }
            acc[0] = acc[1] = acc[2] = acc[3] = 0.f;
        }
        if (more) {
#pragma unroll
            for (int i = 0; i < 8; ++i) { w8[i] = w8n[i]; o8[i] = o8n[i]; }
        }
        grp = ngrp; ch = nch;
    }
}

// ------------------------------------------------------------------------------------------------
// Narrow-input kernel, lane-per-label form: thread <-> label, 32 accumulators (one per batch row of
// the tile), W and idx of the label in registers.  Each lane reads whole 128-byte rows of xs with
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

template <bool VEC4>
__global__ __launch_bounds__(kTileThreads) void fwd_lane32_kernel(const float* __restrict__ xT,
                                                                  const int32_t* __restrict__ idx,
                                                                  const float* __restrict__ w,
                                                                  float* __restrict__ out, int B, int N,
                                                                  int L, int K, int nbt, int labels_per_stream) {
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
        if (valid) {
            const unsigned lane_off = (unsigned)j * 4u;
            const unsigned stride = (unsigned)L * 4u;
#pragma unroll
            for (int b = 0; b < 32; ++b)
                __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(int, acc[b]), orsrc, lane_off, (unsigned)b * stride, 0);
        }
    }
}

// ------------------------------------------------------------------------------------------------
// Generic kernel: one thread owns label j and kFwdBatch batch rows; W/idx of the row are walked
// once per batch block, x is gathered from global memory, out[b, j..j+63] is one 256-byte store.
// ------------------------------------------------------------------------------------------------
constexpr int kFwdBlock = 256;
constexpr int kFwdBatch = 8;

template <bool TP>
__global__ __launch_bounds__(kFwdBlock) void fwd_label_lane(const float* __restrict__ x,
                                                             const int32_t* __restrict__ idx,
                                                             const float* __restrict__ w,
                                                             float* __restrict__ out, int B, int N,
                                                             int L, int K) {
    const int j = blockIdx.x * kFwdBlock + threadIdx.x;
    if (j >= L) return;
    const int b0 = blockIdx.y * kFwdBatch;
    const int nb = min(kFwdBatch, B - b0);
    const int32_t* ip = idx + (size_t)j * K;
    const float* wp = w + (size_t)j * K;
    float acc[kFwdBatch];
#pragma unroll
    for (int q = 0; q < kFwdBatch; ++q) acc[q] = 0.f;
    for (int k = 0; k < K; ++k) {
        const uint32_t n = (uint32_t)ip[k];
        const float wv = wp[k];
#pragma unroll
        for (int q = 0; q < kFwdBatch; ++q) {
            if (q < nb) {
                const float xv = TP ? x[(size_t)n * B + (b0 + q)] : x[(size_t)(b0 + q) * N + n];
                acc[q] = fmaf(wv, xv, acc[q]);
            }
        }
    }
#pragma unroll
    for (int q = 0; q < kFwdBatch; ++q)
        if (q < nb) out[(size_t)(b0 + q) * L + j] = acc[q];
}

}  // namespace

int launch_forward(const float* x, const int32_t* idx, const float* w, float* out, const Dims& d,
                   hipStream_t s) {
    if (tile_path_fits(d.N)) {
        const float* xT = x;
        if (!d.tp) {
            float* ws = nullptr;
            FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)d.N * d.B * sizeof(float), (void**)&ws));
            FFI_TRY(launch_transpose(x, ws, d.B, d.N, s));   // [B,N] -> [N,B]
            xT = ws;
        }
        const size_t lds = tile_lds_bytes(d.N);
        const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)w | (uintptr_t)idx) % 16 == 0);
        static const bool use_quads = getenv("FFI_FWD_QUADS") != nullptr;
        if (!use_quads && d.L < (1 << 25)) {
            const int cus = device_cu_count();
            const int nbt = (d.B + kTileBatch - 1) / kTileBatch;
            int streams = std::max(1, cus / nbt);
            int per_stream = (d.L + streams - 1) / streams;
            streams = (d.L + per_stream - 1) / per_stream;
            const int blocks = streams * nbt;
            if (vec4) {
                FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_lane32_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                hipLaunchKernelGGL(fwd_lane32_kernel<true>, dim3(blocks), dim3(kTileThreads), lds, s, xT, idx, w, out, d.B, d.N, d.L, d.K, nbt, per_stream);
            } else {
                FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_lane32_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
                hipLaunchKernelGGL(fwd_lane32_kernel<false>, dim3(blocks), dim3(kTileThreads), lds, s, xT, idx, w, out, d.B, d.N, d.L, d.K, nbt, per_stream);
            }
            FFI_HIP_TRY(hipGetLastError());
            return FFI_OK;
        }
        TileGrid tg;
        FFI_TRY(tile_grid(d.B, d.L, &tg));
        if (vec4) {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_rows32_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(fwd_rows32_kernel<true>, dim3(tg.blocks), dim3(kTileThreads), lds, s, xT, idx, w, out, d.B, d.N, d.L, d.K, tg.nbt, tg.groups_per_stream);
        } else {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)fwd_rows32_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(fwd_rows32_kernel<false>, dim3(tg.blocks), dim3(kTileThreads), lds, s, xT, idx, w, out, d.B, d.N, d.L, d.K, tg.nbt, tg.groups_per_stream);
        }
        FFI_HIP_TRY(hipGetLastError());
        return FFI_OK;
    }
    dim3 grid((d.L + kFwdBlock - 1) / kFwdBlock, (d.B + kFwdBatch - 1) / kFwdBatch);
    if (grid.y > 65535u) return FFI_ERR_TOO_LARGE;
    if (d.tp)
        hipLaunchKernelGGL(fwd_label_lane<true>, grid, dim3(kFwdBlock), 0, s, x, idx, w, out, d.B, d.N, d.L, d.K);
    else
        hipLaunchKernelGGL(fwd_label_lane<false>, grid, dim3(kFwdBlock), 0, s, x, idx, w, out, d.B, d.N, d.L, d.K);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

}  // namespace ffi
