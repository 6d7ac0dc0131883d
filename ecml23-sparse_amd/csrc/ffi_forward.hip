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
template <bool FULL>
__device__ __forceinline__ void fwd_chunk(const char* __restrict__ xs_bytes, const float (&w8)[8],
                                          const unsigned (&o8)[8], unsigned myoff, int kvalid,
                                          float (&acc)[4]) {
#define FFI_FWD_STEP(Q, I)                                                       \
    if (FULL || (Q * 8 + I) < kvalid) {                                          \
        const float wk = quad_bcast<Q>(w8[I]);                                   \
        const unsigned a = quad_bcast<Q>(o8[I]) + myoff;                         \
        const float4 xv = *reinterpret_cast<const float4*>(xs_bytes + a);        \
        acc[0] = fmaf(wk, xv.x, acc[0]);                                         \
        acc[1] = fmaf(wk, xv.y, acc[1]);                                         \
        acc[2] = fmaf(wk, xv.z, acc[2]);                                         \
        acc[3] = fmaf(wk, xv.w, acc[3]);                                         \
    }
#define FFI_FWD_ROW(Q) \
    FFI_FWD_STEP(Q, 0) FFI_FWD_STEP(Q, 1) FFI_FWD_STEP(Q, 2) FFI_FWD_STEP(Q, 3) \
    FFI_FWD_STEP(Q, 4) FFI_FWD_STEP(Q, 5) FFI_FWD_STEP(Q, 6) FFI_FWD_STEP(Q, 7)
    FFI_FWD_ROW(0) FFI_FWD_ROW(1) FFI_FWD_ROW(2) FFI_FWD_ROW(3)
#undef FFI_FWD_ROW
#undef FFI_FWD_STEP
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
    stage_rows32(xs, xT, N, B, b0);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int g = lane >> 3, s = lane & 7, sq = lane & 3;
    const unsigned myoff = (unsigned)s * 16u;
    const char* xs_bytes = reinterpret_cast<const char*>(xs);
    const int total_groups = (L + kLabelsPerWave - 1) / kLabelsPerWave;
    const int g_begin = stream * groups_per_stream;
    const int g_end = min(g_begin + groups_per_stream, total_groups);
    const int nfull = K / 32, ktail = K - nfull * 32;

    for (int grp = g_begin + wave; grp < g_end; grp += kTileThreads / 64) {
        const int j = grp * kLabelsPerWave + g;
        const bool valid = j < L;
        const size_t row = (size_t)(valid ? j : L - 1) * K;   // keep every lane's loads in bounds
        float acc[4] = {0.f, 0.f, 0.f, 0.f};
        for (int ch = 0; ch < nfull; ++ch) {
            float w8[8];
            unsigned o8[8];
            load_chunk8<VEC4, true>(w + row, idx + row, ch * 32 + sq * 8, K, w8, o8);
            fwd_chunk<true>(xs_bytes, w8, o8, myoff, 32, acc);
        }
        if (ktail) {
            float w8[8];
            unsigned o8[8];
            load_chunk8<VEC4, false>(w + row, idx + row, nfull * 32 + sq * 8, K, w8, o8);
            fwd_chunk<false>(xs_bytes, w8, o8, myoff, ktail, acc);
        }
        if (valid) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int b = b0 + 4 * s + c;
                if (b < B) out[(size_t)b * L + j] = acc[c];
            }
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
        TileGrid tg;
        FFI_TRY(tile_grid(d.B, d.L, &tg));
        const size_t lds = tile_lds_bytes(d.N);
        const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)w | (uintptr_t)idx) % 16 == 0);
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
