// Weight gradient of the fixed-fan-in sparse layer for gfx950:
//   gw[j,k] = sum_b g[b,j] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/backward.cpp:8-36 in the reference).
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

namespace ffi {
namespace {

// ------------------------------------------------------------------------------------------------
// Narrow-input kernel: lane <-> label, 32 connections of the label per pass held as 32 fp32
// accumulators, xs[n][32 batch rows] in LDS.  A workgroup owns a range of labels and makes one
// sweep over it per batch tile: xs is staged once per sweep, and inside a sweep there is no
// barrier, so the wavefronts drift apart and the out_grad/idx loads of some overlap the LDS work of
// the others.  The first sweep writes gw, every later sweep adds its partial sum to what the same
// thread wrote before (plain read-modify-write: no atomics, fixed order, bit-reproducible).
// Each lane reads whole 128-byte rows with the chunk order skewed by its lane id (see
// ffi_lds_tile.h), and out_grad is permuted in registers to match.
// ------------------------------------------------------------------------------------------------
constexpr int kWgChunk = 32;   // connections per register pass

// acc += <row chunk C, gb group C>
template <int C>
__device__ __forceinline__ void wgrad_step(const char* __restrict__ xs_bytes, unsigned base, const float (&gb)[32],
                                           float& acc) {
    const float4 xv = *reinterpret_cast<const float4*>(xs_bytes + skew_addr<C>(base));
    acc = fmaf(xv.x, gb[4 * C + 0], acc);
    acc = fmaf(xv.y, gb[4 * C + 1], acc);
    acc = fmaf(xv.z, gb[4 * C + 2], acc);
    acc = fmaf(xv.w, gb[4 * C + 3], acc);
}

template <bool VEC4>
__global__ __launch_bounds__(kTileThreads) void wgrad_rows32_kernel(const float* __restrict__ xT,
                                                                    const int32_t* __restrict__ idx,
                                                                    const float* __restrict__ g,
                                                                    float* __restrict__ gw, int B, int N,
                                                                    int L, int K, int labels_per_block) {
    extern __shared__ __align__(16) float xs[];
    const char* xs_bytes = reinterpret_cast<const char*>(xs);
    const int lane = threadIdx.x & 63;
    const unsigned skew = (unsigned)(lane & 7) * 16u;
    const int l_begin = blockIdx.x * labels_per_block;
    const int l_end = min(l_begin + labels_per_block, L);
    const int nbt = (B + kTileBatch - 1) / kTileBatch;
    const int nchunks = (K + kWgChunk - 1) / kWgChunk;

    for (int bt = 0; bt < nbt; ++bt) {
        const int b0 = bt * kTileBatch;
        __syncthreads();                                   // everyone is done with the previous tile
        stage_rows32<kTileThreads>(xs, xT, N, B, b0);
        __syncthreads();
        for (int base = l_begin; base < l_end; base += kTileThreads) {
            if (base + (int)(threadIdx.x & ~63u) >= l_end) break;   // nothing left for this wavefront
            const int j = base + (int)threadIdx.x;
            const bool valid = j < l_end;
            const int jj = valid ? j : l_end - 1;          // keep loads in bounds
            const int32_t* irow = idx + (size_t)jj * K;
            float* grow = gw + (size_t)jj * K;
            // out_grad of this label for the tile's 32 batch rows: coalesced across lanes
            float gb[32];
            load_rows32(g, L, b0, B, (unsigned)jj, gb);
            xor_permute_groups(gb, lane & 7);              // match the skewed chunk order of the gathers
            for (int ch = 0; ch < nchunks; ++ch) {
                const int k0 = ch * kWgChunk;
                const bool full = VEC4 && k0 + kWgChunk <= K;
                // column ids of this pass, two 16-bit ids per register (ids < 2^16 on this path)
                unsigned idp[kWgChunk / 2];
                float acc[kWgChunk];
                if (full) {
#pragma unroll
                    for (int q = 0; q < kWgChunk / 4; ++q) {
                        const int4 v = *reinterpret_cast<const int4*>(irow + k0 + 4 * q);
                        idp[2 * q + 0] = (unsigned)v.x | ((unsigned)v.y << 16);
                        idp[2 * q + 1] = (unsigned)v.z | ((unsigned)v.w << 16);
                    }
                } else {
#pragma unroll
                    for (int q = 0; q < kWgChunk / 2; ++q) {
                        const unsigned a = (k0 + 2 * q < K) ? (unsigned)irow[k0 + 2 * q] : 0u;
                        const unsigned b = (k0 + 2 * q + 1 < K) ? (unsigned)irow[k0 + 2 * q + 1] : 0u;
                        idp[q] = a | (b << 16);
                    }
                }
                // partial sums of the earlier batch tiles (written by this same thread)
                if (bt == 0) {
#pragma unroll
                    for (int k = 0; k < kWgChunk; ++k) acc[k] = 0.f;
                } else if (full) {
#pragma unroll
                    for (int q = 0; q < kWgChunk / 4; ++q) {
                        const float4 v = *reinterpret_cast<const float4*>(grow + k0 + 4 * q);
                        acc[4 * q] = v.x; acc[4 * q + 1] = v.y; acc[4 * q + 2] = v.z; acc[4 * q + 3] = v.w;
                    }
                } else {
#pragma unroll
                    for (int k = 0; k < kWgChunk; ++k) acc[k] = (k0 + k < K) ? grow[k0 + k] : 0.f;
                }
#pragma unroll
                for (int k = 0; k < kWgChunk; ++k) {
                    const unsigned id = (k & 1) ? (idp[k >> 1] >> 16) : (idp[k >> 1] & 0xffffu);
                    const unsigned rb = (id << 7) | skew;
                    wgrad_step<0>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<1>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<2>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<3>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<4>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<5>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<6>(xs_bytes, rb, gb, acc[k]);
                    wgrad_step<7>(xs_bytes, rb, gb, acc[k]);
                }
                if (valid) {
                    if (full) {
#pragma unroll
                        for (int q = 0; q < kWgChunk / 4; ++q)
                            *reinterpret_cast<float4*>(grow + k0 + 4 * q) = make_float4(acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
                    } else {
#pragma unroll
                        for (int k = 0; k < kWgChunk; ++k)
                            if (k0 + k < K) grow[k0 + k] = acc[k];
                    }
                }
            }
        }
    }
}

}  // namespace

int launch_weight_grad(const float* x, const int32_t* idx, const float* g, float* gw, const Dims& d,
                       hipStream_t s) {
    // (32 rows of out_grad must be reachable through 32-bit byte offsets)
    if (tile_path_fits(d.N) && d.L < (1 << 25)) {
        const float* xT = x;
        if (!d.tp) {
            float* ws = nullptr;
            FFI_TRY(workspace_get(s, kWsFeaturesT, (size_t)d.N * d.B * sizeof(float), (void**)&ws));
            FFI_TRY(launch_transpose(x, ws, d.B, d.N, s));
            xT = ws;
        }
        const int cus = device_cu_count();
        // one workgroup per CU, equal label ranges (the last pass of a range may be partly filled)
        const int per_block = (d.L + cus - 1) / cus;
        const int blocks = (d.L + per_block - 1) / per_block;
        const size_t lds = tile_lds_bytes(d.N);
        const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)gw | (uintptr_t)idx) % 16 == 0);
        if (vec4) {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_rows32_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(wgrad_rows32_kernel<true>, dim3(blocks), dim3(kTileThreads), lds, s, xT, idx, g, gw, d.B, d.N, d.L, d.K, per_block);
        } else {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_rows32_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(wgrad_rows32_kernel<false>, dim3(blocks), dim3(kTileThreads), lds, s, xT, idx, g, gw, d.B, d.N, d.L, d.K, per_block);
        }
        FFI_HIP_TRY(hipGetLastError());
        return FFI_OK;
    }
    return launch_weight_grad_wide(x, idx, g, gw, d, s);
}

}  // namespace ffi
