// Weight gradient of the fixed-fan-in sparse layer for gfx950:
//   gw[j,k] = sum_b g[b,j] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/backward.cpp:8-36 in the reference).
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>

namespace ffi {
namespace {

// ------------------------------------------------------------------------------------------------
// Narrow-input kernel, register-resident partial sums.  xs[n][32 batch rows] of one batch tile sits
// in LDS.  A unit is (label, chunk of 32 connections); lane <-> unit.  A thread owns up to kResUnits
// units for the whole kernel and keeps their 32 partial sums each in registers across ALL batch
// tiles, so gw is written exactly once and never read (no atomics, fixed order, bit-reproducible);
// per batch tile the workgroup re-stages xs and every thread re-reads the ids and the out_grad
// column of its units.  512 threads per workgroup (two wavefronts per SIMD) leave 256 registers
// per thread for this.  Inside a batch tile there is no barrier, so the wavefronts drift apart and
// the loads of some overlap the LDS work of the others.  Workgroups [0,n1) own upb1 units each, the
// others upb2 each: one launch covers a first round of full workgroups and a second set that shares
// the remainder evenly.
// Each lane reads whole 128-byte rows of xs with the chunk order skewed by its lane id (see
// ffi_lds_tile.h), and out_grad is permuted in registers to match.
// ------------------------------------------------------------------------------------------------
constexpr int kWgChunk = 32;        // connections per unit
constexpr int kResThreads = 512;
constexpr int kResUnits = 4;        // units per thread

// The eight 16-byte reads of one row, all issued before the first use ...
// `base` = LDS address of the row + (lane & 7) * 16 (rows are 128-byte aligned, so the chunk bits can
// be flipped with XOR).
typedef float lds_v4f __attribute__((ext_vector_type(4)));
typedef const lds_v4f __attribute__((address_space(3)))* lds_v4f_ptr;
template <int C>
__device__ __forceinline__ float4 wgrad_read_chunk(unsigned base) {
    const lds_v4f t = *(lds_v4f_ptr)(size_t)(skew_addr<C>(base));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void wgrad_reads(unsigned base, float4 (&v)[8]) {
    v[0] = wgrad_read_chunk<0>(base); v[1] = wgrad_read_chunk<1>(base);
    v[2] = wgrad_read_chunk<2>(base); v[3] = wgrad_read_chunk<3>(base);
    v[4] = wgrad_read_chunk<4>(base); v[5] = wgrad_read_chunk<5>(base);
    v[6] = wgrad_read_chunk<6>(base); v[7] = wgrad_read_chunk<7>(base);
}
// ... and their dot product with the (equally skewed) out_grad values.
__device__ __forceinline__ float wgrad_dot(const float4 (&v)[8], const float (&gb)[32], float acc) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        acc = fmaf(v[c].x, gb[4 * c + 0], acc);
        acc = fmaf(v[c].y, gb[4 * c + 1], acc);
        acc = fmaf(v[c].z, gb[4 * c + 2], acc);
        acc = fmaf(v[c].w, gb[4 * c + 3], acc);
    }
    return acc;
}

template <bool VEC4>
__global__ __launch_bounds__(kResThreads) void wgrad_resident_kernel(const float* __restrict__ xT,
                                                                     const int32_t* __restrict__ idx,
                                                                     const float* __restrict__ g,
                                                                     float* __restrict__ gw,
                                                                     float* __restrict__ bias_grad, int B, int N,
                                                                     int L, int K, int nchunks, int n1, int upb1,
                                                                     int upb2) {
    extern __shared__ __align__(16) float xs[];
    const int lane = threadIdx.x & 63;
    const int blk = blockIdx.x;
    const long long total_units = (long long)L * nchunks;
    const long long u_begin = blk < n1 ? (long long)blk * upb1 : (long long)n1 * upb1 + (long long)(blk - n1) * upb2;
    const long long u_end = min(u_begin + (blk < n1 ? upb1 : upb2), total_units);
    const int nbt = (B + kTileBatch - 1) / kTileBatch;

    float res[kResUnits][kWgChunk];
#pragma unroll
    for (int q = 0; q < kResUnits; ++q)
#pragma unroll
        for (int k = 0; k < kWgChunk; ++k) res[q][k] = 0.f;
    float gsum[kResUnits];                                 // column sums of out_grad (the bias gradient)
#pragma unroll
    for (int q = 0; q < kResUnits; ++q) gsum[q] = 0.f;

    for (int bt = 0; bt < nbt; ++bt) {
        const int b0 = bt * kTileBatch;
        __syncthreads();                                   // everyone is done with the previous tile
        stage_rows32<kResThreads, 8>(xs, xT, N, B, b0);
        __syncthreads();
        // LDS address of xs plus the lane's skew
        unsigned skew = (unsigned)(size_t)(__attribute__((address_space(3))) float*)xs + (unsigned)(lane & 7) * 16u;
        asm volatile("" : "+v"(skew));                     // keep the LDS addresses out of loop-invariant hoisting
#pragma unroll
        for (int q = 0; q < kResUnits; ++q) {
            const long long ubase = u_begin + (long long)q * kResThreads;
            if (ubase + (long long)(threadIdx.x & ~63u) < u_end) {          // the wavefront has units in this round
                const long long u = min(ubase + (long long)threadIdx.x, u_end - 1);   // clamped: loads stay in bounds
                const int j = (int)(u / nchunks);
                const int k0 = (int)(u - (long long)j * nchunks) * kWgChunk;
                const int32_t* irow = idx + (size_t)j * K + k0;
                // out_grad of this label for the tile's 32 batch rows: coalesced across lanes
                float gb[32];
                load_rows32(g, L, b0, B, (unsigned)j, gb);
                if (bias_grad != nullptr) {
                    float t = gsum[q];
#pragma unroll
                    for (int b = 0; b < 32; ++b) t += gb[b];
                    gsum[q] = t;
                }
                // column ids of the unit, two 16-bit ids per register (ids < 2^16 on this path)
                unsigned idp[kWgChunk / 2];
                if (VEC4 && k0 + kWgChunk <= K) {
#pragma unroll
                    for (int t = 0; t < kWgChunk / 4; ++t) {
                        const int4 v = *reinterpret_cast<const int4*>(irow + 4 * t);
                        idp[2 * t + 0] = (unsigned)v.x | ((unsigned)v.y << 16);
                        idp[2 * t + 1] = (unsigned)v.z | ((unsigned)v.w << 16);
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < kWgChunk / 2; ++t) {
                        const unsigned a = (k0 + 2 * t < K) ? (unsigned)irow[2 * t] : 0u;
                        const unsigned b = (k0 + 2 * t + 1 < K) ? (unsigned)irow[2 * t + 1] : 0u;
                        idp[t] = a | (b << 16);
                    }
                }
                xor_permute_groups(gb, lane & 7);          // match the skewed chunk order of the gathers
#pragma unroll
                for (int k = 0; k < kWgChunk; ++k) {
                    const unsigned id = (k & 1) ? (idp[k >> 1] >> 16) : (idp[k >> 1] & 0xffffu);
                    float4 xv[8];
                    wgrad_reads((id << 7) + skew, xv);
                    __builtin_amdgcn_sched_barrier(0);
                    res[q][k] = wgrad_dot(xv, gb, res[q][k]);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        }
    }
#pragma unroll
    for (int q = 0; q < kResUnits; ++q) {
        const long long u = u_begin + (long long)q * kResThreads + threadIdx.x;
        if (u < u_end) {
            const int j = (int)(u / nchunks);
            const int k0 = (int)(u - (long long)j * nchunks) * kWgChunk;
            float* grow = gw + (size_t)j * K + k0;
            if (bias_grad != nullptr && k0 == 0) bias_grad[j] = gsum[q];
            if (VEC4 && k0 + kWgChunk <= K) {
#pragma unroll
                for (int t = 0; t < kWgChunk / 4; ++t)
                    *reinterpret_cast<float4*>(grow + 4 * t) = make_float4(res[q][4 * t], res[q][4 * t + 1], res[q][4 * t + 2], res[q][4 * t + 3]);
            } else {
#pragma unroll
                for (int k = 0; k < kWgChunk; ++k)
                    if (k0 + k < K) grow[k] = res[q][k];
            }
        }
    }
}


// ------------------------------------------------------------------------------------------------
// The same kernel fed by a plan's arranged copy of the column ids (ffi_plan.hip): entry i of a unit
// is (connection inside the chunk << 11) | column id, in an order in which lanes l and l+8 read
// opposite halves of the LDS banks, and units are numbered chunk-major (u = chunk * L + label) so
// that consecutive lanes work on consecutive labels.  Half the id traffic (16-bit entries), and the
// LDS reads mostly free of bank conflicts.  Partial sum i of a unit belongs to connection
// (entry i >> 11); the sums are put back in connection order through a thread-private 128-byte LDS
// slot before they are stored.
// ------------------------------------------------------------------------------------------------
constexpr unsigned kArrIdMask = (1u << kArrIdBits) - 1;
constexpr int kSlotPitch = kWgChunk + 4;     // floats between the reordering slots of neighbouring threads (16-byte aligned)

template <int NCH, int UNITS>
__global__ __launch_bounds__(kResThreads) void wgrad_arranged_kernel(const float* __restrict__ xT,
                                                                     const unsigned short* __restrict__ idx16,
                                                                     const float* __restrict__ g,
                                                                     float* __restrict__ gw,
                                                                     float* __restrict__ bias_grad, int B, int N,
                                                                     int L, int K, int nchunks, int n1, int ipb1,
                                                                     int ipb2) {
    extern __shared__ __align__(16) float xs[];
    const int lane = threadIdx.x & 63;
    const int blk = blockIdx.x;
    // UNITS: units a thread owns.
    // NCH == 1: an item is a unit (label, chunk) and a thread owns UNITS of them, of UNITS labels;
    // NCH > 1 (= the number of chunks of a label): an item is a label and a thread owns all NCH units of UNITS / NCH
    // labels, so that the label's 32 out_grad values of a batch tile are loaded once for all its chunks.
    static_assert(UNITS % NCH == 0 && UNITS <= kResUnits, "whole labels per thread");
    constexpr int kItems = UNITS / NCH;
    const long long total_items = NCH == 1 ? (long long)L * nchunks : (long long)L;
    const long long i_begin = blk < n1 ? (long long)blk * ipb1 : (long long)n1 * ipb1 + (long long)(blk - n1) * ipb2;
    const long long i_end = min(i_begin + (blk < n1 ? ipb1 : ipb2), total_items);
    const int nbt = (B + kTileBatch - 1) / kTileBatch;

    float res[UNITS][kWgChunk];
#pragma unroll
    for (int q = 0; q < UNITS; ++q)
#pragma unroll
        for (int k = 0; k < kWgChunk; ++k) res[q][k] = 0.f;
    float gsum[kItems];                                    // column sums of out_grad (the bias gradient)
#pragma unroll
    for (int q = 0; q < kItems; ++q) gsum[q] = 0.f;

    for (int bt = 0; bt < nbt; ++bt) {
        const int b0 = bt * kTileBatch;
        __syncthreads();                                   // everyone is done with the previous tile
        stage_rows32<kResThreads, 8>(xs, xT, N, B, b0);
        __syncthreads();
        // LDS address of xs plus the lane's skew
        unsigned skew = (unsigned)(size_t)(__attribute__((address_space(3))) float*)xs + (unsigned)(lane & 7) * 16u;
        asm volatile("" : "+v"(skew));                     // keep the LDS addresses out of loop-invariant hoisting
#pragma unroll
        for (int qq = 0; qq < kItems; ++qq) {
            const long long ibase = i_begin + (long long)qq * kResThreads;
            if (ibase + (long long)(threadIdx.x & ~63u) < i_end) {          // the wavefront has items in this round
                const long long it = min(ibase + (long long)threadIdx.x, i_end - 1);   // clamped: loads stay in bounds
                const int j = NCH == 1 ? (int)(it % L) : (int)it;
                float gb[32];
                load_rows32(g, L, b0, B, (unsigned)j, gb);
                if (bias_grad != nullptr) {
                    float t = gsum[qq];
#pragma unroll
                    for (int b = 0; b < 32; ++b) t += gb[b];
                    gsum[qq] = t;
                }
                xor_permute_groups(gb, lane & 7);          // match the skewed chunk order of the gathers
#pragma unroll
                for (int c = 0; c < NCH; ++c) {
                    const long long u = NCH == 1 ? it : (long long)c * L + it;
                    unsigned idp[kWgChunk / 2];            // two 16-bit entries per register
                    const uint4* erow = reinterpret_cast<const uint4*>(idx16 + (size_t)u * kWgChunk);
#pragma unroll
                    for (int t = 0; t < kWgChunk / 8; ++t) {
                        const uint4 v = erow[t];
                        idp[4 * t] = v.x; idp[4 * t + 1] = v.y; idp[4 * t + 2] = v.z; idp[4 * t + 3] = v.w;
                    }
#pragma unroll
                    for (int k = 0; k < kWgChunk; ++k) {
                        const unsigned e = (k & 1) ? (idp[k >> 1] >> 16) : idp[k >> 1];
                        float4 xv[8];
                        wgrad_reads(((e & kArrIdMask) << 7) + skew, xv);
                        __builtin_amdgcn_sched_barrier(0);
                        res[qq * NCH + c][k] = wgrad_dot(xv, gb, res[qq * NCH + c][k]);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        }
    }
    __syncthreads();                                       // xs is free: its first 72 KB become per-thread slots
    // (a pitch of 36 floats: when the connection numbers are the same in every lane -- a lookup that is already in the
    // arranged order has them 0, 1, 2, ... -- a pitch of 32 would send all lanes of a write to two banks)
    float* slot = xs + (size_t)threadIdx.x * kSlotPitch;
    const bool vec4 = (K % 4 == 0) && (((uintptr_t)gw & 15) == 0);
#pragma unroll
    for (int qq = 0; qq < kItems; ++qq) {
        const long long it = i_begin + (long long)qq * kResThreads + threadIdx.x;
        if (it < i_end) {
#pragma unroll
            for (int cc = 0; cc < NCH; ++cc) {
                const int c = NCH == 1 ? (int)(it / L) : cc;
                const int j = NCH == 1 ? (int)(it - (long long)c * L) : (int)it;
                const long long u = (long long)c * L + j;
                const int k0 = c * kWgChunk;
                if (bias_grad != nullptr && c == 0) bias_grad[j] = gsum[qq];
                const unsigned short* erow = idx16 + (size_t)u * kWgChunk;
#pragma unroll
                for (int i = 0; i < kWgChunk; ++i) slot[erow[i] >> kArrIdBits] = res[qq * NCH + cc][i];
                float* grow = gw + (size_t)j * K + k0;
                if (vec4 && k0 + kWgChunk <= K) {
#pragma unroll
                    for (int t = 0; t < kWgChunk / 4; ++t)
                        *reinterpret_cast<float4*>(grow + 4 * t) = *reinterpret_cast<const float4*>(slot + 4 * t);
                } else {
                    for (int k = 0; k < kWgChunk; ++k)
                        if (k0 + k < K) grow[k] = slot[k];
                }
            }
        }
    }
}

}  // namespace

// Four units per thread or three?  A CU works through its share of the units in workgroups, one at a time (the tile of x
// fills the LDS), each of which stages x once per batch tile and then runs one round per unit of its threads; the last
// workgroup's last round may be partly filled.  Whether 3 x 512 or 4 x 512 units per workgroup leaves the cheaper
// remainder depends on the unit count.  The model is in units of a full four-unit round, from timings at 768 columns,
// batch 128 (524,288 / 393,216 / 131,072 / 145,803 labels, fan-in 32): staging 0.36 (scaled with the column count), a
// round of the three-unit kernel 0.93 (it needs 227 registers instead of 256), a partly filled round 0.33 + 0.084 per
// wavefront.  Three units are taken when the model sees more than 5 % in them (measured then: -2.5 % at 670,091 labels, -5.5 % at 393,216
// labels and 512 columns; where it sees 3-5 %, measurements at other widths went both ways).
bool three_units_cheaper(long long units, int N, int cus) {
    const double stage = 0.36 * (double)N / 768.0;
    auto cost = [&](int u, double round) {
        const long long cap = (long long)u * kResThreads;
        const long long full = units / (cap * cus);                       // whole workgroups per CU
        const long long rest = units - full * cap * cus;
        double c = (double)full * (stage + u * round);
        if (rest > 0) {
            const long long wgs = std::min<long long>(cus, (rest + 63) / 64);
            const long long per = (rest + wgs - 1) / wgs;                  // units of a workgroup of the second set
            const long long part = per % kResThreads;
            c += stage + (double)(per / kResThreads) * round + (part ? 0.33 + 0.084 * (double)((part + 63) / 64) : 0.0);
        }
        return c;
    };
    return cost(3, 0.93) < 0.95 * cost(4, 1.0);
}

int launch_weight_grad(const float* x, const int32_t* idx, const float* g, float* gw, float* bias_grad, const Dims& d,
                       hipStream_t s, const ffi_plan* plan) {
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
        // A first round of full workgroups (kResUnits units per thread), one per CU, as long as whole rounds
        // fit; what is left is shared evenly by a second set of workgroups in the same launch.
        const int nchunks = (d.K + kWgChunk - 1) / kWgChunk;
        int n1 = 0, n2 = 0, ipb = 0, ipb2 = 0;
        auto split = [&](long long items, long long cap) {             // cap: items a workgroup can hold
            n1 = (int)(items / (cap * cus)) * cus;
            const long long rest = items - (long long)n1 * cap;
            n2 = 0; ipb2 = 0;
            if (rest > 0) {
                const long long rounds = (rest + cap * cus - 1) / (cap * cus);
                n2 = (int)std::min<long long>(rounds * cus, (rest + 63) / 64);
                ipb2 = (int)((rest + n2 - 1) / n2);
                n2 = (int)((rest + ipb2 - 1) / ipb2);
            }
            ipb = (int)cap;
        };
        if (plan != nullptr && plan->idx16 != nullptr) {
            // the unit slots of the final reordering need 144 bytes per thread
            const size_t lds = std::max(tile_lds_bytes(d.N), (size_t)kResThreads * kSlotPitch * sizeof(float));
            // a label of two or four chunks: all its units in one thread (its out_grad values are loaded once per
            // batch tile instead of once per chunk); the work is then split by labels, not by units
#define FFI_LAUNCH_ARRANGED(NCH, UNITS)                                                                                                \
            do {                                                                                                                       \
                split(NCH == 1 ? (long long)d.L * nchunks : (long long)d.L, (long long)(UNITS / NCH) * kResThreads);                   \
                FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_arranged_kernel<NCH, UNITS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
                hipLaunchKernelGGL((wgrad_arranged_kernel<NCH, UNITS>), dim3((unsigned)(n1 + n2)), dim3(kResThreads), lds, s, xT, plan->idx16, g, gw, \
                                   bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, ipb, ipb2);                                             \
            } while (0)
            if (nchunks == 2) FFI_LAUNCH_ARRANGED(2, 4);
            else if (nchunks == 4) FFI_LAUNCH_ARRANGED(4, 4);
            else if (three_units_cheaper((long long)d.L * nchunks, d.N, cus)) FFI_LAUNCH_ARRANGED(1, 3);
            else FFI_LAUNCH_ARRANGED(1, 4);
#undef FFI_LAUNCH_ARRANGED
            FFI_HIP_TRY(hipGetLastError());
            return FFI_OK;
        }
        split((long long)d.L * nchunks, (long long)kResUnits * kResThreads);
        const unsigned blocks = (unsigned)(n1 + n2);
        const int upb = ipb, upb2 = ipb2;
        const size_t lds = tile_lds_bytes(d.N);
        const bool vec4 = (d.K % 4 == 0) && (((uintptr_t)gw | (uintptr_t)idx) % 16 == 0);
        if (vec4) {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_resident_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(wgrad_resident_kernel<true>, dim3(blocks), dim3(kResThreads), lds, s, xT, idx, g, gw, bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, upb, upb2);
        } else {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_resident_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(wgrad_resident_kernel<false>, dim3(blocks), dim3(kResThreads), lds, s, xT, idx, g, gw, bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, upb, upb2);
        }
        FFI_HIP_TRY(hipGetLastError());
        return FFI_OK;
    }
    return launch_weight_grad_wide(x, idx, g, gw, bias_grad, d, s);
}

}  // namespace ffi
