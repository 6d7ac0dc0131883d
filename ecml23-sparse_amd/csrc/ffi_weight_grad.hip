// Weight gradient of the fixed-fan-in sparse layer for gfx950:
//   gw[j,k] = sum_b g[b,j] * x[b, idx[j,k]]
// (semantics of tfsparse/cc/kernels/backward.cpp:8-36 in the reference).
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>
#include <type_traits>
#include <utility>

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
                                                                     int upb2, const unsigned long long* __restrict__ only_if_outdated) {
    if (only_if_outdated != nullptr && *only_if_outdated != 0) return;     // (enqueued as a fallback: the plan was current)
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
constexpr size_t kLdsPerWorkgroup = 160 * 1024;   // gfx950: all of a CU's LDS can go to one workgroup
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
#pragma unroll
                    for (int t = 0; t < kWgChunk / 8; ++t) {
                        const uint4 v = *reinterpret_cast<const uint4*>(idx16 + arranged_quarter_offset(u, t));
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
#pragma unroll
                for (int i = 0; i < kWgChunk; ++i)
                    slot[idx16[arranged_quarter_offset(u, i >> 3) + (i & 7)] >> kArrIdBits] = res[qq * NCH + cc][i];
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


// ------------------------------------------------------------------------------------------------
// The arranged kernel with its memory traffic taken off the wavefronts' critical path.  Every wavefront owns a
// [32 batch rows][64 labels] slice of LDS behind the tile of x; the out_grad values of its NEXT step (an item in a
// batch tile) are fetched straight into that slice by LDS-direct buffer loads (no registers, no wait), issued one
// by one between the connections of the current step's walk once the current values have been read out of the
// slice, and the arranged ids of the next chunk travel in a second set of 16 registers.  A step therefore starts
// with everything it needs already on the chip: with two wavefronts per SIMD nothing else hides the stream from
// HBM (per-wavefront phase stamps of the arranged kernel at 670,091 labels x 768 columns x batch 128, fan-in 32:
// of a workgroup's 110 us, 68 are walks, 12 the wait for out_grad, 15 the epilogue, 14 staging and barriers).
// The slice is read in the lane's skewed chunk order, which also replaces the 96 conditional moves that used to
// permute the values in registers; x is staged by LDS-direct 16-byte loads; at the end every wavefront puts its
// sums back in connection order through its own slice (no workgroup barrier) and stores whole rows.
// LDS: N * 128 bytes of x + 8 slices of 8 KB: fits for N <= 768.
// ------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(3))) float* lds_f32_ptr;
constexpr int kSliceFloats = kTileBatch * 64;               // one wavefront's slice of out_grad

// f(integral_constant<int, 0>) ... f(integral_constant<int, N - 1>): a loop whose index is a constant expression
template <class F, int... Is>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, Is...>) { (f(std::integral_constant<int, Is>{}), ...); }
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) { static_for_impl(f, std::make_integer_sequence<int, N>{}); }

// LDS-direct buffer loads put lane i's value at M0 + immediate + i * size, and an M0 that changes between two of them
// costs about 30 ns (measured: 32 loads with one M0 each 0.53 us, with an M0 per 16 of them 0.22 us).  So the
// destination's offset inside a 4-KB window goes into the instruction's immediate -- which the hardware also adds to
// the memory address, hence it is taken back out of the scalar offset.
template <int SIZE, int LDS_BYTES>
__device__ __forceinline__ void load_to_lds(const buffer_rsrc& r, lds_f32_ptr window, unsigned lane_off, unsigned wave_off) {
    static_assert(LDS_BYTES >= 0 && LDS_BYTES < 4096, "immediate offset field");
    static_assert(SIZE == 4 || SIZE == 16, "bytes per lane");
    if constexpr (SIZE == 4) __builtin_amdgcn_raw_ptr_buffer_load_lds(r, window, 4, lane_off, wave_off - (unsigned)LDS_BYTES, LDS_BYTES, 0);
    else __builtin_amdgcn_raw_ptr_buffer_load_lds(r, window, 16, lane_off, wave_off - (unsigned)LDS_BYTES, LDS_BYTES, 0);
}

// xs[r][0..32) = src[r * ld + c0 ...] for r < rows by LDS-direct 16-byte loads: one instruction fills eight rows.
// Needs ld % 4 == 0, c0 + 32 <= ld, rows % 8 == 0, src 16-byte aligned, rows * ld * 4 < 2^32.  The caller waits
// (vmcnt) and synchronises.
template <int THREADS>
__device__ __forceinline__ void stage_rows32_direct(float* xs, const float* __restrict__ src, int rows, int ld, int c0, int wave,
                                                    int lane) {
    const buffer_rsrc r = make_rsrc(src, (size_t)rows * (size_t)ld * sizeof(float));
    const unsigned lane_off = (unsigned)(lane >> 3) * (unsigned)ld * 4u + (unsigned)(lane & 7) * 16u;
    const unsigned step = 8u * (unsigned)ld * 4u;          // eight rows further in memory: 1 KB further in LDS
    const int ninstr = rows / 8;
    for (int i0 = wave * 4; i0 < ninstr; i0 += (THREADS / 64) * 4) {
        const lds_f32_ptr window = (lds_f32_ptr)xs + (size_t)i0 * 256;
        const unsigned off = (unsigned)i0 * step + (unsigned)c0 * 4u;
        load_to_lds<16, 0>(r, window, lane_off, off);
        if (i0 + 1 < ninstr) load_to_lds<16, 1024>(r, window, lane_off, off + step);
        if (i0 + 2 < ninstr) load_to_lds<16, 2048>(r, window, lane_off, off + 2 * step);
        if (i0 + 3 < ninstr) load_to_lds<16, 3072>(r, window, lane_off, off + 3 * step);
    }
}

// WALK: connections walked in a label's last chunk.  A fan-in that is not a multiple of 32 leaves that chunk partly
// filled, and the arranged order puts the real connections first: such launches walk its first 8, 16 or 24 entries only
// (labels of one, two or four chunks, i.e. the launches in which a thread holds whole labels).
template <int NCH, int UNITS, bool QUADS, int WALK = kWgChunk>
__global__ __launch_bounds__(kResThreads) void wgrad_stream_kernel(const float* __restrict__ xT,
                                                                   const unsigned short* __restrict__ idx16,
                                                                   const float* __restrict__ g,
                                                                   float* __restrict__ gw,
                                                                   float* __restrict__ bias_grad, int B, int N,
                                                                   int L, int K, int nchunks, int n1, int ipb1,
                                                                   int ipb2) {
    extern __shared__ __align__(16) float xs[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const int blk = blockIdx.x;
    static_assert(UNITS % NCH == 0 && UNITS <= kResUnits, "whole labels per thread");
    static_assert(WALK == kWgChunk || (QUADS && WALK % 8 == 0 && WALK > 0 && WALK < kWgChunk), "short walks: a thread's units must all end in the same chunk");
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
    float gsum[kItems];
#pragma unroll
    for (int q = 0; q < kItems; ++q) gsum[q] = 0.f;

    // the thread's items (clamped, so that every address stays in bounds), their labels, and which of them the
    // wavefront really has (wave-uniform; once false it stays false)
    long long item[kItems];
    unsigned jq[kItems];
    bool act[kItems];
#pragma unroll
    for (int qq = 0; qq < kItems; ++qq) {
        const long long ibase = i_begin + (long long)qq * kResThreads;
        act[qq] = __builtin_amdgcn_readfirstlane((int)(ibase + (long long)(threadIdx.x & ~63u) < i_end)) != 0;
        item[qq] = max(min(ibase + (long long)threadIdx.x, i_end - 1), 0ll);
        jq[qq] = NCH == 1 ? (unsigned)(item[qq] % L) : (unsigned)item[qq];
    }
    const lds_f32_ptr gslice = (lds_f32_ptr)xs + (size_t)N * kTileBatch + wave * kSliceFloats;
    // byte address of the lane's column of the slice; register group c of the lane holds batch entries 4 (c ^ t) ...
    const unsigned gcol = (unsigned)(size_t)gslice + (unsigned)lane * 4u;
    const unsigned tsk = (unsigned)(lane & 7) << 10;       // 4 rows of 256 bytes per group

    // out_grad rows [32 bt, 32 bt + 32) as a buffer (rows beyond the batch read as zero); bt == nbt: an empty buffer,
    // whose loads write zeros
    auto g_rows = [&](int bt) {
        const int b0 = bt * kTileBatch;
        const int nrows = bt < nbt ? min(kTileBatch, B - b0) : 0;
        return make_rsrc(g + (size_t)(bt < nbt ? b0 : 0) * (size_t)L, (size_t)nrows * (size_t)L * sizeof(float));
    };
    const unsigned gstride = (unsigned)L * 4u;
    // row b of that buffer for the 64 labels `label` of the wavefront -> row b of the slice, without passing through registers
    auto fetch_g_row = [&](const buffer_rsrc& r, unsigned label, auto bc) {
        constexpr int b = decltype(bc)::value;
        load_to_lds<4, (b & 15) * 256>(r, gslice + (b & 16) * 64, label * 4u, (unsigned)b * gstride);
    };
    // The same, four rows per instruction (16 bytes per lane: lanes 16 r ... 16 r + 15 fetch row 4 m + r for the labels
    // first ... first + 63, which land in the slice exactly as the row-by-row loads put them).  For wavefronts whose
    // lanes have consecutive labels; lanes behind the wavefront's last item then receive the out_grad of labels that are
    // not theirs, and never store anything.
    const unsigned quad_off = (unsigned)(lane >> 4) * gstride + (unsigned)(lane & 15) * 16u;
    auto fetch_g_rows4 = [&](const buffer_rsrc& r, unsigned first, auto mc) {
        constexpr int m = decltype(mc)::value;
        load_to_lds<16, (m & 3) * 1024>(r, gslice + (m & 4) * 256, quad_off + first * 4u, (unsigned)(4 * m) * gstride);
    };
    // (QUADS: chosen by the launcher for NCH > 1 or a single chunk; otherwise chunk-major unit numbers wrap from the last
    // label of one chunk to the first of the next inside a wavefront)
    // quarter t of the 32 arranged entries of chunk c of item `it`
    auto fetch_ids_quarter = [&](long long it, int c, int t, unsigned (&dst)[kWgChunk / 2]) {
        const long long u = NCH == 1 ? it : (long long)c * L + it;
        const uint4 v = *reinterpret_cast<const uint4*>(idx16 + arranged_quarter_offset(u, t));
        dst[4 * t] = v.x; dst[4 * t + 1] = v.y; dst[4 * t + 2] = v.z; dst[4 * t + 3] = v.w;
    };
    unsigned idn[kWgChunk / 2];                            // ids of the next chunk, in flight
    if (act[0]) {
        const buffer_rsrc r0 = g_rows(0);
        if constexpr (QUADS) static_for<kTileBatch / 4>([&](auto mc) { fetch_g_rows4(r0, (unsigned)__builtin_amdgcn_readfirstlane((int)jq[0]), mc); });
        else static_for<kTileBatch>([&](auto bc) { fetch_g_row(r0, jq[0], bc); });
#pragma unroll
        for (int t = 0; t < kWgChunk / 8; ++t) fetch_ids_quarter(item[0], 0, t, idn);
    }
    const bool direct = (B % 4 == 0) && (N % 8 == 0) && (((uintptr_t)xT & 15) == 0);
    for (int bt = 0; bt < nbt; ++bt) {
        const int b0 = bt * kTileBatch;
        __syncthreads();                                   // everyone is done with the previous tile
        if (direct && b0 + kTileBatch <= B) {
            stage_rows32_direct<kResThreads>(xs, xT, N, B, b0, wave, lane);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        } else {
            stage_rows32<kResThreads, 8>(xs, xT, N, B, b0);
        }
        __syncthreads();
        unsigned skew = (unsigned)(size_t)(lds_f32_ptr)xs + (unsigned)(lane & 7) * 16u;
        asm volatile("" : "+v"(skew));                     // keep the LDS addresses out of loop-invariant hoisting
#pragma unroll
        for (int qq = 0; qq < kItems; ++qq) {
            if (act[qq]) {
                // what follows this item: the wavefront's next item of this batch tile, or its first of the next tile
                const bool more = qq + 1 < kItems && act[qq + 1 < kItems ? qq + 1 : qq];
                const int nbt_ = more ? bt : bt + 1;
                const unsigned jn = more ? jq[qq + 1 < kItems ? qq + 1 : qq] : jq[0];
                const long long itn = more ? item[qq + 1 < kItems ? qq + 1 : qq] : item[0];
                asm volatile("s_waitcnt vmcnt(0)" ::: "memory");          // the slice and idn have arrived
                float gb[32];
#pragma unroll
                for (int c = 0; c < 8; ++c) {
                    const lds_f32_ptr p = (lds_f32_ptr)(size_t)(gcol + (((unsigned)c << 10) ^ tsk));
#pragma unroll
                    for (int i = 0; i < 4; ++i) gb[4 * c + i] = p[i * 64];
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");        // ... and has been read: refill it
                // the next step's rows are requested one per connection of the walk below (a burst of 32 requests per
                // wavefront finds the CU's memory queue full and stalls)
                const buffer_rsrc rn = g_rows(nbt_);
                const unsigned jn0 = (unsigned)__builtin_amdgcn_readfirstlane((int)jn);
                if (bias_grad != nullptr) {
                    float t = gsum[qq];
#pragma unroll
                    for (int b = 0; b < 32; ++b) t += gb[b];
                    gsum[qq] = t;
                }
                static_for<NCH>([&](auto cc) {
                    constexpr int c = decltype(cc)::value;
                    // connections walked in this chunk (the label's last chunk may be partly filled), and in the walk that follows it
                    constexpr int kWalk = c == NCH - 1 ? WALK : kWgChunk;
                    constexpr int kNextWalk = c + 1 < NCH ? (c + 1 == NCH - 1 ? WALK : kWgChunk) : (NCH == 1 ? WALK : kWgChunk);
                    // the quarters of that walk's entries are requested at even distances, each a few connections before its stretch ends
                    constexpr int kQuarters = kNextWalk / 8, kStep = kWalk / kQuarters, kAt = kStep > 3 ? kStep - 3 : 0;
                    if (c > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    unsigned idp[kWgChunk / 2];
#pragma unroll
                    for (int t = 0; t < kWgChunk / 2; ++t) idp[t] = idn[t];
                    // (no branch in here: the walk stays one basic block; behind the last step it fetches ids nobody uses
                    // and zero rows from an empty buffer)
                    static_for<kWalk>([&](auto kc) {
                        constexpr int k = decltype(kc)::value;
                        const unsigned e = (k & 1) ? (idp[k >> 1] >> 16) : idp[k >> 1];
                        if constexpr (QUADS) {
                            // (the eight four-row requests of the next step, spread evenly over the walk of the first chunk)
                            constexpr int kPer = kWalk / 8;
                            if constexpr (c == 0 && k % kPer == 0) fetch_g_rows4(rn, jn0, std::integral_constant<int, k / kPer>{});
                        } else {
                            if constexpr (c == 0) fetch_g_row(rn, jn, kc);
                        }
                        if constexpr (k % kStep == kAt && k / kStep < kQuarters)
                            fetch_ids_quarter(c + 1 < NCH ? item[qq] : itn, c + 1 < NCH ? c + 1 : 0, k / kStep, idn);
                        float4 xv[8];
                        wgrad_reads(((e & kArrIdMask) << 7) + skew, xv);
                        __builtin_amdgcn_sched_barrier(0);
                        res[qq * NCH + c][k] = wgrad_dot(xv, gb, res[qq * NCH + c][k]);
                        __builtin_amdgcn_sched_barrier(0);
                    });
                    asm volatile("" ::: "memory");
                });
            }
        }
    }
    // Epilogue, each wavefront on its own: the sums go back into connection order through the wavefront's slice (128
    // bytes per lane; the 16-byte groups of a lane's row are swizzled by lane bits 1-3 so that lanes which write the
    // same connection number -- a lookup that already is in arranged order -- spread over the banks).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // nothing is on its way into the slice any more
    const unsigned srow = (unsigned)(size_t)gslice + (unsigned)lane * 128u;
    const unsigned sw = ((unsigned)lane >> 1) & 7u;
    const bool vec4 = (K % 4 == 0) && (((uintptr_t)gw & 15) == 0);
    // (the entries of all the thread's units are requested before the first is used: one memory round trip, not one per unit)
    unsigned ent[UNITS][kWgChunk / 2];
#pragma unroll
    for (int qq = 0; qq < kItems; ++qq)
#pragma unroll
        for (int cc = 0; cc < NCH; ++cc) {
            const long long u = NCH == 1 ? item[qq] : (long long)cc * L + item[qq];
#pragma unroll
            for (int t = 0; t < kWgChunk / 8; ++t) {
                uint4 v = make_uint4(0u, 0u, 0u, 0u);
                if (act[qq]) v = *reinterpret_cast<const uint4*>(idx16 + arranged_quarter_offset(u, t));
                ent[qq * NCH + cc][4 * t] = v.x; ent[qq * NCH + cc][4 * t + 1] = v.y;
                ent[qq * NCH + cc][4 * t + 2] = v.z; ent[qq * NCH + cc][4 * t + 3] = v.w;
            }
        }
#pragma unroll
    for (int qq = 0; qq < kItems; ++qq) {
        if (act[qq]) {
            const long long it = i_begin + (long long)qq * kResThreads + threadIdx.x;
            const bool mine = it < i_end;
#pragma unroll
            for (int cc = 0; cc < NCH; ++cc) {
                const int c = NCH == 1 ? (int)(item[qq] / L) : cc;
                const int j = NCH == 1 ? (int)(item[qq] - (long long)c * L) : (int)item[qq];
                const int k0 = c * kWgChunk;
                if (mine && bias_grad != nullptr && (NCH == 1 ? c == 0 : cc == 0)) bias_grad[j] = gsum[qq];
#pragma unroll
                for (int i = 0; i < kWgChunk; ++i) {
                    const unsigned w = ent[qq * NCH + cc][i >> 1];
                    const unsigned conn = ((i & 1) ? (w >> 16) : (w & 0xffffu)) >> kArrIdBits;
                    *(lds_f32_ptr)(size_t)(srow + ((conn ^ (sw << 2)) << 2)) = res[qq * NCH + cc][i];
                }
                float* grow = gw + (size_t)j * K + k0;
                if (QUADS && vec4 && k0 + kWgChunk <= K) {
                    // lanes of consecutive labels: instruction t stores the rows of lanes 8 t ... 8 t + 7, eight lanes per row,
                    // so that a store covers whole 128-byte rows (1 KB in one piece at fan-in 32) instead of 16 bytes of 64 rows
                    const long long it0 = __builtin_amdgcn_readfirstlane((int)(it - lane));   // (the wavefront's first item, below 2^31: L < 2^25 labels)
                    const int j0 = NCH == 1 ? (int)(it0 % L) : (int)it0;
                    (void)j;
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const unsigned r = (unsigned)(8 * t) + ((unsigned)lane >> 3), q = (unsigned)lane & 7u;
                        const unsigned rsw = (r >> 1) & 7u;
                        const lds_v4f v = *(lds_v4f_ptr)(size_t)((unsigned)(size_t)gslice + r * 128u + ((q ^ rsw) << 4));
                        if (it0 + (long long)r < i_end)
                            *reinterpret_cast<float4*>(gw + (size_t)(j0 + (int)r) * K + k0 + 4 * q) = make_float4(v.x, v.y, v.z, v.w);
                    }
                } else if (vec4) {
                    // (a partly filled chunk of a fan-in that is a multiple of four: its first quads)
#pragma unroll
                    for (int t = 0; t < kWgChunk / 4; ++t) {
                        const lds_v4f v = *(lds_v4f_ptr)(size_t)(srow + (((unsigned)t ^ sw) << 4));
                        if (mine && k0 + 4 * t < K) *reinterpret_cast<float4*>(grow + 4 * t) = make_float4(v.x, v.y, v.z, v.w);
                    }
                } else {
                    for (int k = 0; k < kWgChunk; ++k) {
                        const float v = *(lds_f32_ptr)(size_t)(srow + (((unsigned)k ^ (sw << 2)) << 2));
                        if (mine && k0 + k < K) grow[k] = v;
                    }
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
                       hipStream_t s, const ffi_plan* plan, const unsigned long long* only_if_outdated) {
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
            // with room for the wavefronts' out_grad slices behind the tile of x: the streaming kernel
            // (and rows of out_grad of at least 256 bytes: the LDS-direct loads take their destination's offset inside the
            // slice back out of the scalar offset of the row, which must not become negative)
            const bool stream = tile_lds_bytes(d.N) + (size_t)(kResThreads / 64) * kSliceFloats * sizeof(float) <= kLdsPerWorkgroup &&
                                d.L >= 64 && g_options.wgrad_stream >= 0;
            const size_t lds = std::max(tile_lds_bytes(d.N) + (stream ? (size_t)(kResThreads / 64) * kSliceFloats * sizeof(float) : 0),
                                        (size_t)kResThreads * kSlotPitch * sizeof(float));
            // a label of two or four chunks: all its units in one thread (its out_grad values are loaded once per
            // batch tile instead of once per chunk); the work is then split by labels, not by units
            // connections in a label's last chunk, rounded up to the eights the walk is cut in
            const int last_walk = (d.K - (nchunks - 1) * kWgChunk + 7) / 8 * 8;
#define FFI_LAUNCH_STREAM_WALK(NCH, UNITS, WALK)                                                                                       \
            do {                                                                                                                       \
                FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_stream_kernel<NCH, UNITS, true, WALK>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
                hipLaunchKernelGGL((wgrad_stream_kernel<NCH, UNITS, true, WALK>), dim3((unsigned)(n1 + n2)), dim3(kResThreads), lds, s, xT, plan->idx16, g, gw, \
                                   bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, ipb, ipb2);                                             \
            } while (0)
#define FFI_LAUNCH_ARRANGED(NCH, UNITS)                                                                                                \
            do {                                                                                                                       \
                split(NCH == 1 ? (long long)d.L * nchunks : (long long)d.L, (long long)(UNITS / NCH) * kResThreads);                   \
                if (stream) {                                                                                                          \
                    constexpr bool kQuads = NCH > 1;   /* a wavefront's lanes hold consecutive labels */                               \
                    if ((kQuads || nchunks == 1) && last_walk < kWgChunk) {                                                            \
                        /* the last chunk of every label is partly filled: its walk covers the filled part only */                     \
                        if (last_walk == 8) FFI_LAUNCH_STREAM_WALK(NCH, UNITS, 8);                                                     \
                        else if (last_walk == 16) FFI_LAUNCH_STREAM_WALK(NCH, UNITS, 16);                                              \
                        else FFI_LAUNCH_STREAM_WALK(NCH, UNITS, 24);                                                                   \
                    } else if (kQuads || nchunks == 1) {                                                                               \
                        FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_stream_kernel<NCH, UNITS, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
                        hipLaunchKernelGGL((wgrad_stream_kernel<NCH, UNITS, true>), dim3((unsigned)(n1 + n2)), dim3(kResThreads), lds, s, xT, plan->idx16, g, gw, \
                                           bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, ipb, ipb2);                                     \
                    } else {                                                                                                           \
                        FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_stream_kernel<NCH, UNITS, kQuads>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
                        hipLaunchKernelGGL((wgrad_stream_kernel<NCH, UNITS, kQuads>), dim3((unsigned)(n1 + n2)), dim3(kResThreads), lds, s, xT, plan->idx16, g, gw, \
                                           bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, ipb, ipb2);                                     \
                    }                                                                                                                  \
                } else {                                                                                                               \
                    FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_arranged_kernel<NCH, UNITS>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds)); \
                    hipLaunchKernelGGL((wgrad_arranged_kernel<NCH, UNITS>), dim3((unsigned)(n1 + n2)), dim3(kResThreads), lds, s, xT, plan->idx16, g, gw, \
                                       bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, ipb, ipb2);                                         \
                }                                                                                                                      \
            } while (0)
            // (two chunks per label: one label per thread, 64 sums, measured 2-4 % under two labels per thread, whose 128 sums
            // leave the streaming kernel 92 bytes of spills per lane)
            if (nchunks == 2 && (g_options.wgrad_units == 4 || !stream)) FFI_LAUNCH_ARRANGED(2, 4);
            else if (nchunks == 2) FFI_LAUNCH_ARRANGED(2, 2);
            else if (nchunks == 4) FFI_LAUNCH_ARRANGED(4, 4);
            // the streaming kernel: three units per thread wherever measured (4,000 to 3,000,000 labels, batch 32-512, 64-768
            // columns, fan-in 8-32 and 96: 3-15 % under four units); the kernel without slices: by the model above
            else if (g_options.wgrad_units == 3 ||
                     (g_options.wgrad_units != 4 && (stream || three_units_cheaper((long long)d.L * nchunks, d.N, cus)))) FFI_LAUNCH_ARRANGED(1, 3);
            else FFI_LAUNCH_ARRANGED(1, 4);
#undef FFI_LAUNCH_ARRANGED
#undef FFI_LAUNCH_STREAM_WALK
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
            hipLaunchKernelGGL(wgrad_resident_kernel<true>, dim3(blocks), dim3(kResThreads), lds, s, xT, idx, g, gw, bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, upb, upb2, only_if_outdated);
        } else {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)wgrad_resident_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(wgrad_resident_kernel<false>, dim3(blocks), dim3(kResThreads), lds, s, xT, idx, g, gw, bias_grad, d.B, d.N, d.L, d.K, nchunks, n1, upb, upb2, only_if_outdated);
        }
        FFI_HIP_TRY(hipGetLastError());
        return FFI_OK;
    }
    return launch_weight_grad_wide(x, idx, g, gw, bias_grad, d, s);
}

}  // namespace ffi

