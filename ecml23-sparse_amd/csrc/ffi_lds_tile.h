// Device helpers shared by the kernels that keep a [rows][32] fp32 tile in LDS and gather whole
// 128-byte rows from it, one row per lane (gfx950: 160 KB of LDS per CU, 64 banks x 4 bytes, of
// which a row covers one half; measured delivery to registers: 128 bytes per clock per CU).
#ifndef FFI_LDS_TILE_H
#define FFI_LDS_TILE_H

#include "ffi_internal.h"

namespace ffi {

constexpr int kTileBatch = 32;        // batch entries per LDS row: 128 bytes = one pass over the banks
constexpr int kTileThreads = 1024;    // 16 wavefronts per workgroup, one workgroup per CU
constexpr size_t kTileLdsBudget = 152 * 1024;   // of the 160 KB per CU

__host__ __device__ inline size_t tile_lds_bytes(int rows) { return (size_t)rows * kTileBatch * sizeof(float); }
inline bool tile_path_fits(int rows) { return tile_lds_bytes(rows) <= kTileLdsBudget; }

#if defined(__HIPCC__)

// Workgroups are dealt round-robin to the 8 XCDs; this renumbers them so that consecutive logical
// ids share an XCD (and its L2).
__device__ __forceinline__ int xcd_contiguous_block(int block, int nblocks) {
    return (nblocks & 7) == 0 ? (block & 7) * (nblocks >> 3) + (block >> 3) : block;
}

// xs[r][c] = src[r*ld + c0 + c] for c < 32 (zero beyond column `ld`), r < rows.  src rows are read
// in 128-byte pieces, LDS writes are conflict-free.  All of a thread's loads are issued before its
// first LDS write, so the staging costs one memory round trip, not one per row.
template <int THREADS, int INFLIGHT = 4>
__device__ __forceinline__ void stage_rows32(float* __restrict__ xs, const float* __restrict__ src, int rows,
                                             int ld, int c0) {
    const bool vec = (ld % 4 == 0) && (c0 + kTileBatch <= ld) && (((uintptr_t)src & 15) == 0);
    if (vec) {
        // thread -> (row, 16-byte chunk): 8 threads per row
        constexpr int kRowsPerIter = THREADS / 8;
        constexpr int kInFlight = INFLIGHT;
        const int q = threadIdx.x & 7;
        const float* p = src + c0 + 4 * q;
        for (int r0 = threadIdx.x >> 3; r0 < rows; r0 += kRowsPerIter * kInFlight) {
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
                if (r < rows) *reinterpret_cast<float4*>(xs + r * kTileBatch + 4 * q) = v[i];
            }
        }
    } else {
        const int c = threadIdx.x & 31;
        const bool in = c0 + c < ld;
        const float* p = src + c0 + c;
        for (int r = threadIdx.x >> 5; r < rows; r += THREADS / 32)
            xs[r * kTileBatch + c] = in ? p[(size_t)r * ld] : 0.f;
    }
}

// Raw buffer resource over `bytes` bytes at p (gfx9 family: 32-bit data format word).  Loads
// through it take a per-lane byte offset plus a wave-uniform (scalar) byte offset, and reads
// beyond `bytes` return zero instead of faulting.
using buffer_rsrc = __amdgpu_buffer_rsrc_t;
__device__ __forceinline__ buffer_rsrc make_rsrc(const void* p, size_t bytes) {
    const unsigned n = bytes > 0xfffffffeull ? 0xfffffffeu : (unsigned)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, n, 0x00020000);
}
__device__ __forceinline__ float buffer_load_f32(buffer_rsrc r, unsigned lane_off, unsigned wave_off) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, lane_off, wave_off, 0));
}

// v[b] = m[(b0+b)*ld + col] for b < 32 (zero beyond `rows`); rows of m are reached through the
// scalar offset, `col` is the only per-lane address register.  m + b0*ld is rebased in 64 bits,
// the remaining offsets (< 32*ld*4) must fit 32 bits: callers guarantee ld < 2^25.
__device__ __forceinline__ void load_rows32(const float* __restrict__ m, int ld, int b0, int rows, unsigned col,
                                            float (&v)[32]) {
    const float* base = m + (size_t)b0 * (size_t)ld;
    const int nrows = min(32, rows - b0);
    const buffer_rsrc r = make_rsrc(base, (size_t)nrows * (size_t)ld * sizeof(float));
    const unsigned lane_off = col * 4u;
    const unsigned stride = (unsigned)ld * 4u;
#pragma unroll
    for (int b = 0; b < 32; ++b) v[b] = buffer_load_f32(r, lane_off, (unsigned)b * stride);
}

// ---- lane-per-row gathers -------------------------------------------------------------------------
// Every lane reads its OWN 128-byte row (row ids unrelated between lanes).  Bank conflicts are
// kept low by skewing the order in which a lane walks the eight 16-byte chunks of its row: at step
// c lane l reads chunk c ^ (l & 7).  Rows are 128-byte aligned, so inside one half of the banks
// the bank group depends on the chunk number only, and any eight consecutive lanes hit eight
// different bank groups (4.3x faster than the unskewed order, 1.4x faster than padded rows).
// Consequence: register group c of lane l holds batch entries 4*(c ^ (l&7)) .. +3.
// A 128-byte row covers half of the 64 banks (even rows one half, odd rows the other).  The LDS
// serves a ds_read_b128 at 16 lanes per clock (256 bytes) only when eight of those lanes read each
// half; measured with this access pattern: 4 clocks per wavefront read when the lanes with bit 3 of
// their id clear read even rows and the others odd rows, 8 clocks when row parities are random or
// all equal.  Kernels whose row order is theirs to choose (the input gradient, through its plan)
// arrange that; the forward pass and the weight gradient take rows in the order of the lookup
// matrix and run at the 8-clock rate.

__device__ __forceinline__ void cond_swap(bool p, float& a, float& b) {
    const float t = p ? b : a;
    b = p ? a : b;
    a = t;
}

// v[4c+i] <-> v[4(c ^ r)+i] for r in [0,8): its own inverse; three stages of conditional swaps.
__device__ __forceinline__ void xor_permute_groups(float (&v)[32], int r) {
    const bool b4 = r & 4, b2 = r & 2, b1 = r & 1;
#pragma unroll
    for (int e = 0; e < 32; ++e)
        if (!(e & 16)) cond_swap(b4, v[e], v[e + 16]);
#pragma unroll
    for (int e = 0; e < 32; ++e)
        if (!(e & 8)) cond_swap(b2, v[e], v[e + 8]);
#pragma unroll
    for (int e = 0; e < 32; ++e)
        if (!(e & 4)) cond_swap(b1, v[e], v[e + 4]);
}

// The same permutation applied to the 32 bits of a mask (bit e <-> bit e ^ 4r): halves, bytes, nibbles.
__device__ __forceinline__ unsigned xor_permute_bits(unsigned m, int r) {
    if (r & 4) m = (m >> 16) | (m << 16);
    if (r & 2) m = ((m & 0xff00ff00u) >> 8) | ((m & 0x00ff00ffu) << 8);
    if (r & 1) m = ((m & 0xf0f0f0f0u) >> 4) | ((m & 0x0f0f0f0fu) << 4);
    return m;
}

// Byte address (inside the tile) of the chunk read at step C, given base = row*128 | (lane&7)*16.
template <int C>
__device__ __forceinline__ unsigned skew_addr(unsigned base) { return C == 0 ? base : (base ^ (unsigned)(C * 16)); }

#endif  // __HIPCC__

}  // namespace ffi

#endif  // FFI_LDS_TILE_H
