// Device helpers shared by the kernels that keep a [rows][32] fp32 tile in LDS and gather whole
// 128-byte rows from it with eight lanes per row (gfx950: 32 LDS banks x 4 bytes, 160 KB per CU).
#ifndef FFI_LDS_TILE_H
#define FFI_LDS_TILE_H

#include "ffi_internal.h"

namespace ffi {

constexpr int kTileBatch = 32;        // batch entries per LDS row: 128 bytes = one pass over the banks
constexpr int kTileThreads = 1024;    // 16 wavefronts per workgroup, one workgroup per CU
constexpr int kLabelsPerWave = 8;     // eight lanes share one row
constexpr size_t kTileLdsBudget = 152 * 1024;   // of the 160 KB per CU

__host__ __device__ inline size_t tile_lds_bytes(int rows) { return (size_t)rows * kTileBatch * sizeof(float); }
inline bool tile_path_fits(int rows) { return tile_lds_bytes(rows) <= kTileLdsBudget; }

struct TileGrid {
    int blocks;             // workgroups to launch
    int nbt;                // batch tiles of 32 rows
    int groups_per_stream;  // 8-label groups per label stream
};
// blocks = nbt * streams; the workgroups of one label stream (one per batch tile) sit on one XCD
// so that W/idx rows fetched by one of them are L2 hits for the others.
int tile_grid(int B, int L, TileGrid* out);

#if defined(__HIPCC__)

// Value of `v` in lane Q of the caller's quad (DPP quad_perm broadcast; folds into VOP2 users).
template <int Q>
__device__ __forceinline__ float quad_bcast(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), Q * 0x55, 0xf, 0xf, true));
}
template <int Q>
__device__ __forceinline__ unsigned quad_bcast(unsigned v) {
    return (unsigned)__builtin_amdgcn_update_dpp(0, (int)v, Q * 0x55, 0xf, 0xf, true);
}

// Workgroups are dealt round-robin to the 8 XCDs; this renumbers them so that consecutive logical
// ids share an XCD (and its L2).
__device__ __forceinline__ int xcd_contiguous_block(int block, int nblocks) {
    return (nblocks & 7) == 0 ? (block & 7) * (nblocks >> 3) + (block >> 3) : block;
}

// xs[r][c] = src[r*ld + c0 + c] for c < 32 (zero beyond column `ld`), r < rows.  src rows are read
// in 128-byte pieces, LDS writes are conflict-free.  All of a thread's loads are issued before its
// first LDS write, so the staging costs one memory round trip, not one per row.
template <int THREADS>
__device__ __forceinline__ void stage_rows32(float* __restrict__ xs, const float* __restrict__ src, int rows,
                                             int ld, int c0) {
    const bool vec = (ld % 4 == 0) && (c0 + kTileBatch <= ld) && (((uintptr_t)src & 15) == 0);
    if (vec) {
        // thread -> (row, 16-byte chunk): 8 threads per row
        constexpr int kRowsPerIter = THREADS / 8;
        constexpr int kInFlight = 4;
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

// Loads connections k0..k0+7 of one row: weights as they are, column ids scaled to LDS row byte
// offsets (128 bytes per row).  FULL: all eight are inside the row.
template <bool VEC4, bool FULL>
__device__ __forceinline__ void load_chunk8(const float* __restrict__ wrow, const int32_t* __restrict__ irow,
                                            int k0, int K, float (&w8)[8], unsigned (&o8)[8]) {
    if constexpr (VEC4 && FULL) {
        const float4 a = *reinterpret_cast<const float4*>(wrow + k0);
        const float4 b = *reinterpret_cast<const float4*>(wrow + k0 + 4);
        const int4 c = *reinterpret_cast<const int4*>(irow + k0);
        const int4 d = *reinterpret_cast<const int4*>(irow + k0 + 4);
        w8[0] = a.x; w8[1] = a.y; w8[2] = a.z; w8[3] = a.w;
        w8[4] = b.x; w8[5] = b.y; w8[6] = b.z; w8[7] = b.w;
        o8[0] = (unsigned)c.x << 7; o8[1] = (unsigned)c.y << 7; o8[2] = (unsigned)c.z << 7; o8[3] = (unsigned)c.w << 7;
        o8[4] = (unsigned)d.x << 7; o8[5] = (unsigned)d.y << 7; o8[6] = (unsigned)d.z << 7; o8[7] = (unsigned)d.w << 7;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const bool in = FULL || (k0 + i < K);
            w8[i] = in ? wrow[k0 + i] : 0.f;
            o8[i] = in ? ((unsigned)irow[k0 + i] << 7) : 0u;
        }
    }
}

// ---- lane-per-row gathers -------------------------------------------------------------------------
// When every lane reads its OWN 128-byte row (row ids unrelated between lanes), bank conflicts are
// avoided by skewing the order in which a lane walks the eight 16-byte chunks of its row: at step
// c lane l reads chunk c ^ (l & 7).  Rows are 128-byte aligned, so the bank group depends on the
// chunk number only and any eight consecutive lanes hit eight different bank groups.
// Consequence: register group c of lane l holds batch entries 4*(c ^ (l&7)) .. +3.

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

// Byte address (inside the tile) of the chunk read at step C, given base = row*128 | (lane&7)*16.
template <int C>
__device__ __forceinline__ unsigned skew_addr(unsigned base) { return C == 0 ? base : (base ^ (unsigned)(C * 16)); }

#endif  // __HIPCC__

}  // namespace ffi

#endif  // FFI_LDS_TILE_H
