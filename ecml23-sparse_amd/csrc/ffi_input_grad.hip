// Input gradient of the fixed-fan-in sparse layer for gfx950, atomics-free:
//   gx[b,n] = sum over (j,k) with idx[j,k]==n of w[j,k] * g[b,j]
// (semantics of tfsparse/cc/kernels/backward.cpp:39-73 in the reference).
//
// Narrow inputs use the tiled plan: it is the forward pass of the transposed sparse matrix, done
// tile by tile.  A workgroup keeps gs[label in tile][32 batch rows] in LDS, thread n owns input
// column n and walks the tile's connections of that column, gathering whole 128-byte rows of gs
// (chunk order skewed per lane, see ffi_lds_tile.h) into 32 accumulators that live in registers
// across all the tiles of the workgroup's label stream.  Streams are then summed in a fixed order.
#include "ffi_internal.h"
#include "ffi_lds_tile.h"

#include <algorithm>

namespace ffi {
namespace {

// ---- tiled plan ---------------------------------------------------------------------------------

// wp[slot] = w at the connection stored in that slot (0 in padding slots): brings the weights into
// the plan's slot order so that the main kernel reads them coalesced.  One workgroup per label
// tile, one thread per column.  The tile's weights pass through LDS in pieces of kPermChunk floats
// (read from HBM fully coalesced).  The wavefront walks the slice's rows together (every load is
// one coalesced 128-byte row), kPermRows rows per step; a lane stores the slots whose position lies in
// the staged piece.  A column's positions ascend inside each label parity and the two parities
// alternate, so nothing of a later piece sits before the first step in which some lane met a
// position beyond the current piece: the next piece resumes there.
constexpr int kPermChunk = 16384;     // 64 KB of LDS per piece: two workgroups fit on a CU and overlap each other
constexpr int kPermRows = 24;          // slot rows a wavefront handles per step
constexpr int kPermChunkBig = 32768;  // 128 KB: a whole tile of 1024 labels x 32 connections in one piece
__global__ __launch_bounds__(1024) void igrad_permute_weights_kernel(
    const unsigned short* __restrict__ pos16, const unsigned* __restrict__ slice_off, const float* __restrict__ w,
    float* __restrict__ wp, int L, int K, int tile_labels, int chunk) {
    extern __shared__ __align__(16) float ws[];
    const int t = blockIdx.x, nthreads = blockDim.x;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const size_t sl = (size_t)t * (nthreads >> 6) + wave;
    const unsigned row0 = slice_off[sl], rows = slice_off[sl + 1] - row0;
    const int nl = min(tile_labels, L - t * tile_labels);
    const unsigned npos = (unsigned)nl * (unsigned)K;
    const float* wt = w + (size_t)t * tile_labels * K;
    const bool vec = ((((uintptr_t)wt) & 15) == 0);
    const unsigned short* ep = pos16 + (size_t)row0 * 64 + lane;
    float* op = wp + (size_t)row0 * 64 + lane;
    unsigned lo = 0;                 // wave-uniform: rows below lo hold nothing of this or a later piece
    for (unsigned c0 = 0; c0 < npos; c0 += (unsigned)chunk) {
        const unsigned n = min((unsigned)chunk, npos - c0);
        __syncthreads();
        if (vec) {
            // all of a thread's loads go out before its first LDS write: one round trip per piece
            const unsigned nv = n / 4;
            const float4* src4 = reinterpret_cast<const float4*>(wt + c0);
            float4* dst4 = reinterpret_cast<float4*>(ws);
            for (unsigned q0 = threadIdx.x; q0 < nv; q0 += nthreads * 8) {
                float4 v[8];
#pragma unroll
                for (int r = 0; r < 8; ++r) v[r] = src4[min(q0 + r * nthreads, nv - 1)];
#pragma unroll
                for (int r = 0; r < 8; ++r)
                    if (q0 + r * nthreads < nv) dst4[q0 + r * nthreads] = v[r];
            }
            for (unsigned r = nv * 4 + threadIdx.x; r < n; r += nthreads) ws[r] = wt[c0 + r];
        } else {
            for (unsigned q = threadIdx.x; q < n; q += nthreads) ws[q] = wt[c0 + q];
        }
        __syncthreads();
        const unsigned hi = c0 + n;
        unsigned resume = 0xffffffffu;
        // kPermRows rows per step: all of a step's slot loads are in flight together
        for (unsigned i = lo; i < rows; i += kPermRows) {
            unsigned e[kPermRows];
#pragma unroll
            for (int q = 0; q < kPermRows; ++q) e[q] = ep[(size_t)min(i + q, rows - 1) * 64];
            bool any_later = false;
#pragma unroll
            for (int q = 0; q < kPermRows; ++q) {
                const unsigned pos = e[q];
                const bool real = i + q < rows && pos != kPadPos;
                if (real && pos >= c0 && pos < hi) op[(size_t)(i + q) * 64] = ws[pos - c0];
                if (c0 == 0 && i + q < rows && !real) op[(size_t)(i + q) * 64] = 0.f;     // padding slots
                any_later |= real && pos >= hi;
            }
            if (resume == 0xffffffffu && __any(any_later)) resume = i;
        }
        lo = (resume == 0xffffffffu) ? rows : resume;
    }
}

// The eight 16-byte reads of one row (chunk order skewed by the lane id) ...
// `skewbase` = LDS address of the tile + (lane & 7) * 16; the tile is 128-byte aligned, so the chunk
// bits can be flipped with XOR after the row offset has been added (one add + seven XORs per row).
typedef float lds_v4f __attribute__((ext_vector_type(4)));
typedef const lds_v4f __attribute__((address_space(3)))* lds_v4f_ptr;
template <int C>
__device__ __forceinline__ float4 igrad_read_chunk(unsigned base) {
    const lds_v4f t = *(lds_v4f_ptr)(size_t)(skew_addr<C>(base));
    return make_float4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void igrad_reads_at(unsigned base, float4 (&v)[8]) {
    v[0] = igrad_read_chunk<0>(base); v[1] = igrad_read_chunk<1>(base);
    v[2] = igrad_read_chunk<2>(base); v[3] = igrad_read_chunk<3>(base);
    v[4] = igrad_read_chunk<4>(base); v[5] = igrad_read_chunk<5>(base);
    v[6] = igrad_read_chunk<6>(base); v[7] = igrad_read_chunk<7>(base);
}
__device__ __forceinline__ void igrad_reads(unsigned e, unsigned skewbase, float4 (&v)[8]) {
    const unsigned base = (e << 7) + skewbase;
    v[0] = igrad_read_chunk<0>(base); v[1] = igrad_read_chunk<1>(base);
    v[2] = igrad_read_chunk<2>(base); v[3] = igrad_read_chunk<3>(base);
    v[4] = igrad_read_chunk<4>(base); v[5] = igrad_read_chunk<5>(base);
    v[6] = igrad_read_chunk<6>(base); v[7] = igrad_read_chunk<7>(base);
}
// ... and the 32 multiply-adds that consume them.
__device__ __forceinline__ void igrad_fmas(const float4 (&v)[8], float wv, float (&acc)[32]) {
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        acc[4 * c + 0] = fmaf(wv, v[c].x, acc[4 * c + 0]);
        acc[4 * c + 1] = fmaf(wv, v[c].y, acc[4 * c + 1]);
        acc[4 * c + 2] = fmaf(wv, v[c].z, acc[4 * c + 2]);
        acc[4 * c + 3] = fmaf(wv, v[c].w, acc[4 * c + 3]);
    }
}

// partial[stream][n][b] over the stream's tiles.  grid = streams * batch tiles.
// MAXT: largest workgroup the instantiation is launched with (sets the register budget);
// LPT: labels of a tile staged per thread (tile_labels <= LPT * blockDim.x).
// WLDS: `wp` is the weight matrix itself and `slot32` holds one word per slot, (position in the tile's [tile_labels][K]
// block of the weights << 17) | (LDS row << 7), in place of lab16:
// the tile's weights are staged in LDS behind the rows of out_grad (with a zero word at tile_labels * K that
// padding slots read) and every slot fetches its weight from there, so no slot-ordered copy of the weights exists.
// PERM (with WLDS and LPT == 1): `colperm` names, per tile, the column each thread walks -- the plan sorts a tile's columns by
// length so that the 64 columns of a wavefront are about equally long.  The thread's sums over one tile then belong to
// another thread's column: after every tile they pass through LDS (the tile's rows and weights are dead by then; row n of
// the exchange = column n, chunks skewed like every other row) to the column's own thread, which adds them to the
// sums it keeps over the whole label stream.
template <int MAXT, int LPT, bool WLDS, bool PERM = false>
__global__ __launch_bounds__(MAXT) void igrad_tile_kernel(const unsigned short* __restrict__ lab16, const float* __restrict__ wp,
                                  const unsigned* __restrict__ slice_off,
                                  const float* __restrict__ g, float* __restrict__ partial, int B, int L,
                                  int tile_labels, int tiles, int tiles_per_stream, int nbt, unsigned total_rows,
                                  const unsigned short* __restrict__ rowpos, int zero_row,
                                  const unsigned* __restrict__ slot32, int K, const unsigned short* __restrict__ colperm = nullptr) {
    static_assert(!PERM || (WLDS && LPT == 1), "the exchange of sums is built for the weights-in-LDS form");
    extern __shared__ __align__(16) float gs[];
    char* gs_bytes = reinterpret_cast<char*>(gs);
    const int nthreads = blockDim.x;
    const int u = xcd_contiguous_block(blockIdx.x, gridDim.x);
    const int bt = u % nbt, stream = u / nbt;
    const int b0 = bt * kTileBatch;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned skew = (unsigned)(lane & 7) * 16u;
    // LDS address of gs (a 32-bit offset inside the workgroup's LDS) plus the lane's skew
    const unsigned skewbase = (unsigned)(size_t)(__attribute__((address_space(3))) float*)gs + skew;
    const int t_begin = stream * tiles_per_stream, t_end = min(t_begin + tiles_per_stream, tiles);
    // plan slots and permuted weights, addressed as (scalar row offset) + (lane offset); 4-GB buffers at most
    const buffer_rsrc lab_rsrc = WLDS ? make_rsrc(slot32, (size_t)total_rows * 256u) : make_rsrc(lab16, (size_t)total_rows * 128u);
    const buffer_rsrc wp_rsrc = make_rsrc(wp, WLDS ? 0 : (size_t)total_rows * 256u);
    const unsigned lane2 = (unsigned)lane * 2u, lane4 = (unsigned)lane * 4u;
    // (WLDS) the tile's weights behind the rows of out_grad and the two zero rows
    float* ws = gs + (size_t)(zero_row + 2) * kTileBatch;
    const unsigned wsbase = (unsigned)(size_t)(__attribute__((address_space(3))) float*)ws;
    const unsigned tile_w = (unsigned)tile_labels * (unsigned)K;       // floats of a full tile; index of the zero word
    constexpr int kWRegs = PERM ? 1 : 8;                                           // 16-byte pieces of the tile's weights a thread carries

    float acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = 0.f;
    // (PERM) the sums of the thread's own column over the tiles so far; `acc` holds one tile's sums of whatever column
    // the thread walks in it
    float home[PERM ? 32 : 1];
#pragma unroll
    for (int i = 0; i < (PERM ? 32 : 1); ++i) home[i] = 0.f;
    unsigned walked = 0;                                   // (PERM) the column of the tile just walked
    // acc -> row `walked` of the exchange; a barrier; row threadIdx.x -> home.  Called between two barriers that keep
    // the tile's rows from being read or written meanwhile.
    auto hand_over = [&]() __attribute__((always_inline)) {
        char* rowp = gs_bytes + ((size_t)walked << 7);
        const int r = lane & 7;
#pragma unroll
        for (int c = 0; c < 8; ++c)
            *reinterpret_cast<float4*>(rowp + ((c ^ r) << 4)) = make_float4(acc[4 * c], acc[4 * c + 1], acc[4 * c + 2], acc[4 * c + 3]);
        __syncthreads();
        const char* mine = gs_bytes + ((size_t)threadIdx.x << 7);
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const float4 v = *reinterpret_cast<const float4*>(mine + ((c ^ r) << 4));
            // (group c of `home`, like group c of `acc`, holds batch entries 4 (c ^ r) ...: undone once, at the end)
            home[PERM ? 4 * c : 0] += v.x; home[PERM ? 4 * c + 1 : 0] += v.y;
            home[PERM ? 4 * c + 2 : 0] += v.z; home[PERM ? 4 * c + 3 : 0] += v.w;
        }
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] = 0.f;
    };

    for (int t = t_begin; t < t_end; ++t) {
        const int j0 = t * tile_labels;
        const int nl = min(tile_labels, L - j0);
        // out_grad rows of this tile: requested before the barrier, so the loads are in flight
        // while the slower wavefronts finish the previous tile
        float gbn[LPT][32];
        unsigned rowp_of[LPT];                   // the LDS row of each staged label (the plan's choice), fetched with its out_grad values
#pragma unroll
        for (int p = 0; p < LPT; ++p) {
            const int jl = (int)threadIdx.x + p * nthreads;
            rowp_of[p] = 0;
            if (jl < nl) {
                load_rows32(g, L, b0, B, (unsigned)(j0 + jl), gbn[p]);
                rowp_of[p] = rowpos[j0 + jl];
            }
        }
        const size_t sl = (size_t)t * (nthreads >> 6) + wave;
        const unsigned row0 = __builtin_amdgcn_readfirstlane(slice_off[sl]);
        const unsigned rows = __builtin_amdgcn_readfirstlane(slice_off[sl + 1]) - row0;
        // The slice's first slot rows are requested here, before the barriers and the staging of the tile: they do not
        // depend on LDS, and their round trip then runs beside that of the tile's rows instead of after it.
        // Slots are fetched from memory kAhead rows ahead of the multiply-adds that use them, through
        // buffer loads whose row offset is a scalar (row indices clamped, not predicated, so the loads
        // carry neither branches nor per-lane address arithmetic).
        constexpr int kAhead = MAXT <= 768 ? 6 : 4;     // (six rows ahead: 0.9 % of the whole step at 670,091 labels; the 1024-thread form has the registers for four)
        const unsigned last = rows ? rows - 1 : 0u;     // (an empty slice: the loads land on the next slice's first row, or beyond the buffer, and are not used)
        // per slot: the label's LDS row and the weight (the forms whose weights are in slot order), or (WLDS) the packed
        // word whose bits 7..16 are the row's byte offset and whose bits 17..31 are the weight's position
        auto load_lab = [&](unsigned r) {
            if (WLDS) return (unsigned)__builtin_amdgcn_raw_buffer_load_b32(lab_rsrc, lane4, (row0 + r) * 256u, 0);
            return (unsigned)(unsigned short)__builtin_amdgcn_raw_buffer_load_b16(lab_rsrc, lane2, (row0 + r) * 128u, 0);
        };
        auto load_w = [&](unsigned r) { return WLDS ? 0.f : buffer_load_f32(wp_rsrc, lane4, (row0 + r) * 256u); };
        unsigned e4[kAhead];
        float w4[kAhead];
#pragma unroll
        for (int q = 0; q < kAhead; ++q) {
            const unsigned r = min((unsigned)q, last);
            e4[q] = load_lab(r);
            w4[q] = load_w(r);
        }
        // (WLDS) the tile's block of the weight matrix, contiguous: requested with the rows of out_grad
        float4 wreg[kWRegs];
        const unsigned nw = (unsigned)nl * (unsigned)K;
        const float* wt = wp + (size_t)j0 * K;
        const bool wvec = WLDS && (nw % 4 == 0) && ((((uintptr_t)wt) & 15) == 0);
        const unsigned nw4 = wvec ? nw / 4 : 0u;                         // 16-byte pieces; the first kWRegs * nthreads of them travel in registers
#pragma unroll
        for (int r = 0; r < kWRegs; ++r) {
            const unsigned q = threadIdx.x + r * nthreads;
            wreg[r] = make_float4(0.f, 0.f, 0.f, 0.f);
            if (WLDS && !PERM && q < nw4) wreg[r] = reinterpret_cast<const float4*>(wt)[q];
        }
        unsigned next_walked = 0;
        if (PERM) next_walked = colperm[(size_t)t * nthreads + threadIdx.x];
        __syncthreads();                       // the previous tile is no longer being read
        // (PERM, 16-byte aligned weights) the tile's weights go from memory straight into LDS, a wavefront 1 KB per instruction
        // -- the registers hold two sets of sums here, not a third of weights; pieces [from, to), waited for in front of the
        // barrier that ends the staging
        auto weights_to_lds = [&](unsigned from, unsigned to) __attribute__((always_inline)) {
            const buffer_rsrc wr = make_rsrc(wt, (size_t)nw * sizeof(float));
            for (unsigned i = from + (unsigned)__builtin_amdgcn_readfirstlane(wave); i < to; i += (unsigned)nthreads >> 6) {
                if (i * 256u + (unsigned)lane * 4u < nw)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (__attribute__((address_space(3))) float*)ws + (size_t)i * 256, 16,
                                                             (unsigned)lane * 16u, i * 1024u, 0, 0);
            }
        };
        const unsigned wpieces = (nw + 255u) / 256u;
        if (PERM) {
            if (t > t_begin) {
                hand_over();
                __syncthreads();               // the exchange has been read: the tile may be staged over it
            }
            // (requested only now that the exchange is over: asked for in front of it, the pieces that land behind the
            // exchange's rows made the kernel 4 % slower)
            if (wvec) weights_to_lds(0u, wpieces);
            walked = next_walked;
        }
        // rows `zero_row` (even) and `zero_row + 1` (odd) are all zero: the targets of padding slots
        // (PERM: the exchange overwrites them after every tile)
        if ((PERM || t == t_begin) && threadIdx.x < 64) gs[zero_row * kTileBatch + threadIdx.x] = 0.f;
        if (WLDS) {
            if ((PERM || t == t_begin) && threadIdx.x == 0) ws[tile_w] = 0.f;
            if (wvec && PERM) {
                // (requested above)
            } else if (wvec) {
#pragma unroll
                for (int r = 0; r < kWRegs; ++r) {
                    const unsigned q = threadIdx.x + r * nthreads;
                    if (q < nw4) reinterpret_cast<float4*>(ws)[q] = wreg[r];
                }
                // (tiles whose weights exceed that: the rest directly, one more round trip)
                for (unsigned q = threadIdx.x + kWRegs * nthreads; q < nw4; q += nthreads)
                    reinterpret_cast<float4*>(ws)[q] = reinterpret_cast<const float4*>(wt)[q];
            } else {
                for (unsigned q = threadIdx.x; q < nw; q += nthreads) ws[q] = wt[q];
            }
        }
        // gs[jl][c] = g[b0+c][j0+jl]: the rows were loaded coalesced along labels; 16-byte LDS writes
        // whose chunk order is skewed by the label id (no bank conflicts)
#pragma unroll
        for (int p = 0; p < LPT; ++p) {
            const int jl = (int)threadIdx.x + p * nthreads;
            if (jl < nl) {
                const int r = jl & 7;
                xor_permute_groups(gbn[p], r);
                // the label's row in LDS is the plan's choice (it balances the bank halves of every column)
                char* rowp = gs_bytes + (rowp_of[p] << 7);
#pragma unroll
                for (int c = 0; c < 8; ++c)
                    *reinterpret_cast<float4*>(rowp + ((c ^ r) << 4)) =
                        make_float4(gbn[p][4 * c], gbn[p][4 * c + 1], gbn[p][4 * c + 2], gbn[p][4 * c + 3]);
            }
        }
        if (PERM) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");      // the weights have arrived in LDS
        __syncthreads();
        if (rows == 0) continue;               // wave-uniform: no column of this slice is used in the tile
        for (unsigned i = 0; i < rows; i += kAhead) {
            unsigned en[kAhead];
            float wn[kAhead];
#pragma unroll
            for (int q = 0; q < kAhead; ++q) {
                const unsigned r = min(i + kAhead + q, last);
                en[q] = load_lab(r);
                wn[q] = load_w(r);
            }
            // keep these loads here, a whole group of rows ahead of their use (left alone, the
            // scheduler sinks them below the multiply-adds and every group waits a full round trip)
            __builtin_amdgcn_sched_barrier(0);
            // Padding slots inside the slice carry weight 0 (or the position of a zero word) and point at an all-zero
            // LDS row.  The rows past the slice's end: the weights-in-LDS form does not walk them (a wave-uniform branch
            // per row; against redirecting them to the zero row it saves two selects per row and 2.5 rows per slice,
            // 5 us of a 0.66-ms step at 670,091 labels); the forms with weights in slot order redirect them, branch-free
            // (there the branch measured 0.4 % slower at fan-in 64 and 501,070 labels).
#pragma unroll
            for (int q = 0; q < kAhead; ++q) {
                const bool in = i + q < rows;                       // wave-uniform
                float4 xv[8];
                if (WLDS) {
                    if (!in) break;
                    // (the tile starts at LDS address 0 -- the kernel has no other LDS -- so the row's byte offset and the
                    // lane's skew, which share no bit, combine with an OR: one instruction with the mask)
                    const float wv = *(const float __attribute__((address_space(3)))*)(size_t)(wsbase + (e4[q] >> 17) * 4u);
                    igrad_reads_at((e4[q] & 0x1ff80u) | skewbase, xv);
                    igrad_fmas(xv, wv, acc);
                } else {
                    igrad_reads(in ? e4[q] : (unsigned)zero_row, skewbase, xv);
                    igrad_fmas(xv, in ? w4[q] : 0.f, acc);
                }
            }
#pragma unroll
            for (int q = 0; q < kAhead; ++q) { e4[q] = en[q]; w4[q] = wn[q]; }
        }
    }
    if (PERM) {
        __syncthreads();                       // the last tile is no longer being read
        if (t_begin < t_end) hand_over();
#pragma unroll
        for (int i = 0; i < 32; ++i) acc[i] = home[PERM ? i : 0];
    }
    // back to natural batch order, then one 128-byte row per thread
    xor_permute_groups(acc, lane & 7);
    float* out = partial + ((size_t)stream * nthreads + threadIdx.x) * ((size_t)nbt * kTileBatch) + b0;
#pragma unroll
    for (int c = 0; c < 8; ++c)
        *reinterpret_cast<float4*>(out + 4 * c) = make_float4(acc[4 * c], acc[4 * c + 1], acc[4 * c + 2], acc[4 * c + 3]);
}

// gx = sum over streams, ascending: a fixed order, so results are reproducible.
template <bool TP>
__global__ __launch_bounds__(256) void igrad_reduce_kernel(const float* __restrict__ partial, float* __restrict__ gx,
                                                           int B, int N, int streams, int nthreads, int bpad,
                                                           const unsigned long long* __restrict__ verdict, int col_lo) {
    const int b = blockIdx.x * 256 + threadIdx.x;
    const int n = blockIdx.y;                          // column inside the plan's window; gx column n + col_lo
    if (b >= B) return;
    gx += TP ? (size_t)col_lo * B : (size_t)col_lo;
    // the plan is known to be outdated: zeros, for the kernel that recomputes the gradient from the lookup to add to
    if (verdict != nullptr && *verdict == 0) {
        if (TP) gx[(size_t)n * B + b] = 0.f; else gx[(size_t)b * N + n] = 0.f;
        return;
    }
    float v = 0.f;
    const size_t step = (size_t)nthreads * bpad;
    const float* p = partial + (size_t)n * bpad + b;
    int r = 0;
    for (; r + 8 <= streams; r += 8) {                 // eight loads in flight, added in ascending order
        float t[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) t[q] = p[(size_t)(r + q) * step];
#pragma unroll
        for (int q = 0; q < 8; ++q) v += t[q];
    }
    for (; r < streams; ++r) v += p[(size_t)r * step];
    if (TP) gx[(size_t)n * B + b] = v; else gx[(size_t)b * N + n] = v;
}

int launch_tiled(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp, hipStream_t s,
                 const unsigned long long* verdict) {
    const int nbt = (B + kTileBatch - 1) / kTileBatch;
    const int cus = device_cu_count();
    const int per_cu = tiled_workgroups_per_cu(p->threads, p->tile_labels, p->K, p->w_in_lds, nbt);
    int streams = std::max(1, std::min(p->tiles, per_cu * cus / std::max(1, nbt)));
    const int tps = (p->tiles + streams - 1) / streams;
    streams = (p->tiles + tps - 1) / tps;
    const int bpad = nbt * kTileBatch;
    const size_t slots = (size_t)p->total_rows * 64;
    float* wp = nullptr;
    float* partial = nullptr;
    if (!p->w_in_lds) FFI_TRY(workspace_get(s, kWsFeaturesT, std::max<size_t>(slots, 1) * sizeof(float), (void**)&wp));
    FFI_TRY(workspace_get(s, kWsPartials, (size_t)streams * p->threads * bpad * sizeof(float), (void**)&partial));
    // large pieces (a whole tile of 1024 labels x 32 connections in one) as soon as the small one does not hold the
    // tile: every piece costs a walk over the tile's slots
    const int chunk = ((long long)p->tile_labels * p->K <= kPermChunk) ? kPermChunk : kPermChunkBig;
    if (!p->w_in_lds) {
        FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_permute_weights_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, chunk * 4));
        hipLaunchKernelGGL(igrad_permute_weights_kernel, dim3(p->tiles), dim3(p->threads), chunk * sizeof(float), s, p->pos16,
                           p->slice_off, w, wp, p->L, p->K, p->tile_labels, chunk);
    }
    // the tile's rows + the two all-zero rows (+ the tile's weights)
    const size_t lds = tiled_lds_bytes(p->tile_labels, p->K, p->w_in_lds);
    const dim3 grid(streams * nbt), block(p->threads);
#define FFI_LAUNCH_TILE(MAXT, LPT, WLDS)                                                                                \
    do {                                                                                                                \
        FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_tile_kernel<MAXT, LPT, WLDS>,                                \
                                        hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));                        \
        hipLaunchKernelGGL((igrad_tile_kernel<MAXT, LPT, WLDS>), grid, block, lds, s, p->lab16, WLDS ? w : wp, p->slice_off, g, \
                           partial, B, p->L, p->tile_labels, p->tiles, tps, nbt, (unsigned)p->total_rows, p->rowpos, p->zero_row, \
                           p->slot32, p->K);                                                                             \
    } while (0)
    // the plan sizes its tiles so that one of these fits: tile_labels <= LPT * threads
    if (p->w_in_lds) {
        // (plans take that form only with workgroups of at most 768 threads that stage one label each)
        if (p->threads > 768 || p->tile_labels > p->threads) return FFI_ERR_BAD_ARGUMENT;
        if (p->colperm != nullptr) {
            // (the exchange of sums between the threads takes a 128-byte row per thread, wherever the tile ends)
            const size_t lds_x = std::max(lds, (size_t)p->threads * kTileBatch * sizeof(float));
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_tile_kernel<768, 1, true, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_x));
            hipLaunchKernelGGL((igrad_tile_kernel<768, 1, true, true>), grid, block, lds_x, s, p->lab16, w, p->slice_off, g, partial, B, p->L,
                               p->tile_labels, p->tiles, tps, nbt, (unsigned)p->total_rows, p->rowpos, p->zero_row, p->slot32, p->K, p->colperm);
        } else {
            FFI_LAUNCH_TILE(768, 1, true);
        }
    } else if (per_cu > 1) {
        FFI_LAUNCH_TILE(1024, 1, false);                 // (the instantiation of at most 128 registers)
    } else if (p->threads <= 768) {
        if (p->tile_labels <= p->threads) FFI_LAUNCH_TILE(768, 1, false); else FFI_LAUNCH_TILE(768, 2, false);
    } else {
        FFI_LAUNCH_TILE(1024, 1, false);
    }
#undef FFI_LAUNCH_TILE
    dim3 rgrid((B + 255) / 256, p->col_n ? p->col_n : p->N);
    if (tp)
        hipLaunchKernelGGL(igrad_reduce_kernel<true>, rgrid, dim3(256), 0, s, partial, gx, B, p->N, streams, p->threads, bpad, verdict, p->col_lo);
    else
        hipLaunchKernelGGL(igrad_reduce_kernel<false>, rgrid, dim3(256), 0, s, partial, gx, B, p->N, streams, p->threads, bpad, verdict, p->col_lo);
    FFI_HIP_TRY(hipGetLastError());
    return FFI_OK;
}

// ---- without a plan --------------------------------------------------------------------------------
// The input gradient straight from the lookup, for the one call after the lookup was edited behind the library's back:
// the kernel runs only if *verdict == 0 ("the cached plan is outdated") and returns at once otherwise.  A workgroup takes a
// stream of label tiles for one batch tile, as igrad_tile_kernel does, and sorts each tile's connections by column itself:
// counts per column (integer LDS atomics), an exclusive scan, then every connection takes the next free place of its
// column's bucket.  Thread t then walks the bucket of column col_lo + t, gathering rows of the tile's out_grad from LDS.
// No slot balancing (rows lie in label order, so row parities are random and the reads run at the 8-clock rate; a
// wavefront walks as long as its longest bucket), and the order inside a bucket is whatever the atomics gave: sums are
// not reproducible bit for bit.  Measured at 670,091 labels x fan-in 32 over 768 columns, batch 128, against float
// atomics into an LDS tile of gx (ds_add_f32 retires a third of a lane per clock and CU here, integer atomics seven
// lanes): 14.3 ms before.  gx must be zero; the workgroups add their sums with one global atomic per (column, sample).
// LDS: gs[tile_labels][32] | ws[tile_labels * K] | lst[tile_labels * K] | cursor[threads] | wave sums[16].
template <bool TP>
__global__ __launch_bounds__(1024) void igrad_unplanned_kernel(const unsigned long long* __restrict__ verdict,
                                                               const int32_t* __restrict__ idx, const float* __restrict__ w,
                                                               const float* __restrict__ g, float* __restrict__ gx, int B, int N,
                                                               int L, int K, int tile_labels, int tiles, int tiles_per_stream,
                                                               int nbt, int col_lo, int ncols) {
    if (*verdict != 0) return;
    extern __shared__ __align__(16) float gs[];
    const int nthreads = blockDim.x;
    float* ws = gs + (size_t)tile_labels * kTileBatch;
    unsigned* lst = reinterpret_cast<unsigned*>(ws + (size_t)tile_labels * K);
    int* cursor = reinterpret_cast<int*>(lst + (size_t)tile_labels * K);
    int* wave_sum = cursor + nthreads;
    const int bt = blockIdx.x % nbt, stream = blockIdx.x / nbt;
    const int b0 = bt * kTileBatch;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const unsigned skewbase = (unsigned)(size_t)(__attribute__((address_space(3))) float*)gs + (unsigned)(lane & 7) * 16u;
    char* gs_bytes = reinterpret_cast<char*>(gs);
    const int t_begin = stream * tiles_per_stream, t_end = min(t_begin + tiles_per_stream, tiles);
    float acc[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) acc[i] = 0.f;
    for (int t = t_begin; t < t_end; ++t) {
        const int j0 = t * tile_labels;
        const int nl = min(tile_labels, L - j0);
        const int total = nl * K;
        const int32_t* src = idx + (size_t)j0 * K;
        __syncthreads();                                   // the previous tile is no longer being read
        cursor[threadIdx.x] = 0;
        for (int jl = threadIdx.x; jl < nl; jl += nthreads) {
            float gb[32];
            load_rows32(g, L, b0, B, (unsigned)(j0 + jl), gb);
            const int r = jl & 7;
            xor_permute_groups(gb, r);
            char* rowp = gs_bytes + ((size_t)jl << 7);
#pragma unroll
            for (int c = 0; c < 8; ++c)
                *reinterpret_cast<float4*>(rowp + ((c ^ r) << 4)) = make_float4(gb[4 * c], gb[4 * c + 1], gb[4 * c + 2], gb[4 * c + 3]);
        }
        for (int q = threadIdx.x; q < total; q += nthreads) ws[q] = w[(size_t)j0 * K + q];
        __syncthreads();
        for (int e = threadIdx.x; e < total; e += nthreads) {
            const unsigned c = (unsigned)(src[e] - col_lo);             // (ids outside [0, N) or outside the window: skipped)
            if (c < (unsigned)ncols) atomicAdd(&cursor[c], 1);
        }
        __syncthreads();
        // exclusive scan of the counts over the workgroup
        const int mine = cursor[threadIdx.x];
        int incl = mine;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int v = __shfl_up(incl, off, 64);
            if (lane >= off) incl += v;
        }
        if (lane == 63) wave_sum[wave] = incl;
        __syncthreads();
        int before = 0;
        for (int q = 0; q < wave; ++q) before += wave_sum[q];
        const int begin = before + incl - mine;
        cursor[threadIdx.x] = begin;
        __syncthreads();
        {
            // (label of entry e without a division per entry: the thread's entries are nthreads apart)
            int l = (int)threadIdx.x / K, k = (int)threadIdx.x - l * K;
            const int dl = nthreads / K, dk = nthreads - dl * K;
            for (int e = threadIdx.x; e < total; e += nthreads) {
                const unsigned c = (unsigned)(src[e] - col_lo);
                if (c < (unsigned)ncols) lst[atomicAdd(&cursor[c], 1)] = ((unsigned)e << 10) | (unsigned)l;
                l += dl; k += dk;
                if (k >= K) { k -= K; ++l; }
            }
        }
        __syncthreads();
        const int len = cursor[threadIdx.x] - begin;
        int longest = len;
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) longest = max(longest, __shfl_xor(longest, off, 64));
        for (int i = 0; i < longest; ++i) {
            if (i < len) {
                const unsigned entry = lst[begin + i];
                const float wv = ws[entry >> 10];
                float4 xv[8];
                igrad_reads(entry & 1023u, skewbase, xv);
                igrad_fmas(xv, wv, acc);
            }
        }
    }
    xor_permute_groups(acc, lane & 7);
    if ((int)threadIdx.x < ncols) {
        const int n = col_lo + (int)threadIdx.x;
#pragma unroll
        for (int c = 0; c < 32; ++c)
            if (b0 + c < B) atomicAdd(&gx[TP ? (size_t)n * B + (b0 + c) : (size_t)(b0 + c) * N + n], acc[c]);
    }
}

}  // namespace

// LDS of igrad_unplanned_kernel for tiles of `tile_labels` labels
static size_t unplanned_lds_bytes(int tile_labels, int K, int threads) {
    return (size_t)tile_labels * (kTileBatch * sizeof(float) + 8u * (size_t)K) + (size_t)threads * 4u + 64u;
}

bool input_grad_unplanned_fits(int N, int K) {
    const int threads = std::min(1024, (N + 63) / 64 * 64);
    return tile_path_fits(N) && N <= 2048 && unplanned_lds_bytes(1, K, threads) <= (size_t)kPlanLdsBudget;
}

int launch_input_grad_unplanned(const unsigned long long* verdict, const int32_t* idx, const float* w, const float* g, float* gx,
                                const Dims& d, hipStream_t s) {
    if (!input_grad_unplanned_fits(d.N, d.K)) return FFI_ERR_BAD_ARGUMENT;
    const int nbt = (d.B + kTileBatch - 1) / kTileBatch;
    const int cus = device_cu_count();
    // inputs of more than 1,024 columns: one launch per half of the columns (a thread per column)
    const int windows = d.N > 1024 ? 2 : 1;
    const int lower = windows == 1 ? d.N : ((d.N + 1) / 2 + 63) / 64 * 64;
    for (int win = 0; win < windows; ++win) {
        const int col_lo = win == 0 ? 0 : lower, ncols = win == 0 ? lower : d.N - lower;
        const int threads = (ncols + 63) / 64 * 64;
        // as many labels per tile as the LDS holds (entries keep the label in 10 bits), then evened out so that every
        // workgroup of a batch tile gets the same number of tiles
        const size_t per_label = kTileBatch * sizeof(float) + 8u * (size_t)d.K;
        int tl = (int)std::min<size_t>(1023, ((size_t)kPlanLdsBudget - (size_t)threads * 4u - 64u) / per_label);
        const int streams0 = std::max(1, cus / std::max(1, nbt));
        const int tiles0 = (d.L + tl - 1) / tl;
        const int tps = (tiles0 + streams0 - 1) / streams0;
        if (tiles0 > streams0) tl = std::min(tl, (int)(((long long)d.L + (long long)tps * streams0 - 1) / ((long long)tps * streams0)));
        const int tiles = (d.L + tl - 1) / tl;
        const int streams = (tiles + tps - 1) / tps;
        const size_t lds = unplanned_lds_bytes(tl, d.K, threads);
        const dim3 grid((unsigned)(streams * nbt)), block((unsigned)threads);
        if (d.tp) {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_unplanned_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(igrad_unplanned_kernel<true>, grid, block, lds, s, verdict, idx, w, g, gx, d.B, d.N, d.L, d.K, tl, tiles, tps, nbt,
                               col_lo, ncols);
        } else {
            FFI_HIP_TRY(hipFuncSetAttribute((const void*)igrad_unplanned_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
            hipLaunchKernelGGL(igrad_unplanned_kernel<false>, grid, block, lds, s, verdict, idx, w, g, gx, d.B, d.N, d.L, d.K, tl, tiles, tps, nbt,
                               col_lo, ncols);
        }
        FFI_HIP_TRY(hipGetLastError());
    }
    return FFI_OK;
}

int launch_input_grad(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp,
                      hipStream_t s, const unsigned long long* verdict, bool* zeroed_if_outdated) {
    if (zeroed_if_outdated) *zeroed_if_outdated = false;
    // (a plan whose last build failed holds no arrays)
    if (p->lookup == nullptr) return FFI_ERR_BAD_ARGUMENT;
    if (p->tiled) {
        if (!p->slice_off || !p->rowpos || (p->w_in_lds ? !p->slot32 : (!p->lab16 || !p->pos16))) return FFI_ERR_BAD_ARGUMENT;
        if (zeroed_if_outdated) *zeroed_if_outdated = verdict != nullptr;
        FFI_TRY(launch_tiled(p, w, g, gx, B, tp, s, verdict));
        // inputs wider than one workgroup has threads: the second half of the columns has a tiled form of its own
        if (p->upper != nullptr) {
            const ffi_plan* u = p->upper;
            if (!u->tiled || !u->slice_off || !u->rowpos || (u->w_in_lds ? !u->slot32 : (!u->lab16 || !u->pos16))) return FFI_ERR_BAD_ARGUMENT;
            return launch_tiled(u, w, g, gx, B, tp, s, verdict);
        }
        return FFI_OK;
    }
    if (!p->perm || !p->col_ptr) return FFI_ERR_BAD_ARGUMENT;
    return launch_input_grad_wide(p, w, g, gx, B, tp, s);
}

}  // namespace ffi
