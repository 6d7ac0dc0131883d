// Internal declarations shared by the translation units of libffi_hip.so (gfx950 only).
#ifndef FFI_INTERNAL_H
#define FFI_INTERNAL_H

#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstddef>
#include <vector>

#include "ffi_hip.h"

struct ffi_plan;

namespace ffi {

// Shape bundle, validated on the host before any launch.
struct Dims {
    int B;   // batch
    int N;   // num_features
    int L;   // num_units (labels)
    int K;   // fan_in
    bool tp; // features / feature_grad are [N,B]
};

// Overrides of the launchers' choices, set through ffi_set_option (benchmark sweeps re-check each choice against its
// alternative with them); all zero = the library decides.
struct Options {
    int wgrad_units = 0;            // 3 or 4 units per thread of the arranged weight-gradient kernels
    int wgrad_stream = 0;           // -1: never the streaming weight-gradient kernel
    int fwd_lane64 = 0;             // -1: never the 64-sample forward kernel
    int plan_weights_in_lds = 0;    // -1: never / 1: whenever the tile fits
    int workgroups_per_cu = 0;      // upper limit for the kernel that walks a tiled plan
    int plan_sorted_columns = 0;    // -1: never / 1: always (in the weights-in-LDS form) the plans that hand the columns to the walking kernel's threads tile by tile, by length
};
extern Options g_options;

// Records a failing HIP call for ffi_last_hip_error() and maps it to FFI_ERR_HIP.
int hip_fail(hipError_t e);

#define FFI_HIP_TRY(expr)                                   \
    do {                                                    \
        hipError_t e__ = (expr);                            \
        if (e__ != hipSuccess) return ::ffi::hip_fail(e__); \
    } while (0)

#define FFI_TRY(expr)                 \
    do {                              \
        int s__ = (expr);             \
        if (s__ != FFI_OK) return s__; \
    } while (0)

// Held by every entry point that enqueues work, from its first launch to its last: calls on one stream share that
// stream's workspaces, so the kernels of one call must not be interleaved with those of another call made from a
// second thread on the same stream (TensorFlow enters an op's Compute from several threads at once).  Calls on
// different streams do not wait for each other.  Recursive: an entry point may be built from others.
class StreamCall {
public:
    explicit StreamCall(hipStream_t s);
    ~StreamCall();
    StreamCall(const StreamCall&) = delete;
    StreamCall& operator=(const StreamCall&) = delete;
private:
    void* mutex_;
};

// Library-owned device scratch, one buffer per (device, stream, slot), grown on demand and kept.
// Work that uses a buffer is ordered by the stream it belongs to.
enum WorkspaceSlot { kWsFeaturesT = 0, kWsPartials = 1, kWsSlots = 2, kWsLoss = 3, kWsNonzero = 4, kWsGradients = 5, kWsRewire = 6, kWsTopk = 7, kWsScores = 8 };
int workspace_get(hipStream_t s, int slot, size_t bytes, void** out);
void workspace_clear(int device);
size_t workspace_bytes(int device);
int device_cu_count();

// inference variant: bf16 features / weights (raw 16-bit patterns), fp32 accumulation
int launch_forward_bf16(const unsigned short* features, const int32_t* idx, const unsigned short* w, float* out,
                        const Dims& d, hipStream_t s);
int launch_forward_topk_bf16(const unsigned short* features, const int32_t* idx, const unsigned short* w, float* values,
                             int32_t* indices, int k, const Dims& d, hipStream_t s);
int launch_topk_f32(const float* scores, int B, int L, int k, float* values, int32_t* indices, hipStream_t s);

// dst[c][r] = src[r][c] for a row-major [rows, cols] matrix.
// dst[c * dst_ld + r] = src[r * src_ld + c] for r < rows, c < cols (leading dimensions default to the dense ones)
int launch_transpose(const float* src, float* dst, int rows, int cols, hipStream_t s, int src_ld = 0, int dst_ld = 0);

// ---- launchers (each validates nothing; callers pass validated Dims) ---------------------------
// bias ([L], added to every row of out) and bias_grad ([L], column sums of g) may be null
int launch_forward(const float* x, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d,
                   hipStream_t s);
// `plan` (may be null): a plan of the same lookup whose arranged copy of the column ids the kernel may use
// `only_if_outdated` (may be null; without a plan only): device word of a lookup check -- the kernel returns at once unless it is 0
int launch_weight_grad(const float* x, const int32_t* idx, const float* g, float* gw, float* bias_grad, const Dims& d,
                       hipStream_t s, const ffi_plan* plan = nullptr, const unsigned long long* only_if_outdated = nullptr);
// any shape (the tile kernels cover narrow inputs only)
int launch_forward_wide(const float* x, const int32_t* idx, const float* w, const float* bias, float* out, const Dims& d,
                        hipStream_t s);
int launch_weight_grad_wide(const float* x, const int32_t* idx, const float* g, float* gw, float* bias_grad, const Dims& d,
                            hipStream_t s);


// ---- loss gradient (ffi_loss.hip) ---------------------------------------------------------------
struct LossArgs {
    const int64_t* indices;   // [nnz,2] (row, column) of the listed label positions
    const float* values;      // [nnz] or null (all 1)
    int nnz;
    int kind;                 // ffi_loss_kind
    float scale;              // factor on the gradient
    float* loss_sum;          // device float or null
    unsigned* nz_words;       // [ceil(B/32)][L] non-zero masks of the gradient to fill in, or null
    bool skip_zero_stores;    // leave out the stores of zero gradients (fused forward kernel only; needs nz_words)
};
// partial[npartial] loss sums, corr[nnz] loss corrections and saved[nnz] scores of the listed positions
int loss_partial_buffer(hipStream_t s, int npartial, int nnz, double** partial, double** corr, float** saved);
// g at the listed positions, loss corrections, final loss sum; the score of a listed position comes from
// saved[p], else scores[b,j], else from its row of idx / w (+ bias) and x
int launch_loss_positives(const LossArgs& la, const float* saved, const float* scores, const float* x, const int32_t* idx,
                          const float* w, const float* bias, float* g, const Dims& d, const double* partial, int npartial,
                          double* corr, hipStream_t s);
// g = scale * dloss/dscore for a whole score matrix (g may be the score buffer itself)
int launch_loss_grad(const LossArgs& la, const float* scores, float* g, int B, int L, hipStream_t s);
// out[3] (device doubles): scores above the threshold, sum of label values at such positions, sum of label values
int launch_threshold_metrics(const float* scores, const int64_t* indices, const float* values, int nnz, float threshold, int B,
                             int L, double* out, hipStream_t s);
// per-sample top-k wanted from a forward pass: values / indices are [B, k], 1 <= k <= 8
struct TopkArgs {
    int k;
    float* values;
    int32_t* indices;
};
// forward pass whose epilogue turns the scores into loss gradients (scores may be null; tk may be null)
int launch_forward_loss(const float* x, const int32_t* idx, const float* w, const float* bias, const LossArgs& la,
                        float* scores, float* g, const TopkArgs* tk, const Dims& d, hipStream_t s);
// forward pass with per-sample top-k; the score matrix is written only if `scores` is given
int launch_forward_topk(const float* x, const int32_t* idx, const float* w, const float* bias, float* scores, const TopkArgs& tk,
                        const Dims& d, hipStream_t s);
// Candidate lists for a threshold-based top-k: count[B] appended entries, cand_val / cand_idx [B][kTopkCap].
constexpr int kTopkCap = 8192;          // candidate slots per sample (a multiple of 8)
int launch_topk_candidates_init(int* count, int* cand_idx, int B, int cap, hipStream_t s);
// Where the scores of a whole row come from when a sample's candidate list has overflowed: the score matrix [B,L],
// or (scores == null) the layer itself, features as xT [N][B].
struct TopkRowSource {
    const float* scores = nullptr;
    const float* xT = nullptr;
    const int32_t* idx = nullptr;
    const float* w = nullptr;
    const float* bias = nullptr;
    int N = 0, L = 0, K = 0;
};
// the k best candidates of every sample; a sample whose count exceeds cap is answered from its whole row (src)
int launch_topk_candidates_select(const float* cand_val, const int* cand_idx, const int* count, int B, int cap, int k,
                                  float* values, int32_t* indices, hipStream_t s, const TopkRowSource& src);
// the k best of nlists * 8 (score, label) candidates per sample (label -1 = empty slot)
int launch_topk_merge(const float* part_val, const int* part_idx, int B, int nlists, int k, float* values, int32_t* indices,
                      hipStream_t s);

// ---- backward pass over the non-zero entries of out_grad only (ffi_sparse_grad.hip) -------------
// words[t][j]: bit i set <=> out_grad[32 t + i, j] may be non-zero
constexpr int kSparseMaxFeatures = 4096;   // the sparse input gradient keeps 8 x N floats in LDS
constexpr float kSparseDefaultMaxDensity = 0.01f;   // above this share of non-zeros the dense kernels are used
// fills words from g
int launch_nonzero_scan(const float* g, unsigned* words, int B, int L, hipStream_t s);
// the masks to use (the caller's, or a scan of g into a workspace) and their number of set bits.  Synchronises the
// stream, unless `lagged` and an earlier call of the same shape on this stream has left its count: that one is
// returned then, without waiting (this call's count is left for the next one)
int nonzero_count(const float* g, const unsigned* given_words, int B, int L, hipStream_t s, bool lagged,
                  const unsigned** words_out, unsigned long long* count_out);
// drops the counts remembered for a device (the next lagged call waits again)
void nonzero_count_forget(int device);
// active == null: every row of gw is written (zeros for labels without a set bit).  active != null ([L] bytes):
// only the rows of labels with a set bit are written and active[j] tells which
int launch_weight_grad_sparse(const float* x, const int32_t* idx, const float* g, const unsigned* words, float* gw,
                              float* bias_grad, unsigned char* active, const Dims& d, hipStream_t s);
bool sparse_input_grad_fits(int N, int K);
bool sparse_weight_grad_fits(int B, int N);   // x within 32-bit byte offsets
bool sparse_weight_grad_fits(int B, int N);   // x within 32-bit byte offsets
// g[b,j] = 0 wherever the mask bit of (b,j) is clear
int launch_zero_unmasked(float* g, const unsigned* words, int B, int L, hipStream_t s);
int launch_input_grad_sparse(const int32_t* idx, const float* w, const float* g, const unsigned* words, float* gx,
                             const Dims& d, hipStream_t s);

// ---- optimizer (ffi_optimizer.hip) ---------------------------------------------------------------
// one Adam step (Keras' update rule) on `count` float32 variables; arrays 16-byte aligned; step is 1-based
int launch_adam_step(float* var, float* m, float* v, const float* g, size_t count, float lr, float beta_1, float beta_2,
                     float eps, long long step, hipStream_t s);
// the same for a [rows, row_len] variable whose gradient rows are valid only where active[row] != 0 (zero elsewhere)
int launch_adam_step_rows(float* var, float* m, float* v, const float* g, const unsigned char* active, int rows, int row_len,
                          float lr, float beta_1, float beta_2, float eps, long long step, hipStream_t s);

// ---- rewiring (ffi_rewire.hip) -------------------------------------------------------------------
// *threshold (device) = the k-th smallest |w| (k counted from 1; k == 0 gives 0)
int launch_select_threshold(const float* w, size_t count, unsigned long long k, float* threshold, hipStream_t s);
// positions with |w| < *threshold get a new source in [0, num_features) and zeros in the listed arrays;
// *rewired (device, may be null) receives their number
int launch_rewire(int32_t* lookup, const float* w, float* const* arrays, int n_arrays, size_t count, unsigned num_features,
                  const float* threshold, unsigned long long seed, long long* rewired, hipStream_t s);

}  // namespace ffi

// Column-ordered view of one lookup matrix, in one of two forms.
//
// tiled == true (narrow inputs): labels are cut into tiles of `tile_labels`; inside a tile the
// connections are grouped by column, and the columns into slices of 64 (one per wavefront).  A
// slice is stored slot-major (two 16-bit arrays): row i of the slice holds the i-th connection of each of its 64
// columns (so a wavefront reads 256 contiguous bytes per step), padded to the longest column of
// the slice.  Inside a column the slots alternate between even and odd labels (which parity comes
// first depends on the lane, see ffi_plan.hip), positions ascend inside each parity, and holes are
// padding slots: a fixed order, but not the ascending-position order in which the reference's CPU
// kernel accumulates (tfsparse/cc/kernels/backward.cpp:64-72).
//
// tiled == false (any shape): a CSC per block of `block_labels` labels.  perm[e] = flat position of
// the e-th connection in (label block, column, position) order;
// col_ptr[blk*N + n] .. col_ptr[blk*N + n + 1] are the connections of column n inside block blk.
struct ffi_plan {
    int device = -1;
    int L = 0, K = 0, N = 0;
    const int32_t* lookup = nullptr;  // the buffer this plan was built from (cache key)
    unsigned long long fingerprint = 0;
    bool tiled = false;
    // tiled form
    int tile_labels = 0;      // labels per tile (<= 1024)
    int threads = 0;          // workgroup size of the kernels walking the plan: N rounded up to 64
    int slices = 0;           // threads / 64
    int tiles = 0;            // ceil(L / tile_labels)
    long long total_rows = 0; // rows of 64 entries over all slices
    unsigned* slice_off = nullptr;       // [tiles*slices + 1] first row of each slice
    unsigned short* lab16 = nullptr;     // [total_rows*64] LDS row (of the walking kernel's tile) of each slot's label;
                                         // padding slots hold zero_row + parity (two all-zero rows)
    unsigned short* rowpos = nullptr;    // [L] LDS row each label is staged into, inside its tile (see ffi_plan.hip)
    int zero_row = 0;                    // first of the two all-zero rows = rows of the tile in LDS before them
    // plans whose columns are handed to the walking kernel's threads anew in every tile, longest first (so that the 64
    // columns a wavefront walks together are about equally long): [tiles * threads] the column of each thread, a
    // permutation of 0 ... threads - 1 per tile; null in plans whose thread t always walks column t
    unsigned short* colperm = nullptr;
    unsigned* slot32 = nullptr;          // plans with w_in_lds, instead of lab16 and pos16: [total_rows*64] (position << 17) | (LDS row << 7)
    unsigned short* pos16 = nullptr;     // [total_rows*64] position (inside the tile's rows of lookup) of each slot;
                                         // kPadPos in padding slots
    // arranged copy of the column ids for the weight gradient (narrow inputs only, else null): per unit u = chunk * L +
    // label (a chunk = 32 connections) 32 entries of (connection inside the chunk << 11) | column id, each label's
    // connections reordered so that even and odd columns alternate (see ffi_plan.hip); stored in blocks of 64 units,
    // quarter by quarter (ffi::arranged_quarter_offset), so that the 64 lanes of a wavefront load 1 KB in one piece
    unsigned short* idx16 = nullptr;
    // blocked global form
    int block_labels = 0;     // labels per block (bounds the part of out_grad that is live at a time)
    int nblocks = 0;
    int32_t* perm = nullptr;
    int32_t* col_ptr = nullptr;
    unsigned long long* d_scratch = nullptr;  // counters of the build, fingerprint partial sums (device)
    unsigned long long* h_scratch = nullptr;  // pinned mirror
    hipEvent_t fp_done = nullptr;             // recorded behind the fingerprint kernel and its copy to h_scratch
    int fp_blocks = 0;                        // workgroups of the fingerprint kernel in flight: that many pairs of partial sums
    // Check of the lookup's content on the device, without a host wait (plan_guard_*): device words
    // {unused, unused, workgroups finished, expected fingerprint, verdict (1 = the plan is current), fingerprint found,
    // bad ids found, unused, then a pair of partial sums per workgroup}; the pinned mirror holds one word that the
    // check writes last: (number of the check << 2) | (verdict << 1) | (bad ids seen)
    unsigned long long* d_guard = nullptr;
    unsigned long long* h_guard = nullptr;
    unsigned long long guard_seq = 0;         // checks enqueued so far
    unsigned long long guard_seen = 0;        // number of the last check whose result the host has looked at
    bool guard_stale = false;                 // such a look found the plan outdated and nobody has acted on it yet
    bool edited_by_library = false;           // the library itself has enqueued an in-place edit of `lookup` since the plan was built
    hipStream_t guard_stream = nullptr;       // the stream of that check
    size_t bytes = 0;
    // Device buffers behind the arrays above (`owned`) and buffers of an earlier build kept for the next one (`spare`):
    // a rebuild after rewiring needs arrays of nearly the same sizes, and hipMalloc / hipFree of 100-MB buffers cost
    // more than the kernels that fill them.
    struct Buffer { void* ptr; size_t bytes; };
    std::vector<Buffer> owned, spare;
    hipStream_t helper_stream = nullptr;      // the arranged ids are built beside the tiled form (created on first use)
    hipEvent_t helper_event = nullptr;
    int batch_hint = 0;                       // batch size the plan is expected to be used with (0 = unknown); steers layout choices only
    bool w_in_lds = false;                    // tiled form: tiles small enough for the walking kernel to keep the tile's weights in LDS too
    // Inputs of 1,025 to 1,216 columns (the LDS tile holds them, a workgroup of one thread per column does not): the tiled
    // form is built twice, for the lower and the upper half of the columns.  This plan's tiled arrays then cover columns
    // [col_lo, col_lo + col_n) = the lower half, and `upper` (tiled arrays only; everything else of it is unused) the rest.
    int col_lo = 0, col_n = 0;                // col_n == 0: all N columns
    ffi_plan* upper = nullptr;
};

namespace ffi {
constexpr int kPlanTileLabels = 1024;     // a [1024+1][32] fp32 tile fits LDS
constexpr unsigned kPadPos = 0xffffu;      // pos16 of a padding slot; real positions are below it (tile_labels * K <= 0xffff)
// LDS of the kernel that walks the tiled form: the tile's rows of out_grad (per bank half: half the tile plus some room
// for the balancing) and two all-zero rows, 128 bytes each; with the tile's weights behind them, tile_labels * K floats
// and one zero word that padding slots read.
constexpr size_t kPlanLdsBudget = 163700;      // of the 163,840 bytes a workgroup can have (the walking kernel has no other LDS)
inline int tiled_rows_per_half(int tile_labels) { return tile_labels / 2 + (tile_labels / 32 < 64 ? tile_labels / 32 : 64); }
inline size_t tiled_lds_bytes(int tile_labels, int K, bool with_weights) {
    return (size_t)(2 * tiled_rows_per_half(tile_labels) + 2) * 128 + (with_weights ? ((size_t)tile_labels * K + 4) * 4 : 0);
}
// Workgroups of the walking kernel that one CU holds at a time: as many as fit its LDS and its wavefront slots at the
// kernel's register count (16 wavefronts per CU for the instantiation of at most 128 registers that the forms with
// weights in slot order have, 12 for the weights-in-LDS instantiation).  Plans size their tiles for that: one label per
// thread for workgroups of at most 512 threads (slot-ordered weights: two workgroups of 512, four of 256, ...), and for
// weights-in-LDS plans of at most 256 threads a share of the LDS (three workgroups of 256, six of 128).
// Measured, input gradient at 300,000-501,070 labels against one workgroup per CU: slot-ordered weights at eight batch
// tiles -9 % at 512 columns / fan-in 64, -22 % at 256 columns, -51 % at 128, -74 % at 64; weights in LDS with two to
// four batch tiles -28 % at 256 columns, -40...-60 % at 64-128 columns, but +16 % with two workgroups of 384 threads
// (half-size tiles pad more than the sharing gains) and 0...+30 % with a single batch tile (nothing to overlap): those
// two cases keep one workgroup per CU.
inline int tiled_workgroups_per_cu(int threads, int tile_labels, int K, bool with_weights, int batch_tiles) {
    if (threads > 512 || tile_labels > threads) return 1;
    if (with_weights && (threads > 256 || batch_tiles < 2)) return 1;
    const size_t lds = tiled_lds_bytes(tile_labels, K, with_weights);
    const int by_lds = (int)((size_t)160 * 1024 / (lds > 0 ? lds : 1));
    const int by_waves = (with_weights ? 768 : 1024) / (threads > 0 ? threads : 1);
    int n = by_lds < by_waves ? by_lds : by_waves;
    if (g_options.workgroups_per_cu > 0 && n > g_options.workgroups_per_cu) n = g_options.workgroups_per_cu;
    return n < 1 ? 1 : n;
}
// Whether a tiled plan hands its columns to the walking kernel's threads tile by tile, sorted by length (ffi_plan.hip,
// tile_perm_kernel): the weights-in-LDS form with six or more slices, where every workgroup walks two tiles or more.
inline bool plan_sorts_columns(int threads, int tile_labels, int K, bool weights_in_lds, int tiles, int batch_hint) {
    if (!weights_in_lds || g_options.plan_sorted_columns < 0) return false;
    if (g_options.plan_sorted_columns > 0) return true;                 // (tests: whenever the form allows)
    if (threads < 384) return false;
    const int nbt = batch_hint > 32 ? (batch_hint + 31) / 32 : 1;
    const int per_stream = tiled_workgroups_per_cu(threads, tile_labels, K, true, nbt) * device_cu_count() / nbt;
    return tiles >= 2 * (per_stream > 1 ? per_stream : 1);
}
constexpr int kArrIdBits = 11;            // column-id field of an arranged entry (narrow inputs: ids < 1216)
// 16-bit word at which quarter t (entries 8 t ... 8 t + 7) of unit u starts in ffi_plan::idx16: units in blocks of 64, a
// block = [quarter][unit][8 entries]
__host__ __device__ inline size_t arranged_quarter_offset(long long u, int t) {
    return ((size_t)(u >> 6) * 4 + (size_t)t) * 512 + (size_t)(u & 63) * 8;
}
inline size_t arranged_words(long long units) { return (size_t)((units + 63) / 64) * 64 * 32; }
int plan_build(ffi_plan* p, const int32_t* lookup, hipStream_t s);
int plan_tile_labels(int N, int K, int L, int batch_hint, bool* weights_in_lds);
int launch_arrange_in_place(int32_t* lookup, float* const* arrays, int n_arrays, int L, int K, hipStream_t s);
// Content fingerprint of `lookup` (and the count of ids outside [0,N)).  _begin enqueues the kernel
// on `s` and returns; _end waits for that kernel only, not for what the caller enqueued on `s`
// after it, so the host learns the result while later kernels are still running.
int plan_fingerprint_begin(ffi_plan* p, const int32_t* lookup, hipStream_t s);
int plan_fingerprint_end(ffi_plan* p, unsigned long long* out, unsigned long long* bad_ids);
int plan_fingerprint(ffi_plan* p, const int32_t* lookup, hipStream_t s, unsigned long long* out,
                     unsigned long long* bad_ids);
int plan_scratch_alloc(ffi_plan* p);
// Enqueues a check of `lookup` against the plan's fingerprint on `s`: the verdict lands in p->d_guard[kGuardVerdict]
// (device) for the kernels enqueued behind it, and in the pinned mirror for a later call of the host.
constexpr int kGuardVerdict = 4;
int plan_guard_enqueue(ffi_plan* p, const int32_t* lookup, hipStream_t s);
// What the last finished check found, if the host has not seen it yet: *seen = false when no check has finished
// since the last poll.  Never waits.
int plan_guard_poll(ffi_plan* p, bool* seen, bool* current, unsigned long long* bad_ids);
// Both gradients recomputed straight from `lookup` by plain kernels that run only if *verdict == 0 (and return at
// once otherwise): enqueued behind plan-driven kernels, they overwrite what an outdated plan produced.  features /
// weight_grad / bias_grad may be null (no weight gradient wanted), feature_grad may be null.
int launch_backward_if_outdated(const unsigned long long* verdict, const float* features, const int32_t* lookup,
                                const float* weights, const float* out_grad, float* feature_grad, float* weight_grad,
                                float* bias_grad, const Dims& d, hipStream_t s, bool feature_grad_is_zeroed);
void plan_free(ffi_plan* p);
// `verdict` (may be null): device word of a lookup check enqueued ahead; where the kernels can, they leave zeros in gx
// when it says the plan is outdated (*zeroed_if_outdated tells whether they could)
int launch_input_grad(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp,
                      hipStream_t s, const unsigned long long* verdict = nullptr, bool* zeroed_if_outdated = nullptr);
// The input gradient straight from the lookup (no plan), added into a zeroed gx by a kernel that runs only if *verdict == 0;
// for inputs that fit the LDS tile and fan-ins whose tile of one label fits beside it (input_grad_unplanned_fits).
bool input_grad_unplanned_fits(int N, int K);
int launch_input_grad_unplanned(const unsigned long long* verdict, const int32_t* idx, const float* w, const float* g, float* gx,
                                const Dims& d, hipStream_t s);
int launch_input_grad_wide(const ffi_plan* p, const float* w, const float* g, float* gx, int B, bool tp, hipStream_t s);
}  // namespace ffi

#endif  // FFI_INTERNAL_H
