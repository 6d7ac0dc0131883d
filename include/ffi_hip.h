/*
 * C ABI of the MI355X (gfx950) fixed-fan-in sparse layer kernels.
 *
 * This is the boundary a host framework binds to.  It replaces the GPU half of the reference's
 * kernel functors
 *     FixedFanInSparseMatmulKernel<GPUDevice,...>::operator()      tfsparse/cc/kernels/common.h:20-26
 *     FixedFanInSparseMatmulGradKernel<GPUDevice,...>::operator()  tfsparse/cc/kernels/common.h:28-37
 * as they are called from the TensorFlow op kernels in tfsparse/cc/kernels/register.cpp:18-39,48-72.
 *
 * Conventions
 *   - all pointers are DEVICE pointers to dense, contiguous, row-major buffers owned by the caller;
 *   - features is [batch, num_features], or [num_features, batch] when `transposed` != 0
 *     (the reference's "Tp" ops); lookup, weights, weight_grad are [num_units, fan_in];
 *     result / out_grad are [batch, num_units]; feature_grad has the shape of features;
 *   - lookup holds column ids in [0, num_features); int32 and uint32 share the entry points
 *     (same bits for valid ids), duplicates inside a row are legal and accumulate.  The backward entry points
 *     report ids outside that range as FFI_ERR_BAD_LOOKUP: at once when they build their view of the lookup (first
 *     use, after ffi_rewire_f32 / ffi_arrange_connections_f32, ffi_plan_create / ffi_plan_refresh), and one call
 *     late when foreign code wrote the id into a lookup they have already seen (the call that met it skipped the
 *     connection and returned FFI_OK); the forward entry points do not look (neither does the
 *     reference in release builds, kernel_data.cu.h:211) and their results for such a lookup are undefined, not
 *     just for the offending connection: the narrow-input kernels keep two 16-bit ids per register, so an id of
 *     65,536 or more also changes its neighbour, and an id in [num_features, 65,536) reads whatever lies behind
 *     the staged features in LDS (reads past the end of LDS return zero; no device memory outside the call's
 *     buffers is touched).  ffi_check_lookup audits a matrix;
 *   - outputs are fully overwritten; work is enqueued on `stream` (a hipStream_t passed as void*,
 *     NULL = the default stream) and, with two documented exceptions, never synchronises the host;
 *   - every function returns FFI_OK (0) or a negative ffi_status instead of aborting, where the
 *     reference fail-fasts through gsl_Expects (forward.cu:19-28, backward.cu:27-40):
 *     null pointers, any dimension <= 0 or > INT32_MAX, num_units*fan_in > INT32_MAX.
 *   - the library is thread-safe, as an op kernel that TensorFlow enters from several threads at once has to be
 *     (the reference's kernels are stateless, register.cpp:18-72): calls that share a plan or the internal plan
 *     cache serialise, and calls on the same stream serialise for the time it takes to enqueue their work (they
 *     share that stream's internal workspaces; the stream then runs them one after the other).  Calls on different
 *     streams do not wait for each other.
 */
#ifndef FFI_HIP_H
#define FFI_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ffi_stream_t;           /* hipStream_t */
typedef struct ffi_plan ffi_plan;     /* column-ordered view of one lookup matrix (opaque) */

enum ffi_status {
    FFI_OK = 0,
    FFI_ERR_NULL_POINTER = -1,
    FFI_ERR_BAD_SHAPE = -2,       /* a dimension is <= 0, or shapes disagree */
    FFI_ERR_TOO_LARGE = -3,       /* a size does not fit the 32-bit contract of the reference */
    FFI_ERR_HIP = -4,             /* a HIP runtime call failed; see ffi_last_hip_error() */
    FFI_ERR_OUT_OF_MEMORY = -5,
    FFI_ERR_BAD_LOOKUP = -6,      /* a column id is outside [0, num_features) */
    FFI_ERR_NO_DEVICE = -7,
    FFI_ERR_BAD_ARGUMENT = -8
};

/* Library identification: ABI version (bumped on incompatible changes) and the code-object target. */
int ffi_abi_version(void);
const char* ffi_target_arch(void);
const char* ffi_status_string(int status);
/* hipError_t of the last failing runtime call on the calling thread (0 if none). */
int ffi_last_hip_error(void);

/*
 * Forward:  result[b,j] = sum_k weights[j,k] * features[b, lookup[j,k]].
 * Replaces FixedFanInSparseMatmulKernel<GPUDevice,float,Int,*,Transposed>::operator()
 * (tfsparse/cc/kernels/forward.cu:36-74; CPU semantics tfsparse/cc/kernels/forward.cpp:9-44),
 * i.e. the compute of ops FanInSparseMatmul / FanInSparseMatmulTp
 * (tfsparse/cc/ops/fixed_fan_in_ops.cpp:55-71).
 */
int ffi_forward_f32(const float* features, const int32_t* lookup, const float* weights, float* result,
                    int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                    int transposed, ffi_stream_t stream);

/*
 * ffi_forward_f32 for callers that cannot allocate device memory while they run: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart in the reference.
 * Same arguments and results (bit for bit) as ffi_forward_f32, but the call allocates nothing: the one buffer
 * the kernels need beyond inputs and outputs -- the [num_features, batch] copy of [batch, num_features]
 * features -- lives in a fixed 4 MiB array inside the library's code object (one per GPU, held until the
 * process ends).  Limits: num_features <= 1216 (the kernel that keeps a tile of the features in LDS) and
 * batch * num_features <= 1,048,576; anything larger returns FFI_ERR_TOO_LARGE.  Every call on a GPU uses
 * that GPU's one array (it is overwritten, never read before it is written, so nothing needs clearing):
 * calls that overlap on one GPU -- two streams, or two threads -- race, and the caller must serialise them.
 */
int ffi_forward_noalloc_f32(const float* features, const int32_t* lookup, const float* weights, float* result,
                            int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                            int transposed, ffi_stream_t stream);

/*
 * Backward, both gradients from one call, as the reference's grad op does:
 *   feature_grad[b,n] = sum over (j,k) with lookup[j,k]==n of weights[j,k] * out_grad[b,j]
 *   weight_grad[j,k]  = sum_b features[b, lookup[j,k]] * out_grad[b,j]
 * Replaces FixedFanInSparseMatmulGradKernel<GPUDevice,float,Int,*,Transposed>::operator()
 * (tfsparse/cc/kernels/backward.cu:49-133; CPU semantics tfsparse/cc/kernels/backward.cpp:8-73),
 * i.e. ops FanInSparseMatmulGrad / FanInSparseMatmulGradTp (fixed_fan_in_ops.cpp:73-93).
 * Either output pointer may be NULL to skip that gradient.  The input gradient uses no float
 * atomics: results are bit-identical from run to run.  It needs a column-ordered view of `lookup`
 * which is built on the device on first use and cached inside the library, keyed on the lookup
 * pointer and shape, so in-place edits of lookup (rewiring, sparse/custom_layer.py:32-43) must be picked up:
 *   - edits made through this library (ffi_rewire_f32, ffi_arrange_connections_f32) mark the cached view outdated
 *     on the host, and the next backward call rebuilds it before it enqueues anything (that call synchronises
 *     `stream` and takes the time of a plan build, about 2 ms at 670,091 x 32 connections; results stay
 *     bit-reproducible);
 *   - edits by foreign code are caught by a content fingerprint that a kernel re-checks on every call, on the
 *     device, without a host wait: every call enqueued before the host has seen the verdict -- the first call after
 *     the edit and as many more as the host runs ahead of the GPU -- computes correct results by kernels that read
 *     the lookup directly (the input gradient sorts each label tile's connections by column on the fly: about
 *     2 ms at that size instead of 0.5, and its sums are not reproducible bit for bit); the first call made after the verdict has reached
 *     the host rebuilds the view.  Callers that edit the lookup themselves and care should hold an explicit plan
 *     (ffi_plan_create / ffi_plan_refresh) or call ffi_arrange_connections_f32 afterwards.
 */
int ffi_backward_f32(const float* features, const int32_t* lookup, const float* weights,
                     const float* out_grad, float* feature_grad, float* weight_grad,
                     int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                     int transposed, ffi_stream_t stream);

/* The two halves of ffi_backward_f32 on their own (backward.cpp:8-36 and :39-73). */
int ffi_weight_grad_f32(const float* features, const int32_t* lookup, const float* out_grad,
                        float* weight_grad,
                        int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                        int transposed, ffi_stream_t stream);
int ffi_input_grad_f32(const int32_t* lookup, const float* weights, const float* out_grad,
                       float* feature_grad,
                       int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                       int transposed, ffi_stream_t stream);

/*
 * Explicit plans, for callers that know when lookup changes (e.g. once per rewire interval,
 * sparse/optimizer.py:68-74) and want to skip the per-call fingerprint.  No counterpart in the
 * reference, whose input gradient scatters with atomicAdd (backward.cu.h:119,139,161,182).
 * ffi_plan_create synchronises `stream` once.  A plan is tied to the device it was made on.
 * `batch_hint` is the batch size the plan will mostly be used with (0 = unknown).  It steers the plan's layout only:
 * for batches of at most 128 (at most 256 with fan_in <= 32 and num_features <= 256 or 448 < num_features <= 768)
 * and num_features <= 768 the plan uses smaller label tiles whose weights the input-gradient kernel keeps on chip,
 * which needs no slot-ordered copy of the weights per call;
 * any batch size may be used with any plan, a mismatch costs time (up to 30 %), not correctness.  The plans the stateless
 * entry points cache take the batch size of the call that builds them.
 */
int ffi_plan_create(const int32_t* lookup, int64_t num_units, int64_t fan_in, int64_t num_features,
                    int64_t batch_hint, ffi_stream_t stream, ffi_plan** plan);
int ffi_plan_refresh(ffi_plan* plan, const int32_t* lookup, ffi_stream_t stream);
int ffi_plan_destroy(ffi_plan* plan);
/*
 * What a plan looks like (for benchmarks and logs; no counterpart in the reference).  info[0] = 1 for the tiled form
 * (narrow inputs) or 0 for the blocked global form; [1] = 1 if the input-gradient kernel keeps a tile's weights in LDS;
 * [2] labels per tile; [3] threads of the walking kernel; [4] tiles; [5] slot rows (64 slots each; slots / connections
 * is the padding the walk pays); [6] bytes the plan holds on the device; [7] = 1 if it holds arranged column ids for
 * the weight gradient.
 */
int ffi_plan_info(const ffi_plan* plan, int64_t info[8]);
int ffi_input_grad_planned_f32(const ffi_plan* plan, const float* weights, const float* out_grad,
                               float* feature_grad, int64_t batch, int transposed, ffi_stream_t stream);

/*
 * Weight gradient with an explicit plan of the same lookup matrix: for narrow inputs the kernel then
 * reads the plan's 16-bit copy of the column ids, reordered per label so that its LDS reads are free
 * of bank conflicts (ffi_backward_f32 does the same through its cached plan).  `lookup` is still
 * needed for shapes the plan holds no such copy for.  No counterpart in the reference.
 */
int ffi_weight_grad_planned_f32(const ffi_plan* plan, const float* features, const int32_t* lookup,
                                const float* out_grad, float* weight_grad, int64_t batch, int transposed,
                                ffi_stream_t stream);

/*
 * Optional layout help for the caller (no counterpart in the reference).  The order of a label's
 * connections inside its row of lookup / weights carries no meaning, and the kernels run faster when
 * even and odd column ids alternate along a row, starting with an even id in labels whose index has
 * bit 3 clear and with an odd id in the others (the forward pass and the weight gradient then read
 * both halves of the LDS banks in every clock).  This reorders every row of `lookup` that way, in
 * place, per chunk of 32 connections, and applies the same permutation to up to four float matrices
 * of the same shape (weights, optimizer moments, ...; `arrays` is a HOST array of `n_arrays` device
 * pointers).  Results of all entry points are unchanged up to summation order; the call is
 * idempotent.  A caller that rewires (sparse/custom_layer.py:32-43) may call it again afterwards.  Like
 * ffi_rewire_f32 it marks any cached plan of `lookup` outdated.
 */
int ffi_arrange_connections_f32(int32_t* lookup, float* const* arrays, int n_arrays,
                                int64_t num_units, int64_t fan_in, ffi_stream_t stream);

/*
 * Tells the library that the caller has edited (or is about to edit, on the stream of its next backward call) the
 * lookup at this address in place with code of its own: cached plans of that buffer are marked outdated, and the next
 * backward call rebuilds before it runs, as after ffi_rewire_f32.  Optional: without it the device-side check
 * described at the top finds the edit, at the price of one backward call through the recomputing kernels.  No
 * counterpart in the reference, whose TensorFlow variables are simply read anew by every kernel.  Host-side only;
 * enqueues nothing.
 */
int ffi_lookup_edited(const int32_t* lookup);

/*
 * Overrides one of the library's kernel choices, process-wide (for benchmark sweeps that re-check a choice against its
 * alternative; no counterpart in the reference).  0 always means "the library decides".
 *   "wgrad_units"          3 or 4: units per thread of the weight-gradient kernels that read arranged column ids
 *   "wgrad_stream"         -1: never the weight-gradient kernel that streams out_grad through LDS
 *   "fwd_lane64"           -1: never the forward kernel that holds 64 samples per workgroup
 *   "plan_weights_in_lds"  -1: never / 1: whenever it fits: the input-gradient form that keeps a tile's weights in LDS
 *   "workgroups_per_cu"    n > 0: at most n workgroups per CU for the kernel that walks a tiled plan
 *   "plan_sorted_columns"  -1: never / 1: whenever the weights-in-LDS form is taken: plans that hand a tile's columns to the
 *                          walking kernel's threads sorted by length (fewer padded slots; the sums pass through LDS after every tile)
 * Drops the cached plans and workspaces of the current device first (as ffi_cache_clear, with its rule about calls in
 * flight).  Unknown names and values outside the ranges above return FFI_ERR_BAD_ARGUMENT and change nothing.
 */
int ffi_set_option(const char* name, int value);

/* Drops every cached plan and workspace of the calling thread's current device.  Waits for the device first; no other
   call of this library may be in flight on that device (from another thread) while it runs. */
int ffi_cache_clear(void);
/* Device bytes currently held by the library (plans + workspaces) on the current device. */
size_t ffi_cache_bytes(void);
/*
 * What the library will hold on the device, beside the caller's tensors, once ffi_forward_f32 (FFI_PASS_FORWARD) and / or
 * ffi_backward_f32 (FFI_PASS_BACKWARD) have run at this shape on one stream: the cached plan of the lookup matrix and
 * the per-stream workspaces.  The reference's op owns no memory (TensorFlow allocates every buffer,
 * tfsparse/cc/kernels/register.cpp:29,59-60); this lets a caller budget for what this library adds.  The plan's size
 * depends on the lookup's content: the figure assumes column ids drawn uniformly (as the reference draws them,
 * sparse/custom_layer.py:15,38) and is an estimate; ffi_cache_bytes() reports the actual amount afterwards.  Needs a
 * current device only for the number of compute units; returns 0 for shapes the entry points reject.
 */
enum ffi_pass_flags { FFI_PASS_FORWARD = 1, FFI_PASS_BACKWARD = 2 };
size_t ffi_workspace_bytes(int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed, int passes);

/*
 * Host-side audit of a lookup matrix (the reference checks index ranges only in audit builds,
 * tfsparse/cc/kernels/kernel_data.cu.h:26-43,211).  Synchronises `stream`.
 * Returns FFI_OK, or FFI_ERR_BAD_LOOKUP if any id is >= num_features (as unsigned).
 */
int ffi_check_lookup(const int32_t* lookup, int64_t num_units, int64_t fan_in, int64_t num_features,
                     ffi_stream_t stream);

/*
 * The layer as its caller uses it: the op followed by tf.nn.bias_add (sparse/layer.py:239-249,
 * sparse/custom_layer.py:45-50), fused.  result[b,j] = (sum_k ...) + bias[j]; bias is [num_units].
 * The backward variant also returns bias_grad[j] = sum_b out_grad[b,j] (the gradient TensorFlow
 * registers for bias_add), computed by the weight-gradient kernel from the out_grad values it
 * loads anyway; weight_grad and bias_grad must both be given, feature_grad may be NULL.
 */
int ffi_forward_bias_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                         float* result,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                         int transposed, ffi_stream_t stream);
int ffi_backward_bias_f32(const float* features, const int32_t* lookup, const float* weights,
                          const float* out_grad, float* feature_grad, float* weight_grad, float* bias_grad,
                          int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                          int transposed, ffi_stream_t stream);

/*
 * Inference variant (no counterpart in the reference, whose ops are registered for float only,
 * tfsparse/cc/kernels/register.cpp:79-109): features and weights are bfloat16 (raw 16-bit
 * patterns, same layouts as above), products are accumulated in fp32, result is fp32.
 */
int ffi_forward_bf16_f32(const uint16_t* features, const int32_t* lookup, const uint16_t* weights, float* result,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                         int transposed, ffi_stream_t stream);

/*
 * The same forward pass fused with a per-sample top-k (1 <= k <= 8): topk_values / topk_indices are
 * [batch, k], scores descending, equal scores ordered by ascending label (the rule of tf.nn.top_k,
 * which the reference uses in sparse/metrics.py:19).  The [batch, num_units] score matrix is never
 * written.  Rows with fewer than k labels are padded with (-inf, -1).
 */
int ffi_forward_topk_bf16(const uint16_t* features, const int32_t* lookup, const uint16_t* weights,
                          float* topk_values, int32_t* topk_indices,
                          int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                          int k, int transposed, ffi_stream_t stream);

/* Per-row top-k (1 <= k <= 8) of an fp32 score matrix scores[batch, num_units], same ordering rule. */
int ffi_topk_f32(const float* scores, int64_t batch, int64_t num_units, int k,
                 float* topk_values, int32_t* topk_indices, ffi_stream_t stream);

/*
 * The loss the reference trains the layer with, and its gradient with respect to the scores: the
 * producer of out_grad.  Restates SparseLossBase.call (sparse/metrics.py:136-139) on top of
 * dense_sparse_cwise_op (sparse/utils.py:11-17): every (b,j) is charged loss(score, 0), except the
 * positions listed in the sparse label matrix, which are charged loss(score, value).
 *   label_indices  [nnz, 2] int64 (row, column) pairs, the layout of tf.sparse.SparseTensor.indices;
 *   label_values   [nnz] float (NULL = all 1.0); nnz may be 0 (both may then be NULL).
 * A position must not be listed twice (TensorFlow's scatter update leaves the outcome open as
 * well); pairs outside [0,batch) x [0,num_units) are skipped, as TensorFlow's GPU gather does.
 *   out_grad[b,j]  = grad_scale * d loss / d score  (Keras' mean over labels, then over the batch,
 *                    is grad_scale = 1 / (batch * num_units)); may alias `scores`;
 *   loss_sum       one float on the device: the un-scaled sum of the element losses; may be NULL.
 *   nz_words       [ceil(batch/32), num_units] uint32, may be NULL: bit i of nz_words[t, j] is set where
 *                  out_grad[32 t + i, j] is not zero, the masks ffi_backward_sparse_f32 accepts.
 * Sums are formed in a fixed order (no atomics).
 */
enum ffi_loss_kind {
    FFI_LOSS_HINGE = 1,           /* SparseHingeLoss          sparse/metrics.py:147-154 */
    FFI_LOSS_SQUARED_HINGE = 2,   /* SparseSquaredHingeLoss   sparse/metrics.py:157-164 */
    FFI_LOSS_BCE = 3,             /* SparseBinaryCrossEntropyLoss  sparse/metrics.py:167-173 */
    /* flag for ffi_forward_loss_f32, OR-ed into loss_kind: gradients that are exactly zero are not stored
       (out_grad keeps what it held there); needs nz_words, which then says which entries were written.
       Such an out_grad goes to ffi_backward_sparse_f32 with FFI_SPARSE_GRAD_IS_PARTIAL. */
    FFI_LOSS_SKIP_ZERO_STORES = 0x100
};
int ffi_loss_grad_f32(const float* scores, const int64_t* label_indices, const float* label_values, int64_t nnz,
                      int loss_kind, float grad_scale, float* out_grad, float* loss_sum, uint32_t* nz_words,
                      int64_t batch, int64_t num_units, ffi_stream_t stream);

/*
 * The counts behind the reference's thresholded metrics (SparsePrecision.update_state, sparse/metrics.py:88-96;
 * SparseRecall.update_state, :119-126), from one pass over the scores.  counts (three doubles on the device):
 *   counts[0]  number of scores > threshold                        (precision's denominator)
 *   counts[1]  sum of label values at listed positions whose score > threshold   (the numerator of both)
 *   counts[2]  sum of all label values                             (recall's denominator)
 * label_indices / label_values / nnz as for ffi_loss_grad_f32.
 */
int ffi_threshold_metrics_f32(const float* scores, const int64_t* label_indices, const float* label_values, int64_t nnz,
                              float threshold, double* counts, int64_t batch, int64_t num_units, ffi_stream_t stream);

/*
 * Forward pass, bias add and loss gradient in one pass (no counterpart in the reference, where they
 * are three TensorFlow ops and the [batch, num_units] score matrix makes two more trips through
 * memory): the forward kernel turns each finished score into its loss gradient before storing it.
 * `bias` may be NULL; `scores` may be NULL when only the gradient and the loss are wanted (the
 * scores of the listed label positions are then recomputed from their rows of lookup / weights).
 * With FFI_LOSS_SKIP_ZERO_STORES in loss_kind the kernel leaves out the stores of zero gradients: with
 * a hinge loss late in training that is nearly all of the [batch, num_units] matrix.
 */
int ffi_forward_loss_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                         const int64_t* label_indices, const float* label_values, int64_t nnz,
                         int loss_kind, float grad_scale, float* scores, float* out_grad, float* loss_sum,
                         uint32_t* nz_words,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                         int transposed, ffi_stream_t stream);

/*
 * Forward pass with a per-sample top-k in fp32 (1 <= k <= 8), same ordering rule as ffi_forward_topk_bf16 (scores
 * descending, equal scores by ascending label: tf.nn.top_k, sparse/metrics.py:19).  `bias` may be NULL.  The
 * [batch, num_units] score matrix is written only if `scores` is given.  How: a sample of the labels is scored
 * first and fixes, per sample, a threshold that k labels are known to reach; the forward kernel then appends
 * every score at or above its sample's threshold to a candidate list (a tiny share of all labels), and the k
 * best candidates are selected.  The result is exact.  A sample whose candidates overflow its list (8192 slots;
 * e.g. thousands of labels tied with the k-th score, as an all-zero feature row gives) is answered from a scan of its
 * whole row instead (on the device, without a host wait; slower for that sample only), so ties still resolve to the
 * lower labels as tf.nn.top_k resolves them.
 * ffi_forward_loss_topk_f32 is ffi_forward_loss_f32 with the same top-k of the scores as a by-product: what a
 * training step needs for the loss, the backward pass and the P@k metrics (sparse/metrics.py:31-71) without
 * the score matrix ever being stored.  No counterpart in the reference.
 */
int ffi_forward_topk_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                         float* scores, float* topk_values, int32_t* topk_indices,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                         int k, int transposed, ffi_stream_t stream);
int ffi_forward_loss_topk_f32(const float* features, const int32_t* lookup, const float* weights, const float* bias,
                              const int64_t* label_indices, const float* label_values, int64_t nnz,
                              int loss_kind, float grad_scale, float* scores, float* out_grad, float* loss_sum,
                              uint32_t* nz_words, float* topk_values, int32_t* topk_indices, int k,
                              int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                              int transposed, ffi_stream_t stream);

/*
 * Backward pass that skips the exact zeros of out_grad, as the reference's GPU kernels do entry by
 * entry (`if(out == 0) continue`, tfsparse/cc/kernels/backward.cu.h:73,94,131,151): with a hinge loss
 * every satisfied margin has gradient 0, and late in training that is nearly all of them.  Same
 * results as ffi_backward_bias_f32 (bias_grad may be NULL here) up to summation order.
 *   nz_words      the masks of the non-zero entries as ffi_forward_loss_f32 / ffi_loss_grad_f32 write
 *                 them (a set bit over a zero entry is allowed, a clear bit over a non-zero entry is
 *                 not), or NULL: out_grad is then scanned first (one read of the matrix);
 *   flags         FFI_SPARSE_GRAD_IS_PARTIAL: out_grad holds values only where nz_words (required then) has a
 *                 bit set, as ffi_forward_loss_f32 leaves it with FFI_LOSS_SKIP_ZERO_STORES; if the dense
 *                 kernels have to run, the call first writes zeros into out_grad wherever the bit is clear.
 *                 FFI_SPARSE_DECIDE_FROM_PREVIOUS: choose the kernels from the number of set bits that the
 *                 previous call of the same shape on this stream found, without waiting for this call's
 *                 number (the first call of a shape still waits).  Results are the same either way -- the
 *                 sparse kernels are correct at any density -- only a sudden jump in density costs one slow
 *                 call; sparse_path_taken then reports the choice made;
 *   max_density   share of set bits up to which the sparse kernels are used (<= 0: library default);
 *                 above it the call runs the dense kernels of ffi_backward_bias_f32;
 *   sparse_path_taken  HOST int, may be NULL: 1 if the sparse kernels ran, 0 if the dense ones did.
 * Synchronises `stream` once (the host reads the number of set bits), except as described under flags.  The sparse input gradient
 * covers num_features <= 4096; wider inputs take the dense input-gradient kernels.  It accumulates
 * with LDS float adds, no global atomics: where two lanes of one instruction add to the same column the
 * hardware picks the order, so its results are reproducible up to summation order only (the dense kernels
 * are bit-reproducible), and FFI_SPARSE_DECIDE_FROM_PREVIOUS, which picks sparse or dense kernels from an
 * earlier call's count, can change the summation order of identical inputs with the call history.
 */
enum ffi_sparse_flags {
    FFI_SPARSE_GRAD_IS_PARTIAL = 1,
    FFI_SPARSE_DECIDE_FROM_PREVIOUS = 2
};
int ffi_backward_sparse_f32(const float* features, const int32_t* lookup, const float* weights,
                            float* out_grad, const uint32_t* nz_words, int flags, float max_density,
                            float* feature_grad, float* weight_grad, float* bias_grad, int* sparse_path_taken,
                            int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                            int transposed, ffi_stream_t stream);

/*
 * Backward pass and optimizer step in one call: the results of ffi_backward_sparse_f32 (feature_grad,
 * from the weights as they are on entry) followed by ffi_adam_step_f32 on `weights` with weight_grad and
 * on `bias` with bias_grad; the two gradients are not returned (they live in a library workspace).
 * When the sparse kernels run, the weight gradient of a label without a non-zero out_grad entry is
 * neither written nor read: the Adam pass takes a zero for it.  `bias` (with bias_m, bias_v) may be
 * NULL; feature_grad may be NULL.  The other arguments are those of the two calls.
 * No counterpart in the reference, where the optimizer is a separate TensorFlow op.
 */
int ffi_backward_sparse_adam_f32(const float* features, const int32_t* lookup, float* weights, float* out_grad,
                                 const uint32_t* nz_words, int flags, float max_density,
                                 float* feature_grad, float* weight_m, float* weight_v,
                                 float* bias, float* bias_m, float* bias_v,
                                 float learning_rate, float beta_1, float beta_2, float epsilon, int64_t step,
                                 int* sparse_path_taken,
                                 int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in,
                                 int transposed, ffi_stream_t stream);

/*
 * One Adam step on `count` float32 variables (weights [num_units * fan_in], or the bias), the
 * optimizer the reference trains the layer with: SparseAdam (sparse/optimizer.py:9-23) is a
 * keras.optimizers.Adam (run.py:126) and this is that class's update rule,
 *   alpha = learning_rate * sqrt(1 - beta_2^step) / (1 - beta_1^step)
 *   m += (gradient - m) * (1 - beta_1);   v += (gradient^2 - v) * (1 - beta_2)
 *   variable -= (m * alpha) / (sqrt(v) + epsilon)
 * with `step` counted from 1.  variable, m and v are updated in place; all four arrays must be
 * 16-byte aligned.  Keras' defaults: beta_1 0.9, beta_2 0.999, epsilon 1e-7.
 */
int ffi_adam_step_f32(float* variable, float* m, float* v, const float* gradient, int64_t count,
                      float learning_rate, float beta_1, float beta_2, float epsilon, int64_t step,
                      ffi_stream_t stream);

/*
 * Rewiring (sparse/layer.py:215-219,236-237; sparse/custom_layer.py:20-43), on the flat per-connection
 * variables of the layer.
 * ffi_select_threshold_f32: *threshold (one float on the device) = the k-th smallest |weights[i]|, k counted
 * from 1 -- the threshold FixedFractionSelector.select (sparse/layer.py:75-86) takes from
 * tf.nn.top_k(-|w|, k) with k = round(fraction * count); k == 0 gives 0 (an empty selection).
 * ffi_rewire_f32: every position with |weights[i]| < *threshold (the strict comparison of
 * sparse/layer.py:57,86; a FixedMagnitudeSelector passes its own threshold) gets a new source drawn
 * uniformly from [0, num_features) in lookup[i] -- by a counter-based generator keyed on (seed, i); the
 * reference draws from TensorFlow's stream, which no other implementation reproduces -- and zeros in
 * arrays[0..n_arrays) (HOST array of up to four device pointers: the optimizer's moments,
 * sparse/optimizer.py:14-21).  Weights keep their values.  *rewired_count (device, may be NULL)
 * receives the number of positions changed.  The call marks any cached plan of `lookup` outdated: the next
 * backward call through the stateless entry points rebuilds it first; an explicit plan needs ffi_plan_refresh.
 */
int ffi_select_threshold_f32(const float* weights, int64_t count, int64_t k, float* threshold, ffi_stream_t stream);
int ffi_rewire_f32(int32_t* lookup, const float* weights, float* const* arrays, int n_arrays, int64_t count,
                   int64_t num_features, const float* threshold, uint64_t seed, int64_t* rewired_count,
                   ffi_stream_t stream);

/*
 * Host (CPU) implementation, for the DEVICE_CPU kernels an op library registers beside the GPU ones
 * (tfsparse/cc/kernels/register.cpp:79-80,88-89,97-98,106-107; CPU functors forward.cpp:9-44, backward.cpp:8-73).
 * All pointers are HOST pointers; nothing touches a GPU and nothing starts a thread: the caller splits the work
 * over its own threads through the ranges -- ffi_host_forward_f32 writes result[:, unit_begin:unit_end);
 * ffi_host_backward_f32 writes weight_grad rows [unit_begin, unit_end) (if weight_grad is given) and the
 * feature_grad entries of batch rows [batch_begin, batch_end) (if feature_grad is given), as the reference splits
 * its two halves (backward.cpp:26-35 by units, :58-72 by batch entries).  Ids outside [0, num_features) return
 * FFI_ERR_BAD_LOOKUP.  These are not fallbacks of the GPU entry points, which never compute on the CPU.
 */
int ffi_host_forward_f32(const float* features, const int32_t* lookup, const float* weights, float* result,
                         int64_t batch, int64_t num_features, int64_t num_units, int64_t fan_in, int transposed,
                         int64_t unit_begin, int64_t unit_end);
int ffi_host_backward_f32(const float* features, const int32_t* lookup, const float* weights, const float* out_grad,
                          float* feature_grad, float* weight_grad, int64_t batch, int64_t num_features,
                          int64_t num_units, int64_t fan_in, int transposed, int64_t unit_begin, int64_t unit_end,
                          int64_t batch_begin, int64_t batch_end);

#ifdef __cplusplus
}
#endif
#endif /* FFI_HIP_H */
