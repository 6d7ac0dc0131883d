"""Fixed-fan-in sparse matmul ops on torch device tensors, backed by the HIP C ABI.

Mirrors the reference's Python op surface (sparse/ops/fixed_fan_in_ops.py:15-40): the same four
functions with the same argument order ``(features, lookup, weights[, out_grad])`` and layouts,
and the same gradient wiring ``[feature_grad, None, weight_grad]``.  Shape rules follow the op
shape functions (tfsparse/cc/ops/fixed_fan_in_ops.cpp:14-53).  torch is used for device memory
and streams only; all arithmetic runs in libffi_hip.so.
"""
from __future__ import annotations

import torch

from . import _lib

_INDEX_DTYPES = (torch.int32, torch.uint32)


def _stream_handle(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _check_inputs(features, lookup, weights, transposed, out_grad=None):
    # rank / shape agreement, as the reference's shape functions demand at graph time
    for name, t in (("features", features), ("lookup", lookup), ("weights", weights)):
        if t.dim() != 2:
            raise ValueError(f"{name} must have rank 2, got shape {tuple(t.shape)}")
    if tuple(lookup.shape) != tuple(weights.shape):
        raise ValueError(f"lookup {tuple(lookup.shape)} and weights {tuple(weights.shape)} must have equal shapes")
    if features.dtype != torch.float32 or weights.dtype != torch.float32:
        raise TypeError("only float32 features/weights are registered (as in the reference)")
    if lookup.dtype not in _INDEX_DTYPES:
        raise TypeError("lookup must be int32 or uint32 (as in the reference)")
    if not features.is_cuda:
        raise RuntimeError("the HIP path needs device tensors; there is no CPU fallback in this package")
    if lookup.device != features.device or weights.device != features.device:
        raise RuntimeError("features, lookup and weights must live on the same device")
    batch = features.shape[1] if transposed else features.shape[0]
    num_features = features.shape[0] if transposed else features.shape[1]
    num_units, fan_in = lookup.shape
    if out_grad is not None:
        if out_grad.dim() != 2 or tuple(out_grad.shape) != (batch, num_units):
            raise ValueError(f"out_grad must have shape {(batch, num_units)}, got {tuple(out_grad.shape)}")
        if out_grad.dtype != torch.float32 or out_grad.device != features.device:
            raise TypeError("out_grad must be float32 on the features' device")
    return batch, num_features, num_units, fan_in


def _forward(features, lookup, weights, transposed):
    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed)
    features = features.contiguous()
    lookup = lookup.contiguous()
    weights = weights.contiguous()
    with torch.cuda.device(features.device):
        result = torch.empty((batch, num_units), dtype=torch.float32, device=features.device)
        _lib.check(_lib.lib().ffi_forward_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), result.data_ptr(),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return result


def _backward(features, lookup, weights, out_grad, transposed):
    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed, out_grad)
    features = features.contiguous()
    lookup = lookup.contiguous()
    weights = weights.contiguous()
    out_grad = out_grad.contiguous()
    with torch.cuda.device(features.device):
        feature_grad = torch.empty_like(features)
        weight_grad = torch.empty_like(weights)
        _lib.check(_lib.lib().ffi_backward_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), out_grad.data_ptr(),
            feature_grad.data_ptr(), weight_grad.data_ptr(),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return feature_grad, weight_grad


def fan_in_sparse_matmul_grad(features, lookup, weights, out_grad):
    """Op FanInSparseMatmulGrad: returns ``(feature_grad [B,N], weight_grad [L,K])``."""
    return _backward(features, lookup, weights, out_grad, False)


def fan_in_sparse_matmul_grad_tp(features, lookup, weights, out_grad):
    """Op FanInSparseMatmulGradTp: features and feature_grad are ``[N,B]``."""
    return _backward(features, lookup, weights, out_grad, True)


class FanInSparseMatmul(torch.autograd.Function):
    """Forward op with the gradient the reference registers for it (fixed_fan_in_ops.py:31-34)."""

    @staticmethod
    def forward(ctx, features, lookup, weights):
        ctx.save_for_backward(features, lookup, weights)
        return _forward(features, lookup, weights, False)

    @staticmethod
    def backward(ctx, grad):
        features, lookup, weights = ctx.saved_tensors
        feature_grad, weight_grad = fan_in_sparse_matmul_grad(features, lookup, weights, grad)
        return feature_grad, None, weight_grad


class FanInSparseMatmulTp(torch.autograd.Function):
    """Transposed-features op and its gradient (fixed_fan_in_ops.py:37-40)."""

    @staticmethod
    def forward(ctx, features, lookup, weights):
        ctx.save_for_backward(features, lookup, weights)
        return _forward(features, lookup, weights, True)

    @staticmethod
    def backward(ctx, grad):
        features, lookup, weights = ctx.saved_tensors
        feature_grad, weight_grad = fan_in_sparse_matmul_grad_tp(features, lookup, weights, grad)
        return feature_grad, None, weight_grad


def fan_in_sparse_matmul(features, lookup, weights):
    """Op FanInSparseMatmul: ``result[b,j] = sum_k weights[j,k] * features[b, lookup[j,k]]``."""
    return FanInSparseMatmul.apply(features, lookup, weights)


def fan_in_sparse_matmul_tp(features, lookup, weights):
    """Op FanInSparseMatmulTp: as above with features given as ``[N,B]``; result is ``[B,L]``."""
    return FanInSparseMatmulTp.apply(features, lookup, weights)


# ------------------------------------------------------------------------------------------------
# Inference variant: bf16 features and weights, fp32 accumulation, optional fused top-k.
# The reference registers its ops for float only (tfsparse/cc/kernels/register.cpp:79-109) and takes
# top-k through tf.nn.top_k in its metrics (sparse/metrics.py:19); these functions have no op there.
# ------------------------------------------------------------------------------------------------
def _check_bf16_inputs(features, lookup, weights, transposed):
    for name, t in (("features", features), ("lookup", lookup), ("weights", weights)):
        if t.dim() != 2:
            raise ValueError(f"{name} must have rank 2, got shape {tuple(t.shape)}")
    if tuple(lookup.shape) != tuple(weights.shape):
        raise ValueError(f"lookup {tuple(lookup.shape)} and weights {tuple(weights.shape)} must have equal shapes")
    if features.dtype != torch.bfloat16 or weights.dtype != torch.bfloat16:
        raise TypeError("features and weights must be bfloat16")
    if lookup.dtype not in _INDEX_DTYPES:
        raise TypeError("lookup must be int32 or uint32")
    if not features.is_cuda:
        raise RuntimeError("the HIP path needs device tensors; there is no CPU fallback in this package")
    if lookup.device != features.device or weights.device != features.device:
        raise RuntimeError("features, lookup and weights must live on the same device")
    batch = features.shape[1] if transposed else features.shape[0]
    num_features = features.shape[0] if transposed else features.shape[1]
    num_units, fan_in = lookup.shape
    return batch, num_features, num_units, fan_in


def fan_in_sparse_matmul_bf16(features, lookup, weights, transposed=False):
    """Scores ``[B,L]`` in fp32 from bf16 features (``[B,N]``, or ``[N,B]`` if ``transposed``) and weights."""
    batch, num_features, num_units, fan_in = _check_bf16_inputs(features, lookup, weights, transposed)
    features, lookup, weights = features.contiguous(), lookup.contiguous(), weights.contiguous()
    with torch.cuda.device(features.device):
        result = torch.empty((batch, num_units), dtype=torch.float32, device=features.device)
        _lib.check(_lib.lib().ffi_forward_bf16_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), result.data_ptr(),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return result


def fan_in_sparse_topk_bf16(features, lookup, weights, k=5, transposed=False):
    """``(values [B,k] fp32, labels [B,k] int32)`` of the k best scores per sample, best first.

    Equal scores are ordered by ascending label; the score matrix is never materialised.
    """
    batch, num_features, num_units, fan_in = _check_bf16_inputs(features, lookup, weights, transposed)
    features, lookup, weights = features.contiguous(), lookup.contiguous(), weights.contiguous()
    with torch.cuda.device(features.device):
        values = torch.empty((batch, k), dtype=torch.float32, device=features.device)
        labels = torch.empty((batch, k), dtype=torch.int32, device=features.device)
        _lib.check(_lib.lib().ffi_forward_topk_bf16(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), values.data_ptr(), labels.data_ptr(),
            batch, num_features, num_units, fan_in, int(k), int(transposed), _stream_handle(features.device)))
    return values, labels


def topk_scores(scores, k=5):
    """Per-row top-k of an fp32 ``[B,L]`` score matrix, same ordering rule as above."""
    if scores.dim() != 2 or scores.dtype != torch.float32:
        raise TypeError("scores must be a float32 matrix")
    if not scores.is_cuda:
        raise RuntimeError("the HIP path needs device tensors; there is no CPU fallback in this package")
    scores = scores.contiguous()
    batch, num_units = scores.shape
    with torch.cuda.device(scores.device):
        values = torch.empty((batch, k), dtype=torch.float32, device=scores.device)
        labels = torch.empty((batch, k), dtype=torch.int32, device=scores.device)
        _lib.check(_lib.lib().ffi_topk_f32(scores.data_ptr(), batch, num_units, int(k), values.data_ptr(),
                                           labels.data_ptr(), _stream_handle(scores.device)))
    return values, labels


# ------------------------------------------------------------------------------------------------
# The op followed by tf.nn.bias_add, as the reference's layer applies it (sparse/layer.py:239-249),
# fused into the kernels: the forward adds bias[j] before it stores a score, the backward returns the
# bias gradient (column sums of out_grad) from the weight-gradient kernel.
# ------------------------------------------------------------------------------------------------
def _check_bias(bias, weights, num_units):
    if bias.dim() != 1 or bias.shape[0] != num_units:
        raise ValueError(f"bias must have shape ({num_units},), got {tuple(bias.shape)}")
    if bias.dtype != torch.float32 or bias.device != weights.device:
        raise TypeError("bias must be float32 on the weights' device")


def _forward_bias(features, lookup, weights, bias, transposed):
    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed)
    _check_bias(bias, weights, num_units)
    features, lookup, weights, bias = features.contiguous(), lookup.contiguous(), weights.contiguous(), bias.contiguous()
    with torch.cuda.device(features.device):
        result = torch.empty((batch, num_units), dtype=torch.float32, device=features.device)
        _lib.check(_lib.lib().ffi_forward_bias_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), bias.data_ptr(), result.data_ptr(),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return result


def _backward_bias(features, lookup, weights, out_grad, transposed, need_feature_grad=True):
    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed, out_grad)
    features, lookup, weights, out_grad = features.contiguous(), lookup.contiguous(), weights.contiguous(), out_grad.contiguous()
    with torch.cuda.device(features.device):
        feature_grad = torch.empty_like(features) if need_feature_grad else None
        weight_grad = torch.empty_like(weights)
        bias_grad = torch.empty((num_units,), dtype=torch.float32, device=features.device)
        _lib.check(_lib.lib().ffi_backward_bias_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), out_grad.data_ptr(),
            feature_grad.data_ptr() if need_feature_grad else None, weight_grad.data_ptr(), bias_grad.data_ptr(),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return feature_grad, weight_grad, bias_grad


class FanInSparseMatmulBiasTp(torch.autograd.Function):
    """``fan_in_sparse_matmul_tp`` + ``bias_add`` as one differentiable op; gradients
    ``[feature_grad, None, weight_grad, bias_grad]``."""

    @staticmethod
    def forward(ctx, features, lookup, weights, bias):
        ctx.save_for_backward(features, lookup, weights)
        return _forward_bias(features, lookup, weights, bias, True)

    @staticmethod
    def backward(ctx, grad):
        features, lookup, weights = ctx.saved_tensors
        feature_grad, weight_grad, bias_grad = _backward_bias(features, lookup, weights, grad, True,
                                                              need_feature_grad=ctx.needs_input_grad[0])
        return feature_grad, None, weight_grad, bias_grad


class FanInSparseMatmulBias(torch.autograd.Function):
    """As above with features given as ``[B,N]``."""

    @staticmethod
    def forward(ctx, features, lookup, weights, bias):
        ctx.save_for_backward(features, lookup, weights)
        return _forward_bias(features, lookup, weights, bias, False)

    @staticmethod
    def backward(ctx, grad):
        features, lookup, weights = ctx.saved_tensors
        feature_grad, weight_grad, bias_grad = _backward_bias(features, lookup, weights, grad, False,
                                                              need_feature_grad=ctx.needs_input_grad[0])
        return feature_grad, None, weight_grad, bias_grad


def fan_in_sparse_matmul_bias(features, lookup, weights, bias):
    """``fan_in_sparse_matmul(features, lookup, weights) + bias`` in one kernel."""
    return FanInSparseMatmulBias.apply(features, lookup, weights, bias)


def fan_in_sparse_matmul_tp_bias(features, lookup, weights, bias):
    """``fan_in_sparse_matmul_tp(features, lookup, weights) + bias`` in one kernel."""
    return FanInSparseMatmulBiasTp.apply(features, lookup, weights, bias)


def backward_sparse(features, lookup, weights, out_grad, nz_words=None, max_density=None, transposed=False,
                    need_feature_grad=True, need_bias_grad=False, grad_is_partial=False, decide_from_previous=False):
    """Backward pass that walks only the non-zero entries of ``out_grad`` (what the reference's GPU
    kernels do entry by entry, tfsparse/cc/kernels/backward.cu.h:73,94,131,151).

    ``nz_words`` ([ceil(B/32), L] int32 bit masks from ``metrics.forward_loss(..., want_masks=True)``)
    saves the scan of ``out_grad``.  Above ``max_density`` (share of non-zeros; default: the
    library's) the dense kernels run instead.  ``grad_is_partial``: ``out_grad`` holds values only where
    ``nz_words`` has a bit set (``metrics.forward_loss(..., skip_zero_stores=True)``); the call may then
    write zeros into the rest of it.  ``decide_from_previous``: choose between sparse and dense kernels
    from the count of non-zeros the previous call of this shape on the stream found, so that the host
    does not wait (same results up to summation order; the first call of a shape still waits).  Returns ``(feature_grad or None, weight_grad,
    bias_grad or None, sparse_kernels_ran)``."""
    import ctypes

    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed, out_grad)
    features, lookup, weights, out_grad = features.contiguous(), lookup.contiguous(), weights.contiguous(), out_grad.contiguous()
    if nz_words is not None:
        if nz_words.dtype != torch.int32 or tuple(nz_words.shape) != ((batch + 31) // 32, num_units) or not nz_words.is_contiguous():
            raise ValueError(f"nz_words must be a contiguous int32 tensor of shape {((batch + 31) // 32, num_units)}")
    taken = ctypes.c_int(-1)
    with torch.cuda.device(features.device):
        feature_grad = torch.empty_like(features) if need_feature_grad else None
        weight_grad = torch.empty_like(weights)
        bias_grad = torch.empty((num_units,), dtype=torch.float32, device=features.device) if need_bias_grad else None
        _lib.check(_lib.lib().ffi_backward_sparse_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), out_grad.data_ptr(),
            nz_words.data_ptr() if nz_words is not None else None,
            int(bool(grad_is_partial)) | (2 if decide_from_previous else 0), float(max_density or 0.0),
            feature_grad.data_ptr() if need_feature_grad else None, weight_grad.data_ptr(),
            bias_grad.data_ptr() if need_bias_grad else None, ctypes.byref(taken),
            batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device)))
    return feature_grad, weight_grad, bias_grad, bool(taken.value)


def arrange_connections(lookup, *arrays):
    """Reorders, in place, the connections inside every row of ``lookup`` ([L,K] int32/uint32) so that
    even and odd column ids alternate (which the kernels read faster), and applies the same
    permutation to every float32 ``[L,K]`` tensor in ``arrays`` (weights, optimizer moments).

    The order of a label's connections carries no meaning, so all results stay the same up to
    summation order.  Idempotent.  Up to four arrays per call.
    """
    import ctypes

    if lookup.dim() != 2 or lookup.dtype not in _INDEX_DTYPES or not lookup.is_cuda or not lookup.is_contiguous():
        raise TypeError("lookup must be a contiguous int32/uint32 [L,K] device tensor")
    if len(arrays) > 4:
        raise ValueError("at most four arrays per call")
    for a in arrays:
        if a.dtype != torch.float32 or tuple(a.shape) != tuple(lookup.shape) or a.device != lookup.device or not a.is_contiguous():
            raise TypeError("arrays must be contiguous float32 tensors of lookup's shape on lookup's device")
    num_units, fan_in = lookup.shape
    ptrs = (ctypes.c_void_p * max(len(arrays), 1))(*[a.data_ptr() for a in arrays])
    with torch.cuda.device(lookup.device):
        _lib.check(_lib.lib().ffi_arrange_connections_f32(lookup.data_ptr(), ptrs, len(arrays), num_units, fan_in,
                                                          _stream_handle(lookup.device)))


def select_threshold(weights, k):
    """Device tensor ``[1]``: the ``k``-th smallest ``|weights|`` (``k`` from 1; 0 gives 0.0), the threshold
    ``FixedFractionSelector`` (sparse/layer.py:75-86) derives from ``tf.nn.top_k(-|w|, k)``."""
    if weights.dtype != torch.float32 or not weights.is_cuda or not weights.is_contiguous():
        raise TypeError("weights must be a contiguous float32 device tensor")
    with torch.cuda.device(weights.device):
        threshold = torch.empty((1,), dtype=torch.float32, device=weights.device)
        _lib.check(_lib.lib().ffi_select_threshold_f32(weights.data_ptr(), weights.numel(), int(k), threshold.data_ptr(),
                                                       _stream_handle(weights.device)))
    return threshold


def rewire_connections(lookup, weights, arrays, num_features, threshold, seed):
    """In place: every connection with ``|weights| < threshold`` (``threshold``: device tensor ``[1]``) gets a
    new source drawn uniformly from ``[0, num_features)`` and zeros in ``arrays`` (up to four float32 tensors
    shaped like ``weights``).  Returns a device int64 tensor ``[1]`` with the number of connections changed."""
    import ctypes

    if lookup.dtype not in _INDEX_DTYPES or not lookup.is_cuda or not lookup.is_contiguous():
        raise TypeError("lookup must be a contiguous int32/uint32 device tensor")
    if weights.dtype != torch.float32 or weights.numel() != lookup.numel() or not weights.is_contiguous():
        raise TypeError("weights must be a contiguous float32 tensor with as many elements as lookup")
    arrays = list(arrays)
    if len(arrays) > 4:
        raise ValueError("at most four arrays per call")
    for a in arrays:
        if a.dtype != torch.float32 or a.numel() != lookup.numel() or a.device != lookup.device or not a.is_contiguous():
            raise TypeError("arrays must be contiguous float32 tensors with as many elements as lookup, on its device")
    ptrs = (ctypes.c_void_p * max(len(arrays), 1))(*[a.data_ptr() for a in arrays])
    with torch.cuda.device(lookup.device):
        changed = torch.empty((1,), dtype=torch.int64, device=lookup.device)
        _lib.check(_lib.lib().ffi_rewire_f32(lookup.data_ptr(), weights.data_ptr(), ptrs, len(arrays), lookup.numel(),
                                             int(num_features), threshold.data_ptr(), int(seed) & (2**64 - 1), changed.data_ptr(),
                                             _stream_handle(lookup.device)))
    return changed


def lookup_edited(lookup):
    """Call after editing ``lookup`` in place with torch operations: the library then rebuilds its cached view of the
    connections before the next backward pass, instead of finding the edit on the device one call late."""
    _lib.check(_lib.lib().ffi_lookup_edited(lookup.data_ptr()))


def fan_in_sparse_topk(features, lookup, weights, bias=None, k=5, transposed=False, want_scores=False):
    """``(values [B,k], labels [B,k] int32)`` of the k best fp32 scores per sample (best first, equal scores
    by ascending label), and the score matrix as a third result if ``want_scores``.  Without
    ``want_scores`` the ``[B,L]`` matrix is never written.  A sample whose candidate list overflows (see
    the C header) is answered from a scan of its whole row."""
    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed)
    if bias is not None:
        _check_bias(bias, weights, num_units)
        bias = bias.contiguous()
    features, lookup, weights = features.contiguous(), lookup.contiguous(), weights.contiguous()
    with torch.cuda.device(features.device):
        values = torch.empty((batch, k), dtype=torch.float32, device=features.device)
        labels = torch.empty((batch, k), dtype=torch.int32, device=features.device)
        scores = torch.empty((batch, num_units), dtype=torch.float32, device=features.device) if want_scores else None
        _lib.check(_lib.lib().ffi_forward_topk_f32(
            features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), bias.data_ptr() if bias is not None else None,
            scores.data_ptr() if want_scores else None, values.data_ptr(), labels.data_ptr(),
            batch, num_features, num_units, fan_in, int(k), int(transposed), _stream_handle(features.device)))
    return (values, labels, scores) if want_scores else (values, labels)
