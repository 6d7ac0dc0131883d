"""Losses and P@k of the reference's training loop, on sparse label matrices.

Mirrors sparse/metrics.py: ``SparseHingeLoss`` (:147-154), ``SparseSquaredHingeLoss`` (:157-164),
``SparseBinaryCrossEntropyLoss`` (:167-173) on ``SparseLossBase`` (:132-144), and ``PrecisionAtK``
(:31-71).  A loss object is called as ``loss(y_true, y_pred)`` with ``y_true`` a sparse
``[batch, num_units]`` matrix (a torch sparse COO tensor, or a pair ``(indices [nnz,2] int64,
values [nnz] float32 or None)`` in the layout of ``tf.sparse.SparseTensor``) and returns the mean
over labels, then over the batch (Keras' default reduction), as a differentiable scalar.  The loss
sum and the gradient with respect to the scores come from one pass in libffi_hip.so; torch holds
the tensors.
"""
from __future__ import annotations

import torch

from . import _lib
from .fixed_fan_in_ops import _check_bias, _check_inputs, _stream_handle, backward_sparse, topk_scores

LOSS_HINGE, LOSS_SQUARED_HINGE, LOSS_BCE = 1, 2, 3
SKIP_ZERO_STORES = 0x100      # flag on the loss kind of forward_loss: zero gradients are not stored


def _labels(y_true, device):
    """``(indices [nnz,2] int64 contiguous, values [nnz] float32 or None)`` on ``device``."""
    if isinstance(y_true, torch.Tensor):
        if not y_true.is_sparse:
            raise TypeError("y_true must be a sparse COO tensor or an (indices, values) pair")
        y_true = y_true.coalesce()
        indices, values = y_true.indices().t(), y_true.values()
    else:
        indices, values = y_true
    indices = indices.to(device=device, dtype=torch.int64).contiguous()
    if indices.dim() != 2 or indices.shape[1] != 2:
        raise ValueError(f"label indices must have shape [nnz, 2], got {tuple(indices.shape)}")
    if values is not None:
        values = values.to(device=device, dtype=torch.float32).contiguous()
        if values.dim() != 1 or values.shape[0] != indices.shape[0]:
            raise ValueError("label values must have shape [nnz]")
    return indices, values


def sparse_loss_grad(scores, y_true, kind, grad_scale=None, in_place=False, want_masks=False):
    """``(out_grad [B,L], loss_sum [1])``: ``out_grad = grad_scale * d loss / d scores`` and the
    un-scaled sum of the element losses.  ``grad_scale`` defaults to ``1 / (B * L)``;
    ``in_place`` overwrites ``scores`` with the gradient.  With ``want_masks`` a third result holds
    the bit masks of the non-zero gradients (``[ceil(B/32), L]`` int32) for ``backward_sparse``."""
    if scores.dim() != 2 or scores.dtype != torch.float32:
        raise TypeError("scores must be a float32 [batch, num_units] matrix")
    if not scores.is_cuda:
        raise RuntimeError("the HIP path needs device tensors; there is no CPU fallback in this package")
    scores = scores if in_place else scores.contiguous()
    if not scores.is_contiguous():
        raise ValueError("in_place needs contiguous scores")
    batch, num_units = scores.shape
    indices, values = _labels(y_true, scores.device)
    scale = 1.0 / (batch * num_units) if grad_scale is None else float(grad_scale)
    with torch.cuda.device(scores.device):
        out_grad = scores if in_place else torch.empty_like(scores)
        loss_sum = torch.empty((1,), dtype=torch.float32, device=scores.device)
        masks = torch.empty(((batch + 31) // 32, num_units), dtype=torch.int32, device=scores.device) if want_masks else None
        _lib.check(_lib.lib().ffi_loss_grad_f32(
            scores.data_ptr(), indices.data_ptr() if indices.numel() else None,
            values.data_ptr() if values is not None and values.numel() else None, indices.shape[0], int(kind), scale,
            out_grad.data_ptr(), loss_sum.data_ptr(), masks.data_ptr() if want_masks else None, batch, num_units,
            _stream_handle(scores.device)))
    return (out_grad, loss_sum, masks) if want_masks else (out_grad, loss_sum)


def forward_loss(features, lookup, weights, bias, y_true, kind, grad_scale=None, transposed=False, want_scores=False,
                 want_masks=False, skip_zero_stores=False, topk=0):
    """Forward pass, bias add and loss gradient in one kernel: ``(scores or None, out_grad, loss_sum)``,
    plus the bit masks of the non-zero gradients with ``want_masks``.  With ``skip_zero_stores`` (needs
    ``want_masks``) ``out_grad`` is written only where its mask bit is set and is undefined elsewhere:
    hand it to ``backward_sparse(..., grad_is_partial=True)``.  With ``topk`` = k (1..8) the per-sample k best
    scores and their labels (``[B,k]`` each) are appended to the results as a pair: the P@k metrics of the step
    without the score matrix."""
    batch, num_features, num_units, fan_in = _check_inputs(features, lookup, weights, transposed)
    if bias is not None:
        _check_bias(bias, weights, num_units)
        bias = bias.contiguous()
    features, lookup, weights = features.contiguous(), lookup.contiguous(), weights.contiguous()
    if skip_zero_stores and not want_masks:
        raise ValueError("skip_zero_stores needs want_masks: the masks say which entries of out_grad were written")
    indices, values = _labels(y_true, features.device)
    scale = 1.0 / (batch * num_units) if grad_scale is None else float(grad_scale)
    with torch.cuda.device(features.device):
        out_grad = torch.empty((batch, num_units), dtype=torch.float32, device=features.device)
        scores = torch.empty_like(out_grad) if want_scores else None
        loss_sum = torch.empty((1,), dtype=torch.float32, device=features.device)
        masks = torch.empty(((batch + 31) // 32, num_units), dtype=torch.int32, device=features.device) if want_masks else None
        common = (features.data_ptr(), lookup.data_ptr(), weights.data_ptr(), bias.data_ptr() if bias is not None else None,
                  indices.data_ptr() if indices.numel() else None,
                  values.data_ptr() if values is not None and values.numel() else None, indices.shape[0],
                  int(kind) | (SKIP_ZERO_STORES if skip_zero_stores else 0), scale,
                  scores.data_ptr() if want_scores else None, out_grad.data_ptr(), loss_sum.data_ptr(),
                  masks.data_ptr() if want_masks else None)
        shape = (batch, num_features, num_units, fan_in, int(transposed), _stream_handle(features.device))
        top = None
        if topk:
            top = (torch.empty((batch, topk), dtype=torch.float32, device=features.device),
                   torch.empty((batch, topk), dtype=torch.int32, device=features.device))
            _lib.check(_lib.lib().ffi_forward_loss_topk_f32(*common, top[0].data_ptr(), top[1].data_ptr(), int(topk), *shape))
        else:
            _lib.check(_lib.lib().ffi_forward_loss_f32(*common, *shape))
    result = (scores, out_grad, loss_sum, masks) if want_masks else (scores, out_grad, loss_sum)
    return result + (top,) if topk else result


def _upstream_is_one(upstream):
    """True where the factor autograd hands to ``backward`` is known ON THE HOST to be 1: reading a device scalar
    here would make every training step wait for the GPU."""
    if not isinstance(upstream, torch.Tensor):
        return float(upstream) == 1.0
    return upstream.device.type == "cpu" and upstream.numel() == 1 and float(upstream) == 1.0


def _scaled(out_grad, upstream):
    # multiplied on the device, whatever the factor (a host-side scalar equal to 1 is the one case that can be
    # skipped without looking at the device); out of place, since a retained graph may run backward again
    return out_grad if _upstream_is_one(upstream) else out_grad * upstream


class _SparseLossFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, scores, indices, values, kind):
        out_grad, loss_sum = sparse_loss_grad(scores, (indices, values), kind)
        ctx.save_for_backward(out_grad)
        return loss_sum[0] / (scores.shape[0] * scores.shape[1])

    @staticmethod
    def backward(ctx, grad):
        (out_grad,) = ctx.saved_tensors
        return _scaled(out_grad, grad), None, None, None


class _LayerLossFn(torch.autograd.Function):
    """Layer forward + bias + loss as one op: the loss gradient is formed inside the forward kernel."""

    @staticmethod
    def forward(ctx, features, lookup, weights, bias, indices, values, kind, transposed, want_scores):
        scores, out_grad, loss_sum, masks = forward_loss(features, lookup, weights, bias, (indices, values), kind,
                                                         transposed=transposed, want_scores=want_scores, want_masks=True,
                                                         skip_zero_stores=True)
        ctx.save_for_backward(features, lookup, weights, out_grad, masks)
        ctx.transposed = transposed
        ctx.has_bias = bias is not None
        batch = features.shape[1] if transposed else features.shape[0]
        loss = loss_sum[0] / (batch * lookup.shape[0])
        if want_scores:
            ctx.mark_non_differentiable(scores)
            return loss, scores
        return loss, torch.empty(0, device=features.device)

    @staticmethod
    def backward(ctx, grad, _grad_scores):
        features, lookup, weights, out_grad, masks = ctx.saved_tensors
        # The upstream factor never touches the [B,L] gradient matrix (mostly unwritten entries, hundreds of MB):
        # all three results are linear in it, so the factor goes on the small operands instead.  The weight
        # gradient is linear in the features ([B,N]); the feature and bias gradients are scaled as results.
        one = _upstream_is_one(grad)
        # the masks say where the gradient is not zero: the backward pass skips the rest when they are few
        feature_grad, weight_grad, bias_grad, _ = backward_sparse(features if one else features * grad, lookup, weights,
                                                                  out_grad, nz_words=masks,
                                                                  transposed=ctx.transposed,
                                                                  need_feature_grad=ctx.needs_input_grad[0],
                                                                  need_bias_grad=ctx.has_bias, grad_is_partial=True,
                                                                  decide_from_previous=True)
        if not one:
            if feature_grad is not None:
                feature_grad.mul_(grad)
            if bias_grad is not None:
                bias_grad.mul_(grad)
        return feature_grad, None, weight_grad, bias_grad, None, None, None, None, None


class SparseLossBase:
    """``loss(y_true, y_pred)`` on a sparse label matrix (sparse/metrics.py:132-144; the base class
    itself computes the hinge loss, as in the reference)."""

    kind = LOSS_HINGE

    def __init__(self, name="sparse_loss"):
        self.name = name

    def __call__(self, y_true, y_pred):
        indices, values = _labels(y_true, y_pred.device)
        return _SparseLossFn.apply(y_pred, indices, values, self.kind)

    def fused(self, features, lookup, weights, bias, y_true, transposed=False, want_scores=False):
        """The same loss of ``fan_in_sparse_matmul[_tp](features, lookup, weights) + bias`` without
        writing the scores (unless asked for): returns ``(loss, scores or None)``."""
        indices, values = _labels(y_true, features.device)
        loss, scores = _LayerLossFn.apply(features, lookup, weights, bias, indices, values, self.kind, transposed, want_scores)
        return loss, (scores if want_scores else None)


class SparseHingeLoss(SparseLossBase):
    kind = LOSS_HINGE

    def __init__(self, name="sparse_hinge_loss"):
        super().__init__(name)


class SparseSquaredHingeLoss(SparseLossBase):
    kind = LOSS_SQUARED_HINGE

    def __init__(self, name="sparse_hinge_loss"):
        super().__init__(name)


class SparseBinaryCrossEntropyLoss(SparseLossBase):
    kind = LOSS_BCE

    def __init__(self, name="sparse_bce_loss"):
        super().__init__(name)


def topk_as_matrix(data, k):
    """The positions of the k best scores of every row as a sparse 0/1 matrix of ``data``'s shape
    (sparse/metrics.py:9-28): ``(indices [B*k, 2] int64 in row-major order, values [B*k] of ones, dense_shape)``,
    the triple a ``tf.sparse.SparseTensor`` holds.  Equal scores go to the lower label."""
    _, top = topk_scores(data, int(k))
    batch = data.shape[0]
    cols, _ = torch.sort(top.to(torch.int64), dim=1)                           # tf.sparse.reorder: ascending columns
    rows = torch.arange(batch, device=data.device).unsqueeze(1).expand_as(cols)
    indices = torch.stack([rows.reshape(-1), cols.reshape(-1)], dim=1)
    return indices, torch.ones(indices.shape[0], dtype=torch.float32, device=data.device), tuple(data.shape)


class PrecisionAtK:
    """Fraction of the k best-scored labels of each sample that are true labels, accumulated over
    ``update_state`` calls (sparse/metrics.py:31-71: label values at the top-k positions are summed,
    and every sample counts k in the denominator, also when it has fewer than k labels)."""

    def __init__(self, k=1, name=None):
        self.name = name or "P_at_{}".format(k)
        self._k = int(k)
        self.reset_state()

    def reset_state(self):
        self._correct = 0.0
        self._total = 0.0

    def update_state(self, y_true, y_pred, sample_weight=None):
        assert sample_weight is None
        _, top = topk_scores(y_pred, self._k)                  # [B,k] labels, device top-k
        self.update_from_topk(y_true, top, y_pred.shape[1])

    def update_from_topk(self, y_true, top_labels, num_units):
        """As ``update_state`` for callers that already hold the top-k labels ``[B, >=k]``."""
        indices, values = _labels(y_true, top_labels.device)
        batch = top_labels.shape[0]
        top = top_labels[:, :self._k].to(torch.int64)
        if indices.shape[0]:
            keys = indices[:, 0] * num_units + indices[:, 1]
            order = torch.argsort(keys)
            keys = keys[order]
            vals = torch.ones_like(keys, dtype=torch.float32) if values is None else values[order]
            rows = torch.arange(batch, device=top.device).unsqueeze(1).expand_as(top)
            want = (rows * num_units + top).reshape(-1)
            pos = torch.searchsorted(keys, want).clamp_(max=keys.numel() - 1)
            hit = (keys[pos] == want) & (top.reshape(-1) >= 0)
            self._correct += float((vals[pos] * hit).sum())
        self._total += float(batch * self._k)

    def result(self):
        return self._correct / self._total if self._total else 0.0


def threshold_counts(scores, y_true, threshold):
    """Device tensor of three doubles: number of scores above ``threshold``, sum of the label values at
    listed positions whose score is above it, sum of all label values (one pass over the scores)."""
    if scores.dim() != 2 or scores.dtype != torch.float32 or not scores.is_cuda:
        raise TypeError("scores must be a float32 [batch, num_units] device matrix")
    scores = scores.contiguous()
    batch, num_units = scores.shape
    indices, values = _labels(y_true, scores.device)
    with torch.cuda.device(scores.device):
        counts = torch.empty((3,), dtype=torch.float64, device=scores.device)
        _lib.check(_lib.lib().ffi_threshold_metrics_f32(
            scores.data_ptr(), indices.data_ptr() if indices.numel() else None,
            values.data_ptr() if values is not None and values.numel() else None, indices.shape[0], float(threshold),
            counts.data_ptr(), batch, num_units, _stream_handle(scores.device)))
    return counts


class _ThresholdMetric:
    def __init__(self, threshold, name):
        self.name = name
        self._threshold = float(threshold)
        self.reset_state()

    def reset_state(self):
        self._correct = 0.0
        self._total = 0.0

    def result(self):
        return self._correct / self._total if self._total else 0.0     # divide_no_nan


class SparsePrecision(_ThresholdMetric):
    """Label values at predicted positions (score > threshold) over the number of predicted positions,
    accumulated over ``update_state`` calls (sparse/metrics.py:73-98)."""

    def __init__(self, threshold, name=None):
        super().__init__(threshold, name or "Precision")

    def update_state(self, y_true, y_pred, sample_weight=None):
        assert sample_weight is None
        predicted, correct, _ = threshold_counts(y_pred, y_true, self._threshold).tolist()
        self._correct += correct
        self._total += predicted


class SparseRecall(_ThresholdMetric):
    """Label values at predicted positions over the sum of all label values (sparse/metrics.py:101-129)."""

    def __init__(self, threshold, name=None):
        super().__init__(threshold, name or "Recall")

    def update_state(self, y_true, y_pred, sample_weight=None):
        assert sample_weight is None
        _, correct, total = threshold_counts(y_pred, y_true, self._threshold).tolist()
        self._correct += correct
        self._total += total
