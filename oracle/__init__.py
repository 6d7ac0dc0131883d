"""CPU oracle for the fixed-fan-in sparse layer: TEST INFRASTRUCTURE, never the product path.

Thin ctypes binding over ``libffi_oracle.so`` (built from ``ffi_oracle.c`` by ``oracle/Makefile``)
plus a dense numpy restatement of the reference's own ground truth
(tfsparse/cc/kernels/reference.cpp:15-82) for small shapes.

Only the test-suite, ``__graft_entry__.smoke()`` and the CPU-baseline leg of ``bench.py`` import
this package.  All functions take and return numpy arrays.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libffi_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_i32p = ctypes.POINTER(ctypes.c_int32)
_i64 = ctypes.c_int64


def build(force: bool = False) -> str:
    """Compile the C restatement with the Makefile next to it; returns the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        common = [_i64, _i64, _i64, _i64, ctypes.c_int, ctypes.c_int]
        _lib.ffi_oracle_forward_f32.argtypes = [_f32p, _i32p, _f32p, _f32p] + common
        _lib.ffi_oracle_forward_f64.argtypes = [_f32p, _i32p, _f32p, _f64p] + common
        for name, outp in (("ffi_oracle_weight_grad_f32", _f32p), ("ffi_oracle_input_grad_f32", _f32p),
                           ("ffi_oracle_weight_grad_f64", _f64p), ("ffi_oracle_input_grad_f64", _f64p)):
            getattr(_lib, name).argtypes = [_f32p, _i32p, _f32p, _f32p, outp] + common
        _lib.ffi_oracle_backward_f32.argtypes = [_f32p, _i32p, _f32p, _f32p, _f32p, _f32p] + common
        for name in ("ffi_oracle_forward_f32", "ffi_oracle_forward_f64", "ffi_oracle_weight_grad_f32",
                     "ffi_oracle_input_grad_f32", "ffi_oracle_weight_grad_f64", "ffi_oracle_input_grad_f64",
                     "ffi_oracle_backward_f32"):
            getattr(_lib, name).restype = ctypes.c_int
        _lib.ffi_oracle_round_bf16_array.argtypes = [_f32p, _f32p, _i64]
        _lib.ffi_oracle_round_bf16_array.restype = None
        _lib.ffi_oracle_topk_f32.argtypes = [_f32p, _i64, _i64, ctypes.c_int, _f32p, _i32p]
        _lib.ffi_oracle_topk_f32.restype = None
    return _lib


def default_threads() -> int:
    """All hardware threads, as the reference's CPU harness does (testing/cpu.cpp:36-37)."""
    return max(1, os.cpu_count() or 1)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _idx(a):
    a = np.asarray(a)
    if a.dtype == np.uint32:
        a = a.view(np.int32)          # same bits; the C side widens through uint32_t
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a, a.ctypes.data_as(_i32p)


def _dims(features, lookup, transposed):
    if features.ndim != 2 or lookup.ndim != 2:
        raise ValueError("features and lookup must be matrices")
    if transposed:
        N, B = features.shape
    else:
        B, N = features.shape
    L, K = lookup.shape
    return B, N, L, K


def _check(rc, what):
    if rc != 0:
        raise RuntimeError(f"oracle {what} failed with status {rc}")


def forward(features, lookup, weights, transposed=False, threads=None, f64=False):
    """out[b,j] = sum_k weights[j,k] * features[b, lookup[j,k]]  (forward.cpp:9-44)."""
    features, fp = _f32(features)
    lookup, lp = _idx(lookup)
    weights, wp = _f32(weights)
    B, N, L, K = _dims(features, lookup, transposed)
    assert weights.shape == (L, K)
    threads = threads or default_threads()
    if f64:
        out = np.empty((B, L), dtype=np.float64)
        _check(lib().ffi_oracle_forward_f64(fp, lp, wp, out.ctypes.data_as(_f64p), B, N, L, K, int(transposed), threads), "forward_f64")
    else:
        out = np.empty((B, L), dtype=np.float32)
        _check(lib().ffi_oracle_forward_f32(fp, lp, wp, out.ctypes.data_as(_f32p), B, N, L, K, int(transposed), threads), "forward_f32")
    return out


def weight_grad(features, lookup, weights, out_grad, transposed=False, threads=None, f64=False):
    """gw[j,k] = sum_b features[b, lookup[j,k]] * out_grad[b,j]  (backward.cpp:8-36)."""
    features, fp = _f32(features)
    lookup, lp = _idx(lookup)
    weights, wp = _f32(weights)
    out_grad, gp = _f32(out_grad)
    B, N, L, K = _dims(features, lookup, transposed)
    assert out_grad.shape == (B, L)
    threads = threads or default_threads()
    if f64:
        gw = np.empty((L, K), dtype=np.float64)
        _check(lib().ffi_oracle_weight_grad_f64(fp, lp, wp, gp, gw.ctypes.data_as(_f64p), B, N, L, K, int(transposed), threads), "weight_grad_f64")
    else:
        gw = np.empty((L, K), dtype=np.float32)
        _check(lib().ffi_oracle_weight_grad_f32(fp, lp, wp, gp, gw.ctypes.data_as(_f32p), B, N, L, K, int(transposed), threads), "weight_grad_f32")
    return gw


def input_grad(features, lookup, weights, out_grad, transposed=False, threads=None, f64=False):
    """gx[b, lookup[j,k]] += weights[j,k] * out_grad[b,j]  (backward.cpp:39-73)."""
    features, fp = _f32(features)
    lookup, lp = _idx(lookup)
    weights, wp = _f32(weights)
    out_grad, gp = _f32(out_grad)
    B, N, L, K = _dims(features, lookup, transposed)
    assert out_grad.shape == (B, L)
    threads = threads or default_threads()
    # pre-filled with garbage, like the reference's tests do, so an unwritten element shows
    if f64:
        gx = np.full(features.shape, np.nan, dtype=np.float64)
        _check(lib().ffi_oracle_input_grad_f64(fp, lp, wp, gp, gx.ctypes.data_as(_f64p), B, N, L, K, int(transposed), threads), "input_grad_f64")
    else:
        gx = np.full(features.shape, np.nan, dtype=np.float32)
        _check(lib().ffi_oracle_input_grad_f32(fp, lp, wp, gp, gx.ctypes.data_as(_f32p), B, N, L, K, int(transposed), threads), "input_grad_f32")
    return gx


def backward(features, lookup, weights, out_grad, transposed=False, threads=None):
    """(feature_grad, weight_grad) in the order the grad op returns them (register.cpp:59-60)."""
    gw = weight_grad(features, lookup, weights, out_grad, transposed, threads)
    gx = input_grad(features, lookup, weights, out_grad, transposed, threads)
    return gx, gw


def round_bf16(a):
    """fp32 -> bf16 -> fp32 with round-to-nearest-even."""
    a, ap = _f32(a)
    out = np.empty_like(a)
    lib().ffi_oracle_round_bf16_array(ap, out.ctypes.data_as(_f32p), a.size)
    return out


def topk(scores, k):
    """Per-row top-k: values descending, ties resolved towards the lower index."""
    scores, sp = _f32(scores)
    B, L = scores.shape
    values = np.empty((B, k), dtype=np.float32)
    indices = np.empty((B, k), dtype=np.int32)
    lib().ffi_oracle_topk_f32(sp, B, L, int(k), values.ctypes.data_as(_f32p), indices.ctypes.data_as(_i32p))
    return values, indices


# ---- dense ground truth of the reference's own tests (reference.cpp:15-82), numpy float64 -------

def dense_operator(lookup, weights, num_features):
    """D[n, j] = sum of weights[j,k] over the k with lookup[j,k] == n  (reference.cpp:15-27)."""
    lookup = np.asarray(lookup).astype(np.int64)
    L, K = lookup.shape
    D = np.zeros((num_features, L), dtype=np.float64)
    np.add.at(D, (lookup.reshape(-1), np.repeat(np.arange(L), K)), np.asarray(weights, dtype=np.float64).reshape(-1))
    return D


def dense_forward(features, lookup, weights, transposed=False):
    """out = X . D  (reference.cpp:30-45)."""
    X = np.asarray(features, dtype=np.float64)
    if transposed:
        X = X.T
    return X @ dense_operator(lookup, weights, X.shape[1])


def dense_backward(features, lookup, weights, out_grad, transposed=False):
    """gx = G . D^T, gw[j,k] = (X^T G)[lookup[j,k], j]  (reference.cpp:48-82)."""
    X = np.asarray(features, dtype=np.float64)
    if transposed:
        X = X.T
    G = np.asarray(out_grad, dtype=np.float64)
    D = dense_operator(lookup, weights, X.shape[1])
    gx = G @ D.T
    if transposed:
        gx = gx.T
    dense_gw = X.T @ G
    lookup = np.asarray(lookup).astype(np.int64)
    L, K = lookup.shape
    gw = dense_gw[lookup, np.arange(L)[:, None]]
    return gx, gw


# ---- loss and its gradient with respect to the scores (numpy, float64 inside) --------------------
LOSS_HINGE, LOSS_SQUARED_HINGE, LOSS_BCE = 1, 2, 3


def cwise_loss(kind, score, y):
    """Element loss, sparse/metrics.py:142-144 (hinge), :152-154, :162-164 (squared hinge), :172-173 (bce:
    tf.nn.sigmoid_cross_entropy_with_logits = max(x,0) - x*z + log1p(exp(-|x|)))."""
    score = np.asarray(score, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    if kind == LOSS_BCE:
        return np.maximum(score, 0.0) - score * y + np.log1p(np.exp(-np.abs(score)))
    r = np.maximum(1.0 - (2.0 * y - 1.0) * score, 0.0)
    return r if kind == LOSS_HINGE else r * r


def cwise_loss_grad(kind, score, y):
    """d cwise_loss / d score; relu' is 0 at 0 (TensorFlow's ReluGrad passes the gradient where x > 0)."""
    score = np.asarray(score, dtype=np.float64)
    y = np.asarray(y, dtype=np.float64)
    if kind == LOSS_BCE:
        return 1.0 / (1.0 + np.exp(-score)) - y
    sign = 2.0 * y - 1.0
    r = np.maximum(1.0 - sign * score, 0.0)
    if kind == LOSS_HINGE:
        return np.where(r > 0.0, -sign, 0.0)
    return -2.0 * sign * r


def sparse_loss(scores, label_indices, label_values, kind):
    """SparseLossBase.call (sparse/metrics.py:136-139) through dense_sparse_cwise_op (sparse/utils.py:11-17):
    the dense part charges every entry loss(s, 0); the listed positions are overwritten with
    loss(s, value).  Returns (element losses [B,L], d sum(losses) / d scores [B,L]) in float64;
    the reference's per-sample value is ``losses.mean(axis=-1)``."""
    s = np.asarray(scores, dtype=np.float64)
    idx = np.asarray(label_indices, dtype=np.int64).reshape(-1, 2)
    vals = np.ones(len(idx)) if label_values is None else np.asarray(label_values, dtype=np.float64)
    losses = cwise_loss(kind, s, 0.0)
    grad = cwise_loss_grad(kind, s, 0.0)
    if len(idx):
        b, j = idx[:, 0], idx[:, 1]
        losses[b, j] = cwise_loss(kind, s[b, j], vals)
        grad[b, j] = cwise_loss_grad(kind, s[b, j], vals)
    return losses, grad


# ---- Adam (numpy, float32 like the variables) -----------------------------------------------------
def adam_step(variable, m, v, gradient, learning_rate=0.001, beta_1=0.9, beta_2=0.999, epsilon=1e-7, step=1):
    """One step of keras.optimizers.Adam, the base class of the reference's SparseAdam
    (sparse/optimizer.py:9-12; created in run.py:126).  TensorFlow is not part of the reference tree;
    this restates the published update_step of that class (Keras 2.11-2.15, the generation whose
    ``_momentums`` / ``_velocities`` / ``_index_dict`` fields sparse/optimizer.py:16-18 reads):
        alpha = lr * sqrt(1 - beta_2^t) / (1 - beta_1^t)
        m += (g - m) * (1 - beta_1);  v += (g^2 - v) * (1 - beta_2);  var -= (m * alpha) / (sqrt(v) + epsilon)
    all in float32.  Returns new (variable, m, v).  PARITY UNPINNED against the reference itself (it holds
    no optimizer test or vector); tests/test_oracle.py pins the arithmetic against the closed form of the
    first step and against torch.optim.Adam with the epsilon rescaled to Keras' placement."""
    f = np.float32
    var, m, v, g = (np.asarray(a, dtype=f).copy() for a in (variable, m, v, gradient))
    b1p, b2p = f(beta_1) ** f(step), f(beta_2) ** f(step)
    alpha = f(learning_rate) * np.sqrt(f(1) - b2p, dtype=f) / (f(1) - b1p)
    m += (g - m) * (f(1) - f(beta_1))
    v += (g * g - v) * (f(1) - f(beta_2))
    var -= (m * alpha) / (np.sqrt(v, dtype=f) + f(epsilon))
    return var, m, v


# ---- rewiring selection (numpy) --------------------------------------------------------------------
def select_threshold(weights, k):
    """The threshold of FixedFractionSelector.select (sparse/layer.py:75-86): ``tf.nn.top_k(-|w|, k)`` returns
    the k smallest magnitudes in ascending order of |w|, its last value is the k-th smallest; k == 0 is
    taken as 0.0 (nothing has a magnitude below it)."""
    mags = np.abs(np.asarray(weights, dtype=np.float32).reshape(-1))
    if k <= 0:
        return np.float32(0.0)
    return np.partition(mags, k - 1)[k - 1]


def rewire_selection(weights, threshold):
    """Boolean mask of the connections that are rewired: strictly below the threshold (sparse/layer.py:57,86)."""
    return np.abs(np.asarray(weights, dtype=np.float32)) < np.float32(threshold)


def threshold_counts(scores, label_indices, label_values, threshold):
    """(predicted, correct, total_true) as SparsePrecision / SparseRecall accumulate them (sparse/metrics.py:88-96,
    113-126): predicted = count(scores > threshold); correct = sum of label values at listed positions whose score
    is above the threshold; total_true = sum of all label values."""
    s = np.asarray(scores)
    idx = np.asarray(label_indices, dtype=np.int64).reshape(-1, 2)
    vals = np.ones(len(idx)) if label_values is None else np.asarray(label_values, dtype=np.float64)
    predicted = float(np.count_nonzero(s > np.float32(threshold)))
    hit = s[idx[:, 0], idx[:, 1]] > np.float32(threshold) if len(idx) else np.zeros(0, bool)
    return predicted, float((vals * hit).sum()), float(vals.sum())
