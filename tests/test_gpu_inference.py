"""Parity of the bf16 inference variant (scores and fused top-k) with the CPU oracle.

The reference has neither a bf16 registration nor a top-k op, so the expected values come from the
oracle's fp32 forward (tfsparse/cc/kernels/forward.cpp:9-44 restated) applied to inputs rounded to
bf16 with round-to-nearest-even, and from the oracle's top-k, whose tie rule (lower label first,
as tf.nn.top_k) no reference test covers: "parity unpinned" for the tie rule.

Gates: against the oracle on the SAME rounded inputs max|a-b|/max|ref| <= 1e-5 (only the summation
order differs); against the oracle on the unrounded fp32 inputs <= 1e-2, the tolerance the
benchmark configuration names.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import load_package, rel_err

pytestmark = pytest.mark.gpu

SAME_INPUT_RTOL = 1e-5
FP32_INPUT_RTOL = 1e-2

#          B     N     L    K  transposed
SHAPES = [(512, 1000, 3000, 64, False),
          (37, 513, 1001, 7, False),
          (8, 64, 5, 1, False),
          (600, 2000, 700, 72, True),
          (1030, 300, 129, 65, False),
          (512, 4096, 2048, 64, True),    # aligned [N,B] input: used in place, no staging copy
          (130, 70000, 260, 33, False)]   # ids above 16 bits


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


def make_case(shape, seed, sorted_rows=True):
    B, N, L, K, tp = shape
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    lookup = np.stack([rng.choice(N, size=K, replace=False) for _ in range(L)]).astype(np.int32)
    if sorted_rows:
        lookup.sort(axis=1)
    w = (rng.standard_normal((L, K)) / np.sqrt(K)).astype(np.float32)
    if tp:
        x = np.ascontiguousarray(x.T)
    return x, lookup, w


def to_bf16(a):
    """Device bf16 tensor holding exactly the oracle's rounding of `a`."""
    r = oracle.round_bf16(a)
    t = torch.from_numpy(r).cuda().to(torch.bfloat16)
    assert torch.equal(t.float().cpu(), torch.from_numpy(r))     # the conversion lost nothing
    return r, t


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "B%d_N%d_L%d_K%d_%s" % (s[0], s[1], s[2], s[3], "tp" if s[4] else "nt"))
def test_bf16_scores_match_oracle(ffi, shape):
    x, lookup, w = make_case(shape, 11)
    xr, dx = to_bf16(x)
    wr, dw = to_bf16(w)
    got = ffi.fixed_fan_in_ops.fan_in_sparse_matmul_bf16(dx, torch.from_numpy(lookup).cuda(), dw, transposed=shape[4])
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    assert np.isfinite(got).all()
    want_same = oracle.forward(xr, lookup, wr, transposed=shape[4])
    want_fp32 = oracle.forward(x, lookup, w, transposed=shape[4])
    assert rel_err(got, want_same) <= SAME_INPUT_RTOL
    assert rel_err(got, want_fp32) <= FP32_INPUT_RTOL


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "B%d_N%d_L%d_K%d_%s" % (s[0], s[1], s[2], s[3], "tp" if s[4] else "nt"))
@pytest.mark.parametrize("k", [1, 5, 8])
def test_fused_topk_matches_oracle(ffi, shape, k):
    x, lookup, w = make_case(shape, 12)
    xr, dx = to_bf16(x)
    wr, dw = to_bf16(w)
    dl = torch.from_numpy(lookup).cuda()
    ops = ffi.fixed_fan_in_ops
    values, labels = ops.fan_in_sparse_topk_bf16(dx, dl, dw, k=k, transposed=shape[4])
    scores = ops.fan_in_sparse_matmul_bf16(dx, dl, dw, transposed=shape[4])
    torch.cuda.synchronize()
    values, labels, scores = values.cpu().numpy(), labels.cpu().numpy(), scores.cpu().numpy()
    # (1) the fused kernel selects exactly the top-k of the scores the unfused kernel writes
    ov, oi = oracle.topk(scores, k)
    np.testing.assert_array_equal(labels, oi)
    np.testing.assert_array_equal(values, ov)
    # (2) against the oracle's own scores: values within tolerance, and every reported label is a
    #     legitimate member of the oracle's top-k up to that tolerance (near-ties may swap)
    want = oracle.forward(xr, lookup, wr, transposed=shape[4])
    wv, _ = oracle.topk(want, k)
    tol = SAME_INPUT_RTOL * np.abs(want).max()
    kk = min(k, shape[2])
    assert np.abs(values[:, :kk] - wv[:, :kk]).max() <= tol
    picked = np.take_along_axis(want, labels[:, :kk].astype(np.int64), axis=1)
    assert (picked >= wv[:, kk - 1:kk] - tol).all()
    if shape[2] < k:
        assert (labels[:, shape[2]:] == -1).all() and np.isneginf(values[:, shape[2]:]).all()


def test_fused_topk_ties_go_to_lower_label(ffi):
    # small-integer features and weights: scores are exact small integers with many ties
    B, N, L, K = 70, 40, 900, 4
    rng = np.random.default_rng(5)
    x = rng.integers(0, 3, size=(B, N)).astype(np.float32)
    w = rng.integers(-1, 2, size=(L, K)).astype(np.float32)
    lookup = np.stack([rng.choice(N, size=K, replace=False) for _ in range(L)]).astype(np.int32)
    _, dx = to_bf16(x)
    _, dw = to_bf16(w)
    values, labels = ffi.fixed_fan_in_ops.fan_in_sparse_topk_bf16(dx, torch.from_numpy(lookup).cuda(), dw, k=8)
    torch.cuda.synchronize()
    want = oracle.forward(x, lookup, w)
    ov, oi = oracle.topk(want, 8)
    assert (ov[:, :-1] == ov[:, 1:]).any()                      # the case really has ties inside the top 8
    np.testing.assert_array_equal(values.cpu().numpy(), ov)
    np.testing.assert_array_equal(labels.cpu().numpy(), oi)


@pytest.mark.parametrize("B,L,k", [(3, 100000, 5), (64, 5000, 8), (700, 333, 1), (2, 3, 5), (1, 1, 1)])
def test_topk_of_score_matrix(ffi, B, L, k):
    rng = np.random.default_rng(B * 7 + L)
    scores = rng.standard_normal((B, L)).astype(np.float32)
    scores = np.round(scores * 8) / 8 if L > 1000 else scores      # coarse grid: plenty of equal scores
    values, labels = ffi.fixed_fan_in_ops.topk_scores(torch.from_numpy(scores).cuda(), k=k)
    torch.cuda.synchronize()
    ov, oi = oracle.topk(scores, k)
    np.testing.assert_array_equal(values.cpu().numpy(), ov)
    np.testing.assert_array_equal(labels.cpu().numpy(), oi)


def test_inference_argument_errors(ffi):
    ops = ffi.fixed_fan_in_ops
    x = torch.zeros((4, 8), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((5, 2), dtype=torch.bfloat16, device="cuda")
    lookup = torch.zeros((5, 2), dtype=torch.int32, device="cuda")
    with pytest.raises(TypeError):
        ops.fan_in_sparse_matmul_bf16(x.float(), lookup, w)
    with pytest.raises(ffi._lib.FfiError):
        ops.fan_in_sparse_topk_bf16(x, lookup, w, k=9)
    with pytest.raises(ffi._lib.FfiError):
        ops.fan_in_sparse_topk_bf16(x, lookup, w, k=0)
    with pytest.raises(RuntimeError):
        ops.fan_in_sparse_matmul_bf16(x.cpu(), lookup.cpu(), w.cpu())
