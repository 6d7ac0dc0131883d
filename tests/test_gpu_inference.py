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


# ---- fp32 forward with fused top-k (no score matrix) ------------------------------------------------------------
#            B    N     L      K  transposed
TOPK_F32 = [(128, 768, 20000, 32, True),
            (37, 300, 9001, 7, False),
            (64, 512, 12000, 64, True),
            (5, 96, 700, 40, False),          # fewer labels than the threshold sample
            (3, 16, 3, 4, False),             # fewer labels than k: the missing places are (-inf, -1) as in the oracle
            (40, 1216, 6000, 16, True),       # the widest input whose tile of x fits in LDS
            (33, 3000, 5000, 12, True)]       # wide inputs: scores, then their top-k


@pytest.mark.parametrize("k", [1, 5, 8])
@pytest.mark.parametrize("shape", TOPK_F32)
def test_fp32_topk_without_the_score_matrix(ffi, shape, k):
    # exact: the labels and scores are those of the top-k (tf.nn.top_k order) of the scores the same kernel writes
    B, N, L, K, tp = shape
    rng = np.random.default_rng(sum(shape[:4]) + k)
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = rng.standard_normal((L, K)).astype(np.float32)
    bias = (rng.standard_normal(L) * 0.3).astype(np.float32)
    feats = np.ascontiguousarray(x.T) if tp else x
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    v1, i1, scores = ffi.fan_in_sparse_topk(dev(feats), dev(lookup), dev(w), dev(bias), k=k, transposed=tp, want_scores=True)
    v2, i2 = ffi.fan_in_sparse_topk(dev(feats), dev(lookup), dev(w), dev(bias), k=k, transposed=tp)
    torch.cuda.synchronize()
    sc = scores.cpu().numpy()
    ref_v, ref_i = oracle.topk(sc, k)
    assert np.array_equal(i1.cpu().numpy(), ref_i) and np.array_equal(v1.cpu().numpy(), ref_v)
    assert np.array_equal(i2.cpu().numpy(), ref_i) and np.array_equal(v2.cpu().numpy(), ref_v)
    # and the scores are the layer's
    assert rel_err(sc, oracle.forward(feats, lookup, w, transposed=tp) + bias[None, :]) <= 1e-5


def test_fp32_topk_with_ties_and_cancellation(ffi):
    # many exactly equal scores (ties broken by label) and scores that are sums of large cancelling terms
    B, N, L, K = 40, 64, 9000, 4
    rng = np.random.default_rng(3)
    x = rng.integers(-3, 4, (B, N)).astype(np.float32) * 1000.0
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = rng.integers(-2, 3, (L, K)).astype(np.float32)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    v, i, scores = ffi.fan_in_sparse_topk(dev(x), dev(lookup), dev(w), None, k=8, want_scores=True)
    v2, i2 = ffi.fan_in_sparse_topk(dev(x), dev(lookup), dev(w), None, k=8)
    torch.cuda.synchronize()
    ref_v, ref_i = oracle.topk(scores.cpu().numpy(), 8)
    assert np.array_equal(i.cpu().numpy(), ref_i) and np.array_equal(v.cpu().numpy(), ref_v)
    assert np.array_equal(i2.cpu().numpy(), ref_i)


def test_fp32_topk_with_a_run_of_high_scores(ffi):
    # 300 neighbouring labels beat every other one: one workgroup meets far more candidates of a sample than it parks
    B, N, L, K = 6, 128, 30000, 8
    rng = np.random.default_rng(11)
    x = np.abs(rng.standard_normal((B, N))).astype(np.float32)
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = rng.standard_normal((L, K)).astype(np.float32)
    w[7000:7300] = np.abs(w[7000:7300]) + 5.0
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    v, i, scores = ffi.fan_in_sparse_topk(dev(x), dev(lookup), dev(w), None, k=8, want_scores=True)
    v2, i2 = ffi.fan_in_sparse_topk(dev(x), dev(lookup), dev(w), None, k=8)
    torch.cuda.synchronize()
    ref_v, ref_i = oracle.topk(scores.cpu().numpy(), 8)
    assert (ref_i >= 7000).all() and (ref_i < 7300).all()
    assert np.array_equal(i.cpu().numpy(), ref_i) and np.array_equal(v.cpu().numpy(), ref_v)
    assert np.array_equal(i2.cpu().numpy(), ref_i) and np.array_equal(v2.cpu().numpy(), ref_v)


def test_fp32_topk_argument_errors(ffi):
    x = torch.zeros((4, 16), device="cuda")
    lookup = torch.zeros((5, 2), dtype=torch.int32, device="cuda")
    w = torch.zeros((5, 2), device="cuda")
    for k in (0, 9):
        with pytest.raises(ffi._lib.FfiError):
            ffi.fan_in_sparse_topk(x, lookup, w, None, k=k)
    with pytest.raises(ValueError):
        ffi.fan_in_sparse_topk(x, lookup, w, torch.zeros(4, device="cuda"), k=1)      # bias of the wrong length
    with pytest.raises(RuntimeError):
        ffi.fan_in_sparse_topk(x.cpu(), lookup.cpu(), w.cpu(), None, k=1)


def test_fp32_topk_when_a_candidate_list_overflows(ffi):
    # every label ties with the best score: no list of 8192 candidates can hold them; the sample is then answered from a
    # scan of its whole row, and ties go to the lower labels as tf.nn.top_k (sparse/metrics.py:19) resolves them
    B, N, L, K = 3, 16, 20000, 2
    x = torch.ones((B, N), device="cuda")
    lookup = torch.zeros((L, K), dtype=torch.int32, device="cuda")
    w = torch.ones((L, K), device="cuda")
    for want_scores in (False, True):
        out = ffi.fan_in_sparse_topk(x, lookup, w, None, k=3, want_scores=want_scores)
        torch.cuda.synchronize()
        v, i = out[0], out[1]
        assert i.cpu().numpy().tolist() == [[0, 1, 2]] * B
        assert bool((v == 2.0).all())


def test_fp32_topk_of_an_all_zero_feature_row(ffi):
    # what validation data does hold: a sample without features.  Its scores are the bias (zero-initialised: all labels
    # tie), while the other samples of the batch take the fast path.  ffi_topk_f32 on the stored scores (L > 65536:
    # the threshold filter) and the forward pass without a score matrix must both answer labels 0..k-1 for it
    B, N, L, K, k = 5, 96, 70000, 8, 5
    rng = np.random.default_rng(8)
    x = np.abs(rng.standard_normal((B, N))).astype(np.float32)
    x[2] = 0.0
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = rng.standard_normal((L, K)).astype(np.float32)
    bias = np.zeros(L, dtype=np.float32)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    v1, i1, scores = ffi.fan_in_sparse_topk(dev(x), dev(lookup), dev(w), dev(bias), k=k, want_scores=True)
    v2, i2 = ffi.fan_in_sparse_topk(dev(x), dev(lookup), dev(w), dev(bias), k=k)
    v3 = torch.empty((B, k), device="cuda")
    i3 = torch.empty((B, k), dtype=torch.int32, device="cuda")
    ffi._lib.check(ffi._lib.lib().ffi_topk_f32(scores.data_ptr(), B, L, k, v3.data_ptr(), i3.data_ptr(),
                                              torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    ref_v, ref_i = oracle.topk(scores.cpu().numpy(), k)
    assert ref_i[2].tolist() == list(range(k))
    for v, i in ((v1, i1), (v2, i2), (v3, i3)):
        assert np.array_equal(i.cpu().numpy(), ref_i) and np.array_equal(v.cpu().numpy(), ref_v)


def test_inference_config_full_size(ffi):
    # c5 at its full size (batch 512, 100,000 inputs, 670,091 labels, fan-in 64, sorted rows, bf16): the fused top-5 equals
    # the top-5 of the score matrix the unfused kernel writes, and a label slice of those scores meets both oracle gates
    from ecml23_sparse_amd import synth
    cfg = synth.CONFIGS["c5"]
    t = synth.make_inputs(cfg, seed=42, device="cuda", transposed=True)
    x, lookup, w = t["features"].to(torch.bfloat16), t["lookup"], t["weights"].to(torch.bfloat16)
    print("case config=c5 full size", flush=True)
    vals, labels = ffi.fan_in_sparse_topk_bf16(x, lookup, w, k=5, transposed=True)
    scores = ffi.fan_in_sparse_matmul_bf16(x, lookup, w, transposed=True)
    ref_v, ref_i = ffi.topk_scores(scores, 5)
    torch.cuda.synchronize()
    assert torch.equal(labels, ref_i) and torch.equal(vals, ref_v)
    # the device top-k itself, on a few samples, against the oracle's
    rows = scores[:4].cpu().numpy()
    o_v, o_i = oracle.topk(rows, 5)
    assert np.array_equal(ref_i[:4].cpu().numpy(), o_i) and np.array_equal(ref_v[:4].cpu().numpy(), o_v)
    sl = slice(123_000, 123_500)
    xs = x.float().cpu().numpy()
    ls, ws = lookup[sl].cpu().numpy(), w[sl].float().cpu().numpy()
    got = scores[:, sl].cpu().numpy()
    assert rel_err(got, oracle.forward(xs, ls, ws, transposed=True)) <= SAME_INPUT_RTOL
    x32 = t["features"].cpu().numpy()
    assert rel_err(got, oracle.forward(x32, ls, t["weights"][sl].cpu().numpy(), transposed=True)) <= FP32_INPUT_RTOL
