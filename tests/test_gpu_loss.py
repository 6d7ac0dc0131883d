"""The producer of out_grad: losses on sparse label matrices (sparse/metrics.py:132-173) through the
C ABI, alone (`ffi_loss_grad_f32`) and fused into the forward kernel (`ffi_forward_loss_f32`),
against the numpy oracle (pinned in tests/test_oracle.py by known values, a dense autograd
restatement and central differences).

Gates: gradients and loss sums within 1e-5 of the largest reference magnitude; where the loss
consumes scores computed on the GPU, the oracle is fed the oracle's own forward scores, and
entries within 1e-5 of a kink of the hinge (margin exactly 1) are left out of the comparison.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from conftest import load_package, rel_err

pytestmark = pytest.mark.gpu

RTOL = 1e-5
KINDS = [oracle.LOSS_HINGE, oracle.LOSS_SQUARED_HINGE, oracle.LOSS_BCE]


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


def label_list(rng, B, L, per_sample=5, values=True):
    rows, cols = [], []
    for b in range(B):
        c = rng.choice(L, size=min(per_sample, L), replace=False)
        rows += [b] * len(c)
        cols += list(np.sort(c))
    indices = np.stack([np.array(rows), np.array(cols)], axis=1).astype(np.int64)
    vals = rng.choice([1.0, 1.0, 1.0, 0.5], size=len(rows)).astype(np.float32) if values else None
    return indices, vals


def away_from_kinks(scores, indices, values, kind, tol=1e-5):
    """Mask of entries whose hinge margin is not within `tol` of 1 (where the hinge slope jumps)."""
    if kind != oracle.LOSS_HINGE:
        return np.ones(scores.shape, bool)
    y = np.zeros(scores.shape)
    if len(indices):
        y[indices[:, 0], indices[:, 1]] = 1.0 if values is None else values
    return np.abs(1.0 - (2.0 * y - 1.0) * scores) > tol


def call_loss_grad(ffi, scores_t, indices, values, kind, scale, in_place=False):
    lib = ffi._lib.lib()
    B, L = scores_t.shape
    idx_t = torch.from_numpy(indices).cuda() if len(indices) else None
    val_t = torch.from_numpy(values).cuda() if values is not None and len(values) else None
    g = scores_t if in_place else torch.full_like(scores_t, float("nan"))
    loss = torch.full((1,), float("nan"), device="cuda")
    ffi._lib.check(lib.ffi_loss_grad_f32(scores_t.data_ptr(), idx_t.data_ptr() if idx_t is not None else None,
                                         val_t.data_ptr() if val_t is not None else None, len(indices), kind,
                                         ctypes.c_float(scale), g.data_ptr(), loss.data_ptr(), None, B, L,
                                         torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return g.cpu().numpy(), float(loss.cpu()[0])


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(128, 5000), (37, 1001), (3, 7), (1, 1), (64, 4099)])
def test_loss_grad_against_oracle(ffi, kind, shape):
    B, L = shape
    rng = np.random.default_rng(B * 131 + L + kind)
    scores = rng.normal(-0.5, 1.5, (B, L)).astype(np.float32)
    indices, values = label_list(rng, B, L, per_sample=min(5, L))
    scale = 1.0 / (B * L)
    losses, grad = oracle.sparse_loss(scores, indices, values, kind)
    g, loss_sum = call_loss_grad(ffi, torch.from_numpy(scores).cuda(), indices, values, kind, scale)
    ok = away_from_kinks(scores, indices, values, kind)
    assert rel_err(np.where(ok, g, 0), np.where(ok, grad * scale, 0)) <= RTOL
    assert abs(loss_sum - losses.sum()) <= RTOL * abs(losses.sum())


@pytest.mark.parametrize("kind", KINDS)
def test_loss_grad_in_place_and_default_values(ffi, kind):
    # out_grad may be the score buffer itself; label_values NULL means all ones
    B, L = 33, 777
    rng = np.random.default_rng(kind)
    scores = rng.normal(0, 1, (B, L)).astype(np.float32)
    indices, _ = label_list(rng, B, L, values=False)
    losses, grad = oracle.sparse_loss(scores, indices, None, kind)
    g, loss_sum = call_loss_grad(ffi, torch.from_numpy(scores).cuda(), indices, None, kind, 0.25, in_place=True)
    ok = away_from_kinks(scores, indices, None, kind)
    assert rel_err(np.where(ok, g, 0), np.where(ok, grad * 0.25, 0)) <= RTOL
    assert abs(loss_sum - losses.sum()) <= RTOL * abs(losses.sum())


def test_loss_grad_no_labels_and_skipped_pairs(ffi):
    # nnz = 0 (NULL lists); pairs outside the matrix are skipped and change nothing
    B, L = 16, 300
    rng = np.random.default_rng(9)
    scores = rng.normal(0, 1, (B, L)).astype(np.float32)
    empty = np.zeros((0, 2), np.int64)
    losses, grad = oracle.sparse_loss(scores, empty, None, oracle.LOSS_SQUARED_HINGE)
    g, loss_sum = call_loss_grad(ffi, torch.from_numpy(scores).cuda(), empty, None, oracle.LOSS_SQUARED_HINGE, 1.0)
    assert rel_err(g, grad) <= RTOL and abs(loss_sum - losses.sum()) <= RTOL * losses.sum()
    good = np.array([[2, 5], [7, 299]], np.int64)
    bad = np.array([[B, 0], [0, L], [-1, 3], [3, -1]], np.int64)
    losses, grad = oracle.sparse_loss(scores, good, None, oracle.LOSS_SQUARED_HINGE)
    g, loss_sum = call_loss_grad(ffi, torch.from_numpy(scores).cuda(), np.concatenate([good, bad]), None,
                                 oracle.LOSS_SQUARED_HINGE, 1.0)
    assert rel_err(g, grad) <= RTOL and abs(loss_sum - losses.sum()) <= RTOL * losses.sum()


def test_loss_grad_argument_errors(ffi):
    lib = ffi._lib.lib()
    s = torch.zeros((4, 8), device="cuda")
    g = torch.zeros_like(s)
    sh = torch.cuda.current_stream().cuda_stream
    one = ctypes.c_float(1.0)
    assert lib.ffi_loss_grad_f32(None, None, None, 0, 2, one, g.data_ptr(), None, None, 4, 8, sh) == -1
    assert lib.ffi_loss_grad_f32(s.data_ptr(), None, None, 3, 2, one, g.data_ptr(), None, None, 4, 8, sh) == -1   # nnz without a list
    assert lib.ffi_loss_grad_f32(s.data_ptr(), None, None, 0, 7, one, g.data_ptr(), None, None, 4, 8, sh) == -8   # unknown loss
    assert lib.ffi_loss_grad_f32(s.data_ptr(), None, None, 0, 2, one, g.data_ptr(), None, None, 0, 8, sh) == -2
    assert lib.ffi_loss_grad_f32(s.data_ptr(), None, None, -1, 2, one, g.data_ptr(), None, None, 4, 8, sh) == -2
    assert lib.ffi_loss_grad_f32(s.data_ptr(), None, None, 0, 2, one, g.data_ptr(), None, None, 4, 8, sh) == 0    # loss_sum may be NULL
    f = lib.ffi_forward_loss_f32
    assert f(s.data_ptr(), s.data_ptr(), s.data_ptr(), None, None, None, 0, 2, one, g.data_ptr(), g.data_ptr(), None, None,
             4, 8, 4, 2, 0, sh) == -8                                                                        # scores == out_grad


#           B    N     L     K  transposed
FUSED = [(128, 768, 5000, 32, True),
         (37, 300, 1001, 7, False),
         (64, 512, 2100, 64, True),
         (33, 3000, 333, 12, True),        # wide inputs: forward kernel, then the loss as a pass of its own
         (130, 2048, 260, 72, False),
         (1, 17, 65, 3, False),            # one sample
         (65, 1216, 1025, 33, True),       # the widest LDS tile, three batch tiles with one row in the last
         (50, 1217, 700, 16, False),       # one column more: the wide kernels
         (200, 64, 3000, 100, True),       # four register chunks per label
         (31, 768, 1023, 32, False)]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", FUSED)
@pytest.mark.parametrize("want_scores,use_bias", [(False, True), (True, True), (False, False)])
def test_forward_loss_fused_against_oracle(ffi, kind, shape, want_scores, use_bias):
    B, N, L, K, tp = shape
    rng = np.random.default_rng(B + N + L + K + kind)
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = (rng.standard_normal((L, K)) * 0.4).astype(np.float32)
    bias = (rng.standard_normal(L) * 0.5 - 0.5).astype(np.float32) if use_bias else None
    indices, values = label_list(rng, B, L)
    feats = np.ascontiguousarray(x.T) if tp else x
    ref_scores = oracle.forward(feats, lookup, w, transposed=tp)
    if use_bias:
        ref_scores = ref_scores + bias[None, :]
    losses, grad = oracle.sparse_loss(ref_scores, indices, values, kind)
    scale = 1.0 / (B * L)

    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    scores_t, g_t, loss_t = ffi.metrics.forward_loss(dev(feats), dev(lookup), dev(w), dev(bias) if use_bias else None,
                                                     (dev(indices), dev(values)), kind, transposed=tp, want_scores=want_scores)
    torch.cuda.synchronize()
    if want_scores:
        assert rel_err(scores_t.cpu().numpy(), ref_scores) <= RTOL
    else:
        assert scores_t is None
    # a score differs from the oracle's by rounding (1e-5 gate); the gradient inherits that difference,
    # scaled by the loss's curvature (at most 2), except across a kink of the hinge
    ok = away_from_kinks(ref_scores, indices, values, kind, tol=2 * RTOL * max(1.0, float(np.abs(ref_scores).max())))
    g = g_t.cpu().numpy()
    assert np.abs(np.where(ok, g - grad * scale, 0)).max() <= 4 * RTOL * scale * max(1.0, np.abs(ref_scores).max())
    assert abs(float(loss_t.cpu()[0]) - losses.sum()) <= RTOL * abs(losses.sum())


def test_fused_loss_trains_like_the_unfused_ops(ffi):
    # loss.fused(...) and loss(y, op(...) ) are the same differentiable function: equal value and gradients
    B, N, L, K = 64, 256, 3000, 16
    g = torch.Generator(device="cuda").manual_seed(5)
    x = torch.rand((B, N), device="cuda", generator=g)
    lookup = torch.randint(0, N, (L, K), device="cuda", generator=g, dtype=torch.int64).to(torch.int32)
    rng = np.random.default_rng(1)
    indices, _ = label_list(rng, B, L, values=False)
    y = (torch.from_numpy(indices).cuda(), None)
    loss_fn = ffi.SparseSquaredHingeLoss()
    results = []
    for fused in (False, True):
        w = ((torch.arange(L * K, device="cuda", dtype=torch.float32).reshape(L, K) % 13) / 13 - 0.5).requires_grad_(True)
        bias = torch.full((L,), -0.3, device="cuda", requires_grad=True)
        xin = x.clone().requires_grad_(True)
        if fused:
            loss, _ = loss_fn.fused(xin, lookup, w, bias, y)
        else:
            loss = loss_fn(y, ffi.fan_in_sparse_matmul_bias(xin, lookup, w, bias))
        loss.backward()
        torch.cuda.synchronize()
        results.append((float(loss.detach()), w.grad.cpu().numpy(), bias.grad.cpu().numpy(), xin.grad.cpu().numpy()))
    (l0, gw0, gb0, gx0), (l1, gw1, gb1, gx1) = results
    assert abs(l0 - l1) <= 1e-5 * abs(l0)
    assert rel_err(gw1, gw0) <= 1e-4 and rel_err(gb1, gb0) <= 1e-4 and rel_err(gx1, gx0) <= 1e-4
    # and the value is the reference's: mean over labels, then over the batch
    scores = oracle.forward(x.cpu().numpy(), lookup.cpu().numpy(), w.detach().cpu().numpy()) - 0.3
    losses, _ = oracle.sparse_loss(scores, indices, None, oracle.LOSS_SQUARED_HINGE)
    assert abs(l0 - losses.mean(axis=-1).mean()) <= 1e-5 * losses.mean()


@pytest.mark.parametrize("fused", [False, True])
def test_upstream_factor_scales_every_gradient(ffi, fused):
    # (factor * loss).backward(): autograd hands the factor to the loss op as a device scalar; all gradients
    # carry it, checked against the oracle's backward pass of the oracle's loss gradient
    B, N, L, K, factor = 48, 200, 2500, 12, 3.5
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.rand((B, N), device="cuda", generator=g)
    lookup = torch.randint(0, N, (L, K), device="cuda", generator=g, dtype=torch.int64).to(torch.int32)
    rng = np.random.default_rng(4)
    indices, _ = label_list(rng, B, L, values=False)
    y = (torch.from_numpy(indices).cuda(), None)
    w = ((torch.arange(L * K, device="cuda", dtype=torch.float32).reshape(L, K) % 11) / 11 - 0.5).requires_grad_(True)
    bias = torch.full((L,), -0.2, device="cuda", requires_grad=True)
    xin = x.clone().requires_grad_(True)
    loss_fn = ffi.SparseSquaredHingeLoss()
    if fused:
        loss, _ = loss_fn.fused(xin, lookup, w, bias, y)
    else:
        loss = loss_fn(y, ffi.fan_in_sparse_matmul_bias(xin, lookup, w, bias))
    (loss * factor).backward()
    torch.cuda.synchronize()
    xn, ln, wn = x.cpu().numpy(), lookup.cpu().numpy(), w.detach().cpu().numpy()
    scores = oracle.forward(xn, ln, wn) - 0.2
    _, grad = oracle.sparse_loss(scores, indices, None, oracle.LOSS_SQUARED_HINGE)
    out_grad = (grad * (factor / (B * L))).astype(np.float32)
    ref_gx, ref_gw = oracle.backward(xn, ln, wn, out_grad)
    assert rel_err(w.grad.cpu().numpy(), ref_gw) <= 1e-4
    assert rel_err(xin.grad.cpu().numpy(), ref_gx) <= 1e-4
    assert rel_err(bias.grad.cpu().numpy(), out_grad.sum(axis=0)) <= 1e-4


def test_loss_sum_is_reproducible(ffi):
    B, L = 128, 20000
    rng = np.random.default_rng(2)
    scores = torch.from_numpy(rng.normal(0, 1, (B, L)).astype(np.float32)).cuda()
    indices, values = label_list(rng, B, L)
    a = call_loss_grad(ffi, scores, indices, values, oracle.LOSS_SQUARED_HINGE, 1.0)
    b = call_loss_grad(ffi, scores, indices, values, oracle.LOSS_SQUARED_HINGE, 1.0)
    assert a[1] == b[1] and np.array_equal(a[0], b[0])


@pytest.mark.parametrize("k", [1, 3, 5])
def test_precision_at_k(ffi, k):
    # sparse/metrics.py:31-71: label values at the k best-scored positions, over batch * k
    B, L = 50, 4000
    rng = np.random.default_rng(k)
    scores = rng.normal(0, 1, (B, L)).astype(np.float32)
    indices, _ = label_list(rng, B, L, per_sample=4, values=False)
    for b in range(0, B, 2):                      # make some labels rank high
        scores[b, indices[indices[:, 0] == b][0, 1]] += 10.0
    truth = np.zeros((B, L), bool)
    truth[indices[:, 0], indices[:, 1]] = True
    top = np.argsort(-scores, axis=1, kind="stable")[:, :k]
    expected = truth[np.arange(B)[:, None], top].sum() / (B * k)
    metric = ffi.PrecisionAtK(k=k)
    metric.update_state((torch.from_numpy(indices).cuda(), None), torch.from_numpy(scores).cuda())
    assert abs(metric.result() - expected) < 1e-12
    metric.update_state((torch.from_numpy(indices).cuda(), None), torch.from_numpy(scores).cuda())
    assert abs(metric.result() - expected) < 1e-12          # accumulates numerator and denominator


@pytest.mark.parametrize("shape", [(128, 5000), (37, 1001), (1, 3)])
@pytest.mark.parametrize("threshold", [0.0, 0.7])
def test_threshold_metrics_against_oracle(ffi, shape, threshold):
    # SparsePrecision / SparseRecall (sparse/metrics.py:73-129): exact counts, so exact equality
    B, L = shape
    rng = np.random.default_rng(B + L)
    scores = rng.normal(0, 1, (B, L)).astype(np.float32)
    scores[0, 0] = threshold                                   # on the threshold is not above it
    indices, values = label_list(rng, B, L, per_sample=min(4, L))
    values = np.round(values * 4) / 4                          # exactly representable sums
    predicted, correct, total = oracle.threshold_counts(scores, indices, values, threshold)
    y = (torch.from_numpy(indices).cuda(), torch.from_numpy(values).cuda())
    got = ffi.metrics.threshold_counts(torch.from_numpy(scores).cuda(), y, threshold).cpu().numpy()
    assert tuple(got) == (predicted, correct, total)
    prec, rec = ffi.SparsePrecision(threshold), ffi.SparseRecall(threshold)
    for _ in range(2):
        prec.update_state(y, torch.from_numpy(scores).cuda())
        rec.update_state(y, torch.from_numpy(scores).cuda())
    assert abs(prec.result() - (correct / predicted if predicted else 0.0)) < 1e-12
    assert abs(rec.result() - correct / total) < 1e-12


def test_unaligned_score_buffers(ffi):
    # scores / out_grad that start 4 bytes into an allocation (a view): no 16-byte accesses may be assumed
    B, L = 19, 1003
    rng = np.random.default_rng(77)
    scores = rng.normal(0, 1, (B, L)).astype(np.float32)
    indices, values = label_list(rng, B, L)
    y = (torch.from_numpy(indices).cuda(), torch.from_numpy(values).cuda())
    base = torch.empty(B * L + 1, device="cuda")
    view = base[1:].view(B, L)
    view.copy_(torch.from_numpy(scores))
    assert view.data_ptr() % 16 == 4
    losses, grad = oracle.sparse_loss(scores, indices, values, oracle.LOSS_SQUARED_HINGE)
    g, loss_sum = ffi.metrics.sparse_loss_grad(view, y, oracle.LOSS_SQUARED_HINGE, grad_scale=1.0)
    torch.cuda.synchronize()
    assert rel_err(g.cpu().numpy(), grad) <= RTOL and abs(float(loss_sum) - losses.sum()) <= RTOL * losses.sum()
    got = ffi.metrics.threshold_counts(view, y, 0.0).cpu().numpy()
    assert tuple(got) == oracle.threshold_counts(scores, indices, values, 0.0)
    g2, _ = ffi.metrics.sparse_loss_grad(view, y, oracle.LOSS_SQUARED_HINGE, grad_scale=1.0, in_place=True)
    torch.cuda.synchronize()
    assert g2.data_ptr() == view.data_ptr() and rel_err(view.cpu().numpy(), grad) <= RTOL


@pytest.mark.parametrize("shape", [(128, 768, 20000, 32, True), (37, 300, 9001, 7, False), (33, 3000, 5000, 12, True)])
def test_forward_loss_with_topk_by_product(ffi, shape):
    # loss gradient, masks, loss sum and the top-5 of the scores from one forward pass; the top-5 equals that of the
    # separately written score matrix, the rest is unchanged by asking for it
    B, N, L, K, tp = shape
    rng = np.random.default_rng(sum(shape[:4]))
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = (rng.standard_normal((L, K)) * 0.4).astype(np.float32)
    bias = np.full(L, -1.0, np.float32)
    indices, values = label_list(rng, B, L)
    feats = np.ascontiguousarray(x.T) if tp else x
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    y = (dev(indices), dev(values))
    args = (dev(feats), dev(lookup), dev(w), dev(bias), y, oracle.LOSS_SQUARED_HINGE)
    scores, g0, l0, m0 = ffi.metrics.forward_loss(*args, transposed=tp, want_scores=True, want_masks=True)
    none, g1, l1, m1, (tv, ti) = ffi.metrics.forward_loss(*args, transposed=tp, want_masks=True, topk=5)
    torch.cuda.synchronize()
    assert none is None
    ref_v, ref_i = oracle.topk(scores.cpu().numpy(), 5)
    assert np.array_equal(ti.cpu().numpy(), ref_i) and np.array_equal(tv.cpu().numpy(), ref_v)
    assert torch.equal(m0, m1) and float(l0) == float(l1)
    assert rel_err(g1.cpu().numpy(), g0.cpu().numpy()) <= RTOL
    p5 = ffi.PrecisionAtK(k=5)
    p5.update_from_topk(y, ti, L)
    truth = np.zeros((B, L), np.float32)
    truth[indices[:, 0], indices[:, 1]] = values
    assert abs(p5.result() - truth[np.arange(B)[:, None], ref_i].sum() / (B * 5)) < 1e-9


def test_topk_as_matrix(ffi):
    # sparse/metrics.py:9-28: a 0/1 matrix with k ones per row at the best scores, indices in row-major order
    rng = np.random.default_rng(8)
    scores = rng.standard_normal((9, 300)).astype(np.float32)
    indices, values, shape = ffi.topk_as_matrix(torch.from_numpy(scores).cuda(), 3)
    torch.cuda.synchronize()
    assert shape == (9, 300) and values.tolist() == [1.0] * 27
    _, oi = oracle.topk(scores, 3)
    expect = np.stack([np.repeat(np.arange(9), 3), np.sort(oi, axis=1).reshape(-1)], axis=1)
    assert np.array_equal(indices.cpu().numpy(), expect)
