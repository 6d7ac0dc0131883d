"""Pins the CPU oracle (oracle/ffi_oracle.c) with evidence that does not come from the oracle:
the reference's known-answer test, committed dense-formulation fixtures, the dense and
scipy.sparse formulations on the reference's shape grid, and algebraic invariants chosen so that a
dropped term, a wrong index or a transposed operand fails at least one of them."""
import glob
import json
import os

import numpy as np
import pytest
import scipy.sparse as sp

import oracle
from conftest import GOLDEN, REFERENCE_SHAPES, reference_law_inputs, rel_err

SMALL_SHAPES = [s for s in REFERENCE_SHAPES if s[2] < 1_000_000]


def test_known_answer_forward_exact():
    # testing/test.cpp:13-47: exact equality, both layouts
    with open(os.path.join(GOLDEN, "kat_forward.json")) as f:
        kat = json.load(f)
    x = np.array(kat["features"], dtype=np.float32)
    lookup = np.array(kat["lookup"], dtype=np.int32)
    w = np.array(kat["weights"], dtype=np.float32)
    expected = np.array(kat["expected"], dtype=np.float32)
    assert np.array_equal(oracle.forward(x, lookup, w), expected)
    assert np.array_equal(oracle.forward(np.ascontiguousarray(x.T), lookup, w, transposed=True), expected)
    assert np.array_equal(oracle.forward(x, lookup.astype(np.uint32), w), expected)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "dense_*.npz"))))
@pytest.mark.parametrize("transposed", [False, True])
def test_golden_dense_fixtures(path, transposed):
    z = np.load(path)
    x, lookup, w, g = z["features"], z["lookup"], z["weights"], z["out_grad"]
    xin = np.ascontiguousarray(x.T) if transposed else x
    out = oracle.forward(xin, lookup, w, transposed=transposed)
    gx, gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
    if transposed:
        gx = gx.T
    # the reference's own absolute gates (test_case_templates.h:82,139-140), two-sided here
    assert np.abs(out - z["result"]).max() < 1e-5
    assert np.abs(gx - z["feature_grad"]).max() < 1.5e-5
    assert np.abs(gw - z["weight_grad"]).max() < 1.5e-5


@pytest.mark.parametrize("shape", SMALL_SHAPES)
@pytest.mark.parametrize("transposed", [False, True])
def test_against_dense_formulation(shape, transposed):
    # reference.cpp:15-82 restated in numpy float64; inputs follow the reference tests' law
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K)
    xin = np.ascontiguousarray(x.T) if transposed else x
    out = oracle.forward(xin, lookup, w, transposed=transposed)
    gx, gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
    d_out = oracle.dense_forward(xin, lookup, w, transposed=transposed)
    d_gx, d_gw = oracle.dense_backward(xin, lookup, w, g, transposed=transposed)
    assert out.shape == (B, L) and gx.shape == xin.shape and gw.shape == (L, K)
    assert np.abs(out - d_out).max() < 1e-5
    assert np.abs(gx - d_gx).max() < 1.5e-5
    assert np.abs(gw - d_gw).max() < 1.5e-5


def test_huge_label_count_against_scipy_sparse():
    # (1, 32, 4_000_000, 4) of the reference grid; D is too big to hold densely, so the check is
    # the CSR product of scipy.sparse, an independent library routine
    B, N, L, K = REFERENCE_SHAPES[-1]
    x, lookup, w, g = reference_law_inputs(B, N, L, K)
    S = sp.csr_matrix((w.reshape(-1).astype(np.float64), lookup.reshape(-1), np.arange(0, L * K + 1, K)), shape=(L, N))
    out = oracle.forward(x, lookup, w)
    assert np.abs(out - (S @ x.astype(np.float64).T).T).max() < 1e-5
    gx = oracle.input_grad(x, lookup, w, g)
    ref_gx = (S.T @ g.astype(np.float64).T).T
    assert rel_err(gx, ref_gx) < 1e-4          # about 250k terms per column: relative gate
    gw = oracle.weight_grad(x, lookup, w, g)
    ref_gw = x.astype(np.float64)[0][lookup] * g.astype(np.float64)[0][:, None]
    assert np.abs(gw - ref_gw).max() < 1.5e-5


@pytest.mark.parametrize("shape", [(17, 12, 63, 44), (127, 254, 513, 73)])
def test_f64_variants_agree_with_dense(shape):
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=7)
    d_out = oracle.dense_forward(x, lookup, w)
    d_gx, d_gw = oracle.dense_backward(x, lookup, w, g)
    assert np.allclose(oracle.forward(x, lookup, w, f64=True), d_out, rtol=0, atol=1e-12)
    assert np.allclose(oracle.input_grad(x, lookup, w, g, f64=True), d_gx, rtol=0, atol=1e-12)
    assert np.allclose(oracle.weight_grad(x, lookup, w, g, f64=True), d_gw, rtol=0, atol=1e-12)


def test_adjoint_identity():
    # the layer is linear in x and in W:  <out, g> = <x, gx> = <W, gW>
    B, N, L, K = 33, 100, 257, 19
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=3)
    out = oracle.forward(x, lookup, w).astype(np.float64)
    gx, gw = oracle.backward(x, lookup, w, g)
    a = float((out * g).sum())
    b = float((x.astype(np.float64) * gx).sum())
    c = float((w.astype(np.float64) * gw).sum())
    assert abs(a - b) < 1e-4 * abs(a) and abs(a - c) < 1e-4 * abs(a)


def test_layouts_agree_bitwise():
    # testing/test.cpp:91-166: [B,N] and [N,B] feature layouts give the same numbers
    B, N, L, K = 12, 8, 32, 16
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=5)
    xt = np.ascontiguousarray(x.T)
    assert np.array_equal(oracle.forward(x, lookup, w), oracle.forward(xt, lookup, w, transposed=True))
    gx, gw = oracle.backward(x, lookup, w, g)
    gxt, gwt = oracle.backward(xt, lookup, w, g, transposed=True)
    assert np.array_equal(gx, gxt.T) and np.array_equal(gw, gwt)


def test_duplicates_and_untouched_columns():
    # duplicates inside a row accumulate (reference.cpp:19-25) and each copy gets the full weight
    # gradient; columns no connection points at receive exactly zero input gradient
    x = np.arange(1, 13, dtype=np.float32).reshape(2, 6)
    lookup = np.array([[1, 1, 3], [0, 3, 3]], dtype=np.int32)       # columns 2, 4, 5 untouched
    w = np.array([[1.0, 2.0, 4.0], [8.0, 16.0, 32.0]], dtype=np.float32)
    g = np.array([[1.0, 10.0], [100.0, 1000.0]], dtype=np.float32)
    out = oracle.forward(x, lookup, w)
    assert np.array_equal(out, np.array([[3 * 2 + 4 * 4, 8 * 1 + 48 * 4], [3 * 8 + 4 * 10, 8 * 7 + 48 * 10]], dtype=np.float32))
    gx, gw = oracle.backward(x, lookup, w, g)
    assert np.array_equal(gx[:, [2, 4, 5]], np.zeros((2, 3), dtype=np.float32))
    assert np.array_equal(gx[:, 1], np.array([3.0, 300.0], dtype=np.float32))
    assert np.array_equal(gx[:, 3], np.array([4 * 1 + 48 * 10, 4 * 100 + 48 * 1000], dtype=np.float32))
    assert np.array_equal(gx[:, 0], np.array([80.0, 8000.0], dtype=np.float32))
    assert gw[0, 0] == gw[0, 1] == 2 * 1 + 8 * 100
    assert gw[1, 1] == gw[1, 2] == 4 * 10 + 10 * 1000


def test_identity_lookup_reduces_to_column_scaling():
    # K = 1 and lookup[j] = j: out = x * w^T column-wise, gx = g * w^T, gw = sum_b x*g
    B, N = 5, 9
    rng = np.random.default_rng(11)
    x = rng.standard_normal((B, N)).astype(np.float32)
    w = rng.standard_normal((N, 1)).astype(np.float32)
    g = rng.standard_normal((B, N)).astype(np.float32)
    lookup = np.arange(N, dtype=np.int32).reshape(N, 1)
    assert np.array_equal(oracle.forward(x, lookup, w), x * w.T)
    gx, gw = oracle.backward(x, lookup, w, g)
    assert np.array_equal(gx, g * w.T)
    assert np.allclose(gw[:, 0], (x.astype(np.float64) * g).sum(0), rtol=1e-6, atol=1e-6)


def test_permuting_a_row_only_reorders():
    B, N, L, K = 9, 40, 21, 12
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=9)
    perm = np.random.default_rng(1).permutation(K)
    out = oracle.forward(x, lookup, w)
    out_p = oracle.forward(x, lookup[:, perm], w[:, perm])
    assert np.abs(out - out_p).max() < 1e-5
    gx, gw = oracle.backward(x, lookup, w, g)
    gx_p, gw_p = oracle.backward(x, lookup[:, perm], w[:, perm], g)
    assert np.abs(gx - gx_p).max() < 1.5e-5
    assert np.array_equal(gw[:, perm], gw_p)      # each weight gradient is its own b-ordered sum


def test_thread_count_does_not_change_results():
    B, N, L, K = 16, 64, 1000, 8
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=13)
    one = (oracle.forward(x, lookup, w, threads=1),) + oracle.backward(x, lookup, w, g, threads=1)
    many = (oracle.forward(x, lookup, w, threads=7),) + oracle.backward(x, lookup, w, g, threads=7)
    for a, b in zip(one, many):
        assert np.array_equal(a, b)


def test_forward_accumulation_order_matches_reference_loop():
    # forward.cpp:29-41: four strided partial sums over the 4-aligned part, tail into the first,
    # then v0+v1+v2+v3.  Restated here in numpy float32 (no FMA), so agreement is to rounding only;
    # magnitudes chosen so that a different association (e.g. one running sum) shows.
    K = 11
    x = np.array([[1e8, 1.0, -1e8, 1.0, 3.0, 1.0, 1.0, 1.0, 1.0, 1.0, 1.0]], dtype=np.float32)
    lookup = np.arange(K, dtype=np.int32).reshape(1, K)
    w = np.ones((1, K), dtype=np.float32)
    v = np.zeros(4, dtype=np.float32)
    for i in range(0, 8, 4):
        for q in range(4):
            v[q] = np.float32(v[q] + x[0, i + q] * w[0, i + q])
    for i in range(8, K):
        v[0] = np.float32(v[0] + x[0, i] * w[0, i])
    expected = np.float32(np.float32(np.float32(v[0] + v[1]) + v[2]) + v[3])
    assert oracle.forward(x, lookup, w)[0, 0] == expected
    assert expected != np.float32(np.cumsum((x[0] * w[0]).astype(np.float32), dtype=np.float32)[-1])


def test_bf16_rounding_closed_form():
    vals = np.array([1.0, 1.00390625, 1.005859375, 1.001953125, -3.1415927, 0.0, 65504.0, 1e-40], dtype=np.float32)
    r = oracle.round_bf16(vals)
    # RNE on the top 16 bits: 1+2^-8 is a tie -> even (1.0); 1+3*2^-9 rounds up to 1+2^-7
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == np.float32(1.0078125) and r[3] == 1.0
    assert (r.view(np.uint32) & 0xFFFF == 0).all()
    assert np.all(np.abs(r[:7] - vals[:7]) <= np.abs(vals[:7]) * 2.0 ** -8)


def test_topk_matches_sort_with_lower_index_first():
    rng = np.random.default_rng(2)
    s = rng.integers(0, 20, (7, 300)).astype(np.float32)          # many ties
    values, indices = oracle.topk(s, 5)
    for b in range(s.shape[0]):
        order = np.lexsort((np.arange(s.shape[1]), -s[b]))[:5]
        assert np.array_equal(indices[b], order)
        assert np.array_equal(values[b], s[b, order])


# ---- loss oracle (sparse/metrics.py:132-173 over sparse/utils.py:11-17) ----------------------------
# Pinned by what the mathematics fixes: known values, a dense torch restatement differentiated by
# autograd (torch's own relu / binary_cross_entropy_with_logits, not the oracle's formulas), and
# central differences.
def _loss_case(seed, B=7, L=23, nnz=19):
    rng = np.random.default_rng(seed)
    scores = rng.normal(0, 1.5, (B, L))
    flat = rng.choice(B * L, size=nnz, replace=False)
    indices = np.stack([flat // L, flat % L], axis=1).astype(np.int64)
    values = rng.choice([1.0, 1.0, 0.5, 2.0], size=nnz)
    return scores, indices, values


def test_loss_oracle_known_values():
    # score 0: hinge 1, squared hinge 1, bce log 2 whatever the label
    for y in (0.0, 1.0):
        assert oracle.cwise_loss(oracle.LOSS_HINGE, 0.0, y) == 1.0
        assert oracle.cwise_loss(oracle.LOSS_SQUARED_HINGE, 0.0, y) == 1.0
        assert abs(oracle.cwise_loss(oracle.LOSS_BCE, 0.0, y) - np.log(2.0)) < 1e-15
    # a satisfied margin costs nothing and has zero gradient: negative at -1.5, positive at +1.5
    for kind in (oracle.LOSS_HINGE, oracle.LOSS_SQUARED_HINGE):
        assert oracle.cwise_loss(kind, -1.5, 0.0) == 0.0 and oracle.cwise_loss_grad(kind, -1.5, 0.0) == 0.0
        assert oracle.cwise_loss(kind, 1.5, 1.0) == 0.0 and oracle.cwise_loss_grad(kind, 1.5, 1.0) == 0.0
    # violated margins: negative at +2 -> relu(1+2) = 3, squared 9, slopes +1 and +6; positive at -2 -> same, slopes negated
    assert oracle.cwise_loss(oracle.LOSS_HINGE, 2.0, 0.0) == 3.0 and oracle.cwise_loss_grad(oracle.LOSS_HINGE, 2.0, 0.0) == 1.0
    assert oracle.cwise_loss(oracle.LOSS_SQUARED_HINGE, 2.0, 0.0) == 9.0 and oracle.cwise_loss_grad(oracle.LOSS_SQUARED_HINGE, 2.0, 0.0) == 6.0
    assert oracle.cwise_loss(oracle.LOSS_SQUARED_HINGE, -2.0, 1.0) == 9.0 and oracle.cwise_loss_grad(oracle.LOSS_SQUARED_HINGE, -2.0, 1.0) == -6.0
    # exactly on the margin the relu gradient is 0
    assert oracle.cwise_loss_grad(oracle.LOSS_HINGE, -1.0, 0.0) == 0.0
    # bce slope = sigmoid(s) - y
    assert abs(oracle.cwise_loss_grad(oracle.LOSS_BCE, 0.0, 1.0) + 0.5) < 1e-15
    assert abs(oracle.cwise_loss(oracle.LOSS_BCE, 30.0, 1.0)) < 1e-12 and abs(oracle.cwise_loss(oracle.LOSS_BCE, 30.0, 0.0) - 30.0) < 1e-12


@pytest.mark.parametrize("kind", [1, 2, 3])
def test_loss_oracle_against_dense_autograd(kind):
    import torch
    scores, indices, values = _loss_case(5 + kind)
    losses, grad = oracle.sparse_loss(scores, indices, values, kind)
    y = torch.zeros(scores.shape, dtype=torch.float64)
    y[indices[:, 0], indices[:, 1]] = torch.from_numpy(values)
    s = torch.from_numpy(scores).requires_grad_(True)
    if kind == oracle.LOSS_BCE:
        dense = torch.nn.functional.binary_cross_entropy_with_logits(s, y, reduction="none")
    else:
        hinge = torch.relu(1.0 - (2.0 * y - 1.0) * s)
        dense = hinge if kind == oracle.LOSS_HINGE else hinge.square()
    dense.sum().backward()
    np.testing.assert_allclose(losses, dense.detach().numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(grad, s.grad.numpy(), rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("kind", [2, 3])
def test_loss_oracle_gradient_is_the_derivative(kind):
    # central differences of the summed loss (smooth kinds; the hinge has kinks)
    scores, indices, values = _loss_case(11)
    _, grad = oracle.sparse_loss(scores, indices, values, kind)
    rng = np.random.default_rng(0)
    for _ in range(40):
        b, j = rng.integers(scores.shape[0]), rng.integers(scores.shape[1])
        h = 1e-6
        up, dn = scores.copy(), scores.copy()
        up[b, j] += h
        dn[b, j] -= h
        fd = (oracle.sparse_loss(up, indices, values, kind)[0].sum() - oracle.sparse_loss(dn, indices, values, kind)[0].sum()) / (2 * h)
        assert abs(fd - grad[b, j]) < 1e-5 * max(1.0, abs(grad[b, j]))


def test_loss_oracle_label_list_overrides_dense_part():
    # an empty label list charges every entry as a negative; a listed entry changes only its own cell
    scores, indices, values = _loss_case(3)
    dense_l, dense_g = oracle.sparse_loss(scores, np.zeros((0, 2), np.int64), None, oracle.LOSS_SQUARED_HINGE)
    np.testing.assert_array_equal(dense_l, np.maximum(1.0 + scores, 0.0) ** 2)
    l, g = oracle.sparse_loss(scores, indices, None, oracle.LOSS_SQUARED_HINGE)
    mask = np.zeros(scores.shape, bool)
    mask[indices[:, 0], indices[:, 1]] = True
    np.testing.assert_array_equal(l[~mask], dense_l[~mask])
    np.testing.assert_array_equal(g[~mask], dense_g[~mask])
    np.testing.assert_array_equal(l[mask], np.maximum(1.0 - scores[mask], 0.0) ** 2)


# ---- Adam oracle: closed form of the first step, torch.optim.Adam with Keras' epsilon placement -----
def test_adam_oracle_first_step_closed_form():
    # from zero moments: m = (1-b1) g, v = (1-b2) g^2, update = lr * g / (|g| + eps / sqrt(1 - b2))
    rng = np.random.default_rng(0)
    w = rng.normal(size=1000).astype(np.float32)
    g = rng.normal(size=1000).astype(np.float32)
    var, m, v = oracle.adam_step(w, np.zeros_like(w), np.zeros_like(w), g, learning_rate=0.01, step=1)
    np.testing.assert_allclose(m, 0.1 * g, rtol=1e-6)
    np.testing.assert_allclose(v, 0.001 * g * g, rtol=1e-4)
    expected = w.astype(np.float64) - 0.01 * g / (np.abs(g) + 1e-7 / np.sqrt(1 - 0.999))
    np.testing.assert_allclose(var, expected, rtol=0, atol=2e-6)
    # a zero gradient moves nothing on the first step
    var, m, v = oracle.adam_step(w, np.zeros_like(w), np.zeros_like(w), np.zeros_like(w), step=1)
    assert np.array_equal(var, w) and not m.any() and not v.any()


def test_adam_oracle_against_torch_adam():
    # torch divides by sqrt(v / (1 - b2^t)) + eps; Keras by sqrt(v) + eps with the bias correction in
    # the step size: the two agree when torch is given eps / sqrt(1 - b2^t)... per step, so compare
    # step by step, handing torch the state the oracle produced
    import torch
    rng = np.random.default_rng(1)
    n, lr, eps = 500, 0.003, 1e-7
    w = rng.normal(size=n).astype(np.float32)
    m, v = np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t in range(1, 8):
        g = (rng.normal(size=n) * (rng.random(n) < 0.7)).astype(np.float32)
        p = torch.nn.Parameter(torch.from_numpy(w.astype(np.float64)))
        opt = torch.optim.Adam([p], lr=lr, betas=(0.9, 0.999), eps=eps / np.sqrt(1 - 0.999 ** t))
        opt.state[p] = {"step": torch.tensor(float(t - 1)), "exp_avg": torch.from_numpy(m.astype(np.float64)),
                        "exp_avg_sq": torch.from_numpy(v.astype(np.float64))}
        p.grad = torch.from_numpy(g.astype(np.float64))
        opt.step()
        w, m, v = oracle.adam_step(w, m, v, g, learning_rate=lr, epsilon=eps, step=t)
        np.testing.assert_allclose(w, p.detach().numpy(), rtol=0, atol=3e-6)
        np.testing.assert_allclose(m, opt.state[p]["exp_avg"].numpy(), rtol=1e-5, atol=1e-7)
        np.testing.assert_allclose(v, opt.state[p]["exp_avg_sq"].numpy(), rtol=1e-4, atol=1e-9)


# ---- rewiring selection oracle ------------------------------------------------------------------------
def test_select_threshold_oracle_is_the_kth_smallest_magnitude():
    rng = np.random.default_rng(4)
    w = rng.normal(size=5000).astype(np.float32)
    w[::7] = 0.25                                       # ties
    w[::11] *= -1
    ordered = np.sort(np.abs(w))
    for k in (1, 2, 50, 2500, 4999, 5000):
        thr = oracle.select_threshold(w, k)
        assert thr == ordered[k - 1]
        sel = oracle.rewire_selection(w, thr)
        # strict comparison: the threshold value itself (and its ties) stays, so fewer than k are selected
        assert sel.sum() == (ordered < thr).sum() <= k - 1
    assert oracle.select_threshold(w, 0) == 0.0 and not oracle.rewire_selection(w, 0.0).any()


def test_threshold_counts_oracle_on_a_hand_made_case():
    # 2 x 4 scores, threshold 0: predicted = {(0,1), (0,3), (1,0)}; labels (0,1) value 1, (1,2) value 2, (1,0) value 0.5
    scores = np.array([[-1.0, 0.5, 0.0, 2.0], [0.1, -0.2, -3.0, 0.0]], np.float32)
    idx = np.array([[0, 1], [1, 2], [1, 0]])
    predicted, correct, total = oracle.threshold_counts(scores, idx, np.array([1.0, 2.0, 0.5]), 0.0)
    assert (predicted, correct, total) == (3.0, 1.5, 3.5)        # precision 1.5 / 3, recall 1.5 / 3.5
    assert oracle.threshold_counts(scores, np.zeros((0, 2), int), None, 0.0) == (3.0, 0.0, 0.0)
