"""Backward pass over the non-zero entries of out_grad only (`ffi_backward_sparse_f32`), against the
oracle's backward (backward.cpp:8-73 restated) on the same inputs: the reference's GPU kernels skip
exact zeros entry by entry (backward.cu.h:73,94,131,151) and get the same sums.

Gate: 1e-4 of the largest reference magnitude, as for the dense gradients.  out_grad is drawn with a
given share of non-zeros; masks are either computed here from out_grad, handed in with extra set
bits, produced by the loss kernels, or left to the library (NULL).
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import load_package, rel_err

pytestmark = pytest.mark.gpu

GRAD_RTOL = 1e-4

#          B    N     L     K  transposed
SHAPES = [(128, 768, 5000, 32, True),
          (37, 300, 1001, 7, False),
          (64, 512, 2100, 64, True),
          (200, 96, 700, 72, False),
          (33, 3000, 333, 12, True),
          (40, 5000, 400, 20, False),       # wider than the sparse input gradient covers: dense kernels for gx
          (1, 16, 70, 3, False)]


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


def make_case(shape, density, seed):
    B, N, L, K, tp = shape
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = rng.standard_normal((L, K)).astype(np.float32)
    g = rng.standard_normal((B, L)).astype(np.float32)
    g[rng.random((B, L)) >= density] = 0.0
    if density > 0 and L > 5:
        g[:, 3] = rng.standard_normal(B)            # one label that every sample pushes on
    feats = np.ascontiguousarray(x.T) if tp else x
    return feats, lookup, w, g


def masks_of(g):
    B, L = g.shape
    nbt = (B + 31) // 32
    words = np.zeros((nbt, L), np.uint32)
    for b in range(B):
        words[b // 32] |= (g[b] != 0).astype(np.uint32) << np.uint32(b % 32)
    return words.view(np.int32)


def run(ffi, feats, lookup, w, g, tp, words=None, max_density=1.0):
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    gx, gw, gb, sparse = ffi.backward_sparse(dev(feats), dev(lookup), dev(w), dev(g),
                                             nz_words=dev(words) if words is not None else None,
                                             max_density=max_density, transposed=tp, need_bias_grad=True)
    torch.cuda.synchronize()
    return gx.cpu().numpy(), gw.cpu().numpy(), gb.cpu().numpy(), sparse


@pytest.mark.parametrize("density", [0.001, 0.02, 0.3])
@pytest.mark.parametrize("given_masks", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_sparse_backward_against_oracle(ffi, shape, density, given_masks):
    tp = shape[4]
    feats, lookup, w, g = make_case(shape, density, seed=sum(shape[:4]))
    ref_gx, ref_gw = oracle.backward(feats, lookup, w, g, transposed=tp)
    gx, gw, gb, sparse = run(ffi, feats, lookup, w, g, tp, words=masks_of(g) if given_masks else None)
    assert sparse                                   # max_density = 1 forces the sparse kernels
    assert rel_err(gw, ref_gw) <= GRAD_RTOL
    assert rel_err(gx, ref_gx) <= GRAD_RTOL
    assert rel_err(gb, g.astype(np.float64).sum(axis=0)) <= GRAD_RTOL


def test_default_threshold_picks_dense_kernels_for_dense_gradients(ffi):
    shape = (128, 768, 5000, 32, True)
    feats, lookup, w, g = make_case(shape, 0.5, seed=1)
    ref_gx, ref_gw = oracle.backward(feats, lookup, w, g, transposed=True)
    gx, gw, gb, sparse = run(ffi, feats, lookup, w, g, True, max_density=None)
    assert not sparse
    assert rel_err(gw, ref_gw) <= GRAD_RTOL and rel_err(gx, ref_gx) <= GRAD_RTOL
    assert rel_err(gb, g.astype(np.float64).sum(axis=0)) <= GRAD_RTOL
    feats, lookup, w, g = make_case(shape, 0.002, seed=2)
    ref_gx, ref_gw = oracle.backward(feats, lookup, w, g, transposed=True)
    gx, gw, gb, sparse = run(ffi, feats, lookup, w, g, True, max_density=None)
    assert sparse
    assert rel_err(gw, ref_gw) <= GRAD_RTOL and rel_err(gx, ref_gx) <= GRAD_RTOL


def test_all_zero_gradient_gives_exact_zeros(ffi):
    shape = (70, 200, 900, 16, False)
    feats, lookup, w, g = make_case(shape, 0.0, seed=3)
    gx, gw, gb, sparse = run(ffi, feats, lookup, w, g, False)
    assert sparse and not gx.any() and not gw.any() and not gb.any()


def test_masks_may_cover_zero_entries(ffi):
    # a set bit over a zero entry only costs time
    shape = (64, 256, 1500, 24, True)
    feats, lookup, w, g = make_case(shape, 0.01, seed=4)
    words = masks_of(g).view(np.uint32).copy()
    rng = np.random.default_rng(0)
    words |= (rng.random(words.shape) < 0.05).astype(np.uint32) << np.uint32(7)
    words[:, 10:20] = 0xFFFFFFFF
    ref_gx, ref_gw = oracle.backward(feats, lookup, w, g, transposed=True)
    gx, gw, gb, sparse = run(ffi, feats, lookup, w, g, True, words=words.view(np.int32))
    assert sparse and rel_err(gw, ref_gw) <= GRAD_RTOL and rel_err(gx, ref_gx) <= GRAD_RTOL


def test_sparse_backward_is_reproducible(ffi):
    shape = (128, 768, 20000, 32, True)
    feats, lookup, w, g = make_case(shape, 0.01, seed=5)
    a = run(ffi, feats, lookup, w, g, True)
    b = run(ffi, feats, lookup, w, g, True)
    assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1]) and np.array_equal(a[2], b[2])


@pytest.mark.parametrize("fused", [True, False])
@pytest.mark.parametrize("shape", [(128, 768, 5000, 32, True), (37, 300, 1001, 7, False), (33, 3000, 333, 12, True)])
def test_loss_kernels_write_the_masks_of_their_gradient(ffi, shape, fused):
    B, N, L, K, tp = shape
    rng = np.random.default_rng(6)
    feats, lookup, w, _ = make_case(shape, 0.0, seed=6)
    w *= 0.3
    bias = np.full(L, -1.5, np.float32)             # most margins satisfied: a sparse gradient
    rows = np.repeat(np.arange(B), 3)
    cols = rng.integers(0, L, B * 3)
    keys = np.unique(rows * L + cols)
    indices = np.stack([keys // L, keys % L], axis=1).astype(np.int64)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    y = (dev(indices), None)
    if fused:
        _, g_t, _, masks = ffi.metrics.forward_loss(dev(feats), dev(lookup), dev(w), dev(bias), y, oracle.LOSS_SQUARED_HINGE,
                                                    transposed=tp, want_masks=True)
    else:
        scores = ffi.fan_in_sparse_matmul_tp_bias(dev(feats), dev(lookup), dev(w), dev(bias)) if tp else \
            ffi.fan_in_sparse_matmul_bias(dev(feats), dev(lookup), dev(w), dev(bias))
        g_t, _, masks = ffi.metrics.sparse_loss_grad(scores, y, oracle.LOSS_SQUARED_HINGE, want_masks=True)
    torch.cuda.synchronize()
    g = g_t.cpu().numpy()
    got = masks.cpu().numpy().view(np.uint32)
    want = masks_of(g).view(np.uint32)
    assert 0 < (g != 0).mean() < 0.5
    assert not (want & ~got).any()                  # every non-zero entry is covered
    # nothing else is, except listed label positions whose gradient as a negative was non-zero
    # and whose gradient as a positive is zero (the fused kernel sets bits before the labels are applied)
    allowed = np.zeros_like(want)
    np.bitwise_or.at(allowed, (indices[:, 0] // 32, indices[:, 1]), np.uint32(1) << (indices[:, 0] % 32).astype(np.uint32))
    assert not (got & ~want & ~allowed).any()


def test_fused_loss_backward_uses_the_sparse_kernels(ffi):
    # end to end through autograd: fused loss forward, masks kept, sparse backward; against the dense route
    B, N, L, K = 64, 256, 4000, 16
    gen = torch.Generator(device="cuda").manual_seed(8)
    x = torch.rand((B, N), device="cuda", generator=gen)
    lookup = torch.randint(0, N, (L, K), device="cuda", generator=gen, dtype=torch.int64).to(torch.int32)
    rows = torch.arange(B, device="cuda").repeat_interleave(2)
    cols = torch.randint(0, L, (B * 2,), device="cuda", generator=gen)
    y = (torch.stack([rows, cols], dim=1), None)
    loss_fn = ffi.SparseSquaredHingeLoss()
    grads = []
    for fused in (False, True):
        w = ((torch.arange(L * K, device="cuda", dtype=torch.float32).reshape(L, K) % 11) / 40 - 0.12).requires_grad_(True)
        bias = torch.full((L,), -1.2, device="cuda", requires_grad=True)
        xin = x.clone().requires_grad_(True)
        loss = loss_fn.fused(xin, lookup, w, bias, y)[0] if fused else loss_fn(y, ffi.fan_in_sparse_matmul_bias(xin, lookup, w, bias))
        loss.backward()
        torch.cuda.synchronize()
        grads.append((w.grad.cpu().numpy(), bias.grad.cpu().numpy(), xin.grad.cpu().numpy()))
    for a, b in zip(grads[1], grads[0]):
        assert rel_err(a, b) <= GRAD_RTOL


@pytest.mark.parametrize("force_dense", [False, True])
@pytest.mark.parametrize("B,kind", [(96, oracle.LOSS_SQUARED_HINGE), (70, oracle.LOSS_SQUARED_HINGE), (33, oracle.LOSS_HINGE),
                                    (64, oracle.LOSS_BCE)])
def test_gradient_stored_only_where_it_is_not_zero(ffi, force_dense, B, kind):
    # forward_loss(skip_zero_stores): out_grad is written at the masks' set bits only; the backward pass, told
    # so, gives the results of the full gradient on the sparse kernels and (zeros filled in first) on the dense ones
    # (batches that fill their last tile of 32 samples and batches that do not; a loss without exact zeros too)
    N, L, K, tp = 384, 3000, 32, True
    rng = np.random.default_rng(12)
    feats, lookup, w, _ = make_case((B, N, L, K, tp), 0.0, seed=12)
    w *= 0.3
    bias = np.full(L, -1.5, np.float32)
    keys = np.unique(np.repeat(np.arange(B), 3) * L + rng.integers(0, L, B * 3))
    indices = np.stack([keys // L, keys % L], axis=1).astype(np.int64)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    y = (dev(indices), None)
    args = (dev(feats), dev(lookup), dev(w), dev(bias), y, kind)
    _, g_full, loss_full, masks_full = ffi.metrics.forward_loss(*args, transposed=tp, want_masks=True)
    _, g_part, loss_part, masks = ffi.metrics.forward_loss(*args, transposed=tp, want_masks=True, skip_zero_stores=True)
    torch.cuda.synchronize()
    # (the two kernels add a label's 32 losses in different orders)
    assert torch.equal(masks, masks_full) and abs(float(loss_full) - float(loss_part)) <= 1e-6 * abs(float(loss_full))
    written = torch.from_numpy(np.unpackbits(masks.cpu().numpy().view(np.uint8).reshape(-1, L, 4), axis=2, bitorder="little")
                               .reshape(-1, L, 32).transpose(0, 2, 1).reshape(-1, L)[:B].astype(bool)).cuda()
    assert torch.equal(g_part[written], g_full[written])
    g_part[~written] = float("nan")                  # whatever was there must not matter
    ref_gx, ref_gw = oracle.backward(feats, lookup, w, g_full.cpu().numpy(), transposed=tp)
    gx, gw, gb, sparse = ffi.backward_sparse(dev(feats), dev(lookup), dev(w), g_part, nz_words=masks, transposed=tp,
                                             max_density=1e-9 if force_dense else 1.0, need_bias_grad=True, grad_is_partial=True)
    torch.cuda.synchronize()
    assert sparse == (not force_dense)
    assert rel_err(gw.cpu().numpy(), ref_gw) <= GRAD_RTOL and rel_err(gx.cpu().numpy(), ref_gx) <= GRAD_RTOL
    assert rel_err(gb.cpu().numpy(), g_full.cpu().numpy().astype(np.float64).sum(axis=0)) <= GRAD_RTOL


def test_deciding_from_the_previous_call_gives_the_same_results(ffi):
    # the first call of a shape waits for its own count; later ones use the count left behind: a dense gradient
    # after sparse ones is still computed correctly (by the sparse kernels, once), then the dense kernels take over
    shape = (64, 256, 1500, 24, True)
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    taken = []
    for density in (0.002, 0.003, 0.4, 0.4, 0.002):
        feats, lookup, w, g = make_case(shape, density, seed=int(density * 1e4))
        ref_gx, ref_gw = oracle.backward(feats, lookup, w, g, transposed=True)
        gx, gw, gb, sparse = ffi.backward_sparse(dev(feats), dev(lookup), dev(w), dev(g), transposed=True, need_bias_grad=True,
                                                 max_density=0.05, decide_from_previous=True)
        torch.cuda.synchronize()
        taken.append(sparse)
        assert rel_err(gw.cpu().numpy(), ref_gw) <= GRAD_RTOL and rel_err(gx.cpu().numpy(), ref_gx) <= GRAD_RTOL
        assert rel_err(gb.cpu().numpy(), g.astype(np.float64).sum(axis=0)) <= GRAD_RTOL
    assert taken == [True, True, True, False, False]


def test_headline_config_full_size_training_step(ffi):
    # 670,091 labels x fan-in 32 x 768 inputs x batch 128, gradient about 0.2 % non-zero: size-independent checks.
    #   the fused loss forward (zero gradients not stored) agrees with forward + loss pass at every mask bit,
    #   the masks cover exactly the non-zero gradients (plus listed positions), the loss sums agree;
    #   the sparse backward agrees with the dense kernels on the same gradient, and with the adjoint identity
    #   <out_grad, W x> = <gW, W> = <gx, x> (the layer is linear in x and in W)
    from ecml23_sparse_amd import synth
    cfg = synth.CONFIGS["c2"]
    t = synth.make_inputs(cfg, seed=42, device="cuda", transposed=True)
    x, lookup, w = t["features"], t["lookup"], t["weights"]
    B, L = cfg.batch, cfg.num_units
    scores0 = ffi.fan_in_sparse_matmul_tp(x, lookup, w)
    gen = torch.Generator(device="cuda").manual_seed(0)
    sample = scores0.flatten()[torch.randint(0, B * L, (1 << 20,), device="cuda", generator=gen)]
    bias = torch.full((L,), -1.0 - float(torch.quantile(sample, 0.998)), device="cuda")
    rows = torch.arange(B, device="cuda").repeat_interleave(5)
    y = (torch.stack([rows, torch.randint(0, L, (B * 5,), device="cuda", generator=gen)], dim=1), None)
    kind = oracle.LOSS_SQUARED_HINGE
    scores = ffi.fan_in_sparse_matmul_tp_bias(x, lookup, w, bias)
    g_ref, loss_ref = ffi.metrics.sparse_loss_grad(scores, y, kind)
    _, g, loss, masks = ffi.metrics.forward_loss(x, lookup, w, bias, y, kind, transposed=True, want_masks=True,
                                                 skip_zero_stores=True)
    torch.cuda.synchronize()
    bit = (masks.view(B // 32, 1, L) >> torch.arange(32, device="cuda", dtype=torch.int32).view(1, 32, 1)) & 1
    written = bit.reshape(B, L).bool()
    density = float(written.float().mean())
    assert 0.001 < density < 0.004
    assert bool((written | (g_ref == 0)).all())                                  # every non-zero gradient is covered
    scale = float(g_ref.abs().max())
    assert float((g[written] - g_ref[written]).abs().max()) <= 4e-5 * scale       # scores differ by rounding only
    assert abs(float(loss) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref))
    gx_s, gw_s, gb_s, sparse = ffi.backward_sparse(x, lookup, w, g, nz_words=masks, transposed=True, need_bias_grad=True,
                                                   grad_is_partial=True)
    assert sparse
    g_full = torch.where(written, g, torch.zeros_like(g))
    gx_d, gw_d = ffi.fan_in_sparse_matmul_grad_tp(x, lookup, w, g_full)
    torch.cuda.synchronize()
    assert rel_err(gw_s.cpu().numpy(), gw_d.cpu().numpy()) <= GRAD_RTOL
    assert rel_err(gx_s.cpu().numpy(), gx_d.cpu().numpy()) <= GRAD_RTOL
    assert rel_err(gb_s.cpu().numpy(), g_full.double().sum(dim=0).cpu().numpy()) <= GRAD_RTOL
    a = float((scores0.double() * g_full.double()).sum())
    b = float((x.double() * gx_s.double()).sum())
    c = float((w.double() * gw_s.double()).sum())
    assert abs(a - b) <= 1e-4 * abs(a) and abs(a - c) <= 1e-4 * abs(a)


def _drawn_shapes(count, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        B = int(rng.choice([1, 7, 31, 32, 33, 64, 65, 100, 128, 200]))
        N = int(rng.choice([3, 64, 255, 512, 768, 1024, 1217, 3000, 4096, 4097]))
        L = int(rng.choice([1, 63, 64, 65, 255, 256, 257, 1025, 3000, 7001, 33000]))
        K = int(rng.choice([1, 3, 4, 15, 16, 32, 33, 64, 65, 100]))
        shapes.append((B, N, L, K, bool(rng.integers(0, 2))))
    return shapes


@pytest.mark.parametrize("density", [0.003, 0.1])
@pytest.mark.parametrize("shape", _drawn_shapes(16, seed=77), ids=lambda s: "B%d_N%d_L%d_K%d_%s" % (s[0], s[1], s[2], s[3], "tp" if s[4] else "nt"))
def test_sparse_backward_drawn_shapes(ffi, shape, density):
    # sizes drawn around the boundaries of the sparse kernels (blocks of 256 labels per wavefront, chunks of 32,768
    # labels of a bit row, 4096 columns for the LDS accumulators, 32-connection register chunks), masks given
    tp = shape[4]
    feats, lookup, w, g = make_case(shape, density, seed=sum(shape[:4]) + 1)
    print(f"case shape={shape} density={density}", flush=True)
    ref_gx, ref_gw = oracle.backward(feats, lookup, w, g, transposed=tp)
    gx, gw, gb, sparse = run(ffi, feats, lookup, w, g, tp, words=masks_of(g))
    assert sparse
    assert rel_err(gw, ref_gw) <= GRAD_RTOL
    assert rel_err(gx, ref_gx) <= GRAD_RTOL
    assert rel_err(gb, g.sum(axis=0)) <= GRAD_RTOL
