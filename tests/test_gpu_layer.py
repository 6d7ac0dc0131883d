"""The layer-level caller (sparse/custom_layer.py:45-50 + the bias add of sparse/layer.py:245-247):
fused-bias entry points through the C ABI, and the torch module built on them, against the oracle.

Expected values: oracle forward (forward.cpp:9-44 restated) plus a numpy bias add; the bias
gradient is the float64 column sum of out_grad (the gradient of tf.nn.bias_add).
Gates as for the ops: forward 1e-5, gradients 1e-4, relative to the largest reference magnitude.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import load_package, rel_err

pytestmark = pytest.mark.gpu

FWD_RTOL = 1e-5
GRAD_RTOL = 1e-4

#          B    N     L     K  transposed      (narrow: tile kernels; wide: N beyond the LDS tile)
SHAPES = [(128, 768, 5000, 32, True),
          (37, 300, 1001, 7, False),
          (64, 512, 2100, 64, True),
          (200, 96, 700, 40, False),
          (33, 3000, 333, 12, True),
          (130, 2048, 260, 72, False)]


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


def make_case(shape, seed):
    B, N, L, K, tp = shape
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)          # with replacement, as the layer draws them
    w = (rng.standard_normal((L, K)) / np.sqrt(K)).astype(np.float32)
    bias = rng.standard_normal(L).astype(np.float32)
    g = (rng.standard_normal((B, L)) * 0.1).astype(np.float32)
    if tp:
        x = np.ascontiguousarray(x.T)
    return x, lookup, w, bias, g


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "B%d_N%d_L%d_K%d_%s" % (s[0], s[1], s[2], s[3], "tp" if s[4] else "nt"))
def test_fused_bias_entry_points(ffi, shape):
    B, N, L, K, tp = shape
    x, lookup, w, bias, g = make_case(shape, 3)
    dx, dl, dw, db, dg = dev(x), dev(lookup), dev(w), dev(bias), dev(g)
    lib, st = ffi._lib.lib(), torch.cuda.current_stream().cuda_stream
    out = torch.full((B, L), float("nan"), device="cuda")
    ffi._lib.check(lib.ffi_forward_bias_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), db.data_ptr(), out.data_ptr(),
                                            B, N, L, K, int(tp), st))
    gx = torch.full(tuple(x.shape), float("nan"), device="cuda")
    gw = torch.full((L, K), float("nan"), device="cuda")
    gb = torch.full((L,), float("nan"), device="cuda")
    ffi._lib.check(lib.ffi_backward_bias_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(),
                                             gw.data_ptr(), gb.data_ptr(), B, N, L, K, int(tp), st))
    torch.cuda.synchronize()
    want = oracle.forward(x, lookup, w, transposed=tp) + bias[None, :]
    assert rel_err(out.cpu().numpy(), want) <= FWD_RTOL
    want_gx, want_gw = oracle.backward(x, lookup, w, g, transposed=tp)
    assert rel_err(gx.cpu().numpy(), want_gx) <= GRAD_RTOL
    assert rel_err(gw.cpu().numpy(), want_gw) <= GRAD_RTOL
    assert rel_err(gb.cpu().numpy(), g.astype(np.float64).sum(axis=0)) <= GRAD_RTOL
    # the stand-alone weight gradient agrees (it sums the batch in another lane order, so not bit for bit),
    # and a second backward call reproduces the first one exactly
    gw2 = torch.empty((L, K), device="cuda")
    ffi._lib.check(lib.ffi_weight_grad_f32(dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), gw2.data_ptr(), B, N, L, K, int(tp), st))
    gx3, gw3, gb3 = torch.empty_like(gx), torch.empty_like(gw), torch.empty_like(gb)
    ffi._lib.check(lib.ffi_backward_bias_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx3.data_ptr(),
                                             gw3.data_ptr(), gb3.data_ptr(), B, N, L, K, int(tp), st))
    torch.cuda.synchronize()
    assert rel_err(gw2.cpu().numpy(), want_gw) <= GRAD_RTOL
    assert torch.equal(gw, gw3) and torch.equal(gx, gx3) and torch.equal(gb, gb3)


def test_fused_bias_null_arguments(ffi):
    lib = ffi._lib.lib()
    t = torch.zeros(8, device="cuda")
    assert lib.ffi_forward_bias_f32(t.data_ptr(), t.data_ptr(), t.data_ptr(), None, t.data_ptr(), 1, 1, 1, 1, 0, None) == -1
    assert lib.ffi_backward_bias_f32(t.data_ptr(), t.data_ptr(), t.data_ptr(), t.data_ptr(), None, t.data_ptr(), None,
                                     1, 1, 1, 1, 0, None) == -1


@pytest.mark.parametrize("use_bias", [True, False])
def test_layer_forward_backward(ffi, use_bias):
    layer_mod = ffi.custom_layer
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7)
    B, N, units, K = 48, 640, 3000, 32
    layer = layer_mod.StratifiedRewireLayerV2(units, N, connections=units * K, use_bias=use_bias, generator=gen)
    assert layer.fan_in == K and layer.kernel_indices.dtype == torch.int32 and layer.kernel_weights.shape == (units * K,)
    if use_bias:
        with torch.no_grad():
            layer.bias.copy_(torch.randn(units, device="cuda", generator=gen))
    x = torch.relu(torch.randn(B, N, device="cuda", generator=gen)).requires_grad_(True)
    g = torch.randn(B, units, device="cuda", generator=gen) * 0.1
    out = layer(x)
    out.backward(g)
    torch.cuda.synchronize()
    xn, gn = x.detach().cpu().numpy(), g.cpu().numpy()
    lookup = layer.kernel_indices.view(-1, K).cpu().numpy()
    w = layer.kernel_weights.detach().view(-1, K).cpu().numpy()
    want = oracle.forward(xn, lookup, w)
    if use_bias:
        want = want + layer.bias.detach().cpu().numpy()[None, :]
    assert rel_err(out.detach().cpu().numpy(), want) <= FWD_RTOL
    want_gx, want_gw = oracle.backward(xn, lookup, w, gn)
    assert rel_err(x.grad.cpu().numpy(), want_gx) <= GRAD_RTOL
    assert rel_err(layer.kernel_weights.grad.view(-1, K).cpu().numpy(), want_gw) <= GRAD_RTOL
    if use_bias:
        assert rel_err(layer.bias.grad.cpu().numpy(), gn.astype(np.float64).sum(axis=0)) <= GRAD_RTOL


def test_layer_rewire(ffi):
    layer_mod = ffi.custom_layer
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    B, N, units, K = 40, 256, 1500, 16
    layer = layer_mod.StratifiedRewireLayerV2(units, N, connections=units * K, rewire_selector=layer_mod.FixedFractionSelector(0.05),
                                              arrange=False, generator=gen)
    x = torch.relu(torch.randn(B, N, device="cuda", generator=gen)).requires_grad_(True)
    g = torch.randn(B, units, device="cuda", generator=gen) * 0.1
    layer(x).backward(g)                      # builds and caches the plan for the current indices
    before_idx = layer.kernel_indices.clone()
    before_w = layer.kernel_weights.detach().clone()
    m = torch.ones(units * K, device="cuda")
    v = torch.full((units * K,), 2.0, device="cuda")
    selected = layer.rewire_selector.select(before_w)
    new_m, new_v = layer.rewire([m, v])
    n_sel = int(selected.sum())
    assert 0 < n_sel <= round(0.05 * units * K)
    assert torch.equal(layer.kernel_weights.detach(), before_w)                      # weights keep their values
    assert torch.equal(layer.kernel_indices[~selected], before_idx[~selected])        # only selected sources change
    assert int((layer.kernel_indices != before_idx).sum()) > 0
    assert float(new_m[selected].abs().sum()) == 0 and float(new_v[selected].abs().sum()) == 0
    assert torch.equal(new_m[~selected], m[~selected]) and torch.equal(new_v[~selected], v[~selected])
    assert float(m.min()) == 1.0                                                      # inputs are not modified
    # gradients after the in-place edit follow the new indices (the cached plan is rebuilt)
    x.grad = None
    layer.kernel_weights.grad = None
    layer(x).backward(g)
    torch.cuda.synchronize()
    lookup = layer.kernel_indices.view(-1, K).cpu().numpy()
    w = layer.kernel_weights.detach().view(-1, K).cpu().numpy()
    want_gx, want_gw = oracle.backward(x.detach().cpu().numpy(), lookup, w, g.cpu().numpy())
    assert rel_err(x.grad.cpu().numpy(), want_gx) <= GRAD_RTOL
    assert rel_err(layer.kernel_weights.grad.view(-1, K).cpu().numpy(), want_gw) <= GRAD_RTOL


def test_selectors(ffi):
    layer_mod = ffi.custom_layer
    w = torch.tensor([0.5, -0.1, 0.3, -0.05, 0.2, 0.05, -0.7, 0.0], device="cuda")
    assert layer_mod.FixedMagnitudeSelector(0.1).select(w).tolist() == [False, False, False, True, False, True, False, True]
    # fraction 0.5 of 8 -> the 4th smallest magnitude (0.1) is the threshold, strictly smaller ones are selected
    assert layer_mod.FixedFractionSelector(0.5).select(w).tolist() == [False, False, False, True, False, True, False, True]
    assert layer_mod.FixedFractionSelector(0.0).select(w).sum().item() == 0


def test_arrange_connections(ffi):
    """Rows are permuted (indices, weights and extra arrays together), even and odd ids alternate as far
    as they pair up, the call is idempotent, and the layer's results do not change beyond rounding."""
    ops = ffi.fixed_fan_in_ops
    rng = np.random.default_rng(3)
    B, N, L, K = 40, 300, 1003, 40                      # two chunks per label, the second one partly filled
    lookup = rng.integers(0, N, size=(L, K)).astype(np.int32)
    w = rng.standard_normal((L, K)).astype(np.float32)
    m = rng.standard_normal((L, K)).astype(np.float32)
    x = np.maximum(rng.standard_normal((B, N)), 0).astype(np.float32)
    g = (rng.standard_normal((B, L)) * 0.1).astype(np.float32)
    dl, dw, dm = dev(lookup), dev(w), dev(m)
    ops.arrange_connections(dl, dw, dm)
    torch.cuda.synchronize()
    al, aw, am = dl.cpu().numpy(), dw.cpu().numpy(), dm.cpu().numpy()
    for lo, hi in ((0, 32), (32, 40)):                  # permutation inside each chunk, the three arrays together
        before = np.stack([lookup[:, lo:hi], w[:, lo:hi].view(np.int32), m[:, lo:hi].view(np.int32)], axis=-1)
        after = np.stack([al[:, lo:hi], aw[:, lo:hi].view(np.int32), am[:, lo:hi].view(np.int32)], axis=-1)
        key = lambda a: np.sort(a.astype(np.int64)[..., 0] * (1 << 40) + (a.astype(np.int64)[..., 1] & 0xffffffff), axis=1)
        np.testing.assert_array_equal(key(before), key(after))
        # alternation: position i holds parity (i + role) & 1 for i < 2 * min(#even, #odd)
        par = al[:, lo:hi] & 1
        role = ((np.arange(L) >> 3) & 1)[:, None]
        n_first = (par == role).sum(1, keepdims=True)
        paired = 2 * np.minimum(n_first, (hi - lo) - n_first)
        pos = np.arange(hi - lo)[None, :]
        assert (((par ^ role ^ (pos & 1)) == 0) | (pos >= paired)).all()
    dl2, dw2, dm2 = dl.clone(), dw.clone(), dm.clone()
    ops.arrange_connections(dl2, dw2, dm2)              # idempotent
    assert torch.equal(dl, dl2) and torch.equal(dw, dw2) and torch.equal(dm, dm2)
    out_a = ops.fan_in_sparse_matmul(dev(x), dl, dw)
    torch.cuda.synchronize()
    assert rel_err(out_a.cpu().numpy(), oracle.forward(x, lookup, w)) <= FWD_RTOL
    gx_a, gw_a = ops.fan_in_sparse_matmul_grad(dev(x), dl, dw, dev(g))
    torch.cuda.synchronize()
    want_gx, want_gw = oracle.backward(x, al, aw, g)
    assert rel_err(gx_a.cpu().numpy(), want_gx) <= GRAD_RTOL and rel_err(gw_a.cpu().numpy(), want_gw) <= GRAD_RTOL
    assert rel_err(want_gx, oracle.input_grad(x, lookup, w, g)) <= 1e-5     # same operator, rows reordered


def test_layer_keeps_connections_arranged(ffi):
    layer_mod = ffi.custom_layer
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    units, N, K = 700, 128, 32
    layer = layer_mod.StratifiedRewireLayerV2(units, N, connections=units * K, rewire_selector=layer_mod.FixedFractionSelector(0.1),
                                              generator=gen)
    def alternates(idx):
        par = idx.view(-1, K).cpu().numpy() & 1
        role = ((np.arange(units) >> 3) & 1)[:, None]
        n_first = (par == role).sum(1, keepdims=True)
        paired = 2 * np.minimum(n_first, K - n_first)
        pos = np.arange(K)[None, :]
        return bool((((par ^ role ^ (pos & 1)) == 0) | (pos >= paired)).all())
    assert alternates(layer.kernel_indices)
    w_before = layer.kernel_weights.detach().clone()
    mom = torch.arange(units * K, device="cuda", dtype=torch.float32)
    selected = layer.rewire_selector.select(w_before)
    (new_mom,) = layer.rewire([mom])
    assert alternates(layer.kernel_indices)
    # per label: the same weights as before (reordered), and the moment entries travel with their weights
    wb, wa = w_before.view(units, K).cpu().numpy(), layer.kernel_weights.detach().view(units, K).cpu().numpy()
    np.testing.assert_array_equal(np.sort(wb, 1), np.sort(wa, 1))
    want_mom = torch.where(selected, torch.zeros_like(mom), mom).view(units, K).cpu().numpy()
    order_b, order_a = np.argsort(wb, 1, kind="stable"), np.argsort(wa, 1, kind="stable")
    np.testing.assert_array_equal(np.take_along_axis(want_mom, order_b, 1), np.take_along_axis(new_mom.view(units, K).cpu().numpy(), order_a, 1))


def test_layer_forward_loss_matches_loss_of_forward(ffi):
    # one fused call (scores never written) against loss(y, layer(x)), values and parameter gradients
    gen = torch.Generator(device="cuda").manual_seed(3)
    layer = ffi.StratifiedRewireLayerV2(units=1500, input_dim=200, connections=1500 * 24, generator=gen)
    with torch.no_grad():
        layer.bias.fill_(-0.2)
    x = torch.rand((48, 200), device="cuda", generator=gen)
    rows = torch.arange(48, device="cuda").repeat_interleave(3)
    cols = torch.randint(0, 1500, (48 * 3,), device="cuda", generator=gen)
    y = (torch.stack([rows, cols], dim=1), None)
    loss_fn = ffi.SparseSquaredHingeLoss()
    plain = loss_fn(y, layer(x))
    plain.backward()
    gw0, gb0 = layer.kernel_weights.grad.clone(), layer.bias.grad.clone()
    layer.zero_grad()
    fused, scores = layer.forward_loss(x, y, loss_fn, want_scores=True)
    fused.backward()
    torch.cuda.synchronize()
    assert abs(float(plain.detach()) - float(fused.detach())) <= 1e-5 * abs(float(plain.detach()))
    assert rel_err(layer.kernel_weights.grad.cpu().numpy(), gw0.cpu().numpy()) <= GRAD_RTOL
    assert rel_err(layer.bias.grad.cpu().numpy(), gb0.cpu().numpy()) <= GRAD_RTOL
    assert rel_err(scores.cpu().numpy(), layer(x).detach().cpu().numpy()) <= FWD_RTOL


def test_dense_stratified_block_trains_end_to_end(ffi):
    # run.py:63-66 ("dense-stratified"): Dense(intermediate, relu) -> StratifiedRewireLayerV2(num_labels); the sparse
    # layer's input gradient has to reach the dense layer.  torch supplies the dense layer, the library the sparse one.
    gen = torch.Generator(device="cuda").manual_seed(31)
    B, D, H, L = 48, 64, 96, 1500
    dense = torch.nn.Linear(D, H).cuda()
    sparse = ffi.StratifiedRewireLayerV2(units=L, input_dim=H, connections=L * 8, generator=gen,
                                         rewire_selector=ffi.FixedFractionSelector(0.02))
    opt_dense = torch.optim.Adam(dense.parameters(), lr=0.01)
    opt_sparse = ffi.SparseAdam(list(sparse.parameters()), learning_rate=0.01)
    loss_fn = ffi.SparseSquaredHingeLoss()
    x = torch.rand((B, D), device="cuda", generator=gen)
    rows = torch.arange(B, device="cuda").repeat_interleave(2)
    cols = torch.randint(0, L, (B * 2,), device="cuda", generator=gen)
    y = (torch.stack([rows, cols], dim=1), None)
    p1 = ffi.PrecisionAtK(k=1)
    losses = []
    for it in range(1, 61):
        opt_dense.zero_grad()
        opt_sparse.zero_grad()
        hidden = torch.relu(dense(x))
        loss, scores = sparse.forward_loss(hidden, y, loss_fn, want_scores=(it == 60))
        loss.backward()
        assert dense.weight.grad is not None and torch.isfinite(dense.weight.grad).all() and dense.weight.grad.abs().sum() > 0
        opt_dense.step()
        opt_sparse.step()
        if it % 20 == 1:
            opt_sparse.update_sparse(sparse)
        losses.append(float(loss.detach()))
    p1.update_state(y, scores)
    assert losses[-1] < 0.3 * losses[0]
    assert 0.0 <= p1.result() <= 1.0
    # the listed labels are being pulled apart from the rest
    assert float(scores[rows, cols].mean()) > float(scores.mean()) + 0.1


def test_training_loop_wrapper_rewires_on_schedule(ffi):
    # SparseOptWrapper.train_step (sparse/optimizer.py:43-74): forward, loss, backward, optimizer step, and a rewire of
    # every sparse layer whenever optimizer.iterations % rewire_interval == 1; RewireCallback rewires at epoch starts.
    gen = torch.Generator(device="cuda").manual_seed(5)
    B, D, H, L = 32, 48, 64, 800

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.dense = torch.nn.Linear(D, H)
            # (arrange=False: connections keep their places, so a changed index is a redrawn connection)
            self.sparse = ffi.StratifiedRewireLayerV2(units=L, input_dim=H, connections=L * 8, generator=gen, arrange=False,
                                                      rewire_selector=ffi.FixedFractionSelector(0.05))

        def forward(self, x):
            return self.sparse(torch.relu(self.dense(x)))

    net = Net().cuda()
    model = ffi.SparseOptWrapper(rewire_interval=4, base_model=net)
    with pytest.raises(TypeError):
        model.compile(torch.optim.Adam(net.dense.parameters(), lr=0.01), ffi.SparseSquaredHingeLoss())
    sparse_opt = ffi.SparseAdam(list(net.sparse.parameters()), learning_rate=0.01)
    model.compile([torch.optim.Adam(net.dense.parameters(), lr=0.01), sparse_opt], ffi.SparseSquaredHingeLoss(),
                  metrics=[ffi.PrecisionAtK(k=1)])
    assert model.optimizer is sparse_opt and model.sparse_layers() == [net.sparse]
    x = torch.rand((B, D), device="cuda", generator=gen)
    rows = torch.arange(B, device="cuda").repeat_interleave(2)
    cols = torch.randint(0, L, (B * 2,), device="cuda", generator=gen)
    y = (torch.stack([rows, cols], dim=1), None)
    rewired_at, losses = [], []
    for it in range(1, 13):
        before = net.sparse.kernel_indices.clone()
        out = model.train_step((x, y))
        assert sparse_opt.iterations == it
        if not torch.equal(before, net.sparse.kernel_indices):
            rewired_at.append(it)
            # the optimizer's moments are cleared where connections were redrawn
            changed = before != net.sparse.kernel_indices
            i = sparse_opt._index_of(net.sparse.sparse_weights)
            assert float(sparse_opt._momentums[i][changed].abs().max()) == 0.0
            assert float(sparse_opt._velocities[i][changed].abs().max()) == 0.0
        losses.append(out["loss"])
        assert 0.0 <= out["P_at_1"] <= 1.0
    assert rewired_at == [1, 5, 9]
    assert losses[-1] < losses[0]
    cb = ffi.RewireCallback(model)
    before = net.sparse.kernel_indices.clone()
    cb.on_epoch_begin(0)
    assert torch.equal(before, net.sparse.kernel_indices)
    cb.on_epoch_begin(1)
    assert not torch.equal(before, net.sparse.kernel_indices)


def test_rewire_with_a_selector_that_only_offers_a_mask(ffi):
    # a RewireSelector subclass with select() alone (sparse/layer.py:30-44): the layer redraws exactly the selected
    # connections, keeps their weights, and returns optimizer state cleared at those places
    class EveryThird(ffi.RewireSelector):
        def select(self, weight_values):
            return (torch.arange(weight_values.numel(), device=weight_values.device) % 3) == 0

    gen = torch.Generator(device="cuda").manual_seed(9)
    units, N, K = 40, 50, 6
    layer = ffi.StratifiedRewireLayerV2(units, N, connections=units * K, rewire_selector=EveryThird(), arrange=False,
                                        generator=gen)
    before_idx, before_w = layer.kernel_indices.clone(), layer.kernel_weights.detach().clone()
    m = torch.ones(units * K, device="cuda")
    (new_m,) = layer.rewire([m])
    picked = EveryThird().select(before_w)
    assert torch.equal(layer.kernel_weights.detach(), before_w)
    assert torch.equal(layer.kernel_indices[~picked], before_idx[~picked])
    assert int((layer.kernel_indices[picked] != before_idx[picked]).sum()) > 0.8 * int(picked.sum())
    assert bool(((layer.kernel_indices >= 0) & (layer.kernel_indices < N)).all())
    assert torch.equal(new_m, torch.where(picked, torch.zeros_like(m), m))
    # and the layer still computes what its (edited) variables say
    x = torch.rand((8, N), device="cuda", generator=gen)
    out = layer(x)
    ref = oracle.forward(x.cpu().numpy(), layer.kernel_indices.view(units, K).cpu().numpy().astype(np.int32),
                         layer.kernel_weights.detach().view(units, K).cpu().numpy()) + layer.bias.detach().cpu().numpy()[None, :]
    assert rel_err(out.detach().cpu().numpy(), ref) <= FWD_RTOL


def test_first_generation_layer_keeps_rows_sorted(ffi):
    # StratifiedRewireLayer (sparse/layer.py:339-390): same arithmetic, but a rewiring re-sorts every unit's sources
    # (tf.sparse.reorder) and moves weights and optimizer state with them
    gen = torch.Generator(device="cuda").manual_seed(13)
    units, N, K = 60, 90, 8
    layer = ffi.StratifiedRewireLayer(units, N, connections=units * K, rewire_selector=ffi.FixedFractionSelector(0.2),
                                      generator=gen)
    idx0 = layer.kernel_indices.view(units, K)
    assert bool((idx0[:, 1:] >= idx0[:, :-1]).all())                                  # sorted right after construction
    w_before = layer.kernel_weights.detach().clone()
    idx_before = layer.kernel_indices.clone()
    tag = torch.arange(units * K, device="cuda", dtype=torch.float32) + 1.0          # follows every connection around
    (tag_after,) = layer.rewire([tag])
    idx = layer.kernel_indices.view(units, K)
    assert bool((idx[:, 1:] >= idx[:, :-1]).all())
    # a connection that was not redrawn (tag not cleared) still has its weight and its source, at its new place
    kept = tag_after > 0
    origin = (tag_after[kept] - 1).long()
    assert torch.equal(layer.kernel_weights.detach()[kept], w_before[origin])
    assert torch.equal(layer.kernel_indices[kept], idx_before[origin])
    assert int((~kept).sum()) == int(round(0.2 * units * K)) - 1 or int((~kept).sum()) == int(round(0.2 * units * K))
    # redrawn connections keep their weights too (rows are permutations of the old rows)
    assert torch.equal(torch.sort(layer.kernel_weights.detach().view(units, K), dim=1).values,
                       torch.sort(w_before.view(units, K), dim=1).values)
    x = torch.rand((16, N), device="cuda", generator=gen)
    ref = oracle.forward(x.cpu().numpy(), idx.cpu().numpy().astype(np.int32),
                         layer.kernel_weights.detach().view(units, K).cpu().numpy()) + layer.bias.detach().cpu().numpy()[None, :]
    assert rel_err(layer(x).detach().cpu().numpy(), ref) <= FWD_RTOL
