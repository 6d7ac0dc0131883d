"""Adam step (`ffi_adam_step_f32`) and the SparseAdam object against the numpy oracle
(oracle.adam_step, pinned in tests/test_oracle.py by the closed form of the first step and by
torch.optim.Adam with Keras' epsilon placement).  Gate: 2e-6 absolute on variables of order one,
1e-6 of the largest magnitude on the moments (float32 arithmetic on both sides; fused multiply-adds
differ in the last bit).
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import load_package, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


@pytest.mark.parametrize("count", [1, 3, 4, 1023, 5000 * 32, 1_000_003])
def test_adam_steps_against_oracle(ffi, count):
    rng = np.random.default_rng(count)
    w = rng.normal(size=count).astype(np.float32)
    m, v = np.zeros(count, np.float32), np.zeros(count, np.float32)
    wt, mt, vt = (torch.from_numpy(a.copy()).cuda() for a in (w, m, v))
    for step in range(1, 6):
        g = (rng.normal(size=count) * (rng.random(count) < 0.6)).astype(np.float32)
        w, m, v = oracle.adam_step(w, m, v, g, learning_rate=0.002, step=step)
        ffi.optimizer.adam_step(wt, mt, vt, torch.from_numpy(g).cuda(), 0.002, 0.9, 0.999, 1e-7, step)
        torch.cuda.synchronize()
        np.testing.assert_allclose(wt.cpu().numpy(), w, rtol=0, atol=2e-6)
        assert rel_err(mt.cpu().numpy(), m) <= 1e-6
        assert rel_err(vt.cpu().numpy(), v) <= 1e-6


def test_adam_argument_errors(ffi):
    lib = ffi._lib.lib()
    a = torch.zeros(8, device="cuda")
    p = a.data_ptr()
    sh = torch.cuda.current_stream().cuda_stream
    assert lib.ffi_adam_step_f32(None, p, p, p, 8, 0.1, 0.9, 0.999, 1e-7, 1, sh) == -1
    assert lib.ffi_adam_step_f32(p, p, p, p, 0, 0.1, 0.9, 0.999, 1e-7, 1, sh) == -2
    assert lib.ffi_adam_step_f32(p, p, p, p, 8, 0.1, 0.9, 0.999, 1e-7, 0, sh) == -8       # steps count from 1
    assert lib.ffi_adam_step_f32(p + 4, p, p, p, 4, 0.1, 0.9, 0.999, 1e-7, 1, sh) == -8   # alignment


def test_training_loop_reduces_the_loss_and_rewires(ffi):
    # the reference's train step (sparse/optimizer.py:43-74): forward, loss, gradients, Adam, rewire
    gen = torch.Generator(device="cuda").manual_seed(11)
    B, N, L = 64, 128, 2000
    # arrange=False: positions keep their meaning across a rewire, so the moved ones can be named below
    layer = ffi.StratifiedRewireLayerV2(units=L, input_dim=N, connections=L * 16, generator=gen, arrange=False,
                                        rewire_selector=ffi.FixedFractionSelector(0.05))
    opt = ffi.SparseAdam(list(layer.parameters()), learning_rate=0.01)
    loss_fn = ffi.SparseSquaredHingeLoss()
    x = torch.rand((B, N), device="cuda", generator=gen)
    rows = torch.arange(B, device="cuda").repeat_interleave(3)
    cols = torch.randint(0, L, (B * 3,), device="cuda", generator=gen)
    y = (torch.stack([rows, cols], dim=1), None)
    losses = []
    for it in range(1, 41):
        opt.zero_grad()
        loss, _ = layer.forward_loss(x, y, loss_fn)
        loss.backward()
        opt.step()
        losses.append(float(loss.detach()))
        if it % 10 == 1:
            before = layer.kernel_indices.clone()
            opt.update_sparse(layer)
            moved = (layer.kernel_indices != before)
            i = opt._index_of(layer.kernel_weights)
            if moved.any():
                assert not opt._momentums[i][moved].any() and not opt._velocities[i][moved].any()
    assert losses[-1] < 0.5 * losses[0]
    assert opt.iterations == 40


@pytest.mark.parametrize("force_dense", [False, True])
@pytest.mark.parametrize("shape", [(96, 384, 3000, 32, True), (37, 300, 1001, 7, False), (64, 200, 900, 72, False)])
def test_backward_with_adam_epilogue_matches_backward_then_adam(ffi, shape, force_dense):
    # ffi_backward_sparse_adam_f32 against ffi_backward_sparse_f32 followed by ffi_adam_step_f32 (each of them
    # tested against the oracle on its own), two steps in a row, on the sparse kernels and on the dense ones
    B, N, L, K, tp = shape
    rng = np.random.default_rng(sum(shape[:4]))
    dev = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    x = dev(np.maximum(rng.standard_normal((N, B) if tp else (B, N)), 0).astype(np.float32))
    lookup = dev(rng.integers(0, N, size=(L, K)).astype(np.int32))
    state = {}
    for fused in (False, True):
        w = dev(rng.standard_normal((L, K)).astype(np.float32)) if not state else state["w0"].clone()
        bias = dev(rng.standard_normal(L).astype(np.float32)) if not state else state["b0"].clone()
        if not state:
            state["w0"], state["b0"] = w.clone(), bias.clone()
            state["g"] = []
            for _ in range(2):
                g = rng.standard_normal((B, L)).astype(np.float32)
                g[rng.random((B, L)) >= 0.01] = 0.0
                g[:, 3] = rng.standard_normal(B)
                state["g"].append(dev(g))
        mw, vw, mb, vb = torch.zeros_like(w), torch.zeros_like(w), torch.zeros_like(bias), torch.zeros_like(bias)
        gxs = []
        for step, g in enumerate(state["g"], start=1):
            md = 1e-9 if force_dense else 1.0
            if fused:
                gx, sparse = ffi.optimizer.backward_sparse_adam(x, lookup, w, g.clone(), None, mw, vw, bias, mb, vb,
                                                                0.01, 0.9, 0.999, 1e-7, step, transposed=tp, max_density=md)
            else:
                gx, gw, gb, sparse = ffi.backward_sparse(x, lookup, w, g, transposed=tp, max_density=md, need_bias_grad=True)
                ffi.optimizer.adam_step(w, mw, vw, gw, 0.01, 0.9, 0.999, 1e-7, step)
                ffi.optimizer.adam_step(bias, mb, vb, gb, 0.01, 0.9, 0.999, 1e-7, step)
            assert sparse == (not force_dense)
            gxs.append(gx)
        torch.cuda.synchronize()
        state["fused" if fused else "plain"] = [t.cpu().numpy() for t in (w, mw, vw, bias, mb, vb, *gxs)]
    for a, b in zip(state["fused"], state["plain"]):
        assert rel_err(a, b) <= 1e-5


def test_fused_train_step_follows_the_unfused_loop(ffi):
    # layer.fused_train_step + optimizer.step() against forward_loss / backward / optimizer.step(), three steps
    B, N, L = 64, 128, 2000
    x = torch.rand((B, N), device="cuda", generator=torch.Generator(device="cuda").manual_seed(3))
    rows = torch.arange(B, device="cuda").repeat_interleave(3)
    cols = torch.randint(0, L, (B * 3,), device="cuda", generator=torch.Generator(device="cuda").manual_seed(4))
    y = (torch.stack([rows, cols], dim=1), None)
    loss_fn = ffi.SparseSquaredHingeLoss()
    runs = []
    for fused in (False, True):
        layer = ffi.StratifiedRewireLayerV2(units=L, input_dim=N, connections=L * 16,
                                            generator=torch.Generator(device="cuda").manual_seed(5))
        with torch.no_grad():
            layer.bias.fill_(-1.05)
        opt = ffi.SparseAdam(list(layer.parameters()), learning_rate=0.01)
        losses = []
        for _ in range(3):
            opt.zero_grad()
            if fused:
                loss, _ = layer.fused_train_step(x, y, loss_fn, opt)
            else:
                loss, _ = layer.forward_loss(x, y, loss_fn)
                loss.backward()
            opt.step()
            losses.append(float(loss.detach()))
        torch.cuda.synchronize()
        runs.append((losses, layer.kernel_weights.detach().cpu().numpy(), layer.bias.detach().cpu().numpy()))
    (l0, w0, b0), (l1, w1, b1) = runs
    assert np.allclose(l0, l1, rtol=1e-5)
    assert rel_err(w1, w0) <= 1e-5 and rel_err(b1, b0) <= 1e-5
    assert l0[2] < l0[0]
