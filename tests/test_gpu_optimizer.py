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
