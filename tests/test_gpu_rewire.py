"""Rewiring kernels (`ffi_select_threshold_f32`, `ffi_rewire_f32`): the threshold is an exact value (the
k-th smallest magnitude, sparse/layer.py:75-86) and is compared bit for bit with the numpy oracle; the set
of rewired positions is exact too (strict comparison).  The new sources come from a counter-based generator
of this library (TensorFlow's stream cannot be reproduced): they are checked for range, uniformity
(chi-square), determinism per seed and independence between seeds -- PARITY UNPINNED against the
reference's draws by construction.
"""
import numpy as np
import pytest
import torch

import oracle
from conftest import load_package

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


def weights_case(n, seed):
    rng = np.random.default_rng(seed)
    w = (rng.normal(size=n) * rng.choice([1e-3, 1.0, 50.0], size=n)).astype(np.float32)
    w[rng.integers(0, n, n // 10)] = 0.0                 # exact zeros
    w[rng.integers(0, n, n // 10)] = 0.125               # ties
    w[rng.integers(0, n, n // 20)] = -0.125
    return w


@pytest.mark.parametrize("n", [1, 5, 1000, 32 * 5000 + 3, 1 << 21])
def test_threshold_is_the_kth_smallest_magnitude(ffi, n):
    w = weights_case(n, n)
    wt = torch.from_numpy(w).cuda()
    for k in sorted({0, 1, 2, n // 100, n // 3, n - 1, n} & set(range(0, n + 1))):
        thr = ffi.fixed_fan_in_ops.select_threshold(wt, k)
        torch.cuda.synchronize()
        assert thr.cpu().numpy()[0] == oracle.select_threshold(w, k), (n, k)


def test_threshold_argument_errors(ffi):
    lib = ffi._lib.lib()
    w = torch.zeros(8, device="cuda")
    t = torch.zeros(1, device="cuda")
    sh = torch.cuda.current_stream().cuda_stream
    assert lib.ffi_select_threshold_f32(None, 8, 1, t.data_ptr(), sh) == -1
    assert lib.ffi_select_threshold_f32(w.data_ptr(), 0, 0, t.data_ptr(), sh) == -2
    assert lib.ffi_select_threshold_f32(w.data_ptr(), 8, 9, t.data_ptr(), sh) == -8
    assert lib.ffi_rewire_f32(None, w.data_ptr(), None, 0, 8, 4, t.data_ptr(), 0, None, sh) == -1
    assert lib.ffi_rewire_f32(w.data_ptr(), w.data_ptr(), None, 5, 8, 4, t.data_ptr(), 0, None, sh) == -1


def test_rewire_changes_exactly_the_selected_positions(ffi):
    L, K, N = 3000, 32, 768
    n = L * K
    w = weights_case(n, 7)
    rng = np.random.default_rng(8)
    lookup = rng.integers(0, N, n).astype(np.int32)
    m, v = rng.normal(size=n).astype(np.float32), rng.random(n).astype(np.float32) + 0.1
    k = n // 3                                          # beyond the exact zeros, which nothing is strictly below
    thr = oracle.select_threshold(w, k)
    sel = oracle.rewire_selection(w, thr)
    lt, wt, mt, vt = (torch.from_numpy(a.copy()).cuda() for a in (lookup, w, m, v))
    thr_t = ffi.fixed_fan_in_ops.select_threshold(wt, k)
    changed = ffi.fixed_fan_in_ops.rewire_connections(lt, wt, [mt, vt], N, thr_t, seed=1234)
    torch.cuda.synchronize()
    new = lt.cpu().numpy()
    assert int(changed.cpu()[0]) == sel.sum()
    assert np.array_equal(new[~sel], lookup[~sel])                       # untouched elsewhere
    assert new[sel].min() >= 0 and new[sel].max() < N
    assert np.array_equal(wt.cpu().numpy(), w)                           # weights keep their values
    for arr_t, arr in ((mt, m), (vt, v)):
        got = arr_t.cpu().numpy()
        assert not got[sel].any() and np.array_equal(got[~sel], arr[~sel])
    # the same seed gives the same draws, another seed different ones
    lt2 = torch.from_numpy(lookup.copy()).cuda()
    ffi.fixed_fan_in_ops.rewire_connections(lt2, wt, [], N, thr_t, seed=1234)
    lt3 = torch.from_numpy(lookup.copy()).cuda()
    ffi.fixed_fan_in_ops.rewire_connections(lt3, wt, [], N, thr_t, seed=1235)
    torch.cuda.synchronize()
    assert np.array_equal(lt2.cpu().numpy(), new)
    assert (lt3.cpu().numpy()[sel] != new[sel]).mean() > 0.99


def test_new_sources_are_uniform(ffi):
    # everything is rewired (threshold above every magnitude): chi-square of the sources against uniform
    n, N = 1 << 22, 1000
    wt = torch.zeros(n, device="cuda")
    lt = torch.zeros(n, dtype=torch.int32, device="cuda")
    thr = torch.ones(1, device="cuda")
    ffi.fixed_fan_in_ops.rewire_connections(lt, wt, [], N, thr, seed=99)
    torch.cuda.synchronize()
    counts = np.bincount(lt.cpu().numpy(), minlength=N)
    assert counts.shape[0] == N
    expected = n / N
    chi2 = ((counts - expected) ** 2 / expected).sum()
    # N - 1 = 999 degrees of freedom: mean 999, standard deviation 44.7; 6 sigma
    assert abs(chi2 - (N - 1)) < 6 * np.sqrt(2 * (N - 1))
    # neighbouring positions are not correlated
    a = lt.cpu().numpy().astype(np.float64)
    assert abs(np.corrcoef(a[:-1], a[1:])[0, 1]) < 0.005


def test_layer_rewire_through_the_library(ffi):
    gen = torch.Generator(device="cuda").manual_seed(21)
    layer = ffi.StratifiedRewireLayerV2(units=2000, input_dim=300, connections=2000 * 16, generator=gen, arrange=False,
                                        rewire_selector=ffi.FixedFractionSelector(0.1))
    w = layer.kernel_weights.detach().cpu().numpy()
    before = layer.kernel_indices.cpu().numpy().copy()
    m = torch.ones_like(layer.kernel_weights.data)
    sel = oracle.rewire_selection(w, oracle.select_threshold(w, int(round(0.1 * w.size))))
    (new_m,) = layer.rewire([m])
    torch.cuda.synchronize()
    after = layer.kernel_indices.cpu().numpy()
    assert np.array_equal(after[~sel], before[~sel]) and 0 <= after.min() and after.max() < 300
    assert np.array_equal(new_m.cpu().numpy() == 0, sel) and bool((m == 1).all())      # the input is not modified
    # the mask form of the selector selects the same positions
    assert np.array_equal(layer.rewire_selector.select(torch.from_numpy(w).cuda()).cpu().numpy(), sel)
    # the layer still trains after the edit (plan rebuilt through the fingerprint)
    x = torch.rand((8, 300), device="cuda")
    layer(x).sum().backward()
    torch.cuda.synchronize()
    assert torch.isfinite(layer.kernel_weights.grad).all()
