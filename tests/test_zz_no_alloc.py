"""The allocation-free forward entry point gives ffi_forward_f32's results, call after call on one GPU."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import load_package

pytestmark = pytest.mark.gpu


def _inputs(B, N, L, K, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, N)).astype(np.float32)
    lookup = rng.integers(0, N, (L, K), dtype=np.int64).astype(np.int32)
    w = rng.standard_normal((L, K)).astype(np.float32)
    return x, lookup, w


def _run(lib, check, name, x, lookup, w, transposed):
    B, N = x.shape
    L, K = lookup.shape
    feats = np.ascontiguousarray(x.T) if transposed else x
    dx, dl, dw = (torch.from_numpy(a).cuda() for a in (feats, lookup, w))
    out = torch.full((B, L), float("nan"), device="cuda")
    sh = torch.cuda.current_stream().cuda_stream
    check(getattr(lib, name)(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K, int(transposed), sh))
    torch.cuda.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("transposed", [False, True])
def test_two_calls_in_a_row_match_the_allocating_entry_point(transposed):
    pkg = load_package()
    assert torch.cuda.is_available()
    lib, check = pkg._lib.lib(), pkg._lib.check
    # the second call is smaller: it must not see what the first left in the shared array
    for seed, (B, N, L, K) in enumerate([(128, 768, 20000, 32), (37, 254, 513, 12)]):
        x, lookup, w = _inputs(B, N, L, K, seed)
        want = _run(lib, check, "ffi_forward_f32", x, lookup, w, transposed)
        got = _run(lib, check, "ffi_forward_noalloc_f32", x, lookup, w, transposed)
        assert not np.isnan(got).any()
        assert np.array_equal(got, want), f"shape {(B, N, L, K)}"       # same kernels: bit for bit


def test_sizes_beyond_the_fixed_array_are_rejected():
    pkg = load_package()
    lib = pkg._lib.lib()
    one = ctypes.c_void_p(256)                   # never dereferenced: the size checks come first
    assert lib.ffi_forward_noalloc_f32(one, one, one, one, 2048, 768, 64, 32, 0, None) == -3     # batch * num_features too large
    assert lib.ffi_forward_noalloc_f32(one, one, one, one, 8, 4096, 64, 32, 0, None) == -3       # wide inputs
    assert lib.ffi_forward_noalloc_f32(None, one, one, one, 8, 64, 64, 32, 0, None) == -1
    assert lib.ffi_forward_noalloc_f32(one, one, one, one, 0, 64, 64, 32, 0, None) == -2
