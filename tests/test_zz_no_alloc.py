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


def _device_inputs(x, lookup, w, transposed):
    feats = np.ascontiguousarray(x.T) if transposed else x
    return tuple(torch.from_numpy(a).cuda() for a in (feats, lookup, w))


def _call(lib, check, name, dx, dl, dw, out, transposed):
    B, L = out.shape
    N = dx.shape[0] if transposed else dx.shape[1]
    K = dl.shape[1]
    sh = torch.cuda.current_stream().cuda_stream
    check(getattr(lib, name)(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K, int(transposed), sh))
    torch.cuda.synchronize()


def _free_bytes():
    free, _total = torch.cuda.mem_get_info()
    return free


@pytest.mark.parametrize("transposed", [False, True])
def test_two_calls_in_a_row_match_the_allocating_entry_point(transposed):
    import oracle

    pkg = load_package()
    assert torch.cuda.is_available()
    lib, check = pkg._lib.lib(), pkg._lib.check
    shapes = [(128, 768, 20000, 32), (37, 254, 513, 12)]      # the second call is smaller: it must not see what the first
    cases = []                                                # left in the shared array
    # the allocating entry point first, for every shape: its results are stored and its workspaces dropped again
    for seed, (B, N, L, K) in enumerate(shapes):
        x, lookup, w = _inputs(B, N, L, K, seed)
        dx, dl, dw = _device_inputs(x, lookup, w, transposed)
        want = torch.full((B, L), float("nan"), device="cuda")
        _call(lib, check, "ffi_forward_f32", dx, dl, dw, want, transposed)
        got = torch.full((B, L), float("nan"), device="cuda")
        cases.append((x, lookup, w, dx, dl, dw, want.cpu().numpy(), got))
    check(lib.ffi_cache_clear())
    assert lib.ffi_cache_bytes() == 0
    torch.cuda.synchronize()
    free_before = _free_bytes()
    for x, lookup, w, dx, dl, dw, want, got in cases:
        _call(lib, check, "ffi_forward_noalloc_f32", dx, dl, dw, got, transposed)
        # nothing was allocated: the library holds no workspace, and the device's free memory has not moved (the
        # outputs were allocated beforehand; torch's allocator is not called in between)
        assert lib.ffi_cache_bytes() == 0
        assert _free_bytes() == free_before
    for x, lookup, w, dx, dl, dw, want, got in cases:
        got = got.cpu().numpy()
        assert not np.isnan(got).any()
        assert np.array_equal(got, want), f"shape {x.shape} {lookup.shape}"       # same kernels: bit for bit
        feats = np.ascontiguousarray(x.T) if transposed else x
        ref = oracle.forward(feats, lookup, w, transposed=transposed)
        assert np.abs(got - ref).max() <= 1e-5 * np.abs(ref).max()


def test_sizes_beyond_the_fixed_array_are_rejected():
    pkg = load_package()
    lib = pkg._lib.lib()
    one = ctypes.c_void_p(256)                   # never dereferenced: the size checks come first
    assert lib.ffi_forward_noalloc_f32(one, one, one, one, 2048, 768, 64, 32, 0, None) == -3     # batch * num_features too large
    assert lib.ffi_forward_noalloc_f32(one, one, one, one, 8, 4096, 64, 32, 0, None) == -3       # wide inputs
    assert lib.ffi_forward_noalloc_f32(None, one, one, one, 8, 64, 64, 32, 0, None) == -1
    assert lib.ffi_forward_noalloc_f32(one, one, one, one, 0, 64, 64, 32, 0, None) == -2
