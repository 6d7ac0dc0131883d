"""Parity of the HIP kernels (called through the C ABI) with the CPU oracle on identical inputs.

Gates: forward max|a-b|/max|ref| <= 1e-5, gradients <= 1e-4 (fp32); plus the reference's own
absolute gates on its own data law (1e-5 forward, 1.5e-5 gradients,
testing/test_case_templates.h:82,139-140) on the reference's shape grid.
"""
import ctypes
import glob
import json
import os

import numpy as np
import pytest
import torch

import oracle
from conftest import GOLDEN, REFERENCE_SHAPES, load_package, reference_law_inputs, rel_err

pytestmark = pytest.mark.gpu

FWD_RTOL = 1e-5
GRAD_RTOL = 1e-4


@pytest.fixture(scope="module")
def ffi():
    pkg = load_package()
    assert torch.cuda.is_available(), "these tests need the MI355X"
    return pkg


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def stream():
    return torch.cuda.current_stream().cuda_stream


def hip_forward(ffi, x, lookup, w, transposed):
    """Direct C-ABI call; the output buffer is pre-filled with NaN so an unwritten element shows."""
    B = x.shape[1] if transposed else x.shape[0]
    N = x.shape[0] if transposed else x.shape[1]
    L, K = lookup.shape
    dx, dl, dw = dev(x), dev(lookup), dev(w)
    out = torch.full((B, L), float("nan"), device="cuda")
    ffi._lib.check(ffi._lib.lib().ffi_forward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(),
                                                  B, N, L, K, int(transposed), stream()))
    torch.cuda.synchronize()
    return out.cpu().numpy()


def hip_backward(ffi, x, lookup, w, g, transposed):
    B = x.shape[1] if transposed else x.shape[0]
    N = x.shape[0] if transposed else x.shape[1]
    L, K = lookup.shape
    dx, dl, dw, dg = dev(x), dev(lookup), dev(w), dev(g)
    gx = torch.full(tuple(x.shape), float("nan"), device="cuda")
    gw = torch.full((L, K), float("nan"), device="cuda")
    ffi._lib.check(ffi._lib.lib().ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(),
                                                   gx.data_ptr(), gw.data_ptr(), B, N, L, K, int(transposed), stream()))
    torch.cuda.synchronize()
    return gx.cpu().numpy(), gw.cpu().numpy()


def test_known_answer_forward_exact(ffi):
    # testing/test.cpp:13-47, exact equality, both layouts, int32 and uint32 ids
    with open(os.path.join(GOLDEN, "kat_forward.json")) as f:
        kat = json.load(f)
    x = np.array(kat["features"], dtype=np.float32)
    lookup = np.array(kat["lookup"], dtype=np.int32)
    w = np.array(kat["weights"], dtype=np.float32)
    expected = np.array(kat["expected"], dtype=np.float32)
    assert np.array_equal(hip_forward(ffi, x, lookup, w, False), expected)
    assert np.array_equal(hip_forward(ffi, np.ascontiguousarray(x.T), lookup, w, True), expected)
    out = ffi.fan_in_sparse_matmul(dev(x), dev(lookup).view(torch.uint32), dev(w))
    assert np.array_equal(out.cpu().numpy(), expected)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "dense_*.npz"))))
@pytest.mark.parametrize("transposed", [False, True])
def test_golden_dense_fixtures(ffi, path, transposed):
    z = np.load(path)
    x, lookup, w, g = z["features"], z["lookup"], z["weights"], z["out_grad"]
    xin = np.ascontiguousarray(x.T) if transposed else x
    out = hip_forward(ffi, xin, lookup, w, transposed)
    gx, gw = hip_backward(ffi, xin, lookup, w, g, transposed)
    if transposed:
        gx = gx.T
    assert np.abs(out - z["result"]).max() < 1e-5
    assert np.abs(gx - z["feature_grad"]).max() < 1.5e-5
    assert np.abs(gw - z["weight_grad"]).max() < 1.5e-5


@pytest.mark.parametrize("shape", REFERENCE_SHAPES)
@pytest.mark.parametrize("transposed", [False, True])
def test_reference_shape_grid(ffi, shape, transposed):
    # testing/test.cpp:50-89 with the reference tests' own input law and absolute gates
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K)
    xin = np.ascontiguousarray(x.T) if transposed else x
    print(f"case shape={shape} transposed={transposed}", flush=True)
    out = hip_forward(ffi, xin, lookup, w, transposed)
    gx, gw = hip_backward(ffi, xin, lookup, w, g, transposed)
    o_out = oracle.forward(xin, lookup, w, transposed=transposed)
    o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
    assert not np.isnan(out).any() and not np.isnan(gx).any() and not np.isnan(gw).any()
    assert np.abs(out - o_out).max() < 1e-5
    assert np.abs(gw - o_gw).max() < 1.5e-5
    if L < 1_000_000:
        assert np.abs(gx - o_gx).max() < 1.5e-5
    else:
        # 4,000,000 labels onto 32 columns: ~250k terms of size <= 1 per sum, where fp32 sums in a
        # different association differ by more than the absolute gate; compare against the
        # double-precision sum instead, relative to its magnitude
        t_gx = oracle.input_grad(xin, lookup, w, g, transposed=transposed, f64=True)
        assert rel_err(gx, t_gx) < GRAD_RTOL
    assert rel_err(out, o_out) <= FWD_RTOL
    assert rel_err(gw, o_gw) <= GRAD_RTOL


@pytest.mark.parametrize("shape", [(12, 8, 32, 16), (127, 254, 513, 73)])
def test_layouts_agree(ffi, shape):
    # testing/test.cpp:91-166
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=5)
    xt = np.ascontiguousarray(x.T)
    assert np.abs(hip_forward(ffi, x, lookup, w, False) - hip_forward(ffi, xt, lookup, w, True)).max() < 1.5e-5
    gx, gw = hip_backward(ffi, x, lookup, w, g, False)
    gxt, gwt = hip_backward(ffi, xt, lookup, w, g, True)
    assert np.abs(gx - gxt.T).max() < 1.5e-5 and np.abs(gw - gwt).max() < 1.5e-5


# shapes that steer the library through each of its code paths:
#   narrow inputs (LDS tile kernels), wide inputs (generic kernels), the tiled and the global plan,
#   partly filled batch tiles, fan-ins below / across / beyond the 32-connection register chunk,
#   fewer labels than one tile, more than 1024 columns (one tiled plan per half of the columns, tile forward/weight-grad),
#   the forward kernel over batch tiles of 64
PATH_SHAPES = [
    (300, 700, 5000, 32),      # 10 batch tiles, the last one partly filled
    (33, 96, 9, 5),            # fewer labels than lanes, odd fan-in
    (64, 1100, 3000, 12),      # N > 1024: tile forward / weight-grad, a tiled plan for each half of the columns
    (40, 1216, 2500, 36),      # largest N that still fits the LDS tile
    (48, 1300, 2000, 20),      # wide: generic kernels, one batch entry per lane, rows padded to 128 bytes
    (64, 1400, 700, 16),       # wide, rows already aligned: [N,B] features used in place
    (70, 1500, 900, 9),        # wide, two batch entries per lane, the second half nearly empty
    (200, 2000, 600, 33),      # wide, two batch passes
    (7, 64, 70000, 3),         # many tiles of a tiny column set
    (128, 512, 4100, 100),     # four register chunks per label, tail of 4
    (64, 768, 900, 300),       # a tile's weights far beyond what its threads carry in registers: most are copied behind the barrier
    (96, 200, 3000, 7),        # weights of a tile not a multiple of 16 bytes: staged word by word
    # several workgroups of the input-gradient kernel per CU (narrow layers):
    (300, 200, 9000, 16),      # ten batch tiles, weights in slot order: four workgroups of 256 threads
    (96, 128, 12000, 16),      # three batch tiles, weights in LDS: six workgroups of 128 threads, a share of the LDS each
    (160, 256, 9000, 16),      # five batch tiles, weights in LDS (fan-in below 32): three workgroups of 256 threads
    (160, 256, 9000, 32),      # five batch tiles, weights in slot order: four workgroups of 256 threads
    (288, 64, 20000, 8),       # nine batch tiles, weights in slot order: sixteen workgroups of 64 threads
    # forward over batch tiles of 64 (N <= 608; from 192 samples, from 128 with a fan-in of 64 or more, fan-in 48 / 80 / 112):
    (256, 512, 5000, 64),      # whole tiles, vector loads
    (200, 608, 3100, 21),      # the widest input of that path, fourth tile partly filled, odd fan-in (scalar loads)
    (33, 40, 2100, 48),        # one sample beyond a 32-tile; three half chunks of 16
    (193, 300, 1500, 8),       # one sample in the fourth 64-tile; fan-in below a half chunk
    (130, 256, 2000, 72),      # fan-in with a tail of 8 behind four half chunks
    # full chunks loaded by quads from rows that are only 4-byte aligned (fan-in no multiple of four), last chunk one by one:
    (64, 768, 3000, 33), (40, 512, 2000, 63), (200, 300, 1500, 35), (130, 256, 2000, 67),
    # the 32-sample kernel's build for a fan-in below one chunk (loads by quads):
    (100, 608, 3100, 24), (65, 300, 1500, 8), (128, 768, 5000, 16), (50, 1000, 700, 28), (40, 640, 900, 4),
]


@pytest.mark.parametrize("shape", PATH_SHAPES)
@pytest.mark.parametrize("transposed", [False, True])
def test_code_paths(ffi, shape, transposed):
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=B + N)
    xin = np.ascontiguousarray(x.T) if transposed else x
    print(f"case shape={shape} transposed={transposed}", flush=True)
    out = hip_forward(ffi, xin, lookup, w, transposed)
    gx, gw = hip_backward(ffi, xin, lookup, w, g, transposed)
    assert rel_err(out, oracle.forward(xin, lookup, w, transposed=transposed)) <= FWD_RTOL
    o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
    assert rel_err(gw, o_gw) <= GRAD_RTOL
    assert rel_err(gx, o_gx) <= GRAD_RTOL


@pytest.mark.parametrize("shape", [(100, 608, 3100, 21),     # 32-sample tiles, the fourth holds 4 samples; loads one by one
                                   (100, 608, 3100, 24),     # the same with loads by quads (fan-in below one chunk)
                                   (200, 608, 3100, 21),     # 64-sample tiles, the fourth holds 8 samples
                                   (70, 768, 2000, 32),      # 32-sample tiles, full chunks
                                   (70, 2000, 900, 32)])     # wide input
@pytest.mark.parametrize("transposed", [False, True])
def test_partly_filled_batch_tiles_write_nothing_behind_the_result(ffi, shape, transposed):
    # the rows of a batch tile that lie past the batch must not be stored: the result is a view of a larger buffer whose
    # rows behind it (and a guard row in front) hold a sentinel
    B, N, L, K = shape
    x, lookup, w, _ = reference_law_inputs(B, N, L, K, seed=B + K)
    xin = np.ascontiguousarray(x.T) if transposed else x
    dx, dl, dw = dev(xin), dev(lookup), dev(w)
    sentinel = 12345.0
    whole = torch.full((1 + B + 64, L), sentinel, device="cuda")
    out = whole[1:1 + B]
    print(f"case shape={shape} transposed={transposed}", flush=True)
    ffi._lib.check(ffi._lib.lib().ffi_forward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K,
                                                  int(transposed), stream()))
    torch.cuda.synchronize()
    assert bool((whole[0] == sentinel).all()) and bool((whole[1 + B:] == sentinel).all())
    assert rel_err(out.cpu().numpy(), oracle.forward(xin, lookup, w, transposed=transposed)) <= FWD_RTOL


@pytest.mark.parametrize("option", [("wgrad_units", 3), ("wgrad_units", 4), ("wgrad_stream", -1), ("fwd_lane64", -1),
                                    ("plan_weights_in_lds", -1), ("plan_weights_in_lds", 1), ("workgroups_per_cu", 1),
                                    ("plan_sorted_columns", -1), ("plan_sorted_columns", 1)])
@pytest.mark.parametrize("shape", [(128, 512, 9000, 32), (64, 768, 5000, 16), (256, 256, 6000, 32)])
def test_overridden_kernel_choices_keep_parity(ffi, option, shape):
    # every alternative a benchmark sweep can force computes the same layer
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=N + K)
    lib = ffi._lib.lib()
    print(f"case option={option} shape={shape}", flush=True)
    ffi._lib.check(lib.ffi_set_option(option[0].encode(), option[1]))
    try:
        out = hip_forward(ffi, x, lookup, w, False)
        gx, gw = hip_backward(ffi, x, lookup, w, g, False)
    finally:
        ffi._lib.check(lib.ffi_set_option(option[0].encode(), 0))
    assert rel_err(out, oracle.forward(x, lookup, w)) <= FWD_RTOL
    o_gx, o_gw = oracle.backward(x, lookup, w, g)
    assert rel_err(gw, o_gw) <= GRAD_RTOL and rel_err(gx, o_gx) <= GRAD_RTOL


@pytest.mark.parametrize("shape", [(128, 768, 9000, 32),      # the headline's columns and fan-in: 16 tiles of twelve slices
                                   (100, 700, 4000, 24),      # columns no multiple of 64: the last slice's spare threads take part in the sorting
                                   (64, 512, 3000, 64),
                                   (33, 100, 2500, 8),        # two slices, two batch tiles with one sample in the second
                                   (96, 128, 12000, 16),      # several workgroups per CU
                                   (32, 768, 40, 32),         # fewer labels than threads: the exchange of sums needs more LDS than the tile
                                   (7, 64, 70000, 3),         # one slice: nothing to sort into, same results
                                   (64, 1100, 3000, 12),      # two column windows, each with its own order per tile
                                   (128, 768, 2000, 300)])    # tiles of a hundred labels
@pytest.mark.parametrize("ids", ["uniform", "duplicates", "long_tail", "one_parity_per_half"])
def test_plans_that_sort_a_tiles_columns_by_length(ffi, shape, ids):
    # plans in the weights-in-LDS form may hand the columns to the walking kernel's threads anew in every tile, longest
    # first; the library takes them where they pay (many labels), here they are forced on shapes the oracle finishes quickly
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=N + L + K)
    rng = np.random.default_rng(L)
    if ids == "duplicates":                                   # every fourth label lists one of its columns twice
        for j in range(0, L, 4):
            a, b = rng.choice(K, 2, replace=False) if K > 1 else (0, 0)
            lookup[j, a] = lookup[j, b]
    elif ids == "long_tail":                                  # a few columns take most connections: not too skewed for the tiled form
        lookup = np.where(rng.random((L, K)) < 0.3, rng.integers(0, max(1, N // 16), (L, K)), lookup).astype(np.int32)
    elif ids == "one_parity_per_half":                        # see test_columns_fed_by_one_label_parity
        half = max(1, N // 2)
        lookup = (lookup % half + (np.arange(L)[:, None] % 2) * half).astype(np.int32) % N
    lib = ffi._lib.lib()
    print(f"case shape={shape} ids={ids}", flush=True)
    results = {}
    for value in (1, -1):
        ffi._lib.check(lib.ffi_set_option(b"plan_weights_in_lds", 1))
        ffi._lib.check(lib.ffi_set_option(b"plan_sorted_columns", value))
        try:
            dx, dl, dw, dg = dev(x), dev(lookup), dev(w), dev(g)
            plan = ctypes.c_void_p()
            ffi._lib.check(lib.ffi_plan_create(dl.data_ptr(), L, K, N, B, stream(), ctypes.byref(plan)))
            info = (ctypes.c_int64 * 8)()
            ffi._lib.check(lib.ffi_plan_info(plan, info))
            runs = []
            for _ in range(2):
                gx = torch.full_like(dx, float("nan"))
                ffi._lib.check(lib.ffi_input_grad_planned_f32(plan, dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B, 0, stream()))
                torch.cuda.synchronize()
                runs.append(gx.cpu().numpy())
            ffi._lib.check(lib.ffi_plan_destroy(plan))
            assert np.array_equal(runs[0], runs[1])           # reproducible bit for bit
            results[value] = (runs[0], info[0], info[1], info[5])
            # the stateless route, and an edit of the lookup in place behind it
            got_gx, got_gw = hip_backward(ffi, x, lookup, w, g, False)
            o_gx, o_gw = oracle.backward(x, lookup, w, g)
            assert rel_err(got_gx, o_gx) <= GRAD_RTOL and rel_err(got_gw, o_gw) <= GRAD_RTOL
        finally:
            ffi._lib.check(lib.ffi_set_option(b"plan_sorted_columns", 0))
            ffi._lib.check(lib.ffi_set_option(b"plan_weights_in_lds", 0))
    o_gx = oracle.input_grad(x, lookup, w, g)
    assert rel_err(results[1][0], o_gx) <= GRAD_RTOL and rel_err(results[-1][0], o_gx) <= GRAD_RTOL
    if results[1][1] and results[1][2] and N > 64:
        # tiled, weights in LDS: sorting never needs more slot rows than thread t <-> column t
        assert results[1][3] <= results[-1][3]


@pytest.mark.parametrize("shape", [(300, 700, 5000, 32), (33, 96, 9, 5), (128, 512, 4100, 100), (40, 1216, 2500, 36), (64, 1100, 3000, 12),
                                   (48, 1300, 2000, 20),
                                   (96, 512, 20000, 64),     # two chunks per label, both held by one thread
                                   (64, 300, 2600, 128),      # four chunks per label
                                   (32, 64, 360000, 32),      # enough units per CU for the kernel that holds three units per thread
                                   (70, 768, 5000, 96),       # three chunks per label: unit numbers wrap inside a wavefront (row-by-row out_grad fetches)
                                   (129, 763, 70, 32),        # one sample in the fifth batch tile, odd width (x staged through registers), 70 labels
                                   (32, 768, 64, 8),          # the fewest labels the streaming kernel takes
                                   (64, 776, 4000, 32),       # x tile and out_grad slices do not fit the LDS together: the kernel without slices
                                   # a last chunk that is partly filled is walked as far as it is filled (8, 16 or 24 connections):
                                   (64, 768, 4000, 8), (64, 768, 4000, 12), (100, 512, 3000, 20), (33, 640, 5000, 24), (64, 256, 3000, 3),
                                   (96, 512, 3000, 40), (64, 512, 3000, 52), (40, 300, 2600, 63),        # two chunks
                                   (64, 300, 2600, 104), (32, 256, 2000, 97), (48, 200, 1500, 120)])    # four chunks
def test_planned_weight_grad_code_paths(ffi, shape):
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=B + K)
    dl, dg = dev(lookup), dev(g)
    lib = ffi._lib.lib()
    plan = ctypes.c_void_p()
    ffi._lib.check(lib.ffi_plan_create(dl.data_ptr(), L, K, N, B, stream(), ctypes.byref(plan)))
    try:
        for transposed in (0, 1):
            xin = np.ascontiguousarray(x.T) if transposed else x
            dx = dev(xin)
            gw = torch.full((L, K), float("nan"), device="cuda")
            ffi._lib.check(lib.ffi_weight_grad_planned_f32(plan, dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), gw.data_ptr(), B,
                                                           transposed, stream()))
            torch.cuda.synchronize()
            assert rel_err(gw.cpu().numpy(), oracle.weight_grad(xin, lookup, w, g, transposed=bool(transposed))) <= GRAD_RTOL
    finally:
        ffi._lib.check(lib.ffi_plan_destroy(plan))


def test_columns_fed_by_one_label_parity(ffi):
    # even labels connect to the lower half of the columns only, odd labels to the upper half: every
    # column's connections come from labels of one parity, the worst case for the plan's
    # alternating slot order (every second slot of a column is padding)
    B, N, L, K = 70, 256, 5001, 16
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=31)
    half = N // 2
    lookup = (lookup % half + (np.arange(L)[:, None] % 2) * half).astype(np.int32)
    for transposed in (False, True):
        xin = np.ascontiguousarray(x.T) if transposed else x
        gx, gw = hip_backward(ffi, xin, lookup, w, g, transposed)
        o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
        assert rel_err(gx, o_gx) <= GRAD_RTOL
        assert rel_err(gw, o_gw) <= GRAD_RTOL


def test_labels_that_list_a_column_twice(ffi):
    # duplicates inside a row are legal and accumulate (backward.cpp:58-72 adds every connection).  The plan's fast slot
    # placement works on a bitmap of (column, label) and hands tiles with such a label to the exact placement: here
    # every third tile has some, the others none.
    B, N, L, K = 48, 256, 6000, 16
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=123)
    rng = np.random.default_rng(9)
    for j in rng.choice(L, 40, replace=False):
        if (j // 256) % 3 == 0:
            a, b = rng.choice(K, 2, replace=False)
            lookup[j, a] = lookup[j, b]
    lookup[17, :] = 5                                     # and one label that is a single column K times
    gx, gw = hip_backward(ffi, x, lookup, w, g, False)
    o_gx, o_gw = oracle.backward(x, lookup, w, g)
    assert rel_err(gx, o_gx) <= GRAD_RTOL
    assert rel_err(gw, o_gw) <= GRAD_RTOL
    assert rel_err(hip_forward(ffi, x, lookup, w, False), oracle.forward(x, lookup, w)) <= FWD_RTOL


def test_skewed_lookup_uses_the_global_plan(ffi):
    # every connection points at one of two columns: the padded tiled plan would explode, the
    # library must fall back to the global column order and still be exact to tolerance
    B, N, L, K = 40, 200, 6000, 8
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=77)
    lookup = np.where(lookup % 2 == 0, 3, 150).astype(np.int32)
    gx, gw = hip_backward(ffi, x, lookup, w, g, False)
    t_gx = oracle.input_grad(x, lookup, w, g, f64=True)
    assert rel_err(gx, t_gx) <= GRAD_RTOL
    assert np.array_equal(gx[:, [0, 1, 2, 4, 149, 151]], np.zeros((B, 6), dtype=np.float32))
    assert rel_err(gw, oracle.weight_grad(x, lookup, w, g)) <= GRAD_RTOL
    assert rel_err(hip_forward(ffi, x, lookup, w, False), oracle.forward(x, lookup, w)) <= FWD_RTOL


@pytest.mark.parametrize("case", ["uniform", "upper_half_unused", "lower_half_skewed", "upper_half_skewed", "rewired"])
def test_inputs_of_more_than_1024_columns_take_one_plan_per_half(ffi, case):
    # 1,025 to 1,216 columns: the input gradient walks two tiled plans, one per half of the columns (a workgroup has at
    # most 1,024 threads, one per column).  Either half may be unused, or too skewed for the tiled form (then the global
    # column order serves all columns), and a lookup edited in place must be noticed for both.
    B, N, L, K = 70, 1100, 5000, 16
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=55)
    split = ((N + 1) // 2 + 63) // 64 * 64
    if case == "upper_half_unused":
        lookup = (lookup % split).astype(np.int32)
    elif case == "lower_half_skewed":
        lookup = np.where(lookup < split, 7, lookup).astype(np.int32)
    elif case == "upper_half_skewed":
        lookup = np.where(lookup >= split, N - 1, lookup).astype(np.int32)
    lib = ffi._lib.lib()
    dx, dl, dw, dg = dev(x), dev(lookup), dev(w), dev(g)
    plan = ctypes.c_void_p()
    ffi._lib.check(lib.ffi_plan_create(dl.data_ptr(), L, K, N, B, stream(), ctypes.byref(plan)))
    info = (ctypes.c_int64 * 8)()
    ffi._lib.check(lib.ffi_plan_info(plan, info))
    assert info[0] == (0 if case.endswith("skewed") else 1)
    gx = torch.full_like(dx, float("nan"))
    ffi._lib.check(lib.ffi_input_grad_planned_f32(plan, dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B, 0, stream()))
    torch.cuda.synchronize()
    ffi._lib.check(lib.ffi_plan_destroy(plan))
    assert rel_err(gx.cpu().numpy(), oracle.input_grad(x, lookup, w, g)) <= GRAD_RTOL
    if case == "upper_half_unused":
        assert not gx[:, split:].any()
    # the cached route, both layouts; then an edit of the lookup in place that moves connections between the halves
    for transposed in (False, True):
        xin = np.ascontiguousarray(x.T) if transposed else x
        got_gx, got_gw = hip_backward(ffi, xin, lookup, w, g, transposed)
        o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
        assert rel_err(got_gx, o_gx) <= GRAD_RTOL and rel_err(got_gw, o_gw) <= GRAD_RTOL
    if case == "rewired":
        gx2 = torch.empty_like(dx)

        def run():
            ffi._lib.check(lib.ffi_input_grad_f32(dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx2.data_ptr(), B, N, L, K, 0, stream()))
            torch.cuda.synchronize()
            return gx2.cpu().numpy().copy()

        assert rel_err(run(), oracle.input_grad(x, lookup, w, g)) <= GRAD_RTOL
        rng = np.random.default_rng(8)
        lookup2 = lookup.copy()
        lookup2[rng.integers(0, L, 700), rng.integers(0, K, 700)] = rng.integers(0, N, 700)
        dl.copy_(dev(lookup2))
        for _ in range(3):                                   # recomputed from the lookup, then from the rebuilt plans
            assert rel_err(run(), oracle.input_grad(x, lookup2, w, g)) <= GRAD_RTOL
        assert np.array_equal(run(), run())


def test_unaligned_buffers(ffi):
    # pointers that are only 4-byte aligned take the scalar-load variants of the kernels
    B, N, L, K = 64, 128, 1500, 32
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=88)
    lib = ffi._lib.lib()

    def shifted(a):
        flat = torch.empty(a.size + 1, dtype=torch.from_numpy(a).dtype, device="cuda")
        view = flat[1:].view(*a.shape)
        view.copy_(torch.from_numpy(a))
        return flat, view

    keep = [shifted(a) for a in (x, lookup, w, g)]
    dx, dl, dw, dg = (v for _, v in keep)
    assert dw.data_ptr() % 16 == 4
    fo, out = shifted(np.zeros((B, L), np.float32))
    fgx, gx = shifted(np.zeros((B, N), np.float32))
    fgw, gw = shifted(np.zeros((L, K), np.float32))
    ffi._lib.check(lib.ffi_forward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K, 0, stream()))
    ffi._lib.check(lib.ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(),
                                        gw.data_ptr(), B, N, L, K, 0, stream()))
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), oracle.forward(x, lookup, w)) <= FWD_RTOL
    o_gx, o_gw = oracle.backward(x, lookup, w, g)
    assert rel_err(gx.cpu().numpy(), o_gx) <= GRAD_RTOL and rel_err(gw.cpu().numpy(), o_gw) <= GRAD_RTOL


SCALED_CONFIGS = [
    # (config, labels used here) — same B, N, K and input laws as the benchmark configurations,
    # label count cut so that the CPU oracle finishes in seconds
    ("c1", 131_072),
    ("c2", 100_003),
    ("c3", 40_009),
    ("c4", 20_011),
]


@pytest.mark.parametrize("name,labels", SCALED_CONFIGS)
@pytest.mark.parametrize("transposed", [False, True])
def test_benchmark_configs_against_oracle(ffi, name, labels, transposed):
    from ecml23_sparse_amd import synth
    cfg = synth.CONFIGS[name]
    t = synth.make_inputs(cfg, seed=42, device="cpu", transposed=transposed, num_units=labels)
    x, lookup, w, g = (t[k].numpy() for k in ("features", "lookup", "weights", "out_grad"))
    print(f"case config={name} labels={labels} transposed={transposed}", flush=True)
    out = hip_forward(ffi, x, lookup, w, transposed)
    gx, gw = hip_backward(ffi, x, lookup, w, g, transposed)
    assert rel_err(out, oracle.forward(x, lookup, w, transposed=transposed)) <= FWD_RTOL
    o_gx, o_gw = oracle.backward(x, lookup, w, g, transposed=transposed)
    assert rel_err(gw, o_gw) <= GRAD_RTOL
    assert rel_err(gx, o_gx) <= GRAD_RTOL


def test_input_grad_is_deterministic_and_zero_on_untouched_columns(ffi):
    B, N, L, K = 64, 300, 5000, 24
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=21)
    lookup = (lookup % 250).astype(np.int32)          # columns 250..299 never referenced
    gx1, _ = hip_backward(ffi, x, lookup, w, g, False)
    gx2, _ = hip_backward(ffi, x, lookup, w, g, False)
    assert np.array_equal(gx1, gx2)
    assert np.array_equal(gx1[:, 250:], np.zeros((B, 50), dtype=np.float32))
    assert rel_err(gx1, oracle.input_grad(x, lookup, w, g)) <= GRAD_RTOL


@pytest.mark.parametrize("shape", [(32, 128, 3000, 16),
                                   (100, 768, 9000, 32),      # several label streams, a partly filled batch tile
                                   (20, 300, 900, 300),       # the recomputing kernel's tiles hold 64 labels
                                   (8, 64, 40, 5000),         # ... 4 labels
                                   (4, 64, 6, 25000),         # a label's connections alone exceed the LDS: one thread per connection
                                   (40, 2000, 700, 12)])      # wide input
def test_in_place_rewiring_is_picked_up(ffi, shape):
    # the layer rewires by overwriting entries of the same index variable
    # (sparse/custom_layer.py:32-43): same pointer, new contents
    B, N, L, K = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=31)
    dx, dl, dw, dg = dev(x), dev(lookup), dev(w), dev(g)
    gx = torch.empty_like(dx)
    lib = ffi._lib.lib()

    def run():
        ffi._lib.check(lib.ffi_input_grad_f32(dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(),
                                               B, N, L, K, 0, stream()))
        torch.cuda.synchronize()
        return gx.cpu().numpy().copy()

    before = run()
    assert rel_err(before, oracle.input_grad(x, lookup, w, g)) <= GRAD_RTOL
    rng = np.random.default_rng(4)
    rows, cols = rng.integers(0, L, 500), rng.integers(0, K, 500)
    lookup2 = lookup.copy()
    lookup2[rows, cols] = rng.integers(0, N, 500)
    dl.copy_(dev(lookup2))                              # in place: data_ptr unchanged
    after = run()                                       # served by the kernels that recompute from the lookup
    assert rel_err(after, oracle.input_grad(x, lookup2, w, g)) <= GRAD_RTOL
    assert not np.array_equal(before, after)
    rebuilt = run()                                     # the host has seen the verdict: the plan is rebuilt
    assert rel_err(rebuilt, oracle.input_grad(x, lookup2, w, g)) <= GRAD_RTOL
    assert np.array_equal(rebuilt, run())               # plan-driven again: bit-identical from call to call


def _label_sample_errors(lookup, w, g, x, gx, gw, B, N, K, labels):
    """weight gradient of a label sample and the full input gradient against the oracle ([N,B] features)"""
    o_gw = oracle.weight_grad(x, lookup[labels], w[labels], np.ascontiguousarray(g[:, labels]), transposed=True)
    o_gx = oracle.input_grad(x, lookup, w, g, transposed=True)
    return rel_err(gw[labels], o_gw), rel_err(gx, o_gx)


@pytest.mark.parametrize("route", ["library", "foreign", "foreign_announced"])
def test_rewiring_at_scale_both_routes(ffi, route):
    # 262,144 labels x fan-in 32 over 768 columns, batch 64 (weights-in-LDS plan, streaming weight gradient).
    # library: ffi_rewire_f32 edits the lookup and tells the plan cache -- the next backward rebuilds the plan first:
    #   plan-driven kernels, bit-identical from call to call, never the recomputing kernels;
    # foreign: a torch kernel edits the lookup -- the next backward is served by the recomputing kernels (correct up to
    #   the atomics' summation order), the one after it rebuilds;
    # foreign_announced: the same edit followed by ffi_lookup_edited -- as the library route.
    B, N, L, K = 64, 768, 262144, 32
    rng = np.random.default_rng(5)
    lookup = np.argsort(rng.random((L, N), dtype=np.float32), axis=1)[:, :K].astype(np.int32)
    w = (rng.normal(size=(L, K)) / np.sqrt(K)).astype(np.float32)
    x = np.maximum(rng.normal(size=(N, B)), 0).astype(np.float32)
    g = (rng.normal(size=(B, L)) * 1e-2).astype(np.float32)
    dx, dl, dw, dg = dev(x), dev(lookup), dev(w), dev(g)
    gx, gw = torch.empty_like(dx), torch.empty_like(dw)
    lib = ffi._lib.lib()

    def run():
        gx.fill_(float("nan")); gw.fill_(float("nan"))
        ffi._lib.check(lib.ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                                            B, N, L, K, 1, stream()))
        torch.cuda.synchronize()
        return gx.cpu().numpy().copy(), gw.cpu().numpy().copy()

    sample = rng.choice(L, 4096, replace=False)
    a_gx, a_gw = run()
    e = _label_sample_errors(lookup, w, g, x, a_gx, a_gw, B, N, K, sample)
    assert max(e) <= GRAD_RTOL, e
    if route == "library":
        thr = ffi.fixed_fan_in_ops.select_threshold(dw.view(-1), (L * K) // 100)
        ffi._lib.check(lib.ffi_rewire_f32(dl.data_ptr(), dw.data_ptr(), None, 0, L * K, N, thr.data_ptr(), 99, None, stream()))
    else:
        pos = torch.from_numpy(rng.choice(L * K, (L * K) // 100, replace=False)).cuda()
        dl.view(-1)[pos] = torch.from_numpy(rng.integers(0, N, pos.numel()).astype(np.int32)).cuda()
        if route == "foreign_announced":
            ffi._lib.check(lib.ffi_lookup_edited(dl.data_ptr()))
    torch.cuda.synchronize()
    lookup2 = dl.cpu().numpy()
    changed = int((lookup2 != lookup).sum())
    assert changed > (L * K) // 200
    b_gx, b_gw = run()                                   # the first backward after the edit
    e = _label_sample_errors(lookup2, w, g, x, b_gx, b_gw, B, N, K, sample)
    assert max(e) <= GRAD_RTOL, e
    c_gx, c_gw = run()
    e = _label_sample_errors(lookup2, w, g, x, c_gx, c_gw, B, N, K, sample)
    assert max(e) <= GRAD_RTOL, e
    d_gx, d_gw = run()
    assert np.array_equal(c_gx, d_gx) and np.array_equal(c_gw, d_gw)      # plan-driven: bit-identical
    if route != "foreign":
        # the plan was rebuilt before the first backward enqueued anything: that call was plan-driven already
        assert np.array_equal(b_gx, c_gx) and np.array_equal(b_gw, c_gw)


@pytest.mark.parametrize("transposed", [False, True])
def test_backward_after_in_place_rewiring_without_host_wait(ffi, transposed):
    # both gradients of ffi_backward_f32 / ffi_backward_bias_f32 right after the lookup changed under the cached plan,
    # with no synchronisation between the calls (the verdict of the device-side check is all the kernels have)
    B, N, L, K = 40, 200, 5000, 32
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=77)
    xin = np.ascontiguousarray(x.T) if transposed else x
    dx, dl, dw, dg = dev(xin), dev(lookup), dev(w), dev(g)
    lib = ffi._lib.lib()
    gx, gw, gb = torch.empty_like(dx), torch.empty_like(dw), torch.empty(L, device="cuda")

    def call():
        ffi._lib.check(lib.ffi_backward_bias_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(),
                                                  gw.data_ptr(), gb.data_ptr(), B, N, L, K, int(transposed), stream()))

    call()
    rng = np.random.default_rng(5)
    lookup2 = lookup.copy()
    lookup2[rng.integers(0, L, 800), rng.integers(0, K, 800)] = rng.integers(0, N, 800)
    dl.copy_(dev(lookup2), non_blocking=True)
    for _ in range(3):                                  # fallback kernels, then (whenever the host notices) a rebuilt plan
        gx.fill_(float("nan")); gw.fill_(float("nan")); gb.fill_(float("nan"))
        call()
        ref_gx, ref_gw = oracle.backward(xin, lookup2, w, g, transposed=transposed)
        torch.cuda.synchronize()
        assert rel_err(gx.cpu().numpy(), ref_gx) <= GRAD_RTOL
        assert rel_err(gw.cpu().numpy(), ref_gw) <= GRAD_RTOL
        assert rel_err(gb.cpu().numpy(), g.sum(axis=0)) <= GRAD_RTOL


def test_stateless_backward_does_not_wait_for_the_device(ffi):
    # steady state: a call only enqueues (tfsparse/cc/kernels/backward.cu:59-64 never waits either); calls on two
    # streams with two layers are enqueued back to back while the device is still busy with the first
    B, N, L, K = 128, 768, 200_000, 32
    lib = ffi._lib.lib()
    rng = np.random.default_rng(0)
    layers = []
    for i in range(2):
        x = dev(rng.standard_normal((N, B)).astype(np.float32))
        lk = dev(rng.integers(0, N, (L, K)).astype(np.int32))
        w = dev(rng.standard_normal((L, K)).astype(np.float32))
        g = dev(rng.standard_normal((B, L)).astype(np.float32))
        layers.append((x, lk, w, g, torch.empty_like(x), torch.empty_like(w), torch.cuda.Stream()))
    torch.cuda.synchronize()

    def enqueue(rounds):
        for _ in range(rounds):
            for x, lk, w, g, gx, gw, st in layers:
                ffi._lib.check(lib.ffi_backward_f32(x.data_ptr(), lk.data_ptr(), w.data_ptr(), g.data_ptr(), gx.data_ptr(),
                                                     gw.data_ptr(), B, N, L, K, 1, st.cuda_stream))

    enqueue(2)                                          # plans built (that does synchronise), verdicts seen
    torch.cuda.synchronize()
    import time
    t0 = time.perf_counter()
    enqueue(20)
    t_host = time.perf_counter() - t0
    torch.cuda.synchronize()
    t_all = time.perf_counter() - t0
    assert t_host < 0.5 * t_all, f"enqueueing took {t_host * 1e3:.2f} ms of {t_all * 1e3:.2f} ms: the calls waited for the device"
    for x, lk, w, g, gx, gw, st in layers:
        a = [t.cpu().numpy() for t in (x, lk, w, g)]
        ref_gx, ref_gw = oracle.backward(*a, transposed=True)
        assert rel_err(gx.cpu().numpy(), ref_gx) <= GRAD_RTOL
        assert rel_err(gw.cpu().numpy(), ref_gw) <= GRAD_RTOL


def test_one_lookup_used_from_two_streams_in_turn(ffi):
    # the checks of a cached plan share their accumulators; calls that come in on alternating streams must not let two
    # of them overlap, and an in-place edit of the lookup between them is still picked up
    B, N, L, K = 64, 256, 30_000, 16
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=77)
    dx, dl, dw, dg = dev(x), dev(lookup), dev(w), dev(g)
    lib = ffi._lib.lib()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    gx = [torch.empty((B, N), device="cuda") for _ in streams]
    gw = [torch.empty((L, K), device="cuda") for _ in streams]
    ref_gx, ref_gw = oracle.backward(x, lookup, w, g, transposed=False)
    for rnd in range(6):
        if rnd == 3:                                       # rewire in place: a fifth of the rows get new columns
            torch.cuda.synchronize()
            rng = np.random.default_rng(5)
            rows = rng.choice(L, L // 5, replace=False)
            lookup = lookup.copy()
            lookup[rows] = rng.integers(0, N, (rows.size, K)).astype(np.int32)
            dl.copy_(torch.from_numpy(lookup))
            torch.cuda.synchronize()
            ref_gx, ref_gw = oracle.backward(x, lookup, w, g, transposed=False)
        for i, st in enumerate(streams):
            print(f"case round={rnd} stream={i}", flush=True)
            ffi._lib.check(lib.ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx[i].data_ptr(),
                                                 gw[i].data_ptr(), B, N, L, K, 0, st.cuda_stream))
        torch.cuda.synchronize()
        for i in range(2):
            assert rel_err(gx[i].cpu().numpy(), ref_gx) <= GRAD_RTOL, (rnd, i)
            assert rel_err(gw[i].cpu().numpy(), ref_gw) <= GRAD_RTOL, (rnd, i)


def test_plan_is_unusable_after_a_failed_refresh(ffi):
    # a rebuild that fails (here: an id out of range) leaves a plan without arrays; calls through it are refused
    # with a status instead of walking freed memory
    B, N, L, K = 16, 64, 1000, 8
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=3)
    dl, dw, dg = dev(lookup), dev(w), dev(g)
    lib = ffi._lib.lib()
    plan = ctypes.c_void_p()
    ffi._lib.check(lib.ffi_plan_create(dl.data_ptr(), L, K, N, B, stream(), ctypes.byref(plan)))
    try:
        bad = lookup.copy()
        bad[7, 3] = N + 5
        dbad = dev(bad)
        assert lib.ffi_plan_refresh(plan, dbad.data_ptr(), stream()) == -6
        gx = torch.zeros((B, N), device="cuda")
        assert lib.ffi_input_grad_planned_f32(plan, dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B, 0, stream()) == -8
        ffi._lib.check(lib.ffi_plan_refresh(plan, dl.data_ptr(), stream()))          # a good lookup revives it
        ffi._lib.check(lib.ffi_input_grad_planned_f32(plan, dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B, 0, stream()))
        torch.cuda.synchronize()
        assert rel_err(gx.cpu().numpy(), oracle.input_grad(x, lookup, w, g)) <= GRAD_RTOL
    finally:
        lib.ffi_plan_destroy(plan)


def test_explicit_plan_matches_cached_path(ffi):
    B, N, L, K = 48, 96, 2000, 12
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=41)
    dl, dw, dg = dev(lookup), dev(w), dev(g)
    lib = ffi._lib.lib()
    plan = ctypes.c_void_p()
    ffi._lib.check(lib.ffi_plan_create(dl.data_ptr(), L, K, N, B, stream(), ctypes.byref(plan)))
    try:
        for transposed in (0, 1):
            gx = torch.full((N, B) if transposed else (B, N), float("nan"), device="cuda")
            ffi._lib.check(lib.ffi_input_grad_planned_f32(plan, dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B,
                                                          transposed, stream()))
            torch.cuda.synchronize()
            xin = np.ascontiguousarray(x.T) if transposed else x
            ref = oracle.input_grad(xin, lookup, w, g, transposed=bool(transposed))
            assert rel_err(gx.cpu().numpy(), ref) <= GRAD_RTOL
            # the weight gradient fed by the plan's arranged copy of the column ids
            gw = torch.full((L, K), float("nan"), device="cuda")
            dx = dev(xin)
            ffi._lib.check(lib.ffi_weight_grad_planned_f32(plan, dx.data_ptr(), dl.data_ptr(), dg.data_ptr(), gw.data_ptr(), B,
                                                           transposed, stream()))
            torch.cuda.synchronize()
            assert rel_err(gw.cpu().numpy(), oracle.weight_grad(xin, lookup, w, g, transposed=bool(transposed))) <= GRAD_RTOL
    finally:
        ffi._lib.check(lib.ffi_plan_destroy(plan))


@pytest.mark.parametrize("shape", [(768, 3000, 32), (512, 2500, 16), (100, 1800, 21), (300, 1500, 40)])
def test_plan_layouts_serve_any_batch_size(ffi, shape):
    # the batch hint picks the plan's layout (small batches: label tiles whose weights the kernel keeps in LDS, no
    # slot-ordered copy of the weights; large or unknown: 1024-label tiles behind the permutation kernel); either
    # layout must give the oracle's input gradient at any batch size, bit-identically from call to call
    N, L, K = shape
    lib = ffi._lib.lib()
    for hint in (32, 128, 512, 0):
        plan = None
        for B in (20, 150):
            x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=N + hint)
            dl, dw, dg = dev(lookup), dev(w), dev(g)
            if plan is None:
                plan = ctypes.c_void_p()
                ffi._lib.check(lib.ffi_plan_create(dl.data_ptr(), L, K, N, hint, stream(), ctypes.byref(plan)))
                lookup0 = lookup
            else:
                lookup, dl = lookup0, dev(lookup0)          # the plan describes the first lookup
            print(f"case N={N} L={L} K={K} hint={hint} B={B}", flush=True)
            results = []
            for _ in range(2):
                gx = torch.full((B, N), float("nan"), device="cuda")
                ffi._lib.check(lib.ffi_input_grad_planned_f32(plan, dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B, 0, stream()))
                torch.cuda.synchronize()
                results.append(gx.cpu().numpy())
            assert np.array_equal(results[0], results[1])
            assert rel_err(results[0], oracle.input_grad(x, lookup, w, g, transposed=False)) <= GRAD_RTOL
        ffi._lib.check(lib.ffi_plan_destroy(plan))


@pytest.mark.parametrize("shape", [(128, 768, 60_000, 32, True), (32, 768, 40_000, 32, True), (256, 512, 30_000, 64, True),
                                   (64, 300, 20_000, 12, False), (96, 2000, 5_000, 20, False), (40, 1100, 9_000, 16, True),
                                   (160, 128, 40_000, 16, True), (300, 200, 40_000, 16, False),     # (several input-gradient workgroups per CU)
                                   (128, 768, 160_000, 32, True), (64, 1100, 200_000, 16, True)])   # (plans that sort a tile's columns by length; two column windows)
def test_workspace_estimate_brackets_what_the_library_holds(ffi, shape):
    # ffi_workspace_bytes() is asked before anything is allocated; ffi_cache_bytes() says what forward + backward then
    # hold (plans + workspaces).  The estimate models the padding of the plan for uniformly drawn ids.
    B, N, L, K, tp = shape
    lib = ffi._lib.lib()
    torch.cuda.synchronize()
    ffi._lib.check(lib.ffi_cache_clear())
    assert lib.ffi_cache_bytes() == 0
    estimate = lib.ffi_workspace_bytes(B, N, L, K, int(tp), 3)
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=L)
    xin = np.ascontiguousarray(x.T) if tp else x
    hip_forward(ffi, xin, lookup, w, tp)
    hip_backward(ffi, xin, lookup, w, g, tp)
    held = lib.ffi_cache_bytes()
    print(f"case shape={shape} estimate={estimate} held={held}", flush=True)
    assert held > 0 and 0.8 * held <= estimate <= 1.3 * held + (1 << 20)
    ffi._lib.check(lib.ffi_cache_clear())
    assert lib.ffi_cache_bytes() == 0


def test_bad_lookup_is_reported_not_dereferenced(ffi):
    B, N, L, K = 4, 10, 50, 3
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=51)
    lookup[7, 1] = N            # one id out of range
    dl, dw, dg = dev(lookup), dev(w), dev(g)
    lib = ffi._lib.lib()
    assert lib.ffi_check_lookup(dl.data_ptr(), L, K, N, stream()) == -6
    gx = torch.zeros((B, N), device="cuda")
    assert lib.ffi_input_grad_f32(dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(), B, N, L, K, 0, stream()) == -6
    assert lib.ffi_check_lookup(dl.data_ptr(), L, K, N + 1, stream()) == 0


def test_autograd_wiring(ffi):
    # gradient list order [feature_grad, None, weight_grad] (sparse/ops/fixed_fan_in_ops.py:31-40)
    B, N, L, K = 16, 40, 700, 8
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=61)
    for transposed in (False, True):
        xin = np.ascontiguousarray(x.T) if transposed else x
        tx = dev(xin).requires_grad_(True)
        tw = dev(w).requires_grad_(True)
        fn = ffi.fan_in_sparse_matmul_tp if transposed else ffi.fan_in_sparse_matmul
        out = fn(tx, dev(lookup), tw)
        out.backward(dev(g))
        o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
        assert rel_err(out.detach().cpu().numpy(), oracle.forward(xin, lookup, w, transposed=transposed)) <= FWD_RTOL
        assert rel_err(tx.grad.cpu().numpy(), o_gx) <= GRAD_RTOL
        assert rel_err(tw.grad.cpu().numpy(), o_gw) <= GRAD_RTOL


def test_headline_config_full_size_properties(ffi):
    # 670,091 labels x fan-in 32 x 768 inputs x batch 128: size-independent checks
    #   adjoint identity  <out, g> = <x, gx> = <W, gW>   (the layer is linear in x and in W)
    #   a label slice agrees with the oracle run on that slice alone
    from ecml23_sparse_amd import synth
    cfg = synth.CONFIGS["c2"]
    t = synth.make_inputs(cfg, seed=42, device="cuda", transposed=True)
    x, lookup, w, g = t["features"], t["lookup"], t["weights"], t["out_grad"]
    out = ffi.fan_in_sparse_matmul_tp(x, lookup, w)
    gx, gw = ffi.fan_in_sparse_matmul_grad_tp(x, lookup, w, g)
    torch.cuda.synchronize()
    a = float((out.double() * g.double()).sum())
    b = float((x.double() * gx.double()).sum())
    c = float((w.double() * gw.double()).sum())
    assert abs(a - b) <= 1e-4 * abs(a) and abs(a - c) <= 1e-4 * abs(a)
    sl = slice(300_000, 304_000)
    xs, ls, ws, gs = x.cpu().numpy(), lookup[sl].cpu().numpy(), w[sl].cpu().numpy(), g[:, sl].cpu().numpy()
    assert rel_err(out[:, sl].cpu().numpy(), oracle.forward(xs, ls, ws, transposed=True)) <= FWD_RTOL
    assert rel_err(gw[sl].cpu().numpy(), oracle.weight_grad(xs, ls, ws, np.ascontiguousarray(gs), transposed=True)) <= GRAD_RTOL
    # the full input gradient against the oracle (streams all labels on the host: a few seconds)
    o_gx = oracle.input_grad(xs, lookup.cpu().numpy(), w.cpu().numpy(), g.cpu().numpy(), transposed=True)
    assert rel_err(gx.cpu().numpy(), o_gx) <= GRAD_RTOL


@pytest.mark.parametrize("name", ["c3", "c4"])
def test_other_benchmark_configs_full_size_properties(ffi, name):
    # c3 (fan-in 64, unit-norm inputs, batch 256) and c4 (65,536 inputs: the kernels that gather from cache) at their full
    # label counts: the adjoint identity <out, g> = <x, gx> = <W, gW>, and a label slice against the oracle run on that slice
    from ecml23_sparse_amd import synth
    cfg = synth.CONFIGS[name]
    t = synth.make_inputs(cfg, seed=42, device="cuda", transposed=True)
    x, lookup, w, g = t["features"], t["lookup"], t["weights"], t["out_grad"]
    print(f"case config={name} full size", flush=True)
    out = ffi.fan_in_sparse_matmul_tp(x, lookup, w)
    gx, gw = ffi.fan_in_sparse_matmul_grad_tp(x, lookup, w, g)
    torch.cuda.synchronize()
    a = float((out.double() * g.double()).sum())
    b = float((x.double() * gx.double()).sum())
    c = float((w.double() * gw.double()).sum())
    assert abs(a - b) <= 1e-4 * abs(a) and abs(a - c) <= 1e-4 * abs(a)
    sl = slice(400_000, 401_000)
    xs, ls, ws = x.cpu().numpy(), lookup[sl].cpu().numpy(), w[sl].cpu().numpy()
    gs = np.ascontiguousarray(g[:, sl].cpu().numpy())
    assert rel_err(out[:, sl].cpu().numpy(), oracle.forward(xs, ls, ws, transposed=True)) <= FWD_RTOL
    assert rel_err(gw[sl].cpu().numpy(), oracle.weight_grad(xs, ls, ws, gs, transposed=True)) <= GRAD_RTOL
    # the input gradient is a sum over all labels; the part of it that comes from the slice is checked through linearity:
    # gx(g) - gx(g with the slice zeroed) = gx of the slice alone
    g2 = g.clone()
    g2[:, sl] = 0
    gx2, _ = ffi.fan_in_sparse_matmul_grad_tp(x, lookup, w, g2)
    torch.cuda.synchronize()
    part = (gx.double() - gx2.double()).cpu().numpy()
    o_part = oracle.input_grad(xs, ls, ws, gs, transposed=True)
    assert np.abs(part - o_part).max() <= 1e-4 * np.abs(gx.cpu().numpy()).max()


def test_calls_from_two_threads_on_one_stream(ffi):
    # TensorFlow enters an op's Compute from several threads; both calls here use the stream's transpose workspace
    # ([B,N] features) and the plan cache (backward).  Each thread checks every result of its own inputs.
    import threading
    B, N, L, K = 64, 200, 6000, 16
    lib = ffi._lib.lib()
    cases = []
    for seed in (1, 2):
        x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=100 + seed)
        ref_out = oracle.forward(x, lookup, w)
        ref_gx, ref_gw = oracle.backward(x, lookup, w, g)
        cases.append((dev(x), dev(lookup), dev(w), dev(g), ref_out, ref_gx, ref_gw))
    s = stream()
    errors = []

    def worker(case):
        dx, dl, dw, dg, ref_out, ref_gx, ref_gw = case
        out = torch.empty((B, L), device="cuda")
        gx = torch.empty((B, N), device="cuda")
        gw = torch.empty((L, K), device="cuda")
        try:
            for _ in range(40):
                ffi._lib.check(lib.ffi_forward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K, 0, s))
                ffi._lib.check(lib.ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(),
                                                    gw.data_ptr(), B, N, L, K, 0, s))
                torch.cuda.synchronize()
                e = (rel_err(out.cpu().numpy(), ref_out), rel_err(gx.cpu().numpy(), ref_gx), rel_err(gw.cpu().numpy(), ref_gw))
                if not (e[0] <= FWD_RTOL and e[1] <= GRAD_RTOL and e[2] <= GRAD_RTOL):
                    errors.append(e)
                    return
        except Exception as exc:  # noqa: BLE001
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(c,)) for c in cases]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def _random_shapes(count, seed):
    rng = np.random.default_rng(seed)
    shapes = []
    for _ in range(count):
        B = int(rng.choice([1, 2, 7, 31, 32, 33, 50, 64, 65, 100, 128, 200, 257]))
        N = int(rng.choice([1, 3, 17, 64, 100, 255, 512, 768, 1024, 1025, 1216, 1217, 2000, 5000]))
        L = int(rng.choice([1, 2, 63, 64, 65, 500, 1023, 1024, 1025, 3000, 7001]))
        K = int(rng.choice([1, 2, 3, 4, 8, 15, 16, 31, 32, 33, 48, 64, 65, 100]))
        shapes.append((B, N, L, K, bool(rng.integers(0, 2))))
    return shapes


@pytest.mark.parametrize("shape", _random_shapes(36, seed=2024), ids=lambda s: "B%d_N%d_L%d_K%d_%s" % (s[0], s[1], s[2], s[3], "tp" if s[4] else "nt"))
def test_drawn_shapes(ffi, shape):
    # sizes drawn around the boundaries of the kernels' regimes (batch tiles of 32, wavefronts of 64, label tiles of 1024,
    # register chunks of 32 connections, 1216 columns for the LDS tile, 1024 for the tiled plan), either layout
    B, N, L, K, transposed = shape
    x, lookup, w, g = reference_law_inputs(B, N, L, K, seed=B + 3 * N + 5 * L + 7 * K)
    xin = np.ascontiguousarray(x.T) if transposed else x
    print(f"case shape={shape}", flush=True)
    out = hip_forward(ffi, xin, lookup, w, transposed)
    gx, gw = hip_backward(ffi, xin, lookup, w, g, transposed)
    assert rel_err(out, oracle.forward(xin, lookup, w, transposed=transposed)) <= FWD_RTOL
    o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=transposed)
    assert rel_err(gw, o_gw) <= GRAD_RTOL
    assert rel_err(gx, o_gx) <= GRAD_RTOL
