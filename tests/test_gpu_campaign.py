"""Random differential campaign (`-m gpu`): a few hundred shapes drawn around the boundaries of the kernels' regimes, with
differently distributed column ids, through the stateless C-ABI entry points -- forward, backward, and backward again after
the lookup was edited in place (the call served by the recomputing kernels, then the calls served by the rebuilt plan) --
each compared with the CPU oracle.  Semantics: tfsparse/cc/kernels/forward.cpp:9-44, backward.cpp:8-73."""
import numpy as np
import pytest
import torch

import oracle
from conftest import load_package, rel_err

pytestmark = pytest.mark.gpu

FWD_RTOL = 1e-5
GRAD_RTOL = 1e-4

BATCHES = [1, 2, 7, 31, 32, 33, 63, 64, 65, 96, 100, 127, 128, 129, 191, 192, 193, 200, 256, 257, 300]
WIDTHS = [1, 2, 3, 17, 63, 64, 65, 100, 128, 200, 255, 256, 300, 511, 512, 576, 608, 609, 640, 700, 768, 1000, 1023, 1024, 1025,
          1088, 1100, 1216, 1217, 1300, 2000, 3000]
FAN_INS = [1, 2, 3, 4, 5, 7, 8, 12, 15, 16, 17, 20, 24, 28, 31, 32, 33, 35, 36, 40, 48, 63, 64, 65, 67, 72, 80, 96, 100, 112, 128,
           130, 200, 300]
LABELS = [1, 2, 63, 64, 65, 500, 581, 582, 583, 1023, 1024, 1025, 2000, 3000, 5000, 7001, 12000]


def draw_lookup(rng, dist, L, K, N):
    if dist == "uniform":
        ids = rng.integers(0, N, (L, K))
    elif dist == "few_columns":                                     # heavily skewed: the global plan
        ids = rng.integers(0, max(1, min(N, int(rng.integers(1, 9)))), (L, K))
    elif dist == "long_tail":
        ids = np.minimum((rng.pareto(1.2, (L, K)) * 3).astype(np.int64), N - 1)
    elif dist == "even_columns":                                    # every second column unused
        ids = rng.integers(0, N, (L, K)) // 2 * 2 % N
    else:                                                           # no column twice in a label (where the fan-in allows)
        ids = np.stack([rng.permutation(N)[:K] if K <= N else rng.integers(0, N, K) for _ in range(L)])
    return ids.astype(np.int32)


@pytest.mark.parametrize("seed,options", [(11, ()), (12, ()), (13, ()), (14, ()),
                                          # the plan forms the library takes only for large layers, forced onto small ones
                                          (15, (("plan_weights_in_lds", 1), ("plan_sorted_columns", 1))),
                                          (16, (("plan_weights_in_lds", -1), ("wgrad_stream", -1)))])
def test_random_shapes_layouts_and_id_distributions(seed, options):
    ffi = load_package()
    lib = ffi._lib.lib()
    for name, value in options:
        ffi._lib.check(lib.ffi_set_option(name.encode(), value))
    try:
        _campaign(ffi, lib, seed)
    finally:
        for name, _ in options:
            ffi._lib.check(lib.ffi_set_option(name.encode(), 0))


def _campaign(ffi, lib, seed):
    rng = np.random.default_rng(seed)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    stream = lambda: torch.cuda.current_stream().cuda_stream
    failures = []
    for case in range(100):
        B, N, K = int(rng.choice(BATCHES)), int(rng.choice(WIDTHS)), int(rng.choice(FAN_INS))
        L = min(int(rng.choice(LABELS + [int(rng.integers(1, 12001))])), max(1, min(400_000 // K, 3_000_000 // B)))
        tp = bool(rng.integers(0, 2))
        dist = str(rng.choice(["uniform", "few_columns", "long_tail", "even_columns", "no_duplicates"]))
        name = f"seed={seed} case={case} B={B} N={N} L={L} K={K} transposed={tp} ids={dist}"
        print(name, flush=True)
        x = rng.uniform(-1, 1, (B, N)).astype(np.float32)
        w = rng.uniform(-1, 1, (L, K)).astype(np.float32)
        g = np.maximum(rng.uniform(-1, 1, (B, L)), 0).astype(np.float32)
        lookup = draw_lookup(rng, dist, L, K, N)
        xin = np.ascontiguousarray(x.T) if tp else x
        dx, dl, dw, dg = dev(xin), dev(lookup), dev(w), dev(g)
        out = torch.full((B, L), float("nan"), device="cuda")
        gx = torch.full(tuple(xin.shape), float("nan"), device="cuda")
        gw = torch.full((L, K), float("nan"), device="cuda")

        def backward():
            gx.fill_(float("nan"))
            gw.fill_(float("nan"))
            ffi._lib.check(lib.ffi_backward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), dg.data_ptr(), gx.data_ptr(),
                                                gw.data_ptr(), B, N, L, K, int(tp), stream()))
            torch.cuda.synchronize()
            return gx.cpu().numpy(), gw.cpu().numpy()

        ffi._lib.check(lib.ffi_forward_f32(dx.data_ptr(), dl.data_ptr(), dw.data_ptr(), out.data_ptr(), B, N, L, K, int(tp), stream()))
        got_gx, got_gw = backward()
        o_gx, o_gw = oracle.backward(xin, lookup, w, g, transposed=tp)
        errors = {"forward": (rel_err(out.cpu().numpy(), oracle.forward(xin, lookup, w, transposed=tp)), FWD_RTOL),
                  "input_grad": (rel_err(got_gx, o_gx), GRAD_RTOL), "weight_grad": (rel_err(got_gw, o_gw), GRAD_RTOL)}
        # 2 % of the connections redrawn in place, as a rewiring step does (sparse/custom_layer.py:32-43)
        edited = lookup.copy()
        m = max(1, L * K // 50)
        edited[rng.integers(0, L, m), rng.integers(0, K, m)] = rng.integers(0, N, m)
        dl.copy_(dev(edited))
        o_gx, o_gw = oracle.backward(xin, edited, w, g, transposed=tp)
        for call in ("first", "second", "third"):
            got_gx, got_gw = backward()
            errors[f"input_grad, {call} call after the edit"] = (rel_err(got_gx, o_gx), GRAD_RTOL)
            errors[f"weight_grad, {call} call after the edit"] = (rel_err(got_gw, o_gw), GRAD_RTOL)
        failures += [f"{name}: {what} {err:.3g}" for what, (err, tol) in errors.items() if not err <= tol]
        if case % 25 == 24:
            ffi._lib.check(lib.ffi_cache_clear())
    assert not failures, "\n".join(failures)
