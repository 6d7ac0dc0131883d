"""The C-ABI library called from a C++ program with no Python or torch in its process (tests/cpp/cabi_harness.cpp):
the reference's known-answer case (testing/test.cpp:13-47), its shape grid in both layouts (testing/test.cpp:50-59)
against the CPU oracle with the reference's absolute gates, and the status codes that replace its aborts.

The program is built beforehand by ``__graft_entry__.build()`` (``make -C tests/cpp``); this test only runs it.
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HARNESS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "cabi_harness")


def run(args, timeout):
    assert os.path.exists(HARNESS), "tests/cpp/cabi_harness is not built: run __graft_entry__.build()"
    proc = subprocess.run([HARNESS, *args], capture_output=True, text=True, timeout=timeout)
    print(proc.stdout)
    print(proc.stderr)
    return proc


def test_cpp_caller_passes_the_reference_test_cases():
    proc = run(["test"], 300)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert "0 failure(s)" in proc.stdout
    assert proc.stdout.count(" ok") >= 2 + 1 + 16


def test_cpp_caller_benchmark_mode_runs():
    # a small shape: the mode the reference's quick-bench program has, here only checked to run
    proc = run(["bench", "50", "2048", "20000", "32"], 120)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert "forward pass" in proc.stdout and "backward pass" in proc.stdout


def test_cpp_and_python_callers_draw_the_same_tensors():
    # one seeded counter-based generator on both sides: the C++ program's sums of its inputs and of the library's
    # results equal those of the numpy twin's tensors run through the ctypes binding (inputs exactly, results to the
    # last bits the order of a double-precision sum leaves open)
    import re

    import numpy as np
    import torch

    from conftest import load_package
    pkg = load_package()
    from ecml23_sparse_amd import synth
    B, N, L, K, seed = 24, 100, 3000, 12, 1234
    for tp in (0, 1):
        proc = run(["sums", str(B), str(N), str(L), str(K), str(tp), str(seed)], 120)
        assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
        got = dict(re.findall(r"(\w+) (-?[\d.e+-]+)", proc.stdout.split("sums ", 1)[1]))
        x, lookup, w, g = synth.counter_case(B, N, L, K, transposed=bool(tp), seed=seed)
        seq = lambda a: float(np.cumsum(a.astype(np.float64).ravel())[-1])       # noqa: E731  (added in storage order, as the program adds)
        assert float(got["features"]) == seq(x)
        assert int(float(got["lookup"])) == int(lookup.astype(np.int64).sum())
        assert float(got["weights"]) == seq(w)
        assert float(got["out_grad"]) == seq(g)
        dx, dl, dw, dg = (torch.from_numpy(a).cuda() for a in (x, lookup, w, g))
        out = (pkg.fan_in_sparse_matmul_tp if tp else pkg.fan_in_sparse_matmul)(dx, dl, dw)
        gx, gw = (pkg.fan_in_sparse_matmul_grad_tp if tp else pkg.fan_in_sparse_matmul_grad)(dx, dl, dw, dg)
        torch.cuda.synchronize()
        for name, t in (("result", out), ("feature_grad", gx), ("weight_grad", gw)):
            mine = float(t.double().sum())
            assert abs(float(got[name]) - mine) <= 1e-9 * max(1.0, abs(mine)), name
