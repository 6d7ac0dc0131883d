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
