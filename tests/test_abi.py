"""The C-ABI library loads without a GPU and exports every symbol include/ffi_hip.h declares."""
import ctypes
import os
import re

import pytest

from conftest import ROOT, load_package

HEADER = os.path.join(ROOT, "include", "ffi_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ffi_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = declared_symbols()
    for must in ("ffi_forward_f32", "ffi_backward_f32", "ffi_weight_grad_f32", "ffi_input_grad_f32",
                 "ffi_plan_create", "ffi_plan_destroy", "ffi_input_grad_planned_f32"):
        assert must in names


def test_library_exports_every_declared_symbol():
    pkg = load_package()
    handle = ctypes.CDLL(pkg._lib.LIB_PATH)
    missing = [n for n in declared_symbols() if not hasattr(handle, n)]
    assert not missing, f"declared in ffi_hip.h but not exported: {missing}"


def test_python_signatures_cover_the_header():
    pkg = load_package()
    assert sorted(pkg._lib.SIGNATURES) == declared_symbols()


def test_identification_calls_need_no_gpu():
    pkg = load_package()
    lib = pkg._lib.lib()
    assert lib.ffi_abi_version() >= 1
    assert lib.ffi_target_arch() == b"gfx950"
    assert lib.ffi_status_string(0) == b"ok"
    assert b"null" in lib.ffi_status_string(-1)


def test_argument_checks_run_before_any_device_work():
    # contract violations the reference fail-fasts on (forward.cu:19-28) come back as statuses
    pkg = load_package()
    lib = pkg._lib.lib()
    one = ctypes.c_void_p(16)     # never dereferenced: checks fail first
    assert lib.ffi_forward_f32(None, one, one, one, 1, 1, 1, 1, 0, None) == -1
    assert lib.ffi_forward_f32(one, one, one, one, 0, 1, 1, 1, 0, None) == -2
    assert lib.ffi_forward_f32(one, one, one, one, 1, 1, -3, 1, 0, None) == -2
    assert lib.ffi_forward_f32(one, one, one, one, 1, 1, 2**31, 1, 0, None) == -3
    assert lib.ffi_forward_f32(one, one, one, one, 1, 1, 2**30, 4, 0, None) == -3
    assert lib.ffi_backward_f32(one, one, one, one, None, None, 1, 1, 1, 1, 0, None) == -1
    assert lib.ffi_weight_grad_f32(one, one, one, None, 1, 1, 1, 1, 0, None) == -1
    assert lib.ffi_input_grad_f32(one, one, one, one, 1, 0, 1, 1, 0, None) == -2
    assert lib.ffi_plan_destroy(None) == 0
    with pytest.raises(pkg._lib.FfiError):
        pkg._lib.check(-2)


def test_option_names_and_ranges_are_checked():
    # without a GPU there is nothing cached to drop: the setter still validates and stores
    pkg = load_package()
    lib = pkg._lib.lib()
    assert lib.ffi_set_option(None, 0) == -8
    assert lib.ffi_set_option(b"no_such_option", 0) == -8
    assert lib.ffi_set_option(b"wgrad_units", 5) == -8 and lib.ffi_set_option(b"wgrad_units", 2) == -8
    assert lib.ffi_set_option(b"fwd_lane64", 1) == -8 and lib.ffi_set_option(b"plan_sorted_columns", 2) == -8
    for name, value in ((b"wgrad_units", 3), (b"wgrad_stream", -1), (b"fwd_lane64", -1), (b"plan_weights_in_lds", 1),
                        (b"workgroups_per_cu", 2), (b"plan_sorted_columns", -1), (b"plan_sorted_columns", 1)):
        assert lib.ffi_set_option(name, value) == 0
        assert lib.ffi_set_option(name, 0) == 0
