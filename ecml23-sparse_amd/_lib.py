"""ctypes binding of libffi_hip.so (declared in include/ffi_hip.h)."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libffi_hip.so")

_vp = ctypes.c_void_p
_i64 = ctypes.c_int64
_int = ctypes.c_int
_f32 = ctypes.c_float

# name -> (restype, argtypes); the single source of truth for the Python side of the ABI
SIGNATURES = {
    "ffi_abi_version": (_int, []),
    "ffi_target_arch": (ctypes.c_char_p, []),
    "ffi_status_string": (ctypes.c_char_p, [_int]),
    "ffi_last_hip_error": (_int, []),
    "ffi_forward_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_forward_noalloc_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_backward_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_weight_grad_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_input_grad_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_plan_create": (_int, [_vp, _i64, _i64, _i64, _i64, _vp, ctypes.POINTER(_vp)]),
    "ffi_plan_refresh": (_int, [_vp, _vp, _vp]),
    "ffi_plan_destroy": (_int, [_vp]),
    "ffi_plan_info": (_int, [_vp, ctypes.POINTER(_i64)]),
    "ffi_host_forward_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _i64, _i64]),
    "ffi_host_backward_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _i64, _i64, _i64, _i64]),
    "ffi_input_grad_planned_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _int, _vp]),
    "ffi_cache_clear": (_int, []),
    "ffi_lookup_edited": (_int, [_vp]),
    "ffi_set_option": (_int, [ctypes.c_char_p, _int]),
    "ffi_cache_bytes": (ctypes.c_size_t, []),
    "ffi_workspace_bytes": (ctypes.c_size_t, [_i64, _i64, _i64, _i64, _int, _int]),
    "ffi_check_lookup": (_int, [_vp, _i64, _i64, _i64, _vp]),
    "ffi_weight_grad_planned_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _int, _vp]),
    "ffi_arrange_connections_f32": (_int, [_vp, _vp, _int, _i64, _i64, _vp]),
    "ffi_forward_bias_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_backward_bias_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_forward_bf16_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_forward_topk_bf16": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "ffi_topk_f32": (_int, [_vp, _i64, _i64, _int, _vp, _vp, _vp]),
    "ffi_loss_grad_f32": (_int, [_vp, _vp, _vp, _i64, _int, _f32, _vp, _vp, _vp, _i64, _i64, _vp]),
    "ffi_forward_topk_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _int, _vp]),
    "ffi_forward_loss_topk_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _int,
                                         _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_threshold_metrics_f32": (_int, [_vp, _vp, _vp, _i64, _f32, _vp, _i64, _i64, _vp]),
    "ffi_forward_loss_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _int, _f32, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_backward_sparse_adam_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _f32, _vp, _vp, _vp, _vp, _vp, _vp, _f32, _f32, _f32, _f32,
                                            _i64, ctypes.POINTER(_int), _i64, _i64, _i64, _i64, _int, _vp]),
    "ffi_select_threshold_f32": (_int, [_vp, _i64, _i64, _vp, _vp]),
    "ffi_rewire_f32": (_int, [_vp, _vp, _vp, _int, _i64, _i64, _vp, ctypes.c_uint64, _vp, _vp]),
    "ffi_adam_step_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _f32, _f32, _f32, _f32, _i64, _vp]),
    "ffi_backward_sparse_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _int, _f32, _vp, _vp, _vp, ctypes.POINTER(_int), _i64, _i64, _i64, _i64, _int, _vp]),
}

_lib = None


class FfiError(RuntimeError):
    """A C-ABI call returned a negative ffi_status."""

    def __init__(self, status: int, message: str):
        super().__init__(f"ffi_hip status {status}: {message}")
        self.status = status


def lib() -> ctypes.CDLL:
    """Loads the HIP library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python ecml23-sparse_amd/build.py` "
                "(needs hipcc); this package has no CPU or PyTorch fallback")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(status: int) -> None:
    if status != 0:
        l = lib()
        msg = l.ffi_status_string(status).decode()
        if status == -4:
            msg += f" (hipError_t {l.ffi_last_hip_error()})"
        raise FfiError(status, msg)
