"""ctypes binding of libfsadam.so (the C ABI declared in include/fsadam.h).

The library is loaded from ``fairscale_amd/csrc/libfsadam.so``; there is no fallback: when it is
missing, or a call fails, the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch  # noqa: F401  -- first, so that the HIP runtime torch ships is the one this process maps

FULL_PRECISION = 0
MIXED_PRECISION = 1
MEMORY_EFFICIENT_MIXED_PRECISION = 2
PURE_FP16 = 3
FULL_PRECISION_FP16_COPY = 4

ABI_VERSION = 4

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libfsadam.so")


class FsAdamTensor(ctypes.Structure):
    _fields_ = [
        ("p", ctypes.c_void_p),
        ("m", ctypes.c_void_p),
        ("v", ctypes.c_void_p),
        ("g", ctypes.c_void_p),
        ("p_copy", ctypes.c_void_p),
        ("numel", ctypes.c_int64),
    ]


class _Int64Fields(ctypes.Structure):
    def as_dict(self) -> dict:
        return {name: int(getattr(self, name)) for name, _ in self._fields_}


class FsGradTensor(ctypes.Structure):
    _fields_ = [("g", ctypes.c_void_p), ("numel", ctypes.c_int64)]


GRAD_F32 = 0
GRAD_F16 = 1


class FsAdamPlanInfo(_Int64Fields):
    _fields_ = [("mode", ctypes.c_int32), ("device", ctypes.c_int32)] + [
        (name, ctypes.c_int64)
        for name in ("n_tensors", "total_elems", "tile_elems", "large_chunk_elems", "n_descriptors", "n_vector_tensors",
                     "n_scalar_tensors", "n_launches", "grid", "block", "lds_throttle", "uploads", "n_runs")
    ]


class FsAdamLayout(_Int64Fields):
    _fields_ = [
        (name, ctypes.c_int64)
        for name in ("tile_elems", "large_chunk_elems", "n_large_tensors", "n_small_tensors", "n_empty_tensors",
                     "n_large_descriptors", "n_small_descriptors", "grid_large", "grid_small", "mid_chunk_elems", "n_mid_tensors",
                     "n_mid_descriptors", "grid_mid", "n_runs")
    ]


# name -> (restype, argtypes); one entry per function include/fsadam.h declares
_f32, _i32, _i64, _vp = ctypes.c_float, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
_SCALARS = [_f32, _f32, _f32, _f32, _f32, _f32, _f32, _i32, _i32, _i32]
SIGNATURES = {
    "fsadam_version": (_i32, []),
    "fsadam_last_error": (ctypes.c_char_p, []),
    "fsadam_step_size": (_f32, [_f32, _f32, _f32, _i32, _i32]),
    "fsadam_set_option": (_i32, [ctypes.c_char_p, _i64]),
    "fsadam_get_option": (_i32, [ctypes.c_char_p, ctypes.POINTER(_i64)]),
    "fsadam_step": (_i32, [ctypes.POINTER(FsAdamTensor), _i64, _i32] + _SCALARS + [_vp, _vp]),
    "fsadam_plan_create": (_i32, [_i32, ctypes.POINTER(_vp)]),
    "fsadam_plan_set_tensors": (_i32, [_vp, ctypes.POINTER(FsAdamTensor), _i64, _vp]),
    "fsadam_plan_step": (_i32, [_vp] + _SCALARS + [_vp, _vp]),
    # lr, beta1, beta2, eps, grad_scale_dev, optim_scale, decay, step, eps_mode, bias_correction, found_inf, stream
    "fsadam_plan_step_dev_scale": (_i32, [_vp, _f32, _f32, _f32, _f32, _vp, _f32, _f32, _i32, _i32, _i32, _vp, _vp]),
    "fsadam_plan_info": (_i32, [_vp, ctypes.POINTER(FsAdamPlanInfo)]),
    "fsadam_plan_lazy_events": (_i32, [_vp, _i32]),
    "fsadam_plan_zero_state": (_i32, [_vp, _vp]),
    "fsadam_plan_destroy": (_i32, [_vp]),
    "fsadam_head_elems": (_i32, [ctypes.POINTER(FsAdamTensor), _i32, ctypes.POINTER(_i64)]),
    "fsadam_layout": (_i32, [ctypes.POINTER(FsAdamTensor), _i64, _i32, ctypes.POINTER(FsAdamLayout), ctypes.POINTER(ctypes.c_uint8), ctypes.POINTER(ctypes.c_uint8)]),
    "fsadam_grad_pass": (_i32, [ctypes.POINTER(FsGradTensor), _i64, _i32, _f32, _vp, _i32, _vp, _vp, _vp, _vp]),
    "fsadam_grad_pass_noalloc": (_i32, [ctypes.POINTER(FsGradTensor), _i64, _i32, _f32, _vp, _i32, _vp, _vp, _vp, _vp]),
    "fsadam_clear_cache": (_i32, []),
}

_lib: Optional[ctypes.CDLL] = None


class FsAdamError(RuntimeError):
    """A C-ABI call returned a negative code (message from fsadam_last_error)."""


def library_path() -> str:
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    """The loaded library; raises ImportError when it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise ImportError(
                f"{_LIB_PATH} is missing: build it with `python -m fairscale_amd.csrc.build` "
                "(there is no fallback implementation)"
            )
        L = ctypes.CDLL(_LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(L, name)  # AttributeError if the library lacks a declared symbol
            fn.restype = restype
            fn.argtypes = argtypes
        got = L.fsadam_version()
        if got != ABI_VERSION:
            raise ImportError(f"libfsadam.so has ABI version {got}, this package expects {ABI_VERSION}")
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        msg = lib().fsadam_last_error().decode("utf-8", "replace")
        raise FsAdamError(f"fsadam error {rc}: {msg}")


def step_size(lr: float, beta1: float, beta2: float, step: int, bias_correction: int) -> float:
    return float(lib().fsadam_step_size(lr, beta1, beta2, step, bias_correction))


def set_option(name: str, value: int) -> None:
    check(lib().fsadam_set_option(name.encode(), int(value)))


def get_option(name: str) -> int:
    out = ctypes.c_int64(0)
    check(lib().fsadam_get_option(name.encode(), ctypes.byref(out)))
    return int(out.value)
