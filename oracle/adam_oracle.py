"""TEST INFRASTRUCTURE ONLY -- Python face of the CPU oracle.

Three things live here, none of which the product imports:

* ``step_c`` / ``step_size_c`` / ``float_to_half_c`` / ``half_to_float_c``: ctypes bindings of
  ``oracle/adam_oracle.c`` (the plain-C restatement of
  ``fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:94-130,153-162``).
* ``step_numpy`` / ``step_size_numpy``: the same equations written a second time with vectorised
  numpy float32 arithmetic and numpy's own float16 conversions.  It shares no code with the C file,
  so bitwise agreement between the two pins the software half conversions and the evaluation order.
* ``OracleAdam``: the host-side state machine of ``fairscale/optim/adam.py:184-297`` (lazy state,
  step counters, found_inf handling, optimizer-state-scale backoff/growth, state zeroing) over numpy
  arrays, used to check whole trajectories of the GPU optimizer.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Dict, List, Optional, Sequence

import numpy as np

FULL_PRECISION = 0
MIXED_PRECISION = 1
MEMORY_EFFICIENT_MIXED_PRECISION = 2
PURE_FP16 = 3
FULL_PRECISION_FP16_COPY = 4  # extension: fp32 step + fp16 copy of p (see adam_oracle.c)

MODE_NAMES = {
    FULL_PRECISION: "FULL_PRECISION",
    MIXED_PRECISION: "MIXED_PRECISION",
    MEMORY_EFFICIENT_MIXED_PRECISION: "MEMORY_EFFICIENT_MIXED_PRECISION",
    PURE_FP16: "PURE_FP16",
    FULL_PRECISION_FP16_COPY: "FULL_PRECISION_FP16_COPY",
}

# (param dtype, grad dtype, state dtype) per mode: fused_adam_cuda_kernel.cu:172-256
MODE_DTYPES = {
    FULL_PRECISION: (np.float32, np.float32, np.float32),
    MIXED_PRECISION: (np.float32, np.float16, np.float32),
    MEMORY_EFFICIENT_MIXED_PRECISION: (np.float16, np.float16, np.float32),
    PURE_FP16: (np.float16, np.float16, np.float16),
    FULL_PRECISION_FP16_COPY: (np.float32, np.float32, np.float32),
}

# algorithmic bytes per element: reads p,m,v,g + writes p,m,v(,p_copy)
MODE_BYTES = {FULL_PRECISION: 28, MIXED_PRECISION: 28, MEMORY_EFFICIENT_MIXED_PRECISION: 22, PURE_FP16: 14,
              FULL_PRECISION_FP16_COPY: 30}

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libadam_oracle.so")
_lib: Optional[ctypes.CDLL] = None


def build(force: bool = False) -> str:
    """Compile oracle/adam_oracle.c with gcc (see oracle/Makefile)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        f32, i32, i64, vp = ctypes.c_float, ctypes.c_int, ctypes.c_int64, ctypes.c_void_p
        L.fsadam_oracle_step_size.restype = f32
        L.fsadam_oracle_step_size.argtypes = [f32, f32, f32, i32, i32]
        L.fsadam_oracle_step.restype = i32
        L.fsadam_oracle_step.argtypes = [i32, vp, vp, vp, vp, vp, i64, f32, f32, f32, f32, f32, f32, f32, i32, i32, i32, vp]
        L.oracle_float_to_half.restype = ctypes.c_uint16
        L.oracle_float_to_half.argtypes = [f32]
        L.oracle_half_to_float.restype = f32
        L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.fsadam_oracle_threads.restype = i32
        L.oracle_float_to_half_array.restype = None
        L.oracle_float_to_half_array.argtypes = [vp, vp, i64]
        L.oracle_half_to_float_array.restype = None
        L.oracle_half_to_float_array.argtypes = [vp, vp, i64]
        _lib = L
    return _lib


def threads() -> int:
    return int(lib().fsadam_oracle_threads())


def step_size_c(lr: float, beta1: float, beta2: float, step: int, bias_correction: int) -> np.float32:
    return np.float32(lib().fsadam_oracle_step_size(lr, beta1, beta2, step, bias_correction))


def float_to_half_c(x: float) -> int:
    return int(lib().oracle_float_to_half(x))


def half_to_float_c(h: int) -> np.float32:
    return np.float32(lib().oracle_half_to_float(h))


def float_to_half_array_c(x: np.ndarray) -> np.ndarray:
    """float32 array -> uint16 array of half bit patterns, through the C oracle's software conversion."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().oracle_float_to_half_array(x.ctypes.data, out.ctypes.data, x.size)
    return out


def half_to_float_array_c(h: np.ndarray) -> np.ndarray:
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().oracle_half_to_float_array(h.ctypes.data, out.ctypes.data, h.size)
    return out


def _check(arr: np.ndarray, dtype, name: str) -> None:
    if arr.dtype != dtype or not arr.flags["C_CONTIGUOUS"]:
        raise TypeError(f"{name}: expected contiguous {np.dtype(dtype)}, got {arr.dtype}")


def step_c(mode: int, p: np.ndarray, m: np.ndarray, v: np.ndarray, g: np.ndarray, p_copy: Optional[np.ndarray], *,
           lr: float, beta1: float, beta2: float, eps: float, grad_scale: float = 1.0, optim_scale: float = 1.0,
           decay: float = 0.0, step: int, eps_mode: int = 1, bias_correction: int = 1,
           found_inf: Optional[np.ndarray] = None) -> None:
    """One in-place Adam step over one tensor with the C oracle. ``found_inf``: float32[1]."""
    pd, gd, sd = MODE_DTYPES[mode]
    _check(p, pd, "p"); _check(m, sd, "m"); _check(v, sd, "v"); _check(g, gd, "g")
    n = p.size
    assert m.size == n and v.size == n and g.size == n
    pc = None
    if mode in (MIXED_PRECISION, FULL_PRECISION_FP16_COPY):
        assert p_copy is not None
        _check(p_copy, np.float16, "p_copy")
        assert p_copy.size == n
        pc = p_copy.ctypes.data
    fi = None
    if found_inf is not None:
        _check(found_inf, np.float32, "found_inf")
        fi = found_inf.ctypes.data
    rc = lib().fsadam_oracle_step(mode, p.ctypes.data, m.ctypes.data, v.ctypes.data, g.ctypes.data, pc, n,
                                  lr, beta1, beta2, eps, grad_scale, optim_scale, decay, step, eps_mode,
                                  bias_correction, fi)
    if rc != 0:
        raise RuntimeError(f"fsadam_oracle_step failed: {rc}")


# ------------------------------------------------------------------------------------------------
# Second, independent restatement: numpy float32 vector arithmetic.
# ------------------------------------------------------------------------------------------------

def step_size_numpy(lr: float, beta1: float, beta2: float, step: int, bias_correction: int) -> np.float32:
    """fused_adam_cuda_kernel.cu:153-162 with its rounding points (double pow, float the rest)."""
    f = np.float32
    if bias_correction == 1:
        bc1 = f(1.0 - float(np.float64(f(beta1)) ** step))
        bc2 = f(1.0 - float(np.float64(f(beta2)) ** step))
        return f(f(f(lr) * np.sqrt(bc2, dtype=f)) / bc1)
    return f(lr)


def step_numpy(mode: int, p: np.ndarray, m: np.ndarray, v: np.ndarray, g: np.ndarray, p_copy: Optional[np.ndarray], *,
               lr: float, beta1: float, beta2: float, eps: float, grad_scale: float = 1.0, optim_scale: float = 1.0,
               decay: float = 0.0, step: int, eps_mode: int = 1, bias_correction: int = 1,
               found_inf: Optional[np.ndarray] = None, step_size: Optional[np.float32] = None) -> None:
    """Same contract as ``step_c``; numpy float32 ops are individually correctly rounded and unfused."""
    f = np.float32
    b1, b2, e, gs, os_, wd = f(beta1), f(beta2), f(eps), f(grad_scale), f(optim_scale), f(decay)
    ss = step_size if step_size is not None else step_size_numpy(lr, beta1, beta2, step, bias_correction)
    one = f(1)
    with np.errstate(all="ignore"):
        in_p = p.astype(f)
        sg = g.astype(f) / gs
        if mode == PURE_FP16:  # kernel.cu:94-105
            mom = b1 * (m.astype(f) / os_) + (one - b1) * sg
            vel = b2 * (v.astype(f) / os_) + ((one - b2) * sg) * sg
            m[...] = (mom * os_).astype(np.float16)
            v[...] = (vel * os_).astype(np.float16)
            if found_inf is not None and not (np.isfinite(m).all() and np.isfinite(v).all()):
                found_inf[0] = 1.0
        else:  # kernel.cu:115-121
            mom = b1 * m + (one - b1) * sg
            vel = b2 * v + ((one - b2) * sg) * sg
            m[...] = mom
            v[...] = vel
        denom = np.sqrt(vel + e) if eps_mode == 0 else np.sqrt(vel) + e
        update = mom / denom + wd * in_p
        new_p = in_p - ss * update
        assert new_p.dtype == f
        p[...] = new_p.astype(p.dtype)
        if mode in (MIXED_PRECISION, FULL_PRECISION_FP16_COPY):
            p_copy[...] = p.astype(np.float16)  # from the stored fp32 p: kernel.cu:129


# ------------------------------------------------------------------------------------------------
# Host state machine, fairscale/optim/adam.py:184-297, over numpy arrays.
# ------------------------------------------------------------------------------------------------

class OracleAdam:
    """Mirror of the reference optimizer's host logic for ONE param group on one device.

    ``params``: list of numpy arrays (fp32 for FULL, fp16 otherwise), updated in place.
    ``grads`` are handed to ``step`` (None entries are skipped like ``p.grad is None``, adam.py:212).
    """

    def __init__(self, params: Sequence[np.ndarray], mode: int, lr: float = 1e-3, bias_correction: bool = True,
                 betas=(0.9, 0.999), eps: float = 1e-8, eps_inside_sqrt: bool = False, weight_decay: float = 0.0,
                 kernel=step_c):
        self.params = list(params)
        self.mode = mode
        self.lr, self.bias_correction, self.betas, self.eps, self.weight_decay = lr, bias_correction, betas, eps, weight_decay
        self.eps_mode = 0 if eps_inside_sqrt else 1  # adam.py:117
        self.optim_dtype = MODE_DTYPES[mode][2]
        self.optim_scale = float(2 ** 16) if mode == PURE_FP16 else 1.0  # adam.py:101
        self.steps_since_optim_scale_change = 0  # adam.py:102
        self.optim_scale_update_freq = 2000  # adam.py:103
        self.state: List[Dict] = [dict() for _ in self.params]
        self.fp32_params: List[np.ndarray] = []
        if mode == MIXED_PRECISION:  # adam.py:123-129
            self.fp32_params = [p.astype(np.float32) for p in self.params]
        self._kernel = kernel

    def step(self, grads: Sequence[Optional[np.ndarray]], scale: float = 1.0) -> None:
        found_inf = np.zeros(1, np.float32)  # adam.py:256
        last_step = None
        launched = []
        for j, (p, g) in enumerate(zip(self.params, grads)):
            if g is None:
                continue
            st = self.state[j]
            if not st:  # adam.py:223-228
                st["step"] = 0
                st["exp_avg"] = np.zeros(p.shape, self.optim_dtype)
                st["exp_avg_sq"] = np.zeros(p.shape, self.optim_dtype)
            st["step"] += 1  # adam.py:234
            last_step = st["step"]
            launched.append(j)
        if last_step is None:
            raise IndexError("list index out of range")  # adam.py:256 with no grads at all
        for j in launched:  # one kernel call per group with the LAST param's step, adam.py:272
            st = self.state[j]
            p = self.fp32_params[j] if self.mode == MIXED_PRECISION else self.params[j]
            pc = self.params[j].reshape(-1) if self.mode == MIXED_PRECISION else None
            self._kernel(self.mode, p.reshape(-1), st["exp_avg"].reshape(-1), st["exp_avg_sq"].reshape(-1),
                         np.ascontiguousarray(grads[j]).reshape(-1), pc, lr=self.lr, beta1=self.betas[0],
                         beta2=self.betas[1], eps=self.eps, grad_scale=scale, optim_scale=self.optim_scale,
                         decay=self.weight_decay, step=last_step, eps_mode=self.eps_mode,
                         bias_correction=1 if self.bias_correction else 0, found_inf=found_inf)
        if found_inf[0] != 0:  # adam.py:278-288
            self.steps_since_optim_scale_change = 0
            self.optim_scale /= 2
            if self.optim_scale < 1.0:
                raise RuntimeError("Optimizer state scale < 1. This may mean that gradients are exploding")
            for st, p in zip(self.state, self.params):
                # the reference indexes self.state[p] for EVERY param (adam.py:285-288) and so creates
                # exp_avg / exp_avg_sq (without "step") even for params that never had a gradient
                st["exp_avg"] = np.zeros(p.shape, self.optim_dtype)
                st["exp_avg_sq"] = np.zeros(p.shape, self.optim_dtype)
        else:
            self.steps_since_optim_scale_change += 1  # adam.py:290
        if self.steps_since_optim_scale_change == self.optim_scale_update_freq:  # adam.py:292-295
            self.steps_since_optim_scale_change = 0
            if self.optim_scale < 2 ** 16:
                self.optim_scale *= 2
