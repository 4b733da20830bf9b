"""Python face of the native step: same call as ``fairscale.fused_adam_cuda.adam``.

Reference: pybind module ``fairscale/clib/fused_adam_cuda/fused_adam_cuda.cpp:4-8``, dispatcher
``fused_adam_cuda_kernel.cu:137-265``, list validation ``multi_tensor_apply.cuh:49-67``.  Here the
tensor lists are turned into rows of plain pointers and handed to ``libfsadam.so`` through ctypes;
the kernels run on torch's current HIP stream and the call does not wait for them.
"""
from __future__ import annotations

import contextlib
import ctypes
import sys
from typing import List, Optional, Sequence

import numpy as np
import torch

from . import _cabi, _rows

__all__ = ["adam", "TensorListPlan", "mode_of_lists", "rows_of_lists", "checked_rows"]

_ROW_WORDS = ctypes.sizeof(_cabi.FsAdamTensor) // 8
assert _ROW_WORDS == 6, "FsAdamTensor is five pointers and one int64"


def mode_of_lists(tensor_lists: Sequence[Sequence[torch.Tensor]]) -> int:
    """dtype dispatch of fused_adam_cuda_kernel.cu:165-263 (looks at the first tensor of each list)."""
    depth = len(tensor_lists)
    if depth not in (4, 5):
        raise RuntimeError("tensor_lists.size() != depth")  # multi_tensor_apply.cuh:49
    if len(tensor_lists[0]) == 0:
        raise RuntimeError("tensor_lists[0].size() is not > 0")  # multi_tensor_apply.cuh:51
    p, m, v, g = (tensor_lists[d][0].dtype for d in range(4))
    if m != v:
        raise RuntimeError("exp_avg and exp_avg_sq must have the same dtype")  # kernel.cu:167
    if depth == 5:
        if p != torch.float32 or tensor_lists[4][0].dtype != torch.float16 or m != torch.float32 or g not in (torch.float16, torch.float32):
            raise RuntimeError("five lists expect fp32 params/state, fp16 or fp32 grads and fp16 output params")  # kernel.cu:174-176
        # fp32 grads with a copy-out have no case in the reference (its asserts require fp16 grads): extension
        return _cabi.MIXED_PRECISION if g == torch.float16 else _cabi.FULL_PRECISION_FP16_COPY
    if p != g:
        raise RuntimeError("params and grads must have the same dtype")  # kernel.cu:196
    if p == torch.float32:
        if m != torch.float32:
            raise RuntimeError("Optimizer state must be of type float for float parameters")  # kernel.cu:199
        return _cabi.FULL_PRECISION
    if p == torch.float16:
        if m == torch.float32:
            return _cabi.MEMORY_EFFICIENT_MIXED_PRECISION
        if m == torch.float16:
            return _cabi.PURE_FP16
        raise RuntimeError("Optimizer state must be of type float or half")  # kernel.cu:258
    raise RuntimeError("Parameters must be of type float or half")  # kernel.cu:261


_MODE_DTYPES = {
    _cabi.FULL_PRECISION: (torch.float32, torch.float32, torch.float32, torch.float32),
    _cabi.MIXED_PRECISION: (torch.float32, torch.float32, torch.float32, torch.float16, torch.float16),
    _cabi.MEMORY_EFFICIENT_MIXED_PRECISION: (torch.float16, torch.float32, torch.float32, torch.float16),
    _cabi.PURE_FP16: (torch.float16, torch.float16, torch.float16, torch.float16),
    _cabi.FULL_PRECISION_FP16_COPY: (torch.float32, torch.float32, torch.float32, torch.float32, torch.float16),
}


def validate_lists(tensor_lists: Sequence[Sequence[torch.Tensor]], mode: int) -> torch.device:
    """The checks of multi_tensor_apply.cuh:49-67, plus dtype/device uniformity (the kernels index raw
    memory, so what the reference leaves to asserts is enforced here).  Returns the lists' device."""
    dtypes = _MODE_DTYPES[mode]
    if len(tensor_lists) != len(dtypes):
        raise RuntimeError("tensor_lists.size() != depth")
    len0 = len(tensor_lists[0])
    if len0 == 0:
        raise RuntimeError("tensor_lists[0].size() is not > 0")
    device = tensor_lists[0][0].device
    for lst, dtype in zip(tensor_lists, dtypes):
        if len(lst) != len0:
            raise RuntimeError("Size mismatch among tensor lists")
        for t, t0 in zip(lst, tensor_lists[0]):
            if not t.is_contiguous():
                raise RuntimeError("A tensor was not contiguous.")
            if not t.is_cuda:
                raise RuntimeError("A tensor was not cuda.")
            if t.numel() != t0.numel():
                raise RuntimeError("Size mismatch")
            if t.dtype != dtype:
                raise RuntimeError(f"A tensor has dtype {t.dtype}, the list needs {dtype}.")
            if t.device != device:
                raise RuntimeError("Tensors of one call must live on one device.")
    return device


def rows_of_lists(tensor_lists: Sequence[Sequence[torch.Tensor]]) -> np.ndarray:
    """(n, 6) int64: p, m, v, g, p_copy pointers and numel -- the memory layout of FsAdamTensor[n]."""
    n = len(tensor_lists[0])
    rows = np.zeros((n, _ROW_WORDS), dtype=np.int64)
    data_ptr, numel = torch.Tensor.data_ptr, torch.Tensor.numel
    for d, lst in enumerate(tensor_lists):
        rows[:, d] = list(map(data_ptr, lst))  # C-level loop: this runs every step for every tensor
    rows[:, 5] = list(map(numel, tensor_lists[0]))
    return rows


def mode_codes(mode: int) -> tuple:
    """Element-type codes (0 float32, 1 float16) of the lists of a mode, for the C++ helper."""
    return tuple(_rows.dtype_code(dt) for dt in _MODE_DTYPES[mode])


def checked_rows(tensor_lists: Sequence[Sequence[torch.Tensor]], mode: int, rows: Optional[np.ndarray] = None):
    """Validate the lists and return ``(rows, changed, device)``.

    ``rows`` is a buffer of the right shape from an earlier call (or None): it is overwritten in place
    and ``changed`` tells whether any word differs from what it held.  One C++ pass when the helper is
    built; otherwise ``validate_lists`` + ``rows_of_lists``.
    """
    native = _rows.native
    depth_ok = len(tensor_lists) == len(_MODE_DTYPES[mode])
    if native is not None and depth_ok and len(tensor_lists[0]) > 0 and all(type(lst) is list for lst in tensor_lists):
        n = len(tensor_lists[0])
        first = tensor_lists[0][0]
        if isinstance(first, torch.Tensor) and first.is_cuda:
            fresh = rows is None or rows.shape != (n, _ROW_WORDS)
            buf = np.zeros((n, _ROW_WORDS), dtype=np.int64) if fresh else rows
            lists = tensor_lists if type(tensor_lists) is list else list(tensor_lists)
            status = native.fill_rows(lists, mode_codes(mode), first.device.index, buf.ctypes.data, n)[0]
            if status >= 0:
                return buf, bool(fresh or status == native.CHANGED), first.device
            if not fresh:
                buf[:] = 0  # partly overwritten: whatever comes next counts as changed
    # the Python walk raises the reference's messages for whatever the helper refused
    device = validate_lists(tensor_lists, mode)
    new = rows_of_lists(tensor_lists)
    changed = rows is None or rows.shape != new.shape or not np.array_equal(rows, new)
    return new, changed, device


def _rows_ptr(rows: np.ndarray):
    return rows.ctypes.data_as(ctypes.POINTER(_cabi.FsAdamTensor))


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_SAME_DEVICE = contextlib.nullcontext()


def _stream_handle(device: torch.device) -> int:
    """hipStream_t of torch's current stream on ``device`` (without building a Stream object when torch
    offers the raw handle: this runs once per step)."""
    if _raw_stream is not None and device.index is not None:
        return int(_raw_stream(device.index))
    return int(torch.cuda.current_stream(device).cuda_stream)


def _on_device(device: torch.device):
    """Context that makes ``device`` current for the native call; nothing to do when it already is."""
    if device.index is not None and torch.cuda.current_device() == device.index:
        return _SAME_DEVICE
    return torch.cuda.device(device)


def adam(chunk_size: int, noop_flag: Optional[torch.Tensor], tensor_lists: List[List[torch.Tensor]], lr: float,
         beta1: float, beta2: float, eps: float, grad_scale: float, optim_scale: float, found_inf: torch.Tensor,
         step: int, mode: int, bias_correction: int, decay: float) -> None:
    """Drop-in for ``fairscale.fused_adam_cuda.adam`` (fused_adam_cuda.cpp:4-8; call site adam.py:261-276).

    ``tensor_lists`` is ``[p, m, v, g]`` or ``[p32, m, v, g16, p16_out]``; ``mode`` is the eps mode
    (0 inside the square root, 1 outside).  ``chunk_size`` and ``noop_flag`` are accepted for
    signature compatibility and ignored: chunking is internal, and the reference kernel never reads
    ``noop_flag`` (fused_adam_cuda_kernel.cu:26).  ``found_inf`` is a float32[1] device tensor that is
    set to 1.0 when a stored fp16 ``m``/``v`` is non-finite (PURE_FP16 only) and never cleared.
    """
    precision = mode_of_lists(tensor_lists)
    rows, _, device = checked_rows(tensor_lists, precision)
    if found_inf is None or found_inf.dtype != torch.float32 or not found_inf.is_cuda or found_inf.numel() < 1:
        raise RuntimeError("found_inf must be a float32 device tensor with one element")
    if found_inf.device != device:
        raise RuntimeError("found_inf must live on the tensors' device")
    L = _cabi.lib()
    with _on_device(device):
        # float(): pybind narrows whatever has __float__ (numpy scalars, one-element tensors); so does this
        _cabi.check(L.fsadam_step(_rows_ptr(rows), rows.shape[0], precision, float(lr), float(beta1), float(beta2), float(eps),
                                  float(grad_scale), float(optim_scale), float(decay), int(step), int(mode), int(bias_correction),
                                  found_inf.data_ptr(), _stream_handle(device)))


class TensorListPlan:
    """A tensor list whose device-side table is kept between steps (fsadam_plan_* in include/fsadam.h).

    The optimizer holds one per (param group, device).  ``step`` re-reads every pointer, and only
    when one moved (or the list changed length) is the list validated again and its table re-sent.
    """

    def __init__(self, precision: int, device: torch.device, lazy_events: bool = True):
        self.precision = precision
        self.device = device
        self._rows: Optional[np.ndarray] = None
        self._dirty = True  # the device table does not (yet) hold what _rows holds
        self._handle = ctypes.c_void_p()
        _cabi.check(_cabi.lib().fsadam_plan_create(precision, ctypes.byref(self._handle)))
        # The streams this plan is stepped on are torch's, which live as long as the process, so the library may
        # record its events only when something has to wait for them (3 us less per step).  A caller that steps
        # on a torch.cuda.ExternalStream it destroys later passes lazy_events=False.
        if lazy_events:
            _cabi.check(_cabi.lib().fsadam_plan_lazy_events(self._handle, 1))

    def close(self) -> None:
        if self._handle:
            try:
                _cabi.lib().fsadam_plan_destroy(self._handle)
            finally:
                self._handle = ctypes.c_void_p()

    def __del__(self):  # pragma: no cover - interpreter shutdown order is not ours to test
        if sys is None or sys.is_finalizing():
            return  # the process is ending: nothing to give back, and the runtime underneath may be half gone
        try:
            self.close()
        except Exception:
            pass

    def info(self) -> dict:
        out = _cabi.FsAdamPlanInfo()
        _cabi.check(_cabi.lib().fsadam_plan_info(self._handle, ctypes.byref(out)))
        return out.as_dict()

    def rows_buffer(self, n: int) -> np.ndarray:
        """The (n, 6) int64 buffer the C++ walk fills in place; its contents mirror the device table
        unless ``mark_dirty`` was called since."""
        if self._rows is None or self._rows.shape != (n, _ROW_WORDS):
            self._rows = np.zeros((n, _ROW_WORDS), dtype=np.int64)
            self._dirty = True
        return self._rows

    def mark_dirty(self) -> None:
        """The buffer was partly overwritten by a walk that stopped: send the next table regardless."""
        self._dirty = True

    def step_rows(self, changed: bool, lr: float, beta1: float, beta2: float, eps: float, grad_scale: float,
                  optim_scale: float, found_inf: Optional[torch.Tensor], step: int, eps_mode: int, bias_correction: int,
                  decay: float) -> None:
        """Step over the rows already written into ``rows_buffer`` (validated by whoever wrote them).
        ``grad_scale`` is a Python float or a one-element float32 tensor on the plan's device, which the
        kernel reads when it runs (no host synchronisation)."""
        L = _cabi.lib()
        rows = self._rows
        scale_on_device = isinstance(grad_scale, torch.Tensor)
        if scale_on_device and (grad_scale.dtype != torch.float32 or grad_scale.numel() != 1 or grad_scale.device != self.device):
            raise RuntimeError("a tensor scale must be float32 with one element on the parameters' device")
        # a scheduler may leave a numpy scalar or a one-element tensor in the group: float() as pybind would
        lr, beta1, beta2, eps, optim_scale, decay = float(lr), float(beta1), float(beta2), float(eps), float(optim_scale), float(decay)
        with _on_device(self.device):
            stream = _stream_handle(self.device)
            if changed or self._dirty:
                # dirty until the library has taken the table: a call that fails leaves the device table stale (the
                # buffer already holds the new pointers), and the next step must send it again
                self._dirty = True
                _cabi.check(L.fsadam_plan_set_tensors(self._handle, _rows_ptr(rows), rows.shape[0], stream))
                self._dirty = False
            flag = found_inf.data_ptr() if found_inf is not None else None
            if scale_on_device:
                _cabi.check(L.fsadam_plan_step_dev_scale(self._handle, lr, beta1, beta2, eps, grad_scale.data_ptr(), optim_scale,
                                                         decay, int(step), int(eps_mode), int(bias_correction), flag, stream))
            else:
                _cabi.check(L.fsadam_plan_step(self._handle, lr, beta1, beta2, eps, float(grad_scale), optim_scale, decay,
                                               int(step), int(eps_mode), int(bias_correction), flag, stream))

    def current(self) -> bool:
        """The device table holds the rows of the last step (nothing failed or was left half-written since)."""
        return self._rows is not None and not self._dirty

    def holds_state(self, exp_avg_ptrs: List[int], exp_avg_sq_ptrs: List[int]) -> bool:
        """Does the device table point at exactly these m and v tensors, in this order?"""
        rows = self._rows
        return (self.current() and rows.shape[0] == len(exp_avg_ptrs) == len(exp_avg_sq_ptrs)
                and rows[:, 1].tolist() == exp_avg_ptrs and rows[:, 2].tolist() == exp_avg_sq_ptrs)

    def zero_state(self) -> None:
        """m = v = 0 for every tensor of the last step's list, in one launch (fsadam_plan_zero_state)."""
        with _on_device(self.device):
            _cabi.check(_cabi.lib().fsadam_plan_zero_state(self._handle, _stream_handle(self.device)))

    def step(self, tensor_lists: Sequence[Sequence[torch.Tensor]], lr: float, beta1: float, beta2: float, eps: float,
             grad_scale: float, optim_scale: float, found_inf: Optional[torch.Tensor], step: int, eps_mode: int,
             bias_correction: int, decay: float) -> None:
        try:
            rows, changed, device = checked_rows(tensor_lists, self.precision, self._rows)
        except Exception:
            self._dirty = True
            raise
        if device != self.device:
            self._dirty = True
            raise RuntimeError("tensor list moved to another device")
        self._rows = rows
        self.step_rows(changed, lr, beta1, beta2, eps, grad_scale, optim_scale, found_inf, step, eps_mode,
                       bias_correction, decay)
