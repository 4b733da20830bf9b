"""One read of the gradients before the optimizer step: non-finite check, unscale, L2 and max norms.

Host side of ``fsadam_grad_pass`` (include/fsadam.h).  It stands where the reference makes separate
passes over the gradients:

* ``torch._amp_foreach_non_finite_check_and_unscale_`` from the gradient scalers
  (``fairscale/optim/grad_scaler.py:60-68`` and ``:175-224``),
* ``calc_grad_norm`` (``fairscale/internal/params.py:59-76``), the local norm of
  ``OSS.clip_grad_norm`` (``fairscale/optim/oss.py:244-302``) and
  ``FullyShardedDataParallel.clip_grad_norm_`` (``fully_sharded_data_parallel.py:621-687``),
* the in-place multiplication by the clip coefficient (``oss.py:296-300``).

Everything stays on the device and on torch's current stream; only ``clip_grad_norm_`` reads a
scalar back, exactly where the reference does (``if clip_coef < 1``).
"""
from __future__ import annotations

import ctypes
from math import inf
from typing import Dict, Iterable, List, NamedTuple, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from . import _cabi, _rows

__all__ = ["GradStats", "grad_pass", "calc_grad_norm", "clip_grad_norm_"]

_DTYPE_CODE = {torch.float32: _cabi.GRAD_F32, torch.float16: _cabi.GRAD_F16}


class GradStats(NamedTuple):
    """Device-resident results of one pass over a list of gradients."""

    found_inf: torch.Tensor    # float32[1]: 1.0 when an incoming gradient was +-inf/NaN (never cleared here)
    sum_squares: torch.Tensor  # float64[1]: sum of squares of the (unscaled, stored-precision) gradients
    abs_max: torch.Tensor      # float32[1]: their largest magnitude (NaN if any is NaN)


def supported(grad: torch.Tensor) -> bool:
    """Dense, contiguous fp16/fp32 device tensors go through the kernel."""
    return grad.is_cuda and not grad.is_sparse and grad.dtype in _DTYPE_CODE and grad.is_contiguous()


def grad_pass(grads: Sequence[torch.Tensor], inv_scale: Union[float, torch.Tensor] = 1.0, *, write_back: bool = True,
              found_inf: Optional[torch.Tensor] = None) -> GradStats:
    """Run the pass over ``grads`` (one device, one dtype, fp16 or fp32, dense and contiguous).

    ``inv_scale``: a Python float or a one-element float32 tensor on the gradients' device (read on the
    device, no synchronisation).  ``write_back``: store ``dtype(g * inv_scale)`` over ``g`` (what
    unscaling does); with False the gradients are left alone and the norms are those the stored values
    would have had.  ``found_inf``: float32[1] device tensor to raise; a zeroed one is made when None.
    """
    if len(grads) == 0:
        raise RuntimeError("grad_pass needs at least one gradient")
    device, dtype = grads[0].device, grads[0].dtype
    if dtype not in _DTYPE_CODE:
        raise RuntimeError(f"gradients must be float16 or float32, got {dtype}")
    rows = np.empty((len(grads), 2), dtype=np.int64)
    native = _rows.native
    checked = False
    if native is not None and device.type == "cuda":
        # one C++ loop: layout, contiguity, device, dtype, pointer, numel
        status = native.fill_grad_rows(grads if type(grads) is list else list(grads), _rows.dtype_code(dtype), device.index,
                                       rows.ctypes.data)[0]
        checked = status >= 0
    if not checked:  # also names what the helper refused
        for g in grads:
            if g.device != device or g.dtype != dtype:
                raise RuntimeError("gradients of one pass must share device and dtype")
            if not g.is_cuda or g.is_sparse or not g.is_contiguous():
                raise RuntimeError("gradients must be dense, contiguous device tensors")
        rows[:, 0] = list(map(torch.Tensor.data_ptr, grads))
        rows[:, 1] = list(map(torch.Tensor.numel, grads))
    if found_inf is None:
        found_inf = torch.zeros(1, dtype=torch.float32, device=device)
    elif found_inf.dtype != torch.float32 or found_inf.device != device or found_inf.numel() != 1:
        raise RuntimeError("found_inf must be a float32 tensor with one element on the gradients' device")
    scale_value, scale_ptr = 1.0, None
    if isinstance(inv_scale, torch.Tensor):
        if inv_scale.dtype != torch.float32 or inv_scale.numel() != 1 or inv_scale.device != device:
            raise RuntimeError("a tensor inv_scale must be float32 with one element on the gradients' device")
        scale_ptr = inv_scale.data_ptr()
    else:
        scale_value = float(inv_scale)
    sum_squares = torch.empty(1, dtype=torch.float64, device=device)
    abs_max = torch.empty(1, dtype=torch.float32, device=device)
    with torch.cuda.device(device):
        _cabi.check(_cabi.lib().fsadam_grad_pass(
            rows.ctypes.data_as(ctypes.POINTER(_cabi.FsGradTensor)), len(grads), _DTYPE_CODE[dtype], scale_value, scale_ptr,
            1 if write_back else 0, found_inf.data_ptr(), sum_squares.data_ptr(), abs_max.data_ptr(),
            int(torch.cuda.current_stream(device).cuda_stream)))
    return GradStats(found_inf, sum_squares, abs_max)


def _by_device_and_dtype(grads: Iterable[torch.Tensor]) -> Dict[Tuple[torch.device, torch.dtype], List[torch.Tensor]]:
    groups: Dict[Tuple[torch.device, torch.dtype], List[torch.Tensor]] = {}
    for g in grads:
        groups.setdefault((g.device, g.dtype), []).append(g)
    return groups


def calc_grad_norm(parameters: Union[torch.Tensor, Iterable[torch.nn.Parameter]], p: float) -> torch.Tensor:
    """Norm of all gradients viewed as one vector: the contract of ``calc_grad_norm``
    (``fairscale/internal/params.py:59-76``).  p = 2 and p = inf run on the fused pass (one read of the
    gradients, fp32 squares summed in float64); other p use ``torch.norm`` as the reference does."""
    if isinstance(parameters, torch.Tensor):
        parameters = [parameters]
    params = [par for par in parameters if par.grad is not None]
    if len(params) == 0:
        return torch.tensor(0.0)
    p = float(p)
    grads = [par.grad for par in params]  # only read here; nothing below records autograd history
    if p not in (2.0, inf) or not all(map(supported, grads)):
        with torch.no_grad():
            if p == inf:
                return max(g.abs().max() for g in grads)
            return torch.norm(torch.stack([torch.norm(g, p, dtype=torch.float32) for g in grads]), p).to(dtype=params[0].dtype)
    first = grads[0].device
    stats = [grad_pass(group, 1.0, write_back=False) for group in _by_device_and_dtype(grads).values()]
    if p == inf:
        total = stats[0].abs_max.to(first)
        for s in stats[1:]:
            total = torch.maximum(total, s.abs_max.to(first))  # torch.maximum lets NaN through, like max()
        return total.reshape(()).to(dtype=params[0].dtype)
    total = stats[0].sum_squares.to(first)
    for s in stats[1:]:
        total = total + s.sum_squares.to(first)
    return total.sqrt().to(dtype=torch.float32).reshape(()).to(dtype=params[0].dtype)


def clip_grad_norm_(parameters: Union[torch.Tensor, Iterable[torch.nn.Parameter]], max_norm: Union[float, int],
                    norm_type: Union[float, int] = 2.0, *,
                    fold: Union[bool, str] = False) -> Union[torch.Tensor, Tuple[torch.Tensor, Union[float, torch.Tensor]]]:
    """One rank's part of ``OSS.clip_grad_norm`` (``oss.py:244-302``) / FSDP ``clip_grad_norm_``: the total
    norm, and gradients multiplied in place by ``max_norm / (norm + 1e-6)`` when that is below 1.
    (Across ranks the callers all-reduce ``norm**p`` in between; that stays with them.)

    ``fold=True`` skips the multiplication and returns ``(total_norm, grad_scale)`` instead, where
    ``grad_scale`` (>= 1) is the factor to hand to ``Adam.step(scale=...)``: the step then divides by it
    in registers, which saves a read and a write of every gradient.  ``fold="device"`` does the same
    without the host read-back: ``grad_scale`` is then a one-element float32 tensor on the norm's
    device holding the same value, which the step kernel reads when it runs.
    """
    if isinstance(parameters, torch.Tensor):
        parameters = [parameters]
    params = [par for par in parameters if par.grad is not None]
    max_norm, norm_type = float(max_norm), float(norm_type)
    total_norm = calc_grad_norm(params, norm_type)
    if len(params) == 0:
        return (total_norm, 1.0) if fold else total_norm
    clip_coef = torch.tensor(max_norm, dtype=total_norm.dtype, device=total_norm.device) / (total_norm + 1e-6)
    if fold == "device":
        # 1 / clip_coef evaluated in float64 and narrowed, as float(1.0 / float(clip_coef)) is on the host
        factor = clip_coef.double().reciprocal().float()
        return total_norm, torch.where(clip_coef < 1, factor, torch.ones_like(factor)).reshape(1)
    clipping = bool(clip_coef < 1)  # the reference's host read-back (oss.py:297)
    if fold:
        return total_norm, (1.0 / float(clip_coef)) if clipping else 1.0
    if clipping:
        grads = [par.grad for par in params]
        fast = [g for g in grads if supported(g)]
        for group in _by_device_and_dtype(fast).values():
            coef = clip_coef.to(device=group[0].device, dtype=torch.float32).reshape(1)
            grad_pass(group, coef, write_back=True)
        with torch.no_grad():
            for g in grads:
                if not supported(g):
                    g.mul_(clip_coef.to(g.device))
    return total_norm
