"""``GradScaler`` that accepts fp16 gradients, for use with the fp16-parameter precision modes.

Mirror of ``fairscale/optim/grad_scaler.py:60-68``: torch's scaler refuses to unscale fp16
gradients; the memory-efficient and pure-fp16 modes of ``Adam`` keep gradients in fp16, so the
unscale step is told to allow them.  Here the unscale step itself (torch's
``_amp_foreach_non_finite_check_and_unscale_``, one kernel family per dtype) runs on the fused
gradient pass, which also leaves the L2 norm of the unscaled gradients behind
(``unscaled_grad_norm``), so that clipping does not need another read of the gradients.
"""
from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Optional, Tuple

import torch
from torch.amp.grad_scaler import GradScaler as _TorchGradScaler
from torch.amp.grad_scaler import _MultiDeviceReplicator

from ..grad_pass import GradStats, grad_pass, supported

__all__ = ["GradScaler"]


class GradScaler(_TorchGradScaler):
    def _unscale_grads_(self, optimizer: torch.optim.Optimizer, inv_scale: torch.Tensor, found_inf: torch.Tensor,
                        allow_fp16: bool) -> Dict[torch.device, torch.Tensor]:
        per_device_inv_scale = _MultiDeviceReplicator(inv_scale)
        per_device_found_inf = _MultiDeviceReplicator(found_inf)
        buckets: Dict[Tuple[torch.device, torch.dtype], List[torch.Tensor]] = defaultdict(list)
        with torch.no_grad():
            for group in optimizer.param_groups:
                for param in group["params"]:
                    grad = param.grad
                    if grad is None:
                        continue
                    if grad.is_sparse:
                        # duplicate indices of a scaled fp16 gradient may overflow when summed: check the coalesced values
                        if grad.dtype is torch.float16:
                            param.grad = grad = grad.coalesce()
                        grad = grad._values()
                    buckets[(grad.device, grad.dtype)].append(grad)
            stats: List[GradStats] = []
            complete = True
            for (device, _dtype), grads in buckets.items():
                flag, scale = per_device_found_inf.get(device), per_device_inv_scale.get(device)
                if all(supported(g) for g in grads):
                    stats.append(grad_pass(grads, scale, write_back=True, found_inf=flag))
                else:  # other dtypes and layouts: torch's own multi-tensor kernel
                    torch._amp_foreach_non_finite_check_and_unscale_(grads, flag, scale)
                    complete = False
        self.__dict__.setdefault("_fused_stats", {})[id(optimizer)] = stats if complete else None
        return per_device_found_inf._per_device_tensors

    def unscaled_grad_norm(self, optimizer: torch.optim.Optimizer) -> Optional[torch.Tensor]:
        """L2 norm (float32 scalar tensor on the first gradient's device) of the gradients of ``optimizer``
        as the last ``unscale_`` left them, from the sums the unscale pass already took; None when some
        gradients went through torch's kernel instead (nothing was summed for them)."""
        stats = self.__dict__.get("_fused_stats", {}).get(id(optimizer))
        if not stats:
            return None
        total = stats[0].sum_squares
        for s in stats[1:]:
            total = total + s.sum_squares.to(total.device)
        return total.sqrt().to(torch.float32).reshape(())
