"""``GradScaler`` that accepts fp16 gradients, for use with the fp16-parameter precision modes.

Mirror of ``fairscale/optim/grad_scaler.py:60-68``: torch's scaler refuses to unscale fp16
gradients; the memory-efficient and pure-fp16 modes of ``Adam`` keep gradients in fp16, so the
unscale step is told to allow them.
"""
from __future__ import annotations

from typing import Dict

import torch
from torch.amp.grad_scaler import GradScaler as _TorchGradScaler

__all__ = ["GradScaler"]


class GradScaler(_TorchGradScaler):
    def _unscale_grads_(self, optimizer: torch.optim.Optimizer, inv_scale: torch.Tensor, found_inf: torch.Tensor,
                        allow_fp16: bool) -> Dict[torch.device, torch.Tensor]:
        return super()._unscale_grads_(optimizer, inv_scale, found_inf, True)
