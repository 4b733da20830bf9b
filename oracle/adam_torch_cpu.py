"""TEST INFRASTRUCTURE ONLY -- the same Adam math with in-place torch CPU ops (the CPU baseline).

``bench.py`` times this on the host cores next to the GPU number ("a CPU PyTorch run of the same
Adam math"); ``tests/test_oracle.py`` checks it against the C oracle.  Equations:
``fairscale/clib/fused_adam_cuda/fused_adam_cuda_kernel.cu:94-130``; step size ``:153-162``.
torch's fused CPU loops may contract or reorder by an ulp, so this one is compared with a tolerance,
never bitwise, and is never used as the parity checker.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import adam_oracle as O


@torch.no_grad()
def step_torch_cpu(mode: int, p: torch.Tensor, m: torch.Tensor, v: torch.Tensor, g: torch.Tensor,
                   p_copy: Optional[torch.Tensor], *, lr: float, beta1: float, beta2: float, eps: float,
                   grad_scale: float = 1.0, optim_scale: float = 1.0, decay: float = 0.0, step: int,
                   eps_mode: int = 1, bias_correction: int = 1, found_inf: Optional[torch.Tensor] = None) -> None:
    step_size = float(O.step_size_numpy(lr, beta1, beta2, step, bias_correction))
    g32 = g.float() if g.dtype != torch.float32 else g.clone()
    if grad_scale != 1.0:
        g32.div_(grad_scale)
    p32 = p.float() if p.dtype != torch.float32 else p
    if mode == O.PURE_FP16:
        m32 = m.float().div_(optim_scale)
        v32 = v.float().div_(optim_scale)
    else:
        m32, v32 = m, v
    m32.mul_(beta1).add_(g32, alpha=1 - beta1)
    v32.mul_(beta2).addcmul_(g32, g32, value=1 - beta2)
    denom = (v32 + eps).sqrt_() if eps_mode == 0 else v32.sqrt().add_(eps)
    update = m32 / denom
    if decay != 0.0:
        update.add_(p32, alpha=decay)
    if mode == O.PURE_FP16:
        m.copy_(m32.mul_(optim_scale))
        v.copy_(v32.mul_(optim_scale))
        if found_inf is not None and not (torch.isfinite(m).all() and torch.isfinite(v).all()):
            found_inf.fill_(1.0)
    if p32 is p:
        p.add_(update, alpha=-step_size)
    else:
        p.copy_(p32.add_(update, alpha=-step_size))
    if mode == O.MIXED_PRECISION:
        p_copy.copy_(p)
