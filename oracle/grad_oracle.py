"""TEST INFRASTRUCTURE ONLY -- CPU oracle of the pre-step gradient pass.

Restates, over numpy arrays, what the reference's callers compute on the gradients before the step:

* ``torch._amp_foreach_non_finite_check_and_unscale_`` as used by ``fairscale/optim/grad_scaler.py:211-215``
  (per element: raise found_inf when the value is not finite; store ``value * inv_scale`` computed in
  float32 and rounded to the gradient's dtype, or the value itself when ``inv_scale == 1``);
* ``calc_grad_norm`` (``fairscale/internal/params.py:59-76``): the 2-norm and the max-norm of all
  gradients as one vector, "in full precision no matter what".

Squares are taken in float32, as ``torch.norm(..., dtype=torch.float32)`` takes them (a gradient above
1.8e19 squares to infinity there, and the norm is infinite), and summed in float64: up to the order
of the additions this is the value the device result is compared with under a tolerance.  Pinned in
``tests/test_grad_pass_cpu.py`` against torch's own CPU implementation of the unscale op and
``torch.norm``.
"""
from __future__ import annotations

from typing import List, Sequence, Tuple

import numpy as np


def grad_pass_numpy(grads: Sequence[np.ndarray], inv_scale: float, write_back: bool) -> Tuple[float, float, float]:
    """Returns (found_inf, sum_squares, abs_max); rewrites ``grads`` in place when ``write_back``.

    ``abs_max`` is NaN when a stored value is NaN (torch's ``abs().max()`` propagates NaN)."""
    found = 0.0
    total = 0.0
    abs_max = np.float32(0.0)
    inv = np.float32(inv_scale)
    for g in grads:
        if g.size == 0:
            continue
        f = g.astype(np.float32)
        if not np.isfinite(f).all():
            found = 1.0
        with np.errstate(all="ignore"):
            r = g if inv == np.float32(1.0) else (f * inv).astype(g.dtype)
            u = r.astype(np.float32)
            total += float((u * u).astype(np.float64).sum())  # float32 squares, float64 sum
            m = np.abs(u).max()  # numpy's max propagates NaN
        abs_max = m if (np.isnan(m) or m > abs_max) and not np.isnan(abs_max) else abs_max
        if write_back and r is not g:
            g[...] = r
    return found, total, float(abs_max)


def total_norm(sum_squares: float) -> float:
    return float(np.sqrt(sum_squares))
