"""Optimizers: the ``fairscale.optim`` names this package provides (``Adam``, ``Precision``, ``GradScaler``).

Importing this package loads ``libfsadam.so``; when the library has not been built the import fails
with ``ImportError`` rather than hiding the classes.
"""
from ..grad_pass import calc_grad_norm, clip_grad_norm_, grad_pass
from .adam import Adam, Precision
from .grad_scaler import GradScaler

__all__ = ["Adam", "Precision", "GradScaler", "grad_pass", "calc_grad_norm", "clip_grad_norm_"]
