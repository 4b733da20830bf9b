"""Pins the gradient-pass oracle against torch's CPU implementation of the unscale op and torch.norm,
and checks the argument validation of ``fsadam_grad_pass`` (no device is touched)."""
from __future__ import annotations

import ctypes

import numpy as np
import pytest
import torch

from fairscale_amd import _cabi
from oracle import grad_oracle as G


def _grads(dtype, seed, sizes=(1, 7, 1000, 4099), scale=1.0):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal(n).astype(np.float32) * np.float32(1e-3 * scale)).astype(dtype) for n in sizes]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("inv_scale", [1.0, 1.0 / 1024, 1.0 / 3, 2.5])
def test_oracle_unscale_matches_torch_cpu_foreach(dtype, inv_scale):
    scale = 1.0 / inv_scale
    grads = _grads(dtype, 1, scale=scale)
    tg = [torch.from_numpy(g.copy()) for g in grads]
    found = torch.zeros(1)
    torch._amp_foreach_non_finite_check_and_unscale_(tg, found, torch.tensor([inv_scale], dtype=torch.float32))
    f, ss, mx = G.grad_pass_numpy(grads, inv_scale, write_back=True)
    assert f == found.item() == 0.0
    for a, b in zip(grads, tg):
        assert np.array_equal(a.view(np.uint8), b.numpy().view(np.uint8))  # same rounding of value * inv_scale
    want = torch.norm(torch.stack([torch.norm(t.double(), 2) for t in tg]), 2).item()  # calc_grad_norm's formula, in float64
    assert abs(G.total_norm(ss) - want) <= 1e-7 * want  # the squares are rounded to float32 before they are added
    in_float32 = torch.norm(torch.stack([torch.norm(t, 2, dtype=torch.float32) for t in tg]), 2).item()  # params.py:70-74 as written
    assert abs(G.total_norm(ss) - in_float32) <= 1e-6 * in_float32
    assert mx == max(t.abs().max().item() for t in tg)


def test_oracle_norm_overflows_where_the_float32_norm_does():
    """A float32 gradient above 1.8e19 has no float32 square: ``torch.norm(g, 2, dtype=torch.float32)`` is infinite
    (params.py:70-74), and so is the oracle's sum of squares; the largest magnitude stays finite and no
    overflow is flagged, because the incoming values are finite."""
    grads = [np.array([1.0, -3e19, 2.0], np.float32), np.array([0.5], np.float32)]
    tg = [torch.from_numpy(g.copy()) for g in grads]
    assert torch.isinf(torch.norm(tg[0], 2, dtype=torch.float32))
    f, ss, mx = G.grad_pass_numpy(grads, 1.0, write_back=False)
    assert f == 0.0 and np.isinf(ss) and mx == float(np.float32(3e19))


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("bad", [np.inf, -np.inf, np.nan])
def test_oracle_flags_non_finite_like_torch(dtype, bad):
    grads = _grads(dtype, 2)
    grads[2][123] = bad
    tg = [torch.from_numpy(g.copy()) for g in grads]
    found = torch.zeros(1)
    torch._amp_foreach_non_finite_check_and_unscale_(tg, found, torch.tensor([0.5], dtype=torch.float32))
    f, ss, mx = G.grad_pass_numpy(grads, 0.5, write_back=True)
    assert f == found.item() == 1.0
    for a, b in zip(grads, tg):  # the op keeps scaling after it has seen a non-finite value
        assert np.array_equal(np.isnan(a), np.isnan(b.numpy()))
        ok = ~np.isnan(a)
        assert np.array_equal(a[ok], b.numpy()[ok])
    if np.isnan(bad):
        assert np.isnan(ss) and np.isnan(mx)
    else:
        assert np.isinf(ss) and np.isinf(mx)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("inv_scale", [np.inf, -np.inf, np.nan])
@pytest.mark.parametrize("with_zero", [True, False])
def test_oracle_follows_torch_for_a_scale_that_is_not_finite(dtype, inv_scale, with_zero):
    """A degenerate factor: every finite non-zero gradient becomes an infinity (or NaN), and a gradient that is
    exactly zero becomes NaN (0 * inf), so the largest stored magnitude is NOT the image of the largest incoming
    one.  No flag: the incoming values are finite."""
    grads = _grads(dtype, 3)
    if with_zero:
        grads[2][17] = 0.0
    else:
        for g in grads:
            g[g == 0] = 1e-3
    tg = [torch.from_numpy(g.copy()) for g in grads]
    found = torch.zeros(1)
    torch._amp_foreach_non_finite_check_and_unscale_(tg, found, torch.tensor([inv_scale], dtype=torch.float32))
    f, ss, mx = G.grad_pass_numpy(grads, inv_scale, write_back=True)
    assert f == found.item() == 0.0
    for a, b in zip(grads, tg):
        assert np.array_equal(np.isnan(a), np.isnan(b.numpy())) and np.array_equal(a[~np.isnan(a)], b.numpy()[~np.isnan(a)])
    want_max = max(t.abs().max().item() for t in tg)  # Python's max keeps the first NaN it is given first; look at all
    any_nan = any(bool(torch.isnan(t).any()) for t in tg)
    if any_nan:
        assert np.isnan(mx) and np.isnan(ss)
        assert with_zero or np.isnan(inv_scale)
    else:
        assert np.isinf(mx) and np.isinf(ss) and np.isinf(want_max)


def test_oracle_leaves_gradients_alone_without_write_back():
    grads = _grads(np.float16, 3, scale=256.0)
    before = [g.copy() for g in grads]
    _, ss_dry, mx_dry = G.grad_pass_numpy(grads, 1 / 256, write_back=False)
    assert all(np.array_equal(a, b) for a, b in zip(grads, before))
    _, ss_wet, mx_wet = G.grad_pass_numpy(grads, 1 / 256, write_back=True)
    assert ss_dry == ss_wet and mx_dry == mx_wet  # norms are those of the values unscaling stores
    _, ss_again, _ = G.grad_pass_numpy(grads, 1.0, write_back=False)
    assert ss_again == ss_wet


def test_grad_pass_argument_errors_come_back_as_codes():
    L = _cabi.lib()
    A = 0x7000_0000_0000
    row = (_cabi.FsGradTensor * 1)()
    row[0].g, row[0].numel = A, 16
    call = lambda rows, n, dtype: L.fsadam_grad_pass(rows, n, dtype, 1.0, None, 1, None, None, None, None)  # noqa: E731
    assert call(row, 1, 7) == -1 and "dtype" in L.fsadam_last_error().decode()
    assert call(row, 0, _cabi.GRAD_F16) == -1
    assert call(None, 1, _cabi.GRAD_F16) == -1
    row[0].numel = -1
    assert call(row, 1, _cabi.GRAD_F32) == -1
    row[0].g, row[0].numel = A + 2, 16
    assert call(row, 1, _cabi.GRAD_F32) == -1 and "aligned" in L.fsadam_last_error().decode()
    row[0].g = None
    assert call(row, 1, _cabi.GRAD_F16) == -1
    assert ctypes.sizeof(_cabi.FsGradTensor) == 16


def test_python_wrapper_rejects_what_the_kernel_cannot_take():
    from fairscale_amd.grad_pass import grad_pass, supported

    assert not supported(torch.zeros(4))                       # not on a device
    with pytest.raises(RuntimeError):
        grad_pass([])
    with pytest.raises(RuntimeError, match="float16 or float32"):
        grad_pass([torch.zeros(4, dtype=torch.bfloat16)])
    with pytest.raises(RuntimeError, match="device tensors"):
        grad_pass([torch.zeros(4)])
    with pytest.raises(RuntimeError):
        grad_pass([torch.zeros(4), torch.zeros(4, dtype=torch.float16)])
