"""The stand-alone drop-in for ``fairscale.fused_adam_cuda`` (``fairscale_amd/dropin/fused_adam_cuda.py``),
loaded the way a fairscale checkout would load it: as a module of its own that knows nothing of this
package, finding the library through ``FSADAM_LIBRARY``."""
from __future__ import annotations

import importlib.util
import os

import numpy as np
import pytest
import torch

import _cases as C
from _cases import FULL, MEMEFF, MIXED, PURE16

pytestmark = pytest.mark.gpu

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def dropin():
    os.environ["FSADAM_LIBRARY"] = os.path.join(REPO, "fairscale_amd", "csrc", "libfsadam.so")
    spec = importlib.util.spec_from_file_location("fused_adam_cuda", os.path.join(REPO, "fairscale_amd", "dropin", "fused_adam_cuda.py"))
    module = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(module)
    return module


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
def test_reference_call_sequence_through_the_drop_in(oracle, cuda_device, dropin, mode):
    """What fairscale/optim/adam.py:256-276 does per step: zero the flag, call ``adam`` with the 14 positional
    arguments, read the flag back."""
    sizes = [7, 300, 4097, 150001]
    host = C.Tensors(mode, sizes, 5200 + mode)
    to_dev = lambda arrs: [torch.from_numpy(a).to(cuda_device) for a in arrs]  # noqa: E731
    p, m, v = to_dev(host.p), to_dev(host.m), to_dev(host.v)
    p16 = to_dev(host.p16) if mode == MIXED else None
    flag = np.zeros(1, np.float32)
    optim_scale = 65536.0 if mode == PURE16 else 1.0
    noop = torch.zeros(1, dtype=torch.int32, device=cuda_device)
    for step in (1, 2, 3):
        grads = host.grads(step, scale=8.0 if mode != FULL else 1.0)
        g = to_dev(grads)
        found_inf = torch.zeros(1, dtype=torch.float32, device=cuda_device)
        lists = [p, m, v, g] + ([p16] if mode == MIXED else [])
        with torch.cuda.device(cuda_device):
            dropin.adam(2048 * 32, noop, lists, 1e-3, 0.9, 0.999, 1e-8, 8.0 if mode != FULL else 1.0, optim_scale, found_inf,
                        step, 1, 1, 0.01)
        assert found_inf.item() == 0.0
        for i in range(len(sizes)):
            oracle.step_c(mode, host.p[i], host.m[i], host.v[i], grads[i], host.p16[i] if host.p16 else None, lr=1e-3, beta1=0.9,
                          beta2=0.999, eps=1e-8, grad_scale=8.0 if mode != FULL else 1.0, optim_scale=optim_scale, decay=0.01,
                          step=step, eps_mode=1, bias_correction=1, found_inf=flag)
    pairs = [(host.p, p), (host.m, m), (host.v, v)] + ([(host.p16, p16)] if mode == MIXED else [])
    for want_list, got_list in pairs:
        for want, got in zip(want_list, got_list):
            assert np.array_equal(got.cpu().numpy().view(np.uint8), want.view(np.uint8))


def test_drop_in_raises_runtime_error_like_torch_check(dropin, cuda_device):
    mk = lambda *ns: [torch.zeros(n, device=cuda_device) for n in ns]  # noqa: E731
    flag = torch.zeros(1, device=cuda_device)
    with pytest.raises(RuntimeError):
        dropin.adam(0, None, [mk(4, 5), mk(4, 6), mk(4, 5), mk(4, 5)], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 1, 1, 0.0)
    with pytest.raises(RuntimeError, match="eps_mode"):
        dropin.adam(0, None, [mk(4)] * 4, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 7, 1, 0.0)


def test_drop_in_refuses_lists_of_the_wrong_element_type(dropin, cuda_device):
    """What the reference leaves to asserts that a release build compiles out (fused_adam_cuda_kernel.cu:167-199) is
    refused on the host, for every tensor, before anything is launched: a kernel would otherwise read the buffers at
    another element width, past their end."""
    f32 = lambda *ns: [torch.ones(n, device=cuda_device) for n in ns]  # noqa: E731
    f16 = lambda *ns: [torch.ones(n, device=cuda_device, dtype=torch.float16) for n in ns]  # noqa: E731
    flag = torch.zeros(1, device=cuda_device)
    args = (1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 1, 1, 0.0)
    bad_lists = [
        [f32(8), f32(8), f32(8), f16(8)],              # fp32 parameters with fp16 gradients in four lists
        [f32(8), f32(8), f32(8), f32(8), f16(8)],      # five lists with fp32 gradients
        [f32(8), f32(8), f32(8), f16(8), f32(8)],      # copy-out that is not fp16
        [f16(8), f32(8), f16(8), f16(8)],              # m and v of different types
        [f32(8, 8), f32(8, 8), f32(8, 8), f32(8) + f16(8)],  # a later tensor of another type
        [f32(8), f32(8), f32(8)],                      # three lists
        [f32(8, 8), f32(8), f32(8, 8), f32(8, 8)],     # lists of different lengths
    ]
    for lists in bad_lists:
        before = [t.clone() for lst in lists for t in lst]
        with pytest.raises(RuntimeError):
            dropin.adam(0, None, lists, *args)
        torch.cuda.synchronize(cuda_device)
        assert all(torch.equal(a, b) for a, b in zip(before, [t for lst in lists for t in lst]))
    with pytest.raises(RuntimeError, match="found_inf"):
        dropin.adam(0, None, [f32(8)] * 4, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag.double(), 1, 1, 1, 0.0)
