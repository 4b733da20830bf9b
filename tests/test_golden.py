"""The committed vectors (tests/golden/adam_step_vectors.npz): the oracle must still produce them
bit for bit (CPU), and so must the HIP kernels through the C ABI (GPU)."""
from __future__ import annotations

import importlib.util
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(HERE, "golden", "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)


def load():
    with np.load(os.path.join(HERE, "golden", "adam_step_vectors.npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def same_bits(a, b):
    """Bit-identical, except that a NaN matches any NaN (sign and payload of a generated NaN differ
    between x86 and the GPU; which elements are NaN must still agree)."""
    if a.dtype != b.dtype or a.shape != b.shape:
        return False
    nan_a, nan_b = np.isnan(a), np.isnan(b)
    if not np.array_equal(nan_a, nan_b):
        return False
    word = np.uint16 if a.dtype == np.float16 else np.uint32
    return np.array_equal(a.view(word)[~nan_a], b.view(word)[~nan_a])


def test_fixture_covers_every_mode_and_option():
    data = load()
    names = {k.split("/")[0] for k in data}
    assert names == {c[0] for c in make_golden.CASES} and len(names) == 9
    assert data["pure16_overflow_step2/flag1"][0] == 0.0 and data["pure16_overflow_step2/flag2"][0] == 1.0
    assert np.isinf(data["pure16_overflow_step2/v2"]).any() and np.isfinite(data["pure16_overflow_step2/p2"]).all()
    for name in names:
        if not name.startswith("pure16_overflow"):
            assert data[f"{name}/flag3"][0] == 0.0


def test_oracle_reproduces_the_golden_vectors(oracle):
    data = load()
    fresh = make_golden.build()
    assert sorted(fresh) == sorted(data)
    for key in data:
        assert same_bits(fresh[key], data[key]), key


@pytest.mark.gpu
@pytest.mark.parametrize("case", make_golden.CASES, ids=[c[0] for c in make_golden.CASES])
def test_kernels_reproduce_the_golden_vectors(cuda_device, case):
    import torch

    from fairscale_amd import _cabi, fused_adam_hip

    name, mode, hp = case
    data = load()
    p = torch.from_numpy(data[f"{name}/p0"].copy()).to(cuda_device)
    sd = torch.float16 if mode == _cabi.PURE_FP16 else torch.float32
    m = torch.zeros(p.numel(), dtype=sd, device=cuda_device)
    v = torch.zeros_like(m)
    c = p.half() if mode == _cabi.MIXED_PRECISION else None
    flag = torch.zeros(1, device=cuda_device)
    for step in range(1, make_golden.STEPS + 1):
        g = torch.from_numpy(data[f"{name}/g{step}"]).to(cuda_device)
        lists = [[p], [m], [v], [g]] + ([[c]] if c is not None else [])
        fused_adam_hip.adam(65536, None, lists, hp["lr"], hp["beta1"], hp["beta2"], hp["eps"], hp["grad_scale"], hp["optim_scale"],
                            flag, step, hp["eps_mode"], hp["bias_correction"], hp["decay"])
        torch.cuda.synchronize()
        for got, key in ((p, "p"), (m, "m"), (v, "v")):
            assert same_bits(got.cpu().numpy(), data[f"{name}/{key}{step}"]), f"{name} {key}{step}"
        if c is not None:
            assert same_bits(c.cpu().numpy(), data[f"{name}/c{step}"])
        assert flag.item() == data[f"{name}/flag{step}"][0]
