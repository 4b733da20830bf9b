#!/usr/bin/env python3
"""Writes tests/golden/adam_step_vectors.npz: seeded inputs and the CPU oracle's outputs.

The reference publishes no numeric vectors for its fused Adam (its tests are behavioural), and its
kernel is CUDA, which cannot run where this was written.  These vectors therefore come from the CPU
oracle (oracle/adam_oracle.c), after the oracle itself has been pinned by tests/test_oracle.py
(library cross-checks, closed forms, equivariances).  They freeze that pinned behaviour: a later
edit of the oracle, or a kernel change, that alters a single bit of any case fails a test.

    python tests/golden/make_golden.py          # rewrites the .npz next to this script
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import adam_oracle as O  # noqa: E402

N = 1537  # odd on purpose: whole vectors plus a ragged tail
STEPS = 3

CASES = [
    # name, mode, hyper-parameters
    ("full_default", O.FULL_PRECISION, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=1.0, optim_scale=1.0, decay=0.0, eps_mode=1, bias_correction=1)),
    ("full_wd_eps_inside_nobc", O.FULL_PRECISION, dict(lr=3e-4, beta1=0.8, beta2=0.99, eps=1e-6, grad_scale=3.0, optim_scale=1.0, decay=0.01, eps_mode=0, bias_correction=0)),
    ("mixed_scale65536", O.MIXED_PRECISION, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=65536.0, optim_scale=1.0, decay=0.0, eps_mode=1, bias_correction=1)),
    ("mixed_wd_eps_inside", O.MIXED_PRECISION, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=128.0, optim_scale=1.0, decay=0.01, eps_mode=0, bias_correction=1)),
    ("memeff_scale1024", O.MEMORY_EFFICIENT_MIXED_PRECISION, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=1024.0, optim_scale=1.0, decay=0.0, eps_mode=1, bias_correction=1)),
    ("memeff_wd_nonpow2_scale", O.MEMORY_EFFICIENT_MIXED_PRECISION, dict(lr=2e-3, beta1=0.9, beta2=0.95, eps=1e-7, grad_scale=1000.0, optim_scale=1.0, decay=0.1, eps_mode=1, bias_correction=1)),
    ("pure16_scale65536", O.PURE_FP16, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=1.0, optim_scale=65536.0, decay=0.0, eps_mode=1, bias_correction=1)),
    ("pure16_overflow_step2", O.PURE_FP16, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=1.0, optim_scale=65536.0, decay=0.01, eps_mode=0, bias_correction=1)),
    ("pure16_nonpow2_optim_scale", O.PURE_FP16, dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=2.0, optim_scale=1000.0, decay=0.0, eps_mode=1, bias_correction=1)),
]


def build() -> dict:
    out = {}
    for idx, (name, mode, hp) in enumerate(CASES):
        pd, gd, sd = O.MODE_DTYPES[mode]
        rng = np.random.default_rng(9000 + idx)
        p = (rng.standard_normal(N).astype(np.float32) * np.float32(0.02)).astype(pd)
        if mode == O.MIXED_PRECISION:
            p16 = p.astype(np.float16)
            p = p16.astype(np.float32)
        else:
            p16 = None
        m, v = np.zeros(N, sd), np.zeros(N, sd)
        out[f"{name}/p0"] = p.copy()
        flag = np.zeros(1, np.float32)
        for step in range(1, STEPS + 1):
            g = (rng.standard_normal(N).astype(np.float32) * np.float32(1e-3 * hp["grad_scale"])).astype(gd)
            if name == "pure16_overflow_step2" and step == 2:
                g[N - 2] = np.float16(6e4)
            out[f"{name}/g{step}"] = g
            O.step_c(mode, p, m, v, g, p16, step=step, found_inf=flag, **hp)
            out[f"{name}/p{step}"] = p.copy()
            out[f"{name}/m{step}"] = m.copy()
            out[f"{name}/v{step}"] = v.copy()
            out[f"{name}/flag{step}"] = flag.copy()
            if p16 is not None:
                out[f"{name}/c{step}"] = p16.copy()
    return out


if __name__ == "__main__":
    data = build()
    path = os.path.join(HERE, "adam_step_vectors.npz")
    np.savez_compressed(path, **data)
    print(f"{path}: {len(data)} arrays, {os.path.getsize(path)} bytes")
