"""Seeded workloads and comparison helpers shared by the tests (CPU and GPU)."""
from __future__ import annotations

import random
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

FULL, MIXED, MEMEFF, PURE16 = 0, 1, 2, 3
MODE_DTYPES = {
    FULL: (np.float32, np.float32, np.float32),
    MIXED: (np.float32, np.float16, np.float32),
    MEMEFF: (np.float16, np.float16, np.float32),
    PURE16: (np.float16, np.float16, np.float16),
}


def gpt2_small_shapes() -> List[Tuple[int, ...]]:
    """148 tensors, 124 439 808 parameters."""
    shapes: List[Tuple[int, ...]] = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,),
                   (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]
    shapes += [(768,), (768,)]
    return shapes


def llama7b_shapes() -> List[Tuple[int, ...]]:
    """291 tensors, 6 738 415 616 parameters."""
    h, f, vocab = 4096, 11008, 32000
    shapes: List[Tuple[int, ...]] = [(vocab, h)]
    for _ in range(32):
        shapes += [(h, h)] * 4 + [(f, h), (h, f), (f, h), (h,), (h,)]
    shapes += [(h,), (vocab, h)]
    return shapes


def ragged_sizes(count: int = 4096, seed: int = 3000, max_log2: float = 20.0) -> List[int]:
    """numel = max(1, round(2**U(0, max_log2))): log-uniform, mostly not multiples of 4."""
    rng = random.Random(seed)
    return [max(1, round(2 ** rng.uniform(0.0, max_log2))) for _ in range(count)]


def numel(shape: Sequence[int]) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


class Tensors:
    """One tensor list in numpy: p, m, v (and p16 for MIXED) plus a grad generator."""

    def __init__(self, mode: int, sizes: Sequence[int], seed: int, p_std: float = 0.02):
        self.mode = mode
        self.sizes = list(sizes)
        pd, gd, sd = MODE_DTYPES[mode]
        rng = np.random.default_rng(seed)
        self.p = [(rng.standard_normal(n, dtype=np.float32) * np.float32(p_std)).astype(pd) for n in sizes]
        if mode == MIXED:
            # the optimizer builds masters from the fp16 params: start both from the same values
            self.p16 = [x.astype(np.float16) for x in self.p]
            self.p = [x.astype(np.float32) for x in self.p16]
        else:
            self.p16 = None
        self.m = [np.zeros(n, sd) for n in sizes]
        self.v = [np.zeros(n, sd) for n in sizes]
        self.seed = seed

    def grads(self, step: int, g_std: float = 1e-3, scale: float = 1.0) -> List[np.ndarray]:
        gd = MODE_DTYPES[self.mode][1]
        rng = np.random.default_rng(self.seed + step)
        out = []
        for n in self.sizes:
            g = rng.standard_normal(n, dtype=np.float32) * np.float32(g_std * scale)
            out.append(g.astype(gd))
        return out


def ulp_distance_f16(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Distance in fp16 units in the last place between same-shaped float16 arrays (NaN == NaN)."""
    def key(x):
        u = x.view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, 0x8000 - u, u)  # monotone integer line, -0 == +0
    d = np.abs(key(a) - key(b))
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


def assert_close_f32(got: np.ndarray, want: np.ndarray, what: str, rel: float = 1e-6, abs_floor: float = 1e-12) -> int:
    """|got-want| <= rel*|want| + abs_floor elementwise (NaN must match NaN, inf must match inf).
    Returns the number of elements that are not bit-identical."""
    assert got.dtype == np.float32 and want.dtype == np.float32 and got.shape == want.shape, what
    nan_g, nan_w = np.isnan(got), np.isnan(want)
    assert np.array_equal(nan_g, nan_w), f"{what}: NaN pattern differs"
    inf_w = np.isinf(want)
    assert np.array_equal(got[inf_w], want[inf_w]), f"{what}: infinities differ"
    fin = ~(nan_w | inf_w)
    g, w = got[fin].astype(np.float64), want[fin].astype(np.float64)
    err = np.abs(g - w)
    tol = rel * np.abs(w) + abs_floor
    bad = err > tol
    if bad.any():
        k = int(np.argmax(err - tol))
        raise AssertionError(f"{what}: {int(bad.sum())} of {bad.size} outside {rel:g} relative; worst got={g[k]!r} want={w[k]!r}")
    differs = (got.view(np.uint32) != want.view(np.uint32)) & ~nan_w  # NaN payloads are not compared
    return int(differs.sum())


def assert_close_f16(got: np.ndarray, want: np.ndarray, what: str, max_ulp: int = 1) -> int:
    assert got.dtype == np.float16 and want.dtype == np.float16 and got.shape == want.shape, what
    d = ulp_distance_f16(got, want)
    assert np.array_equal(np.isnan(got), np.isnan(want)), f"{what}: NaN pattern differs"
    if d.size and int(d.max()) > max_ulp:
        k = int(np.argmax(d))
        raise AssertionError(f"{what}: {int((d > max_ulp).sum())} of {d.size} more than {max_ulp} fp16 ulp apart; worst got={got[k]!r} want={want[k]!r}")
    return int((d != 0).sum())


def assert_close(got: np.ndarray, want: np.ndarray, what: str) -> int:
    if want.dtype == np.float16:
        return assert_close_f16(got, want, what)
    return assert_close_f32(got, want, what)
