"""GPU parity of the fused gradient pass (``fsadam_grad_pass`` through the C ABI) against its oracle.

Bars: what is stored (unscaled gradients) and the overflow flag are bit-exact; the max norm is exact
(a maximum does not round); the sum of squares is within 1e-6 relative of the oracle (both square in
float32, like ``torch.norm(..., dtype=float32)``, and add in float64; the device in a fixed order of its
own) and bit-identical between runs; where a float32 square overflows both are infinite."""
from __future__ import annotations

import math

import numpy as np
import pytest
import torch

import _cases as C
from oracle import grad_oracle as G

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 7, 8, 9, 255, 2047, 2048, 2049, 4095, 4097, 65535, 65536, 65537, 131071, 131072, 131073, 300001]


def host_grads(dtype, seed, sizes, scale=1.0):
    rng = np.random.default_rng(seed)
    return [(rng.standard_normal(n).astype(np.float32) * np.float32(1e-3 * scale)).astype(dtype) for n in sizes]


def run_both(host, device, inv_scale, write_back, misalign=0, scale_on_device=False):
    from fairscale_amd.grad_pass import grad_pass

    dev = []
    for h in host:
        t = torch.from_numpy(h).to(device)
        if misalign:
            big = torch.empty(h.size + misalign + 8, dtype=t.dtype, device=device)
            view = big[misalign:misalign + h.size]
            view.copy_(t)
            t = view
        dev.append(t)
    inv = torch.tensor([inv_scale], dtype=torch.float32, device=device) if scale_on_device else inv_scale
    stats = grad_pass(dev, inv, write_back=write_back)
    torch.cuda.synchronize()
    want = G.grad_pass_numpy(host, inv_scale, write_back)
    return dev, stats, want


def check(host, dev, stats, want, what):
    found, ss, mx = want
    assert stats.found_inf.item() == found, what
    for i, (h, d) in enumerate(zip(host, dev)):
        got = d.cpu().numpy()
        nan = np.isnan(h)
        assert np.array_equal(np.isnan(got), nan), f"{what} grad[{i}]"
        assert np.array_equal(got[~nan], h[~nan]), f"{what} grad[{i}] n={h.size}"
    got_ss, got_mx = stats.sum_squares.item(), stats.abs_max.item()
    if math.isnan(ss):
        assert math.isnan(got_ss) and math.isnan(got_mx), what
    elif math.isinf(ss):
        assert math.isinf(got_ss) and got_mx == mx, what
    else:
        assert abs(got_ss - ss) <= 1e-6 * ss, f"{what}: sum of squares {got_ss!r} vs {ss!r}"
        assert got_mx == mx, what


@pytest.mark.parametrize("seed", range(50))
def test_random_gradient_lists_match_the_oracle(cuda_device, seed):
    """Drawn configurations: dtype, list, sizes around the tile sizes of both kinds of pass, an element
    offset per tensor, factors that are 1, a power of two, a half, not a half, tiny and huge, with and
    without write-back, the factor on the host or on the device, special values planted."""
    import random

    rng = random.Random(7000 + seed)
    dtype = rng.choice([np.float16, np.float32])

    def draw_size():
        kind = rng.randrange(5)
        if kind == 0:
            return rng.choice([0, 1, 2, 3, 7, 9])
        if kind == 1:
            return rng.choice([1024, 2048, 4096]) * rng.randrange(1, 6) + rng.choice([-1, 0, 1])
        if kind == 2:
            return rng.randrange(10, 5000)
        if kind == 3:
            return 131072 + rng.choice([-1, 0, 1])
        return rng.randrange(131072, 400000)

    sizes = [draw_size() for _ in range(rng.randrange(1, 20))]
    if sum(sizes) == 0:
        sizes.append(33)
    inv_scale = rng.choice([1.0, 2.0 ** -7, 0.75, 1.0 / 3, 1e-4, 3e4 if dtype == np.float16 else 1e35])
    write_back = rng.random() < 0.6
    host = host_grads(dtype, 7100 + seed, sizes, scale=rng.choice([1.0, 1000.0]))
    info = np.finfo(dtype)
    if seed % 2:
        for g in host:
            for value in (np.inf, -np.inf, np.nan, info.max, -info.max, info.tiny, info.smallest_subnormal, 0.0, -0.0):
                if g.size and rng.random() < 0.2:
                    g[rng.randrange(g.size)] = value
    print(f"seed {seed}: {np.dtype(dtype)}, {len(sizes)} tensors, {sum(sizes)} elements, inv_scale {inv_scale}, write_back {write_back}", flush=True)
    from fairscale_amd.grad_pass import grad_pass

    dev = []
    for h in host:
        k = rng.choice([0, 0, 1, 3, 5])
        big = torch.empty(h.size + k + 8, dtype=torch.from_numpy(h).dtype, device=cuda_device)
        view = big[k:k + h.size]
        view.copy_(torch.from_numpy(h))
        dev.append(view)
    inv = torch.tensor([inv_scale], dtype=torch.float32, device=cuda_device) if rng.random() < 0.5 else inv_scale
    stats = grad_pass(dev, inv, write_back=write_back)
    torch.cuda.synchronize()
    want = G.grad_pass_numpy(host, inv_scale, write_back)
    check(host, dev, stats, want, f"seed {seed}")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("items,throttle,waves", [(2, 0, 1), (4, 65536, 4), (8, 13312, 16), (8, 0, 1), (2, 0, 16), (4, 0, 16), (8, 8192, 4)])
def test_every_compiled_shape_of_the_pass_matches_the_oracle(cuda_device, dtype, items, throttle, waves):
    """2, 4 or 8 vectors per lane and 1, 4 or 16 waves per workgroup are compiled; which runs is picked by
    the kind of pass unless the options say otherwise.  Same results for all of them."""
    from fairscale_amd import _cabi

    old = {k: _cabi.get_option(k) for k in ("grad_items", "grad_lds_throttle", "grad_waves")}
    try:
        _cabi.set_option("grad_items", items)
        _cabi.set_option("grad_lds_throttle", throttle)
        _cabi.set_option("grad_waves", waves)
        for write_back in (False, True):
            host = host_grads(dtype, 12, SIZES, scale=3.0)
            dev, stats, want = run_both(host, cuda_device, 1.0 / 3, write_back, misalign=1)
            check(host, dev, stats, want, f"items {items} throttle {throttle} wb {write_back}")
    finally:
        for k, v in old.items():
            _cabi.set_option(k, v)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("mid_tiles", [0, 2, 16, 64])
def test_descriptors_shared_by_a_few_tiles_do_not_change_the_pass(cuda_device, dtype, mid_tiles):
    """Middle-sized gradients share a descriptor among `mid_tiles` tiles (none with 0).  Sizes around the
    chunk boundaries that result for both dtypes and both kinds of pass."""
    from fairscale_amd import _cabi

    sizes = [1, 4095, 4096, 4097, 8191, 8192, 8193, 16384, 32767, 32768, 32769, 65535, 65536, 65537, 100000, 131071, 131072, 200001]
    old = _cabi.get_option("mid_tiles")
    _cabi.set_option("mid_tiles", mid_tiles)
    try:
        for write_back in (False, True):
            host = host_grads(dtype, 14, sizes, scale=64.0)
            dev, stats, want = run_both(host, cuda_device, 1 / 64, write_back, misalign=3)
            check(host, dev, stats, want, f"mid_tiles {mid_tiles} wb {write_back}")
    finally:
        _cabi.set_option("mid_tiles", old)


def test_unscale_by_an_inexact_factor_rounds_twice_on_every_path(cuda_device):
    """half(float32(float(g) * inv_scale)): the float32 rounding comes first, as in torch's kernel.  Many
    tensors just below one tile (element-wise path) plus a large one (vector path), enough elements for
    the one-in-10^4 cases where a single rounding of the exact product would differ."""
    host = host_grads(np.float16, 31, [2047] * 300 + [500003], scale=3.0)
    dev, stats, want = run_both(host, cuda_device, 1.0 / 3, True)
    check(host, dev, stats, want, "inexact factor")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("inv_scale", [1.0, 1.0 / 1024, 1.0 / 3])
@pytest.mark.parametrize("write_back", [True, False])
def test_ragged_list_matches_oracle(cuda_device, dtype, inv_scale, write_back):
    host = host_grads(dtype, 10, SIZES, scale=1.0 / inv_scale)
    dev, stats, want = run_both(host, cuda_device, inv_scale, write_back)
    check(host, dev, stats, want, f"{np.dtype(dtype)} inv={inv_scale} wb={write_back}")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("inv_scale", [np.inf, -np.inf, np.nan])
@pytest.mark.parametrize("write_back", [True, False])
def test_a_scale_that_is_not_finite_follows_torch(cuda_device, dtype, inv_scale, write_back):
    """With an infinite factor a zero gradient stores NaN (0 * inf) while the largest one stores an infinity: the
    maximum is NaN as torch's ``abs().max()`` makes it, although the kernel forms the stored maximum from the largest
    incoming magnitude; without a zero it is an infinity.  From the host and from the device."""
    for with_zero in (True, False):
        for on_device in (False, True):
            host = host_grads(dtype, 12, [5, 4099, 70001])
            for h in host:
                h[h == 0] = 1e-3
            if with_zero:
                host[2][40000] = 0.0
            dev, stats, want = run_both(host, cuda_device, float(inv_scale), write_back, scale_on_device=on_device)
            assert np.isnan(want[2]) == (with_zero or np.isnan(inv_scale))
            check(host, dev, stats, want, f"{np.dtype(dtype)} inv={inv_scale} zero={with_zero} device={on_device}")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_misaligned_views_and_device_resident_scale(cuda_device, dtype):
    host = host_grads(dtype, 11, [5, 4099, 70001, 140001], scale=64.0)
    dev, stats, want = run_both(host, cuda_device, 1 / 64, True, misalign=1, scale_on_device=True)
    check(host, dev, stats, want, "misaligned")


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("write_back", [True, False])
@pytest.mark.parametrize("align_heads", [1, 0])
def test_heads_split_off_gradient_views_between_cache_lines(cuda_device, dtype, write_back, align_heads):
    """Gradients of 8192 elements and more that start off a 1 KiB boundary give up their first elements to a
    descriptor of their own (the tiles behind start aligned); what is stored, the flag and the maximum stay
    exact and the sum of squares within its bar, with the option on and off, for views that start 1, 37 and
    300 elements into their allocations, one of them with a non-finite value inside the head."""
    from fairscale_amd import _cabi

    for shift in (1, 37, 300):
        host = host_grads(dtype, 12 + shift, [8191, 8192, 8193, 131072 + 200, 300001], scale=64.0)
        _cabi.set_option("align_heads", align_heads)
        try:
            dev, stats, want = run_both(host, cuda_device, 1 / 64, write_back, misalign=shift)
            check(host, dev, stats, want, f"shift {shift}")
            bad = host_grads(dtype, 99, [20000], scale=64.0)
            bad[0][3] = np.inf
            dev, stats, want = run_both(bad, cuda_device, 1 / 64, write_back, misalign=shift)
            assert want[0] == 1.0 and stats.found_inf.item() == 1.0
        finally:
            _cabi.set_option("align_heads", 1)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_non_finite_at_every_position_of_a_tile(cuda_device, dtype):
    """One inf or NaN at a time at every lane position of a 16-byte vector, at tile edges and in the
    ragged tail: flag up, norms inf/NaN, everything else still unscaled."""
    per_vec = 8 if dtype == np.float16 else 4
    tile = 64 * per_vec * 4
    n = 2 * tile + 3 * per_vec + 3
    positions = list(range(per_vec)) + [tile - 1, tile, tile + per_vec - 1, n - per_vec - 3, n - 2, n - 1]
    for pos in positions:
        for bad in (np.inf, np.nan):
            host = host_grads(dtype, 12, [n, 17], scale=16.0)
            host[0][pos] = bad
            dev, stats, want = run_both(host, cuda_device, 1 / 16, True)
            assert want[0] == 1.0
            check(host, dev, stats, want, f"{bad} at {pos}")
    host = host_grads(dtype, 12, [n, 17], scale=16.0)
    dev, stats, want = run_both(host, cuda_device, 1 / 16, True)
    assert want[0] == 0.0 and stats.found_inf.item() == 0.0


def test_subnormal_half_gradients_are_not_flushed(cuda_device):
    """Unscaled fp16 gradients below 6.1e-5 are subnormal halves: their squares must still be summed."""
    host = host_grads(np.float16, 13, [100003, 4099], scale=1e-3)  # ~1e-6: every value subnormal or zero
    assert all((np.abs(h.astype(np.float32)) < 6.2e-5).all() for h in host) and any((h != 0).any() for h in host)
    for inv_scale in (1.0, 0.5):
        dev, stats, want = run_both([h.copy() for h in host], cuda_device, inv_scale, True)
        assert want[1] > 0
        assert abs(stats.sum_squares.item() - want[1]) <= 1e-6 * want[1]
        assert stats.abs_max.item() == want[2] > 0


def test_found_inf_is_sticky_and_zero_sized_tensors_are_skipped(cuda_device):
    from fairscale_amd.grad_pass import grad_pass

    flag = torch.ones(1, device=cuda_device)
    g = [torch.zeros(0, device=cuda_device), torch.full((1000,), 3.0, device=cuda_device), torch.zeros(0, device=cuda_device)]
    stats = grad_pass(g, 0.5, found_inf=flag)
    assert stats.found_inf.item() == 1.0  # never cleared by the pass
    assert stats.sum_squares.item() == 1000 * 2.25 and stats.abs_max.item() == 1.5
    assert torch.equal(g[1], torch.full((1000,), 1.5, device=cuda_device))
    empty = grad_pass([torch.zeros(0, device=cuda_device)], 0.5)
    assert empty.sum_squares.item() == 0.0 and empty.abs_max.item() == 0.0 and empty.found_inf.item() == 0.0


def test_shard_sized_fp16_gradients_against_torch_and_determinism(cuda_device):
    """1.63e9 fp16 gradients (the shard of the benchmark): norm against torch's float64 sum over
    chunks, unscale against torch's multiplication, two runs bit-identical."""
    from fairscale_amd.grad_pass import grad_pass

    n = 1_630_000_000
    gen = torch.Generator(device=cuda_device).manual_seed(6000)
    g = torch.empty(n, device=cuda_device, dtype=torch.float16).normal_(0, 1.0, generator=gen)
    a = grad_pass([g], 1.0 / 1024, write_back=False)
    b = grad_pass([g], 1.0 / 1024, write_back=False)
    assert torch.equal(a.sum_squares, b.sum_squares) and torch.equal(a.abs_max, b.abs_max)
    want_ss, want_mx = 0.0, 0.0
    for lo in range(0, n, 1 << 27):
        u = (g[lo:lo + (1 << 27)].float() * (1.0 / 1024)).half().double()
        want_ss += float((u * u).sum().item())
        want_mx = max(want_mx, float(u.abs().max().item()))
        del u
    assert abs(a.sum_squares.item() - want_ss) <= 1e-6 * want_ss
    assert a.abs_max.item() == want_mx and a.found_inf.item() == 0.0
    ref = (g[-5_000_000:].float() * (1.0 / 1024)).half()
    grad_pass([g], 1.0 / 1024, write_back=True)
    assert torch.equal(g[-5_000_000:], ref)


def test_calc_grad_norm_and_clip_follow_the_reference_contract(cuda_device):
    """calc_grad_norm / clip_grad_norm_ against the reference's formulas written with torch ops
    (fairscale/internal/params.py:59-76, fairscale/optim/oss.py:244-302)."""
    from math import inf

    from fairscale_amd.optim import calc_grad_norm, clip_grad_norm_

    torch.manual_seed(3)
    for dtype in (torch.float32, torch.float16):
        params = [torch.nn.Parameter(torch.randn(n, device=cuda_device).to(dtype)) for n in (10, 3001, 200000)]
        params.append(torch.nn.Parameter(torch.randn(5, device=cuda_device).to(dtype)))  # no gradient: filtered out
        for p in params[:3]:
            p.grad = (torch.randn(p.numel(), device=cuda_device) * 0.01).to(dtype)
        grads = [p.grad for p in params[:3]]
        want2 = torch.norm(torch.stack([torch.norm(g.detach(), 2.0, dtype=torch.float32) for g in grads]), 2.0).to(dtype)
        got2 = calc_grad_norm(params, 2.0)
        assert got2.dtype == dtype and got2.shape == ()
        assert abs(got2.item() - want2.item()) <= (2e-3 if dtype == torch.float16 else 2e-6) * want2.item()
        assert calc_grad_norm(params, inf).item() == max(g.abs().max() for g in grads).item()
        want3 = torch.norm(torch.stack([torch.norm(g.detach(), 3.0, dtype=torch.float32) for g in grads]), 3.0).to(dtype)
        assert calc_grad_norm(params, 3.0).item() == want3.item()  # other p: torch.norm, as in the reference
        # clipping: total norm returned, gradients scaled by max_norm / (norm + 1e-6)
        max_norm = got2.item() / 2
        before = [g.clone() for g in grads]
        total = clip_grad_norm_(params, max_norm)
        assert total.item() == got2.item()
        coef = torch.tensor(max_norm, dtype=total.dtype, device=total.device) / (total + 1e-6)
        for g, b in zip(grads, before):
            assert torch.equal(g, b.clone().mul_(coef))
        after = calc_grad_norm(params, 2.0).item()
        assert abs(after - max_norm) <= 5e-3 * max_norm
        # no clipping needed: untouched
        snap = [g.clone() for g in grads]
        clip_grad_norm_(params, 10 * got2.item())
        assert all(torch.equal(g, s) for g, s in zip(grads, snap))
    assert calc_grad_norm([torch.nn.Parameter(torch.zeros(3, device=cuda_device))], 2.0).item() == 0.0


def test_folding_the_clip_into_the_step_matches_clipping_in_float32(cuda_device):
    """clip_grad_norm_(fold=True) + Adam.step(scale=...) on fp32 gradients: the step divides by
    1/clip_coef in registers; clipping first and stepping with scale 1 multiplies by clip_coef and
    stores. Same mathematics, one rounding apart: parameters agree to 1e-6 relative."""
    from fairscale_amd.optim import Adam, clip_grad_norm_

    torch.manual_seed(4)
    base = torch.randn(50000, device=cuda_device) * 0.02
    grad = torch.randn(50000, device=cuda_device) * 0.1
    outs = []
    for fold in (False, True):
        p = torch.nn.Parameter(base.clone())
        p.grad = grad.clone()
        opt = Adam([p], lr=1e-3)
        if fold:
            norm, scale = clip_grad_norm_([p], 1.0, fold=True)
            assert scale > 1.0 and torch.equal(p.grad, grad)
            opt.step(scale=scale)
        else:
            norm = clip_grad_norm_([p], 1.0)
            opt.step()
        outs.append((norm.item(), p.detach().clone()))
    assert outs[0][0] == outs[1][0]
    assert torch.allclose(outs[0][1], outs[1][1], rtol=1e-6, atol=1e-9)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("max_norm", [1.0, 1e6])
def test_clip_factor_kept_on_the_device_gives_the_bits_of_the_host_fold(cuda_device, dtype, max_norm):
    """fold="device": the factor never visits the host; the step kernel reads it from the tensor.  Same
    value as fold=True computes on the host, hence the same parameters bit for bit; with a max_norm
    above the norm the factor is exactly 1."""
    from fairscale_amd.optim import Adam, Precision, clip_grad_norm_

    torch.manual_seed(6)
    base = (torch.randn(300001, device=cuda_device) * 0.02).to(dtype)
    grad = (torch.randn(300001, device=cuda_device) * 0.1).to(dtype)
    precision = Precision.FULL_PRECISION if dtype == torch.float32 else Precision.MEMORY_EFFICIENT_MIXED_PRECISION
    outs = []
    for fold in (True, "device"):
        p = torch.nn.Parameter(base.clone())
        p.grad = grad.clone()
        opt = Adam([p], lr=1e-3, precision=precision)
        norm, scale = clip_grad_norm_([p], max_norm, fold=fold)
        if fold == "device":
            assert isinstance(scale, torch.Tensor) and scale.dtype == torch.float32 and scale.shape == (1,) and scale.is_cuda
        opt.step(scale=scale)
        outs.append((norm.item(), float(scale), p.detach().clone(), opt.state[p]["exp_avg"].clone(), opt.state[p]["exp_avg_sq"].clone()))
    # the host factor is a Python float that the call narrows to float32; the device one already is float32
    assert outs[0][0] == outs[1][0] and float(np.float32(outs[0][1])) == outs[1][1]
    assert (outs[0][1] > 1.0) == (max_norm == 1.0)
    for a, b in zip(outs[0][2:], outs[1][2:]):
        assert torch.equal(a, b)


def test_grad_scaler_unscales_through_the_fused_pass(cuda_device):
    from fairscale_amd.optim import Adam, GradScaler, Precision

    torch.manual_seed(5)
    w = (torch.randn(64, 32, device=cuda_device) * 0.1).half().requires_grad_()
    b = torch.zeros(64, device=cuda_device).half().requires_grad_()
    x = torch.randn(32, device=cuda_device).half()
    opt = Adam([w, b], lr=1e-2, precision=Precision.MEMORY_EFFICIENT_MIXED_PRECISION)
    scaler = GradScaler(init_scale=256.0)
    first = None
    for i in range(6):
        opt.zero_grad()
        loss = (w.mv(x) + b).pow(2).sum()
        first = loss.item() if first is None else first
        scaler.scale(loss).backward()
        scaled = [w.grad.clone(), b.grad.clone()]
        scaler.unscale_(opt)
        inv = 1.0 / scaler.get_scale()
        for g, s in zip((w.grad, b.grad), scaled):
            assert torch.equal(g, (s.float() * inv).half())
        norm = scaler.unscaled_grad_norm(opt)
        want = torch.norm(torch.stack([torch.norm(g.detach(), 2.0, dtype=torch.float32) for g in (w.grad, b.grad)]), 2.0)
        assert abs(norm.item() - want.item()) <= 2e-6 * want.item()
        scaler.step(opt)
        scaler.update()
    assert loss.item() < first
    # an overflowing backward: the flag goes up, the step is skipped and the scale backs off
    opt.zero_grad()
    w.grad = torch.full_like(w, float("inf"))
    b.grad = torch.zeros_like(b)
    before, scale_before = w.detach().clone(), scaler.get_scale()
    scaler.step(opt)
    scaler.update()
    assert torch.equal(w.detach(), before) and scaler.get_scale() == scale_before * 0.5


def test_whole_flow_unscale_norm_clip_on_device_step(oracle, cuda_device):
    """scale(loss).backward() -> unscale_ (fused pass) -> norm from the same pass -> clip factor formed on the
    device -> step(scale=factor) -> update(): the norm and the clip decision never visit the host (torch's scaler
    still reads its own overflow flag inside step()).  Replayed on the host from the scaled gradients: same
    parameters bit for bit."""
    from fairscale_amd.optim import Adam, GradScaler, Precision

    torch.manual_seed(8)
    sizes = [(64, 32), (64,), (300, 128)]
    params = [(torch.randn(*s, device=cuda_device) * 0.1).half().requires_grad_() for s in sizes]
    x = torch.randn(32, device=cuda_device).half()
    opt = Adam(params, lr=1e-2, precision=Precision.MEMORY_EFFICIENT_MIXED_PRECISION)
    ref = oracle.OracleAdam([p.detach().cpu().numpy().reshape(-1).copy() for p in params], oracle.MEMORY_EFFICIENT_MIXED_PRECISION, lr=1e-2)
    scaler = GradScaler(init_scale=256.0, growth_interval=2)
    max_norm = 0.05
    for it in range(5):
        opt.zero_grad()
        w, b, w2 = params
        loss = (w.mv(x) + b).float().pow(2).sum() + w2.float().pow(2).sum() * 0.01
        scaler.scale(loss).backward()
        scale_now = scaler.get_scale()
        scaled = [p.grad.detach().cpu().numpy().reshape(-1).copy() for p in params]
        scaler.unscale_(opt)
        norm = scaler.unscaled_grad_norm(opt)
        assert norm is not None
        factor = torch.clamp(norm / max_norm, min=1.0).reshape(1)
        scaler.step(opt, scale=factor)
        scaler.update()
        # the same on the host: unscale as the pass stores it, float64 sum of squares, the factor in float32
        inv = np.float32(1.0 / scale_now)
        unscaled = [(g.astype(np.float32) * inv).astype(np.float16) for g in scaled]
        total = np.sqrt(sum(float((u.astype(np.float64) ** 2).sum()) for u in unscaled))
        device_norm = np.float32(norm.item())  # read back only here, for the replay
        assert abs(float(device_norm) - total) <= 1e-6 * total, f"iteration {it}"
        host_factor = max(device_norm / np.float32(max_norm), np.float32(1.0))
        assert float(factor) == float(host_factor), f"iteration {it}"
        ref.step(unscaled, scale=float(host_factor))
        for p, want in zip(params, ref.params):
            assert np.array_equal(p.detach().cpu().numpy().reshape(-1).view(np.uint16), want.view(np.uint16)), f"iteration {it}"
    assert scaler.get_scale() > 256.0  # it grew: no overflow was seen
