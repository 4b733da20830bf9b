"""GPU parity: the HIP step, called through the C ABI, against the CPU oracle on the same seeded inputs.

Tolerances (from the task statement): fp32 state within 1e-6 relative of the oracle, fp16 outputs
within 1 fp16 ulp of the oracle's fp32 result rounded to fp16, overflow flag exact.  The kernels are
built to evaluate the same IEEE operations in the same order as the oracle, so the tests also count
how many values are not bit-identical and require that count to be zero.
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

import _cases as C
from _cases import FULL, MEMEFF, MIXED, PURE16

pytestmark = pytest.mark.gpu

TORCH_DTYPE = {np.dtype(np.float32): torch.float32, np.dtype(np.float16): torch.float16}


def to_gpu(arrs, device):
    return [torch.from_numpy(a).to(device) for a in arrs]


def from_gpu(ts):
    return [t.cpu().numpy() for t in ts]


class GpuList:
    """Device copy of a ``_cases.Tensors`` stepped through ``fused_adam_hip.adam``."""

    def __init__(self, host: C.Tensors, device, misalign=None):
        self.mode = host.mode
        self.device = device
        self.misalign = misalign or {}
        self.p = self._place(host.p, "p")
        self.m = self._place(host.m, "m")
        self.v = self._place(host.v, "v")
        self.p16 = self._place(host.p16, "p16") if host.p16 is not None else None
        self.found_inf = torch.zeros(1, dtype=torch.float32, device=device)

    def _place(self, arrs, name):
        """Optionally put every tensor `k` elements into a larger allocation (a misaligned view)."""
        shift = self.misalign.get(name, 0)
        out = []
        for i, a in enumerate(arrs):
            t = torch.from_numpy(a).to(self.device)
            k = shift[i] if isinstance(shift, (list, tuple)) else shift  # one offset for all, or one per tensor
            if k:
                big = torch.empty(a.size + k + 8, dtype=t.dtype, device=self.device)
                view = big[k:k + a.size]
                view.copy_(t)
                t = view
            out.append(t)
        return out

    def step(self, grads_np, **kw):
        from fairscale_amd import fused_adam_hip

        g = self._place(grads_np, "g")
        lists = [self.p, self.m, self.v, g] + ([self.p16] if self.mode == MIXED else [])
        fused_adam_hip.adam(65536, None, lists, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], kw.get("grad_scale", 1.0),
                            kw.get("optim_scale", 1.0), self.found_inf, kw["step"], kw.get("eps_mode", 1),
                            kw.get("bias_correction", 1), kw.get("decay", 0.0))
        torch.cuda.synchronize(self.device)


def oracle_step(oracle, host: C.Tensors, grads, found_inf, **kw):
    for i in range(len(host.sizes)):
        if host.sizes[i] == 0:
            continue
        oracle.step_c(host.mode, host.p[i], host.m[i], host.v[i], grads[i], host.p16[i] if host.p16 else None,
                      found_inf=found_inf, **kw)


def compare(host: C.Tensors, dev: GpuList, tag: str, exact: bool = True):
    inexact = 0
    names = [("p", host.p, dev.p), ("m", host.m, dev.m), ("v", host.v, dev.v)]
    if host.p16 is not None:
        names.append(("p16", host.p16, dev.p16))
    for name, want_list, got_list in names:
        for i, (want, got) in enumerate(zip(want_list, got_list)):
            inexact += C.assert_close(got.cpu().numpy(), want, f"{tag} {name}[{i}] n={want.size}")
    if exact:
        assert inexact == 0, f"{tag}: {inexact} values within tolerance but not bit-identical to the oracle"
    return inexact


def run_case(oracle, device, mode, sizes, steps, seed, hyper, grad_scale=1.0, g_std=1e-3, misalign=None, optim_scale=1.0,
             mutate=None):
    host = C.Tensors(mode, sizes, seed)
    dev = GpuList(host, device, misalign)
    flag = np.zeros(1, np.float32)
    for step in range(1, steps + 1):
        grads = host.grads(step, g_std=g_std, scale=grad_scale)
        if mutate is not None:
            mutate(grads, step)
        kw = dict(hyper, step=step, grad_scale=grad_scale, optim_scale=optim_scale)
        dev.step(grads, **kw)
        oracle_step(oracle, host, grads, flag, **kw)
        compare(host, dev, f"mode={mode} step={step}")
    assert float(dev.found_inf.item()) == float(flag[0])
    return host, dev


DEFAULT = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, eps_mode=1, bias_correction=1, decay=0.0)


def test_c1_full_precision_flat_2pow20(oracle, cuda_device):
    """The CPU-runnable benchmark configuration on the GPU: one fp32 tensor of 2^20, 10 steps, fresh grads per step."""
    run_case(oracle, cuda_device, FULL, [1 << 20], 10, 1000, DEFAULT)


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
@pytest.mark.parametrize("eps_mode", [0, 1])
@pytest.mark.parametrize("bias_correction", [0, 1])
def test_modes_edge_sizes(oracle, cuda_device, mode, eps_mode, bias_correction):
    """Every dtype combination x eps placement x bias correction over sizes around every boundary
    the kernel has: vector width (4/8), tile (256..4096), the reference's 65536 chunk, the
    descriptors shared by 16 tiles (from 4096 elements, 8192 in PURE_FP16), the small/large tensor threshold
    (131072) and a large tensor that ends just into a shared chunk."""
    sizes = [1, 2, 3, 4, 5, 7, 8, 9, 15, 17, 255, 256, 257, 511, 513, 1023, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8192, 8193, 12289,
             16383, 16384, 16385,
             32769, 65535, 65536, 65537, 100003, 131071, 131072, 131073, 196611, 262144 + 5]
    hyper = dict(DEFAULT, eps_mode=eps_mode, bias_correction=bias_correction, decay=0.01)
    gs = 1.0 if mode == FULL else 1024.0
    run_case(oracle, cuda_device, mode, sizes, 3, 4000 + mode, hyper, grad_scale=gs, optim_scale=65536.0 if mode == PURE16 else 1.0)


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
def test_non_power_of_two_scales(oracle, cuda_device, mode):
    """grad_scale / optim_scale that are not powers of two take the true-division path."""
    hyper = dict(DEFAULT, decay=0.003, eps=1e-6)
    run_case(oracle, cuda_device, mode, [70001, 33, 8192], 3, 4100 + mode, hyper, grad_scale=3.0, optim_scale=1000.0 if mode == PURE16 else 1.0)


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
@pytest.mark.parametrize("which", ["p", "g", "m", "all"])
def test_misaligned_views(oracle, cuda_device, mode, which):
    """Views that start 1 element (p: 3) into an allocation, like OSS bucket views: their full tiles use
    the same vector instructions, at element-aligned addresses."""
    mis = {"p": {"p": 3}, "g": {"g": 1}, "m": {"m": 1}, "all": {"p": 1, "g": 1, "m": 1, "v": 1, "p16": 1}}[which]
    run_case(oracle, cuda_device, mode, [5, 4099, 16385, 40000, 140001], 2, 4200 + mode, dict(DEFAULT, decay=0.01),
             grad_scale=1.0 if mode == FULL else 128.0, misalign=mis, optim_scale=65536.0 if mode == PURE16 else 1.0)


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
@pytest.mark.parametrize("which", ["all", "p_and_g"])
@pytest.mark.parametrize("align_heads", [1, 0])
def test_heads_split_off_views_that_start_between_cache_lines(oracle, cuda_device, mode, which, align_heads):
    """Tensors of 8192 elements and more whose streams start off a 128-byte line give up a head of up to 511
    elements so that their tiles start on line boundaries; smaller ones and aligned ones do not.  Every
    stream shifted by the same element count (views into flat buffers: a common head aligns them all),
    or only p and g shifted (state allocated by the optimizer, parameters and gradients views): the
    head's elements, the tiles behind it and the ragged end must all come out as the oracle's, with the
    option on and off."""
    from fairscale_amd import _cabi

    sizes = [8191, 8192, 8193, 20000, 131071 + 300, 131072 + 511, 131072 + 512, 300001]
    shifts = [4, 4, 36, 260, 100, 511, 5, 7]
    names = ("p", "g", "m", "v", "p16") if which == "all" else ("p", "g", "p16")
    _cabi.set_option("align_heads", align_heads)
    try:
        run_case(oracle, cuda_device, mode, sizes, 2, 4300 + mode, dict(DEFAULT, decay=0.01), grad_scale=1.0 if mode == FULL else 128.0,
                 misalign={name: shifts for name in names}, optim_scale=65536.0 if mode == PURE16 else 1.0)
    finally:
        _cabi.set_option("align_heads", 1)


def test_steps_alternating_between_streams(oracle, cuda_device):
    """Every step runs on another stream than the one before.  In the first half the gradient tensors stay
    where they are, so kernels on one stream read a table that was uploaded on another (the library
    orders the two itself); in the second half they move, so each stream uploads its own table."""
    from fairscale_amd import fused_adam_hip

    host = C.Tensors(MEMEFF, [300_000, 5, 70_001, 1 << 18], 77)
    dev = GpuList(host, cuda_device)
    streams = [torch.cuda.Stream(device=cuda_device) for _ in range(3)]
    flag = np.zeros(1, np.float32)
    g = to_gpu(host.grads(1, g_std=1e-3, scale=1.0), cuda_device)
    for step in range(1, 9):
        grads = host.grads(step, g_std=1e-3, scale=1.0)
        if step <= 4:
            for dst, src in zip(g, grads):
                dst.copy_(torch.from_numpy(src))
        else:
            g = to_gpu(grads, cuda_device)
        torch.cuda.synchronize(cuda_device)  # the copies ran on the default stream, the last step on another
        kw = dict(DEFAULT, step=step, grad_scale=1.0, optim_scale=1.0)
        with torch.cuda.stream(streams[step % 3]):
            fused_adam_hip.adam(65536, None, [dev.p, dev.m, dev.v, g], kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], 1.0, 1.0,
                                dev.found_inf, step, 1, 1, 0.0)
        oracle_step(oracle, host, grads, flag, **kw)
        torch.cuda.synchronize(cuda_device)
        compare(host, dev, f"alternating streams, step {step}")


@pytest.mark.parametrize("seed", range(24))
def test_random_lists_match_the_oracle(oracle, cuda_device, seed):
    """Differential test on drawn configurations: mode, list length, sizes around every boundary (empty,
    below a tile, tile multiples +-1, around the large-tensor threshold), a separate element offset for
    every stream of every tensor (every third seed: up to 511 elements, shared by the streams or not),
    eps placement, bias correction, decay, power-of-two or odd scales;
    every second seed also plants infinities, NaNs, the largest and the smallest magnitudes and zeros
    in the gradients of the second step."""
    import random

    rng = random.Random(9000 + seed)
    mode = rng.choice([FULL, MIXED, MEMEFF, PURE16])
    tile = 512 if mode == PURE16 else 256

    def draw_size():
        kind = rng.randrange(6)
        if kind == 0:
            return rng.choice([0, 1, 2, 3])
        if kind == 1:
            return rng.randrange(4, tile)
        if kind == 2:
            return tile * rng.randrange(1, 40) + rng.choice([-1, 0, 1])
        if kind == 3:
            return rng.randrange(tile, 60000)
        if kind == 4:
            return 131072 + rng.choice([-1, 0, 1, 255, 257])
        return rng.randrange(131072, 500000)

    sizes = [draw_size() for _ in range(rng.randrange(1, 25))]
    if sum(sizes) == 0:
        sizes.append(77)
    names = ["p", "m", "v", "g", "p16"]
    misalign = {name: [rng.choice([0, 0, 1, 2, 3, 5, 7]) for _ in sizes] for name in names}
    if seed % 3 == 0:  # farther into the allocation: other heads in front of the aligned tiles (drawn apart, the sequence above stays)
        far = random.Random(77000 + seed)
        same = far.randrange(2) == 0  # one offset per tensor for every stream, or one per stream
        per_tensor = [far.choice([0, 1, 33, 64, 130, 300, 511]) for _ in sizes]
        misalign = {name: (per_tensor if same else [far.choice([0, 1, 33, 64, 130, 300, 511]) for _ in sizes]) for name in names}
    hyper = dict(lr=rng.choice([1e-3, 3e-2]), beta1=rng.choice([0.9, 0.5]), beta2=rng.choice([0.999, 0.95]),
                 eps=rng.choice([1e-8, 1e-3]), eps_mode=rng.randrange(2), bias_correction=rng.randrange(2),
                 decay=rng.choice([0.0, 0.01]))
    grad_scale = rng.choice([1.0, 128.0, 3.0]) if mode != FULL else rng.choice([1.0, 3.0])
    optim_scale = rng.choice([65536.0, 1024.0, 1000.0]) if mode == PURE16 else 1.0
    print(f"seed {seed}: mode {mode}, {len(sizes)} tensors, {sum(sizes)} elements, grad_scale {grad_scale}, optim_scale {optim_scale}, {hyper}",
          flush=True)
    def plant(grads, step):
        if step != 2 or seed % 2 == 0:
            return
        for g in grads:
            if g.size == 0:
                continue
            info = np.finfo(g.dtype)
            for value in (np.inf, -np.inf, np.nan, info.max, -info.max, info.tiny, info.smallest_subnormal, -info.smallest_subnormal, 0.0, -0.0):
                if rng.random() < 0.3:
                    g[rng.randrange(g.size)] = value

    run_case(oracle, cuda_device, mode, sizes, 3, 9100 + seed, hyper, grad_scale=grad_scale, misalign=misalign,
             optim_scale=optim_scale, mutate=plant)


@pytest.mark.parametrize("seed", range(16))
def test_random_packed_lists_match_the_oracle(oracle, cuda_device, seed):
    """Drawn lists whose streams are packed into flat buffers: every stream starts a drawn number of elements into its
    buffer (the same for all streams or one per stream, so that heads differ), and at drawn places a stream skips a few
    elements or a tensor of one stream lives in an allocation of its own, which cuts the list into runs of drawn lengths
    (single tensors, short runs, runs that are large only together).  Sizes around the tile, the shared-descriptor and
    the large-tensor boundaries, empty tensors inside runs.  Two steps against the oracle, and the run count against a
    count made here."""
    import random

    from fairscale_amd import fused_adam_hip

    rng = random.Random(12000 + seed)
    mode = rng.choice([FULL, MIXED, MEMEFF, PURE16])
    tile = 512 if mode == PURE16 else 256
    pd, gd, sd = C.MODE_DTYPES[mode]

    def draw_size():
        kind = rng.randrange(7)
        if kind == 0:
            return rng.choice([0, 1, 2, 3])
        if kind == 1:
            return rng.randrange(4, tile)
        if kind == 2:
            return tile * rng.randrange(1, 40) + rng.choice([-1, 0, 1])
        if kind == 3:
            return rng.randrange(tile, 9000)
        if kind == 4:
            return rng.randrange(9000, 70000)
        if kind == 5:
            return 131072 + rng.choice([-1, 0, 1, 255])
        return rng.randrange(131072, 400000)

    sizes = [draw_size() for _ in range(rng.randrange(2, 40))]
    if sum(sizes) == 0:
        sizes.append(300)
    names = ["p", "m", "v", "g"] + (["p16"] if mode == MIXED else [])
    same_lead = rng.randrange(2) == 0
    lead0 = rng.choice([0, 1, 3, 64, 130, 511])
    lead = {name: (lead0 if same_lead else rng.choice([0, 1, 3, 64, 130, 511])) for name in names}
    # where a stream breaks: ("gap", name, tensor) skips 1-70 elements in front of the tensor; ("own", name, tensor) puts it elsewhere
    breaks = {}
    for t in range(1, len(sizes)):
        if rng.random() < 0.25:
            breaks[(rng.choice(names), t)] = rng.choice(["gap", "own"])
    host = C.Tensors(mode, sizes, 12100 + seed)
    dtype_of = {"p": host.p[0].dtype if sizes else pd, "m": sd, "v": sd, "g": gd, "p16": np.float16}

    def pack(arrs, name):
        dt = TORCH_DTYPE[np.dtype(dtype_of[name])]
        flat = torch.full((sum(sizes) + lead[name] + 80 * len(sizes) + 8,), 7.0, dtype=dt, device=cuda_device)
        out, at = [], lead[name]
        for t, a in enumerate(arrs):
            how = breaks.get((name, t))
            if how == "gap":
                at += 1 + (t * 13 + seed) % 70
            view = torch.empty(a.size, dtype=dt, device=cuda_device) if how == "own" else flat[at:at + a.size]
            view.copy_(torch.from_numpy(a))
            out.append(view)
            if how != "own":
                at += a.size
        return out

    dev = GpuList.__new__(GpuList)
    dev.mode, dev.device, dev.misalign = mode, cuda_device, {}
    dev.p, dev.m, dev.v = pack(host.p, "p"), pack(host.m, "m"), pack(host.v, "v")
    dev.p16 = pack(host.p16, "p16") if host.p16 is not None else None
    dev.found_inf = torch.zeros(1, dtype=torch.float32, device=cuda_device)
    hyper = dict(lr=rng.choice([1e-3, 3e-2]), beta1=rng.choice([0.9, 0.5]), beta2=rng.choice([0.999, 0.95]), eps=rng.choice([1e-8, 1e-3]),
                 eps_mode=rng.randrange(2), bias_correction=rng.randrange(2), decay=rng.choice([0.0, 0.01]))
    grad_scale = rng.choice([1.0, 128.0, 3.0]) if mode != FULL else rng.choice([1.0, 3.0])
    optim_scale = rng.choice([65536.0, 1000.0]) if mode == PURE16 else 1.0
    # runs as the library must see them: a new one wherever any stream breaks in front of a non-empty tensor
    want_runs, open_run, broken = 0, False, False
    for t, n in enumerate(sizes):
        # a gap in front of a tensor stays in the stream whatever the tensor's size; an allocation of its own breaks the
        # sequence in front of and behind that tensor, unless the tensor is empty (an empty row is skipped)
        broken = (broken or any(breaks.get((name, t)) == "gap" for name in names)
                  or (n > 0 and any(breaks.get((name, t)) == "own" for name in names))
                  or (t > 0 and sizes[t - 1] > 0 and any(breaks.get((name, t - 1)) == "own" for name in names)))
        if n == 0:
            continue
        if not open_run or broken:
            want_runs += 1
        open_run, broken = True, False
    print(f"seed {seed}: mode {mode}, {len(sizes)} tensors, {sum(sizes)} elements, leads {lead}, {len(breaks)} breaks, {want_runs} runs", flush=True)
    plan = fused_adam_hip.TensorListPlan(mode, cuda_device)
    flag = np.zeros(1, np.float32)
    for step in (1, 2):
        grads = host.grads(step, scale=grad_scale)
        g = pack(grads, "g")
        lists = [dev.p, dev.m, dev.v, g] + ([dev.p16] if mode == MIXED else [])
        kw = dict(hyper, step=step, grad_scale=grad_scale, optim_scale=optim_scale)
        plan.step(lists, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], grad_scale, optim_scale, dev.found_inf, step, kw["eps_mode"],
                  kw["bias_correction"], kw["decay"])
        torch.cuda.synchronize(cuda_device)
        oracle_step(oracle, host, grads, flag, **kw)
        compare(host, dev, f"packed draw {seed} mode={mode} step={step}")
        # (fewer when the allocator happens to put two of the separately allocated tensors back to back)
        assert 1 <= plan.info()["n_runs"] <= want_runs
    assert float(dev.found_inf.item()) == float(flag[0])
    plan.close()


def test_pure_fp16_odd_optim_scale_rounds_twice_on_every_path(oracle, cuda_device):
    """m and v are stored as half(float32(m' * S)): two roundings (kernel.cu:100-101).  With a scale that is
    not a power of two the float32 product is inexact, and about one element in 10^4 lands exactly between
    two halves, where rounding the exact product once (a fused multiply-convert) gives the other
    neighbour.  Tensors just below one tile run the element-wise path, the large one the vector path."""
    run_case(oracle, cuda_device, PURE16, [511] * 300 + [300001], 3, 4700, dict(DEFAULT, lr=3e-2, beta1=0.5, eps=1e-3),
             grad_scale=3.0, optim_scale=1000.0)


@pytest.fixture
def options():
    """Set tuning options for one test and put the defaults back afterwards."""
    from fairscale_amd import _cabi

    names = ("lds_throttle", "mid_tiles", "upload_stream", "align_heads", "merge_runs")
    old = {k: _cabi.get_option(k) for k in names}

    def set_many(**kw):
        for k, v in kw.items():
            _cabi.set_option(k, v)

    yield set_many
    for k, v in old.items():
        _cabi.set_option(k, v)


@pytest.mark.parametrize("setting", [dict(lds_throttle=0), dict(lds_throttle=65536), dict(mid_tiles=0), dict(mid_tiles=2), dict(mid_tiles=64),
                                     dict(mid_tiles=4, align_heads=0), dict(merge_runs=0)])
def test_launch_geometry_options_do_not_change_results(oracle, cuda_device, options, setting):
    options(**setting)
    for mode in (MEMEFF, PURE16):
        run_case(oracle, cuda_device, mode, [5, 4099, 40000, 16384, 131071, 140001, 524288 + 17], 2, 4900 + mode, DEFAULT, grad_scale=8.0,
                 optim_scale=65536.0 if mode == PURE16 else 1.0)


@pytest.mark.parametrize("lazy_events", [0, 1])
@pytest.mark.parametrize("upload_stream", [1, 0])
def test_event_bookkeeping_eager_and_lazy(oracle, cuda_device, options, lazy_events, upload_stream):
    """The event behind a step is what protects a table that may still be read and what orders a step on
    another stream behind the one before.  Recorded behind every step (a plan's default) or only when
    needed (what this package switches on for its plans, torch's streams being immortal), the results are the same:
    steps hopping between three streams without any synchronisation by the caller, with the gradient
    pointers moving every step (a new table every step, the ring of slots wrapping around).  The tables
    travel on a stream of the library's own (default) or on the caller's."""
    from fairscale_amd import fused_adam_hip

    options(upload_stream=upload_stream)
    host = C.Tensors(FULL, [5, 4099, 140001, 70000], 5100)
    dev = GpuList(host, cuda_device)
    streams = [torch.cuda.Stream(cuda_device) for _ in range(3)]
    flag = np.zeros(1, np.float32)
    plan = fused_adam_hip.TensorListPlan(FULL, cuda_device, lazy_events=bool(lazy_events))
    keep = []
    for step in range(1, 13):
        grads = host.grads(step)
        g = to_gpu(grads, cuda_device)  # fresh allocations: the pointers move
        keep.append(g)
        torch.cuda.synchronize(cuda_device)  # the gradients were written on the default stream
        with torch.cuda.stream(streams[(step * 2) % 3]):
            plan.step([dev.p, dev.m, dev.v, g], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, dev.found_inf, step, 1, 1, 0.0)
        oracle_step(oracle, host, grads, flag, **dict(DEFAULT, step=step))
    torch.cuda.synchronize(cuda_device)
    compare(host, dev, f"lazy_events={lazy_events} upload_stream={upload_stream}")
    assert plan.info()["uploads"] == 12
    plan.close()


def test_pointer_changes_while_earlier_steps_are_in_flight(oracle, cuda_device):
    """Twelve steps enqueued back to back, each with gradient tensors at new addresses and nothing waiting
    in between: every step uploads a new table into the next slot of the plan's ring while the kernels
    of the steps before may still be reading theirs."""
    from fairscale_amd import fused_adam_hip
    from fairscale_amd import _cabi

    host = C.Tensors(MEMEFF, [300, 70001, 1 << 21, 5_000_000], 5300)
    dev = GpuList(host, cuda_device)
    all_grads = [host.grads(step) for step in range(1, 13)]
    on_device = [to_gpu(g, cuda_device) for g in all_grads]
    plan = fused_adam_hip.TensorListPlan(_cabi.MEMORY_EFFICIENT_MIXED_PRECISION, cuda_device)
    torch.cuda.synchronize(cuda_device)
    for step, g in enumerate(on_device, start=1):
        plan.step([dev.p, dev.m, dev.v, g], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, None, step, 1, 1, 0.0)
    assert plan.info()["uploads"] == 12
    torch.cuda.synchronize(cuda_device)
    flag = np.zeros(1, np.float32)
    for step, grads in enumerate(all_grads, start=1):
        oracle_step(oracle, host, grads, flag, **dict(DEFAULT, step=step, grad_scale=1.0, optim_scale=1.0))
    compare(host, dev, "12 steps in flight")
    plan.close()


def test_two_host_threads_step_their_own_lists(oracle, cuda_device):
    """``fsadam_step`` from two threads at once (ctypes releases the interpreter lock during the call), each
    on its own stream with its own list: the shared table cache is locked inside the library, errors are
    kept per thread."""
    import threading

    from fairscale_amd import fused_adam_hip

    cases = []
    for k, mode in enumerate((FULL, MEMEFF)):
        host = C.Tensors(mode, [33 + k, 5000 + k, 200000 + k], 5400 + k)
        cases.append((host, GpuList(host, cuda_device), torch.cuda.Stream(device=cuda_device)))
    all_grads = [[host.grads(step) for step in range(1, 9)] for host, _, _ in cases]
    on_device = [[to_gpu(g, cuda_device) for g in per_case] for per_case in all_grads]
    torch.cuda.synchronize(cuda_device)
    failures = []

    def worker(k):
        try:
            host, dev, stream = cases[k]
            with torch.cuda.device(cuda_device), torch.cuda.stream(stream):
                for step, g in enumerate(on_device[k], start=1):
                    fused_adam_hip.adam(0, None, [dev.p, dev.m, dev.v, g], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, dev.found_inf, step, 1, 1, 0.0)
        except Exception as exc:  # surfaces in the main thread below
            failures.append(exc)

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize(cuda_device)
    assert not failures, failures
    for k, (host, dev, _) in enumerate(cases):
        flag = np.zeros(1, np.float32)
        for step, grads in enumerate(all_grads[k], start=1):
            oracle_step(oracle, host, grads, flag, **dict(DEFAULT, step=step, grad_scale=1.0, optim_scale=1.0))
        compare(host, dev, f"thread {k}")


def test_more_lists_than_the_table_cache_holds(oracle, cuda_device):
    """``adam`` keeps the device tables of the last few lists it saw.  Twelve lists stepped in turn, three
    rounds, two modes: tables are evicted and rebuilt all the time, results stay those of the oracle."""
    cases = []
    for k in range(12):
        mode = MEMEFF if k % 2 else FULL
        host = C.Tensors(mode, [17 + k, 4096 + k, 140000 + 3 * k], 5000 + k)
        cases.append((host, GpuList(host, cuda_device), np.zeros(1, np.float32)))
    for step in (1, 2, 3):
        for host, dev, flag in cases:
            grads = host.grads(step)
            kw = dict(DEFAULT, step=step, grad_scale=1.0, optim_scale=1.0)
            dev.step(grads, **kw)
            oracle_step(oracle, host, grads, flag, **kw)
    for k, (host, dev, _) in enumerate(cases):
        compare(host, dev, f"list {k}")


@pytest.mark.parametrize("seed", range(40))
def test_extreme_states_and_hyperparameters_match_the_oracle(oracle, cuda_device, seed):
    """Drawn once more, now from the edges: infinities, NaNs, the largest and smallest magnitudes, zeros of both
    signs and a negative second moment planted in p, m and v before the first step; lr from 1e-8 to 1,
    betas 0 / 0.5 / 0.999, eps 0 or 1, decay up to 10, scales from 1e-3 to 2^18 (PURE_FP16 optimizer
    scales from 1/8 to 2^16), a step number of 100000.  IEEE arithmetic decides every result, on both
    sides the same."""
    import random

    rng = random.Random(20000 + seed)
    mode = rng.choice([FULL, MIXED, MEMEFF, PURE16])
    tile = 512 if mode == PURE16 else 256
    sizes = [rng.choice([1, 3, tile - 1, tile, tile + 1, 5 * tile + 3, 40000, 131072, 140001]) for _ in range(rng.randrange(1, 8))]
    host = C.Tensors(mode, sizes, 21000 + seed)
    with np.errstate(over="ignore"):
        for arrs in (host.p, host.m, host.v):
            for a in arrs:
                info = np.finfo(a.dtype)
                for value in (np.inf, -np.inf, np.nan, info.max, -info.max, info.tiny, info.smallest_subnormal, -info.smallest_subnormal,
                              0.0, -0.0, 1.0, -1e-30 if a.dtype == np.float32 else -6e-8):
                    if rng.random() < 0.25:
                        a[rng.randrange(a.size)] = value
        if mode == MIXED:
            host.p16 = [x.astype(np.float16) for x in host.p]
    misalign = {name: [rng.choice([0, 0, 1, 3]) for _ in sizes] for name in ("p", "m", "v", "g", "p16")}
    dev = GpuList(host, cuda_device, misalign)
    hyper = dict(lr=rng.choice([1e-3, 1.0, 1e-8]), beta1=rng.choice([0.9, 0.0, 0.999]), beta2=rng.choice([0.999, 0.5, 0.0]),
                 eps=rng.choice([1e-8, 0.0, 1.0]), eps_mode=rng.randrange(2), bias_correction=rng.randrange(2),
                 decay=rng.choice([0.0, 0.01, 10.0]))
    grad_scale = rng.choice([1.0, 128.0, 3.0, 1e-3, 65536.0 * 4])
    optim_scale = rng.choice([65536.0, 1.0, 1000.0, 2.0 ** -3]) if mode == PURE16 else 1.0
    flag = np.zeros(1, np.float32)
    print(f"seed {seed}: mode {mode}, sizes {sizes}, {hyper}, grad_scale {grad_scale}, optim_scale {optim_scale}", flush=True)
    for step in (1, 2, 3):
        with np.errstate(over="ignore"):
            grads = host.grads(step, g_std=rng.choice([1e-3, 1.0, 1e-6]), scale=grad_scale)
        kw = dict(hyper, step=step if rng.random() < 0.8 else 100000, grad_scale=grad_scale, optim_scale=optim_scale)
        dev.step(grads, **kw)
        oracle_step(oracle, host, grads, flag, **kw)
        compare(host, dev, f"seed {seed} mode {mode} step {step}")
    assert float(dev.found_inf.item()) == float(flag[0])


def test_zero_sized_tensors_in_list(oracle, cuda_device):
    run_case(oracle, cuda_device, FULL, [0, 5, 0, 0, 20000, 0], 2, 4300, DEFAULT)


def test_nine_thousand_tiny_tensors(oracle, cuda_device):
    """9000 tensors of 1..37 elements: one descriptor and one ragged tile each, all in the small-tensor launch."""
    sizes = [(i % 37) + 1 for i in range(9000)]
    run_case(oracle, cuda_device, MEMEFF, sizes, 2, 4400, dict(DEFAULT, decay=0.01), grad_scale=64.0)


def test_c3_ragged_4096_tensors(oracle, cuda_device):
    """The ragged-list benchmark configuration (4096 fp32 tensors, log-uniform sizes up to 2^20, wd 0.01, eps inside
    the square root) at full size for 2 steps."""
    sizes = C.ragged_sizes(4096, 3000, 20.0)
    assert sum(1 for n in sizes if n % 4) > 2000
    run_case(oracle, cuda_device, FULL, sizes, 2, 3000, dict(DEFAULT, decay=0.01, eps_mode=0))


def test_c3_ragged_20_steps_smaller(oracle, cuda_device):
    """The same recipe for the full 20 steps on 512 tensors up to 2^16."""
    sizes = C.ragged_sizes(512, 3001, 16.0)
    run_case(oracle, cuda_device, FULL, sizes, 20, 3001, dict(DEFAULT, decay=0.01, eps_mode=0))


def test_c2_gpt2_small_mixed_precision(oracle, cuda_device):
    """The GPT-2-small benchmark configuration at full size: 148 tensors / 124M parameters, fp32 master + fp16 grads scaled by
    65536 (passed as grad_scale) + fp16 copy-out.  Also checks p16 == half(p32) bitwise on the device."""
    sizes = [C.numel(s) for s in C.gpt2_small_shapes()]
    assert len(sizes) == 148 and sum(sizes) == 124_439_808
    host, dev = run_case(oracle, cuda_device, MIXED, sizes, 2, 2000, DEFAULT, grad_scale=65536.0)
    for p32, p16 in zip(dev.p, dev.p16):
        assert torch.equal(p32.half(), p16)


def test_full_precision_with_fp16_copy_out(oracle, cuda_device):
    """The extension mode for FSDP-style shards: fp32 p, g, m, v plus an fp16 copy of p written in the
    same pass.  p, m, v and the copy against the oracle, ragged sizes, one misaligned copy buffer."""
    from fairscale_amd import fused_adam_hip

    sizes = [1, 5, 255, 257, 4099, 70001, 131072, 200003]
    host = C.Tensors(FULL, sizes, 4800)
    copies = [np.zeros(n, np.float16) for n in sizes]
    dev = GpuList(host, cuda_device)
    dcopies = [torch.zeros(n, dtype=torch.float16, device=cuda_device) for n in sizes]
    big = torch.zeros(sizes[5] + 16, dtype=torch.float16, device=cuda_device)
    dcopies[5] = big[3:3 + sizes[5]]  # 6 bytes into its allocation: that tensor takes the element-wise path
    flag = torch.zeros(1, device=cuda_device)
    for step in range(1, 4):
        grads = host.grads(step)
        kw = dict(DEFAULT, decay=0.01, step=step)
        g = to_gpu(grads, cuda_device)
        fused_adam_hip.adam(65536, None, [dev.p, dev.m, dev.v, g, dcopies], kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], 1.0, 1.0,
                            flag, step, 1, 1, 0.01)
        torch.cuda.synchronize()
        for i in range(len(sizes)):
            oracle.step_c(oracle.FULL_PRECISION_FP16_COPY, host.p[i], host.m[i], host.v[i], grads[i], copies[i], **kw)
        compare(host, dev, f"fp16-copy step {step}")
        for i, (want, got) in enumerate(zip(copies, dcopies)):
            assert np.array_equal(got.cpu().numpy().view(np.uint16), want.view(np.uint16)), f"copy[{i}] step {step}"


def test_nonfinite_grads_propagate_without_flag(oracle, cuda_device):
    """inf / NaN gradients flow into p, m, v in the fp32-state modes and never raise the flag
    (only the fp16-state branch writes it, fused_adam_cuda_kernel.cu:103-105)."""
    for mode in (FULL, MIXED, MEMEFF):
        host = C.Tensors(mode, [4096 + 3], 4500 + mode)
        dev = GpuList(host, cuda_device)
        g = host.grads(1)
        g[0][5] = np.inf
        g[0][17] = -np.inf
        g[0][4097] = np.nan
        kw = dict(DEFAULT, step=1)
        dev.step(g, **kw)
        flag = np.zeros(1, np.float32)
        oracle_step(oracle, host, g, flag, **kw)
        compare(host, dev, f"nonfinite mode={mode}")
        assert dev.found_inf.item() == 0.0 and flag[0] == 0.0
        assert not np.isfinite(host.m[0][5])


def test_pure_fp16_flag_set_exactly_when_state_overflows(oracle, cuda_device):
    """A 6e4 gradient overflows fp16 v at any optimizer scale >= 1: the flag must go up, p is still
    updated from the finite fp32 moments, and the flag is never cleared by a later clean call."""
    host = C.Tensors(PURE16, [50000, 7], 4600)
    dev = GpuList(host, cuda_device)
    kw = dict(DEFAULT, step=1, optim_scale=65536.0)
    flag = np.zeros(1, np.float32)
    g = host.grads(1)
    dev.step(g, **kw)
    oracle_step(oracle, host, g, flag, **kw)
    compare(host, dev, "pure16 clean")
    assert dev.found_inf.item() == 0.0 and flag[0] == 0.0
    g = host.grads(2)
    g[0][49999] = np.float16(6e4)
    kw["step"] = 2
    dev.step(g, **kw)
    oracle_step(oracle, host, g, flag, **kw)
    compare(host, dev, "pure16 overflow")
    assert dev.found_inf.item() == 1.0 and flag[0] == 1.0
    assert np.isinf(host.v[0][49999]) and np.isfinite(host.p[0][49999])
    g = host.grads(3)
    kw["step"] = 3
    dev.step(g, **kw)
    assert dev.found_inf.item() == 1.0  # sticky: the caller clears it (adam.py:256)


@pytest.mark.parametrize("misaligned", [False, True])
def test_pure_fp16_flag_for_every_position_in_a_vector(oracle, cuda_device, misaligned):
    """One overflowing element at a time, at every position of a 128-bit packet (8 halves), in the
    ragged tail, in the first and the last chunk: the flag must go up each time, and stay down for
    the clean control.  Guards the in-kernel check against being applied to only part of a packet."""
    n = 3 * 1024 + 8 * 5 + 3  # a few whole tiles, a few whole vectors and a 3-element tail
    positions = list(range(0, 8)) + list(range(1024 - 8, 1024 + 8)) + list(range(n - 11, n)) + [None]
    kw = dict(DEFAULT, step=1, optim_scale=65536.0)
    for pos in positions:
        host = C.Tensors(PURE16, [n], 4700)
        dev = GpuList(host, cuda_device, {"m": 1} if misaligned else None)
        g = host.grads(1)
        if pos is not None:
            g[0][pos] = np.float16(6e4)
        dev.step(g, **kw)
        flag = np.zeros(1, np.float32)
        oracle_step(oracle, host, g, flag, **kw)
        compare(host, dev, f"overflow at {pos}")
        want = 0.0 if pos is None else 1.0
        assert flag[0] == want
        assert dev.found_inf.item() == want, f"overflow injected at element {pos} (misaligned={misaligned})"
        nonfinite = (~torch.isfinite(dev.m[0])).any().item() or (~torch.isfinite(dev.v[0])).any().item()
        assert nonfinite == (pos is not None)


@pytest.mark.parametrize("merge_runs", [0, 1])
def test_flat_vs_split_is_bitwise_identical(cuda_device, options, merge_runs):
    """Chunking/table invariance at a size the oracle is not needed for: one flat 2^24+5 tensor and
    the same memory stepped as 7 uneven tensors give identical bits (elementwise path).  With the rows laid
    out one by one (merge_runs=0) and, the default, merged back into the one run they form."""
    from fairscale_amd import fused_adam_hip

    options(merge_runs=merge_runs)
    n = (1 << 24) + 5
    gen = torch.Generator(device=cuda_device).manual_seed(7)
    base = [torch.randn(n, device=cuda_device, generator=gen) * s for s in (0.02, 1e-3, 1e-6, 1e-3)]
    base[2].abs_()
    flag = torch.zeros(1, device=cuda_device)
    a = [t.clone() for t in base]
    b = [t.clone() for t in base]
    fused_adam_hip.adam(65536, None, [[t] for t in a], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 5, 1, 1, 0.01)
    cuts = [0, 8, 8 + 4096, 100000, 100000 + 65536 * 3, 1 << 23, (1 << 24) - 8, n]  # multiples of 4: views stay aligned
    lists = [[t[cuts[i]:cuts[i + 1]] for i in range(len(cuts) - 1)] for t in b]
    fused_adam_hip.adam(65536, None, lists, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 5, 1, 1, 0.01)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    plan = fused_adam_hip.TensorListPlan(FULL, cuda_device)
    plan.step(lists, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 6, 1, 1, 0.01)
    assert plan.info()["n_runs"] == (1 if merge_runs else 7) and plan.info()["n_tensors"] == 7
    plan.close()
    # and determinism: the same call on the same inputs twice
    c = [t.clone() for t in base]
    fused_adam_hip.adam(65536, None, [[t] for t in c], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 5, 1, 1, 0.01)
    for x, y in zip(a, c):
        assert torch.equal(x, y)


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
@pytest.mark.parametrize("lead", [0, 3])
def test_lists_packed_into_flat_buffers_match_the_oracle(oracle, cuda_device, mode, lead):
    """Every stream of the list packed back to back into a flat buffer of its own (``lead`` elements in), so that the
    whole list is one run; then the same with the second moment of one tensor and the gradient of another in
    allocations of their own, which cuts the list into five runs.  Against the oracle, which knows nothing of runs."""
    from fairscale_amd import fused_adam_hip

    sizes = [5, 4099, 16385, 40000, 140001, 3, 70000]
    total = sum(sizes)
    for stray in ({}, {"v": 2, "g": 4}):
        host = C.Tensors(mode, sizes, 5300 + mode)
        pd, gd, sd = C.MODE_DTYPES[mode]

        def pack(arrs, name, dtype):
            flat = torch.empty(total + lead, dtype=TORCH_DTYPE[np.dtype(dtype)], device=cuda_device)
            out, at = [], lead
            for i, a in enumerate(arrs):
                view = flat[at:at + a.size] if stray.get(name) != i else torch.empty(a.size, dtype=flat.dtype, device=cuda_device)
                view.copy_(torch.from_numpy(a))
                out.append(view)
                at += a.size
            return out

        dev = GpuList.__new__(GpuList)
        dev.mode, dev.device, dev.misalign = mode, cuda_device, {}
        dev.p, dev.m, dev.v = pack(host.p, "p", host.p[0].dtype), pack(host.m, "m", sd), pack(host.v, "v", sd)
        dev.p16 = pack(host.p16, "p16", np.float16) if host.p16 is not None else None
        dev.found_inf = torch.zeros(1, dtype=torch.float32, device=cuda_device)
        plan = fused_adam_hip.TensorListPlan(mode, cuda_device)
        flag = np.zeros(1, np.float32)
        gs = 1.0 if mode == FULL else 64.0
        for step in (1, 2):
            grads = host.grads(step, scale=gs)
            g = pack(grads, "g", gd)
            lists = [dev.p, dev.m, dev.v, g] + ([dev.p16] if mode == MIXED else [])
            kw = dict(DEFAULT, decay=0.01, step=step, grad_scale=gs, optim_scale=65536.0 if mode == PURE16 else 1.0)
            plan.step(lists, kw["lr"], kw["beta1"], kw["beta2"], kw["eps"], gs, kw["optim_scale"], dev.found_inf, step, 1, 1, kw["decay"])
            torch.cuda.synchronize(cuda_device)
            oracle_step(oracle, host, grads, flag, **kw)
            compare(host, dev, f"packed mode={mode} lead={lead} stray={stray} step={step}")
            assert plan.info()["n_runs"] == (5 if stray else 1)  # [0,1] [2] [3] [4] [5,6]
        plan.close()


def test_the_library_refuses_a_stream_that_is_being_captured(cuda_device):
    """Recorded into a graph the step would replay one step's bias correction for ever: FSADAM_EINVAL, nothing enqueued."""
    from fairscale_amd import _cabi, fused_adam_hip

    t = [torch.full((5000,), x, device=cuda_device) for x in (0.5, 0.0, 0.0, 0.01)]
    flag = torch.zeros(1, device=cuda_device)
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(_cabi.FsAdamError, match="captured"):
        with torch.cuda.graph(graph):
            fused_adam_hip.adam(65536, None, [[x] for x in t], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 1, 1, 0.0)
    torch.cuda.synchronize(cuda_device)
    assert float(t[0][0]) == 0.5 and float(t[1].abs().max()) == 0.0
    fused_adam_hip.adam(65536, None, [[x] for x in t], 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 1, 1, 0.0)
    torch.cuda.synchronize(cuda_device)
    assert float(t[0][0]) != 0.5


def test_a_list_that_fails_validation_leaves_the_plans_table(cuda_device):
    """A plan that holds a table and is handed a list with a NULL pointer refuses the list and goes on stepping the
    table it has: validation comes before anything of the plan is touched."""
    import ctypes

    from fairscale_amd import _cabi

    L = _cabi.lib()
    t = [torch.full((5000,), x, device=cuda_device) for x in (0.5, 0.0, 0.0, 0.01)]
    rows = (_cabi.FsAdamTensor * 1)()
    rows[0].p, rows[0].m, rows[0].v, rows[0].g = (x.data_ptr() for x in t)
    rows[0].numel = 5000
    plan = ctypes.c_void_p()
    _cabi.check(L.fsadam_plan_create(_cabi.FULL_PRECISION, ctypes.byref(plan)))
    stream = int(torch.cuda.current_stream(cuda_device).cuda_stream)
    try:
        _cabi.check(L.fsadam_plan_set_tensors(plan, rows, 1, stream))
        bad = (_cabi.FsAdamTensor * 1)()
        bad[0].p, bad[0].m, bad[0].v, bad[0].g, bad[0].numel = t[0].data_ptr(), None, t[2].data_ptr(), t[3].data_ptr(), 5000
        assert L.fsadam_plan_set_tensors(plan, bad, 1, stream) == -1 and b"NULL" in L.fsadam_last_error()
        info = _cabi.FsAdamPlanInfo()
        _cabi.check(L.fsadam_plan_info(plan, ctypes.byref(info)))
        assert info.n_tensors == 1 and info.uploads == 1
        _cabi.check(L.fsadam_plan_step(plan, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, 0.0, 1, 1, 1, None, stream))
        torch.cuda.synchronize(cuda_device)
        assert float(t[0][0]) != 0.5 and float(t[1][0]) != 0.0
    finally:
        _cabi.check(L.fsadam_plan_destroy(plan))


def _window_check(oracle, mode, before, after, grads, windows, kw, what):
    """Re-run the oracle on [lo, hi) windows of the pre-step device state and compare with the
    post-step device state."""
    flag = np.zeros(1, np.float32)
    for lo, hi in windows:
        p, m, v = (before[k][lo:hi].cpu().numpy().copy() for k in ("p", "m", "v"))
        g = grads[lo:hi].cpu().numpy()
        pc = np.zeros(hi - lo, np.float16) if mode == MIXED else None
        oracle.step_c(mode, p, m, v, g, pc, found_inf=flag, **kw)
        for name, want in (("p", p), ("m", m), ("v", v)):
            got = after[name][lo:hi].cpu().numpy()
            bad = C.assert_close(got, want, f"{what} {name}[{lo}:{hi}]")
            assert bad == 0, f"{what} {name}[{lo}:{hi}]: {bad} values not bit-identical"
        if pc is not None:
            assert C.assert_close(after["p16"][lo:hi].cpu().numpy(), pc, f"{what} p16[{lo}:{hi}]") == 0
    return flag[0]


def _windows(n, count, width, seed):
    rng = np.random.default_rng(seed)
    w = [(0, 2 * width), (n - 2 * width, n)]
    for _ in range(count):
        lo = int(rng.integers(0, n - width))
        w.append((lo, lo + width))
    return w


def test_c4_flat_shard_1p63e9_memory_efficient(oracle, cuda_device):
    """The headline benchmark configuration at its real size: one contiguous 1.63e9-element buffer, fp16 params and grads
    (grads scaled by 1024), fp32 m/v.  Data is generated on the device; the oracle re-computes the
    first/last 2*65536 elements and 48 random 65536-element windows from the pre-step state.  Also a
    misaligned sub-view is stepped and checked the same way."""
    from fairscale_amd import fused_adam_hip

    n = 1_630_000_000
    dev = cuda_device
    gen = torch.Generator(device=dev).manual_seed(4000)
    p = (torch.randn(n, device=dev, generator=gen, dtype=torch.float32) * 0.02).half()
    g = (torch.randn(n, device=dev, generator=gen, dtype=torch.float32) * (1e-3 * 1024)).half()
    m = torch.zeros(n, device=dev)
    v = torch.zeros(n, device=dev)
    flag = torch.zeros(1, device=dev)
    windows = _windows(n, 48, 65536, 4001)
    for step in (1, 2):
        before = {"p": p.clone(), "m": m.clone(), "v": v.clone()}
        fused_adam_hip.adam(65536, None, [[p], [m], [v], [g]], 1e-3, 0.9, 0.999, 1e-8, 1024.0, 1.0, flag, step, 1, 1, 0.0)
        torch.cuda.synchronize()
        kw = dict(DEFAULT, step=step, grad_scale=1024.0)
        _window_check(oracle, MEMEFF, before, {"p": p, "m": m, "v": v}, g, windows, kw, f"C4 step {step}")
        del before
    assert flag.item() == 0.0
    # misaligned sub-view of the same buffers (element offset 3 for p and g, 1 for m, v aligned)
    lo, cnt = 1_000_003, 300_001
    sub = {"p": p[lo:lo + cnt], "m": m[lo - 2:lo - 2 + cnt], "v": v[lo + 1:lo + 1 + cnt]}
    gs = g[lo:lo + cnt]
    before = {k: t.clone() for k, t in sub.items()}
    fused_adam_hip.adam(65536, None, [[sub["p"]], [sub["m"]], [sub["v"]], [gs]], 1e-3, 0.9, 0.999, 1e-8, 1024.0, 1.0, flag, 3, 1, 1, 0.0)
    torch.cuda.synchronize()
    _window_check(oracle, MEMEFF, before, sub, gs, [(0, cnt)], dict(DEFAULT, step=3, grad_scale=1024.0), "C4 misaligned view")


def test_c4_size_properties_that_need_no_oracle(cuda_device):
    """The 1.63e9-element shard again, checked through what holds at any size: the same step on the same
    bits gives the same bits (two runs); gradients doubled together with the gradient scale change nothing
    (a power of two moves only the exponent); the buffer stepped as one tensor or as 1000 uneven views that
    start at odd elements (heads, shared and single descriptors, ragged ends at full scale) gives the same
    bits; and in MIXED_PRECISION the fp16 copy is exactly half(p32) everywhere."""
    from fairscale_amd import fused_adam_hip
    import random

    n = 1_630_000_000
    dev = cuda_device
    gen = torch.Generator(device=dev).manual_seed(4100)
    p0 = (torch.randn(n, device=dev, generator=gen, dtype=torch.float32) * 0.02).half()
    g = (torch.randn(n, device=dev, generator=gen, dtype=torch.float32) * (1e-3 * 1024)).half()
    m0 = torch.randn(n, device=dev, generator=gen, dtype=torch.float32) * 1e-3
    v0 = (torch.randn(n, device=dev, generator=gen, dtype=torch.float32) * 1e-3).square_()
    flag = torch.zeros(1, device=dev)

    def step(lists, scale):
        fused_adam_hip.adam(65536, None, lists, 1e-3, 0.9, 0.999, 1e-8, scale, 1.0, flag, 7, 1, 1, 0.01)

    ref = [p0.clone(), m0.clone(), v0.clone()]
    step([[ref[0]], [ref[1]], [ref[2]], [g]], 1024.0)
    # the same again
    again = [p0.clone(), m0.clone(), v0.clone()]
    step([[again[0]], [again[1]], [again[2]], [g]], 1024.0)
    assert all(torch.equal(a, b) for a, b in zip(ref, again)), "two runs differ"
    # doubled gradients, doubled scale (|g| stays far below the fp16 maximum)
    again = [p0.clone(), m0.clone(), v0.clone()]
    g2 = g * 2
    assert torch.isfinite(g2).all()
    step([[again[0]], [again[1]], [again[2]], [g2]], 2048.0)
    assert all(torch.equal(a, b) for a, b in zip(ref, again)), "power-of-two scale changed the result"
    del g2
    # 1000 uneven views, cut at drawn (mostly odd) elements
    rng = random.Random(4101)
    cuts = sorted({0, n} | {rng.randrange(1, n) for _ in range(999)})
    again = [p0.clone(), m0.clone(), v0.clone()]
    lists = [[t[a:b] for a, b in zip(cuts[:-1], cuts[1:])] for t in (again[0], again[1], again[2], g)]
    step(lists, 1024.0)
    assert all(torch.equal(a, b) for a, b in zip(ref, again)), "split into views changed the result"
    del again, lists, ref
    torch.cuda.empty_cache()
    # MIXED_PRECISION: fp32 master, fp16 copy out
    p32 = p0.float()
    p16 = torch.empty_like(p0)
    step([[p32], [m0], [v0], [g], [p16]], 1024.0)
    assert torch.equal(p16, p32.half())
    assert flag.item() == 0.0


def test_single_tensor_beyond_2_to_31_elements(oracle, cuda_device):
    """One fp16 tensor of 2^31 + 2^20 + 5 elements (PURE_FP16, 17 GB): element counts and offsets are 64-bit
    here (the reference keeps them in int, multi_tensor_apply.cuh:21,80).  Windows at the start, across
    the 2^31 boundary and at the ragged end are re-computed by the oracle."""
    from fairscale_amd import fused_adam_hip

    n = (1 << 31) + (1 << 20) + 5
    dev = cuda_device
    free, _ = torch.cuda.mem_get_info(dev)
    if free < n * 2 * 7:
        pytest.skip("not enough device memory")
    gen = torch.Generator(device=dev).manual_seed(7000)
    p = torch.empty(n, device=dev, dtype=torch.float16).normal_(0, 0.02, generator=gen)
    g = torch.empty(n, device=dev, dtype=torch.float16).normal_(0, 1e-3, generator=gen)
    m = torch.zeros(n, device=dev, dtype=torch.float16)
    v = torch.zeros(n, device=dev, dtype=torch.float16)
    flag = torch.zeros(1, device=dev)
    windows = [(0, 70000), ((1 << 31) - 40000, (1 << 31) + 40000), (n - 70000, n)] + _windows(n, 6, 65536, 7001)
    before = {"p": p.clone(), "m": m.clone(), "v": v.clone()}
    fused_adam_hip.adam(65536, None, [[p], [m], [v], [g]], 1e-3, 0.9, 0.999, 1e-8, 1.0, 65536.0, flag, 1, 1, 1, 0.01)
    torch.cuda.synchronize()
    kw = dict(DEFAULT, step=1, optim_scale=65536.0, decay=0.01)
    _window_check(oracle, PURE16, before, {"p": p, "m": m, "v": v}, g, windows, kw, "beyond 2^31")
    assert flag.item() == 0.0
    # nothing outside the tensor was touched and nothing inside was skipped: every m is non-zero where g is
    assert int((m[-(1 << 22):] != 0).sum().item()) == int((g[-(1 << 22):] != 0).sum().item())


def test_c5_llama7b_pure_fp16_with_overflow_injection(oracle, cuda_device):
    """The Llama-7B benchmark configuration at its real size: 291 tensors / 6.74e9 fp16 parameters, fp16 grads and state
    with optimizer-state scaling.  Step 1 is clean; in step 2 one gradient element in 10^6 is set to
    6e4, which must raise the flag.  Windows of several tensors are re-computed by the oracle."""
    from fairscale_amd import fused_adam_hip

    dev = cuda_device
    free, _total = torch.cuda.mem_get_info(dev)
    need = 6_738_415_616 * 8 + (8 << 30)
    if free < need:
        pytest.skip(f"needs {need >> 30} GiB of device memory, {free >> 30} GiB free")
    sizes = [C.numel(s) for s in C.llama7b_shapes()]
    assert len(sizes) == 291 and sum(sizes) == 6_738_415_616
    gen = torch.Generator(device=dev).manual_seed(5000)
    P = [torch.empty(n, device=dev, dtype=torch.float16).normal_(0, 0.02, generator=gen) for n in sizes]
    G = [torch.empty(n, device=dev, dtype=torch.float16).normal_(0, 1e-3, generator=gen) for n in sizes]
    M = [torch.zeros(n, device=dev, dtype=torch.float16) for n in sizes]
    V = [torch.zeros(n, device=dev, dtype=torch.float16) for n in sizes]
    flag = torch.zeros(1, device=dev)
    probe = [0, 1, 5, 8, 9, 145, 289, 290]  # embedding, attention, ffn, norm vectors, head

    def snapshot():
        return {t: {"p": P[t].clone(), "m": M[t].clone(), "v": V[t].clone()} for t in probe}

    scale = 65536.0
    for step in (1, 2):
        if step == 2:
            rng = np.random.default_rng(5002)
            for t in range(len(sizes)):  # 1 element in 10^6, seeded
                k = max(1, sizes[t] // 1_000_000) if sizes[t] >= 1_000_000 else 0
                if k:
                    idx = torch.from_numpy(rng.integers(0, sizes[t], size=k)).to(dev)
                    G[t][idx] = 6e4
        before = snapshot()
        flag.zero_()
        fused_adam_hip.adam(65536, None, [P, M, V, G], 1e-3, 0.9, 0.999, 1e-8, 1.0, scale, flag, step, 1, 1, 0.0)
        torch.cuda.synchronize()
        kw = dict(DEFAULT, step=step, optim_scale=scale)
        want_flag = 0.0
        for t in probe:
            n = sizes[t]
            wins = [(0, n)] if n <= 65536 else _windows(n, 4, 65536, 5100 + t)
            f = _window_check(oracle, PURE16, before[t], {"p": P[t], "m": M[t], "v": V[t]}, G[t], wins, kw, f"C5 step {step} tensor {t}")
            want_flag = max(want_flag, float(f))
        got_flag = flag.item()
        if step == 1:
            assert got_flag == 0.0 and want_flag == 0.0
        else:
            assert got_flag == 1.0  # some injected element overflowed v
            nonfinite = sum(int((~torch.isfinite(v)).sum().item()) for v in V)
            assert nonfinite > 0
        del before


def test_c5_llama7b_dynamic_scaling_through_the_optimizer(oracle, cuda_device):
    """The Llama-7B configuration at its real size through ``Adam(precision=PURE_FP16)``: a clean step, a step in which
    one gradient element in 10^6 is 6e4 (the stored second moment overflows: flag read back, optimizer-state scale halved,
    m and v of ALL 291 tensors zeroed, adam.py:278-288), then a clean step at the halved scale.  Windows of several
    tensors are re-computed by the oracle with the scale and the step count the optimizer used; the scale trajectory
    is exact; after the backoff there is no non-zero m or v anywhere."""
    from fairscale_amd.optim import Adam, Precision

    dev = cuda_device
    free, _total = torch.cuda.mem_get_info(dev)
    need = 6_738_415_616 * 8 + (8 << 30)
    if free < need:
        pytest.skip(f"needs {need >> 30} GiB of device memory, {free >> 30} GiB free")
    shapes = C.llama7b_shapes()
    sizes = [C.numel(s) for s in shapes]
    gen = torch.Generator(device=dev).manual_seed(5050)
    params = [torch.empty(sh, device=dev, dtype=torch.float16).normal_(0, 0.02, generator=gen).requires_grad_() for sh in shapes]
    clean = [torch.empty(sh, device=dev, dtype=torch.float16).normal_(0, 1e-3, generator=gen) for sh in shapes]
    opt = Adam(params, lr=1e-3, precision=Precision.PURE_FP16)
    assert opt._optim_scale == 65536.0
    probe = [0, 1, 5, 8, 9, 145, 289, 290]  # embedding, attention, ffn, norm vectors, head
    rng = np.random.default_rng(5052)
    want_scale = {1: 65536.0, 2: 65536.0, 3: 32768.0}  # the scale each step runs with
    for step in (1, 2, 3):
        for t, p in enumerate(params):
            p.grad = clean[t].clone() if step == 2 else clean[t]
            if step == 2 and sizes[t] >= 1_000_000:  # 1 element in 10^6, seeded
                idx = torch.from_numpy(rng.integers(0, sizes[t], size=sizes[t] // 1_000_000)).to(dev)
                p.grad.view(-1)[idx] = 6e4
        zero = torch.zeros(1, device=dev, dtype=torch.float16)
        before = {}
        for t in probe:
            st = opt.state[params[t]] if step > 1 else {}
            flat = params[t].detach().view(-1)
            before[t] = {"p": flat.clone(), "m": st["exp_avg"].view(-1).clone() if st else zero.expand(sizes[t]).clone(),
                         "v": st["exp_avg_sq"].view(-1).clone() if st else zero.expand(sizes[t]).clone()}
        scale = opt._optim_scale
        assert scale == want_scale[step]
        print(f"[c5 optimizer] step {step} at scale {scale}", flush=True)
        opt.step()
        torch.cuda.synchronize()
        kw = dict(DEFAULT, step=step, optim_scale=scale)
        for t in probe:
            n = sizes[t]
            wins = [(0, n)] if n <= 65536 else _windows(n, 3, 65536, 5200 + t)
            st = opt.state[params[t]]
            if step == 2:
                # m and v were zeroed after the kernel had stored them: only the parameters can be compared, and they
                # come from the unrounded fp32 moments, overflow or not (fused_adam_cuda_kernel.cu:106-112)
                flag = np.zeros(1, np.float32)
                for lo, hi in wins:
                    p, m, v = (before[t][k][lo:hi].cpu().numpy().copy() for k in ("p", "m", "v"))
                    oracle.step_c(PURE16, p, m, v, params[t].grad.view(-1)[lo:hi].cpu().numpy(), None, found_inf=flag, **kw)
                    assert C.assert_close(params[t].detach().view(-1)[lo:hi].cpu().numpy(), p, f"C5 optimizer step 2 tensor {t} p[{lo}:{hi}]") == 0
            else:
                after = {"p": params[t].detach().view(-1), "m": st["exp_avg"].view(-1), "v": st["exp_avg_sq"].view(-1)}
                f = _window_check(oracle, PURE16, before[t], after, params[t].grad.view(-1), wins, kw, f"C5 optimizer step {step} tensor {t}")
                assert f == 0.0
        if step == 2:
            assert opt._optim_scale == 32768.0 and opt._steps_since_optim_scale_change == 0
            for p in params:
                st = opt.state[p]
                assert not bool(st["exp_avg"].any()) and not bool(st["exp_avg_sq"].any()), "state not zeroed after the overflow"
                assert st["step"] == 2
        del before
    assert opt._optim_scale == 32768.0 and opt._steps_since_optim_scale_change == 1
    assert all(opt.state[p]["step"] == 3 for p in params)


@pytest.mark.parametrize("mode", [FULL, MIXED, MEMEFF, PURE16])
def test_zero_state_clears_m_and_v_and_nothing_else(cuda_device, mode):
    """``fsadam_plan_zero_state``: m = v = 0 for every tensor of the plan (sizes around every boundary, views that start
    between cache lines), the bytes around each state tensor, the parameters and the gradients untouched."""
    from fairscale_amd import fused_adam_hip

    sizes = [1, 7, 255, 256, 257, 4095, 4096, 4097, 8191, 16385, 70001, 131072, 131073, 300001, 0, 5]
    host = C.Tensors(mode, sizes, 5400 + mode)
    for arrs in (host.m, host.v):
        for a in arrs:
            a[...] = 3.0
    dev = GpuList(host, cuda_device, misalign={"m": 3, "v": 1, "p": 1})
    # sentinels around the state views: _place puts a view `k` elements into an allocation 8 elements longer than needed
    guards = []
    for lst, k in ((dev.m, 3), (dev.v, 1)):
        for t in lst:
            base = t._base if t._base is not None else t
            base[:k] = 7.0
            base[k + t.numel():] = 7.0
            guards.append((base, k, t.numel()))
    grads = to_gpu(host.grads(1), cuda_device)
    lists = [dev.p, dev.m, dev.v, grads] + ([dev.p16] if mode == MIXED else [])
    before_p = [t.clone() for t in dev.p]
    before_g = [t.clone() for t in grads]
    plan = fused_adam_hip.TensorListPlan(mode, cuda_device)
    with pytest.raises(Exception, match="no tensors"):
        plan.zero_state()
    plan.step(lists, 1e-3, 0.9, 0.999, 1e-8, 1.0, 65536.0 if mode == PURE16 else 1.0, dev.found_inf, 1, 1, 1, 0.0)
    after_p = [t.clone() for t in dev.p]
    assert any(bool(t.any()) for t in dev.m)
    plan.zero_state()
    torch.cuda.synchronize(cuda_device)
    for t in dev.m + dev.v:
        assert not bool(t.any())
    for base, k, n in guards:
        assert bool((base[:k] == 7.0).all()) and bool((base[k + n:] == 7.0).all()), "zero_state wrote outside a state tensor"
    for a, b in zip(after_p, dev.p):
        assert torch.equal(a, b)
    for a, b in zip(before_g, grads):
        assert torch.equal(a, b)
    assert not all(torch.equal(a, b) for a, b in zip(before_p, dev.p))  # the step itself had run
    plan.close()
