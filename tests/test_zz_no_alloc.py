"""``fsadam_grad_pass_noalloc`` (the gradient pass for callers that cannot allocate device memory) against
``fsadam_grad_pass``, both through the C ABI.

Bars: the gradients as stored, the overflow flag and the maximum are bit-identical; the sum of squares is
within 1e-6 relative (the variant always adds 16 tiles per partial, ``fsadam_grad_pass`` one, so the additions
group differently).  Every case runs twice in a row through the variant, the second time on a smaller list,
because the calls share one array per GPU that keeps the first call's table and partial results.  The variant
is also held to the CPU oracle directly (``test_against_the_oracle``)."""
from __future__ import annotations


import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def _rows(tensors):
    from fairscale_amd import _cabi

    rows = (_cabi.FsGradTensor * len(tensors))()
    for r, t in zip(rows, tensors):
        r.g, r.numel = t.data_ptr(), t.numel()
    return rows


def _call(entry, tensors, inv_scale, write_back, inv_on_device=False):
    from fairscale_amd import _cabi

    L = _cabi.lib()
    dev = tensors[0].device
    flag = torch.zeros(1, dtype=torch.float32, device=dev)
    ssq = torch.full((1,), -1.0, dtype=torch.float64, device=dev)
    amax = torch.full((1,), -1.0, dtype=torch.float32, device=dev)
    inv_dev = torch.tensor([inv_scale], dtype=torch.float32, device=dev) if inv_on_device else None
    code = _cabi.GRAD_F16 if tensors[0].dtype == torch.float16 else _cabi.GRAD_F32
    _cabi.check(getattr(L, entry)(_rows(tensors), len(tensors), code, 1.0 if inv_on_device else inv_scale,
                                  inv_dev.data_ptr() if inv_on_device else None, 1 if write_back else 0, flag.data_ptr(),
                                  ssq.data_ptr(), amax.data_ptr(), int(torch.cuda.current_stream(dev).cuda_stream)))
    torch.cuda.synchronize()
    return flag.item(), ssq.item(), amax.item()


def _make(sizes, dtype, seed, device, offset=0, plant=None):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    out = []
    for n in sizes:
        host = torch.randn(n + offset, generator=gen) * 0.05
        if plant is not None and n > 3:
            host[offset + n // 2] = plant
        out.append(host.to(dtype).to(device)[offset:])
    return out


def _bits(t):
    return t.cpu().numpy().view(np.uint16 if t.dtype == torch.float16 else np.uint32)


def _compare(sizes, dtype, inv_scale, write_back, device, seed, offset=0, plant=None, inv_on_device=False):
    a = _make(sizes, dtype, seed, device, offset, plant)
    # A pass that writes nothing runs on the same memory in both entry points.  One that writes back needs a copy of its own.
    writes = write_back and (inv_on_device or inv_scale != 1.0)
    b = a if not writes else [torch.cat([torch.zeros(offset, dtype=dtype, device=device), t])[offset:] for t in a]
    want = _call("fsadam_grad_pass", a, inv_scale, write_back, inv_on_device)
    got = _call("fsadam_grad_pass_noalloc", b, inv_scale, write_back, inv_on_device)
    what = f"sizes={sizes[:4]}.. dtype={dtype} inv={inv_scale} write_back={write_back} offset={offset}"
    for x, y in zip(a, b):
        assert np.array_equal(_bits(x), _bits(y)), what
    assert got[0] == want[0], what
    if np.isnan(want[2]):
        assert np.isnan(got[2]) and np.isnan(got[1]), what
    else:
        assert got[2] == want[2], what
        assert abs(got[1] - want[1]) <= 1e-6 * abs(want[1]) or got[1] == want[1], what


BIG = [3_000_001, 131072, 70001, 4096, 4097, 1, 0, 9, 2049, 650_000]
SMALL = [70001, 5, 2048]


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("write_back", [False, True])
def test_two_calls_in_a_row_the_second_smaller(cuda_device, dtype, write_back):
    for inv in (1.0, 1.0 / 64, 0.3):
        print(f"[noalloc] dtype={dtype} write_back={write_back} inv={inv}", flush=True)
        _compare(BIG, dtype, inv, write_back, cuda_device, seed=1)
        _compare(SMALL, dtype, inv, write_back, cuda_device, seed=2)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("write_back", [False, True])
def test_against_the_oracle(cuda_device, dtype, write_back):
    """The variant against the CPU restatement of the unscale op and the norms, not only against the other entry
    point: stored gradients and flag bit for bit, the maximum exact, the sum of squares to 1e-6 of the float64 sum.
    Twice in a row, the second list smaller, with special values planted in the first."""
    from oracle import grad_oracle as G

    rng = np.random.default_rng(11)
    for sizes, inv_scale, plant in (([700_001, 131072, 4097, 1, 0, 2049], 0.3, True), ([70001, 5], 2.0 ** -7, False)):
        host = [(rng.standard_normal(n) * 0.05).astype(dtype) for n in sizes]
        if plant:
            info = np.finfo(dtype)
            for value, at in ((6.0e4, 17), (-6.0e4, 4000), (info.smallest_subnormal, 12345), (-0.0, 3)):
                host[0][at] = value
        dev = [torch.from_numpy(h.copy()).to(cuda_device) for h in host]
        print(f"[noalloc] oracle {np.dtype(dtype)} write_back={write_back} sizes={sizes[:3]}..", flush=True)
        got = _call("fsadam_grad_pass_noalloc", dev, inv_scale, write_back)
        want = G.grad_pass_numpy(host, inv_scale, write_back)  # rewrites `host` when write_back
        assert got[0] == want[0] == 0.0
        assert got[2] == want[2]
        assert np.isfinite(want[1]) and abs(got[1] - want[1]) <= 1e-6 * abs(want[1])
        for d, h in zip(dev, host):
            assert np.array_equal(_bits(d), h.view(np.uint16 if dtype == np.float16 else np.uint32))
    # an overflowing gradient raises the flag and is stored as the oracle stores it
    host = [(rng.standard_normal(9000) * 0.05).astype(dtype)]
    host[0][77] = np.inf
    dev = [torch.from_numpy(host[0].copy()).to(cuda_device)]
    got = _call("fsadam_grad_pass_noalloc", dev, 0.5, write_back)
    want = G.grad_pass_numpy(host, 0.5, write_back)
    assert got[0] == want[0] == 1.0 and got[2] == want[2] == np.inf and got[1] == want[1] == np.inf
    assert np.array_equal(_bits(dev[0]), host[0].view(np.uint16 if dtype == np.float16 else np.uint32))


def test_views_between_cache_lines_and_a_scale_on_the_device(cuda_device):
    print("[noalloc] misaligned views", flush=True)
    _compare([300_001, 9000, 17], torch.float16, 0.25, True, cuda_device, seed=3, offset=3, inv_on_device=True)
    _compare([9000], torch.float32, 0.3, False, cuda_device, seed=4, offset=1, inv_on_device=True)


def test_non_finite_gradients_raise_the_flag(cuda_device):
    print("[noalloc] non-finite", flush=True)
    _compare([200_000, 77], torch.float16, 0.5, True, cuda_device, seed=5, plant=float("inf"))
    _compare([5000], torch.float32, 1.0, False, cuda_device, seed=6, plant=float("nan"))


def test_a_shard_sized_buffer_then_a_small_one(cuda_device):
    print("[noalloc] shard", flush=True)
    _compare([400_000_000], torch.float16, 1.0 / 1024, False, cuda_device, seed=7)
    _compare([1000], torch.float16, 1.0 / 1024, False, cuda_device, seed=8)


def test_calls_that_overlap_report_nan_or_the_right_numbers(cuda_device):
    """Calls on two streams without an order between them share the GPU's one array; the library cannot prevent that,
    but each call finds out at its end whether it owned the array from beginning to end, and reports NaN in all three
    outputs if it did not.  Here both streams pass the SAME list (so whatever mixture of the two tables a kernel reads
    stays inside the tensors) and nothing is written back; every result must be either all NaN or exactly the result of
    the call made alone, and a call made alone afterwards must be right again (the array was given back)."""
    from fairscale_amd import _cabi

    L = _cabi.lib()
    gen = torch.Generator(device="cpu").manual_seed(21)
    grads = [(torch.randn(n, generator=gen) * 0.05).half().to(cuda_device) for n in (3_000_001, 70_001, 9)]
    grads.append(torch.zeros(60_000_000, dtype=torch.float16, device=cuda_device).normal_(0, 0.05))
    rows = _rows(grads)
    alone = _call("fsadam_grad_pass_noalloc", grads, 0.25, False)
    assert not np.isnan(alone[1]) and alone[0] == 0.0
    streams = [torch.cuda.Stream(cuda_device), torch.cuda.Stream(cuda_device)]
    outs = [[torch.zeros(1, device=cuda_device), torch.zeros(1, device=cuda_device, dtype=torch.float64), torch.zeros(1, device=cuda_device)]
            for _ in streams]
    spoiled = 0
    for rnd in range(8):
        print(f"[noalloc] overlap round {rnd}", flush=True)
        torch.cuda.synchronize(cuda_device)
        for flag, _, _ in outs:
            flag.zero_()
        torch.cuda.synchronize(cuda_device)
        for k in ((0, 1) if rnd % 2 == 0 else (1, 0)):
            flag, ssq, amax = outs[k]
            _cabi.check(L.fsadam_grad_pass_noalloc(rows, len(grads), _cabi.GRAD_F16, 0.25, None, 0, flag.data_ptr(), ssq.data_ptr(),
                                                   amax.data_ptr(), streams[k].cuda_stream))
        torch.cuda.synchronize(cuda_device)
        for flag, ssq, amax in outs:
            got = (flag.item(), ssq.item(), amax.item())
            if all(np.isnan(x) for x in got):
                spoiled += 1
            else:
                assert got == alone, f"round {rnd}: a call that overlapped another reported {got}, alone it reports {alone}"
    print(f"[noalloc] {spoiled} of 16 overlapping calls reported NaN", flush=True)
    again = _call("fsadam_grad_pass_noalloc", grads, 0.25, False)
    if any(np.isnan(x) for x in again):  # at most the first call behind a spoiled pair may still find the array taken
        again = _call("fsadam_grad_pass_noalloc", grads, 0.25, False)
    assert again == alone


def test_lists_beyond_the_scratch_are_refused(cuda_device):
    from fairscale_amd import _cabi

    L = _cabi.lib()
    # more descriptors than the array holds: 5000 small tensors (one descriptor each), no kernel is launched
    many = [torch.zeros(8, dtype=torch.float16, device=cuda_device) for _ in range(5000)]
    rc = L.fsadam_grad_pass_noalloc(_rows(many), len(many), _cabi.GRAD_F16, 1.0, None, 0, None, None, None, None)
    assert rc == -1 and b"descriptors" in L.fsadam_last_error()
    # more workgroups than there are partials: sizes only, the pointer is never followed
    rows = (_cabi.FsGradTensor * 1)()
    rows[0].g, rows[0].numel = many[0].data_ptr(), 3 * 10 ** 9
    rc = L.fsadam_grad_pass_noalloc(rows, 1, _cabi.GRAD_F32, 0.5, None, 1, None, None, None, None)
    assert rc == -1 and b"workgroups" in L.fsadam_last_error()
    torch.cuda.synchronize()


def test_recorded_into_a_graph_and_replayed(cuda_device):
    """What the entry point is for: between the begin and the end of a capture nothing may allocate.  One call outside
    any capture first (it looks the array's address up), then the call is recorded and replayed four times on fresh
    gradients, with eager work and synchronisations in between; every replay against ``fsadam_grad_pass`` run eagerly
    on copies."""
    from fairscale_amd import _cabi

    L = _cabi.lib()
    sizes = [300_001, 70_000, 5, 4096]
    gen = torch.Generator(device="cpu").manual_seed(9)
    grads = [torch.randn(n, generator=gen).half().to(cuda_device) for n in sizes]
    rows = _rows(grads)
    flag = torch.zeros(1, device=cuda_device)
    ssq = torch.zeros(1, device=cuda_device, dtype=torch.float64)
    amax = torch.zeros(1, device=cuda_device)

    def call(stream):
        _cabi.check(L.fsadam_grad_pass_noalloc(rows, len(grads), _cabi.GRAD_F16, 0.5, None, 1, flag.data_ptr(), ssq.data_ptr(), amax.data_ptr(), stream))

    side = torch.cuda.Stream(cuda_device)
    with torch.cuda.stream(side):
        call(side.cuda_stream)
    torch.cuda.synchronize(cuda_device)
    graph = torch.cuda.CUDAGraph()
    print("[noalloc] capture", flush=True)
    with torch.cuda.graph(graph, stream=side):
        call(torch.cuda.current_stream(cuda_device).cuda_stream)
    torch.cuda.synchronize(cuda_device)
    for rep in range(4):
        fresh = [torch.randn(n, generator=gen).half().to(cuda_device) for n in sizes]
        if rep == 2:
            fresh[1][123] = float("inf")
        for t, f in zip(grads, fresh):
            t.copy_(f)
        flag.zero_()
        torch.cuda.synchronize(cuda_device)
        print(f"[noalloc] replay {rep}", flush=True)
        graph.replay()
        torch.cuda.synchronize(cuda_device)
        want = _call("fsadam_grad_pass", fresh, 0.5, True)
        assert flag.item() == want[0] == (1.0 if rep == 2 else 0.0)
        assert amax.item() == want[2]
        assert abs(ssq.item() - want[1]) <= 1e-6 * abs(want[1]) or ssq.item() == want[1]
        for t, f in zip(grads, fresh):
            assert np.array_equal(_bits(t), _bits(f)), f"replay {rep}"
