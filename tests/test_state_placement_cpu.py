"""Host logic that lays optimizer state out like the parameters (``fairscale_amd/optim/adam.py``), on CPU tensors: which
parameters form a run, where a stream that accompanies a run has to start, and when existing state counts as in place.
The reference allocates ``zeros_like`` per parameter (``fairscale/optim/adam.py:226-228``); parameters that are
back-to-back views of one buffer are what OSS makes of a rank's shard (``fairscale/optim/oss.py:630-659``)."""
from __future__ import annotations

import torch

from fairscale_amd.optim import adam as A


def _views(flat, sizes, lead=0):
    out, at = [], lead
    for n in sizes:
        out.append(flat[at:at + n])
        at += n
    return out


def test_adjacent_runs_follow_the_memory_not_the_list():
    flat = torch.zeros(100_000)
    a, b, c, d = _views(flat, [10, 7, 5000, 3], lead=1)
    other = torch.zeros(7)
    assert A._adjacent_runs([a, b, c, d]) == [[0, 1, 2, 3]]
    assert A._adjacent_runs([a, other, c, d]) == [[0], [1], [2, 3]]            # a stranger in the middle
    assert A._adjacent_runs([a, c, d]) == [[0], [1, 2]]                         # b left out (a frozen parameter): a gap
    assert A._adjacent_runs([b, a]) == [[0], [1]]                               # the wrong way round
    assert A._adjacent_runs([a, b.double(), c]) == [[0], [1], [2]]              # another dtype in between breaks the run
    two_d = flat[6000:6000 + 12].view(3, 4)
    tail = flat[6012:6020]
    assert A._adjacent_runs([two_d, tail]) == [[0, 1]]                          # shapes do not matter, bytes do
    assert A._adjacent_runs([two_d.t(), tail]) == [[0], [1]]                    # a non-contiguous tensor is a run of its own
    assert A._adjacent_runs([]) == []
    empty = flat[10:10]
    assert A._adjacent_runs([flat[1:10], empty, flat[10:20]]) == [[0, 1, 2]]    # an empty view continues the run


def test_a_stream_for_a_run_starts_at_the_runs_phase():
    flat = torch.zeros(200_000)  # float32: 512 elements = 2 KiB
    base = flat.data_ptr() // 4
    for lead in (0, 1, 3, 31, 100, 128, 256, 511, 513):  # 128 and 256 elements in: on a cache line, off the 1 KiB boundary
        first = flat[lead:lead + 50_000]
        for dtype in (torch.float32, torch.float16):
            buf = A._buffer_placed_like(first, 50_000, dtype, zero=True)
            assert buf.numel() == 50_000 and buf.dtype == dtype and buf.is_contiguous() and not bool(buf.any())
            # same element offset modulo 512: one head length puts both on 1 KiB boundaries
            assert A._phase(buf) == (base + lead) % 512 == A._phase(first)
            buf = A._buffer_placed_like(first, 50_000, dtype, zero=False)
            assert buf.numel() == 50_000 and A._phase(buf) == A._phase(first)
    # short runs get a plain allocation, whatever their phase
    short = flat[1:1 + 100]
    assert A._buffer_placed_like(short, 100, torch.float32, zero=True).numel() == 100
    assert not A._needs_placing(100) and not A._needs_placing(8191) and A._needs_placing(8192)


def test_a_run_on_a_boundary_gets_state_on_a_boundary():
    """The allocator hands out 512-byte granules: state for a run that starts ON a 1 KiB boundary must not be left half a
    kilobyte off it."""
    flat = torch.zeros(100_000 + 1024)
    lead = (-(flat.data_ptr() // 4)) % 512  # first element on a 2 KiB boundary
    first = flat[lead:lead + 60_000]
    assert A._phase(first) == 0
    for _ in range(4):  # whatever the allocator returns
        keep = torch.zeros(137)  # shift the allocator's next answer
        for dtype in (torch.float32, torch.float16):
            buf = A._buffer_placed_like(first, 60_000, dtype, zero=True)
            assert A._phase(buf) == 0 and buf.data_ptr() % 1024 == 0
        del keep


def test_state_counts_as_placed_only_when_it_follows_the_parameters():
    params = torch.zeros(60_000)
    state = torch.zeros(60_000 + 512)
    sizes = [9000, 20, 30_000]
    lead = 3
    likes = _views(params, sizes, lead=lead)
    want = (likes[0].data_ptr() // 4) % 512
    start = (want - (state.data_ptr() // 4) % 512) % 512
    good = _views(state, sizes, lead=start)
    assert A._placed(good, likes)
    assert not A._placed(_views(state, sizes, lead=(start + 1) % 512), likes)            # packed, at another offset
    assert not A._placed([torch.zeros(n) for n in sizes], likes)                          # one allocation each
    assert not A._placed([good[0], good[1], torch.zeros(sizes[2])], likes)               # the last one elsewhere
    assert not A._placed([good[0], good[1], good[2][:-1]], likes)                         # a size that does not fit
    # a short run: packed is enough
    small_likes = _views(params, [10, 20], lead=1)
    assert A._placed(_views(state, [10, 20], lead=7), small_likes)


def test_empty_parameters_inside_a_run_do_not_unsettle_it():
    params = torch.zeros(1000)
    state = torch.zeros(1000)
    likes = [params[0:100], params[100:100], params[100:300]]
    assert A._adjacent_runs(likes) == [[0, 1, 2]]
    placed = [state[0:100], state[100:100], state[100:300]]
    assert A._placed(placed, likes)
    assert A._placed([state[0:100], torch.zeros(0), state[100:300]], likes)     # wherever the empty one "lies"
    assert not A._placed([state[0:100], state[100:100], state[101:301]], likes)
