"""CPU-only checks of the C ABI and the host logic around it: the library loads, exports what
include/fsadam.h declares, rounds the step size like the oracle, plans tensor lists as documented and
rejects bad arguments with error codes -- no kernel is launched and no device is touched."""
from __future__ import annotations

import ctypes
import os
import re

import numpy as np
import pytest
import torch

from fairscale_amd import _cabi, fused_adam_hip

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(REPO, "include", "fsadam.h")).read()


def declared_functions():
    code = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(fsadam_[a-z_0-9]+)\s*\(", code)))


def header_define(name):
    m = re.search(r"#define\s+%s\s+\(?(-?\d+)\)?" % name, HEADER)
    assert m, name
    return int(m.group(1))


def rows(*tensors):
    """FsAdamTensor array from (p, m, v, g, p_copy, numel) tuples of plain integers."""
    arr = (_cabi.FsAdamTensor * len(tensors))()
    for r, t in zip(arr, tensors):
        r.p, r.m, r.v, r.g, r.p_copy, r.numel = t
    return arr


def last_error():
    return _cabi.lib().fsadam_last_error().decode()


def test_library_exports_every_declared_symbol():
    L = _cabi.lib()
    names = declared_functions()
    assert len(names) >= 14
    for name in names:
        assert hasattr(L, name), f"{name} is declared in include/fsadam.h but not exported by libfsadam.so"
    assert sorted(_cabi.SIGNATURES) == names, "the ctypes binding and the header disagree on the function list"


def test_abi_version_and_constants():
    assert _cabi.lib().fsadam_version() == header_define("FSADAM_ABI_VERSION") == _cabi.ABI_VERSION
    from oracle import adam_oracle as O

    for name, a, b in [("FSADAM_FULL_PRECISION", _cabi.FULL_PRECISION, O.FULL_PRECISION),
                       ("FSADAM_MIXED_PRECISION", _cabi.MIXED_PRECISION, O.MIXED_PRECISION),
                       ("FSADAM_MEMORY_EFFICIENT_MIXED_PRECISION", _cabi.MEMORY_EFFICIENT_MIXED_PRECISION, O.MEMORY_EFFICIENT_MIXED_PRECISION),
                       ("FSADAM_PURE_FP16", _cabi.PURE_FP16, O.PURE_FP16),
                       ("FSADAM_FULL_PRECISION_FP16_COPY", _cabi.FULL_PRECISION_FP16_COPY, O.FULL_PRECISION_FP16_COPY)]:
        assert header_define(name) == a == b
    assert header_define("FSADAM_EPS_INSIDE_SQRT") == 0 and header_define("FSADAM_EPS_OUTSIDE_SQRT") == 1
    assert ctypes.sizeof(_cabi.FsAdamTensor) == 48  # five pointers and an int64, no padding


def test_step_size_is_bit_identical_to_the_oracle(oracle):
    for lr in (1e-3, 3e-4, 0.1, 1.0):
        for b1, b2 in ((0.9, 0.999), (0.95, 0.98), (0.0, 0.5), (0.5, 0.9)):
            for step in (1, 2, 3, 7, 100, 2000, 123456):
                for bc in (0, 1):
                    got = np.float32(_cabi.step_size(lr, b1, b2, step, bc))
                    want = oracle.step_size_c(lr, b1, b2, step, bc)
                    assert got.view(np.uint32) == np.float32(want).view(np.uint32), (lr, b1, b2, step, bc)


def test_options_roundtrip_and_validation():
    names = ("lds_throttle", "grad_waves", "grad_items", "grad_lds_throttle", "align_heads", "merge_runs", "mid_tiles", "upload_stream")
    old = {k: _cabi.get_option(k) for k in names}
    assert old == {"lds_throttle": -1, "grad_waves": 0, "grad_items": 0, "grad_lds_throttle": -1, "align_heads": 1, "merge_runs": 1,
                   "mid_tiles": 16, "upload_stream": 1}
    try:
        _cabi.set_option("lds_throttle", 20480)
        assert _cabi.get_option("lds_throttle") == 20480
        for flag in ("align_heads", "merge_runs", "upload_stream"):
            for value in (0, 1):
                _cabi.set_option(flag, value)
                assert _cabi.get_option(flag) == value
        for name, bad in (("lds_throttle", 1 << 20), ("grad_waves", 3), ("grad_items", 5), ("align_heads", 2), ("merge_runs", -1), ("mid_tiles", 3),
                          ("mid_tiles", 128), ("upload_stream", 2), ("no_such_option", 1),
                          # shapes and orders that were measured and dropped are not options any more
                          ("block", 64), ("groups", 1), ("xcd_remap", 0), ("max_large_chunk", 65536), ("unaligned_vectors", 1), ("lazy_events", 1)):
            with pytest.raises(_cabi.FsAdamError):
                _cabi.set_option(name, bad)
    finally:
        for k, v in old.items():
            _cabi.set_option(k, v)


def layout(tensors, mode):
    arr = rows(*tensors)
    out = _cabi.FsAdamLayout()
    cls = (ctypes.c_uint8 * len(tensors))()
    vec = (ctypes.c_uint8 * len(tensors))()
    _cabi.check(_cabi.lib().fsadam_layout(arr, len(tensors), mode, ctypes.byref(out), cls, vec))
    return out.as_dict(), list(cls), list(vec)


def test_layout_classes_and_descriptor_counts():
    A = 0x7000_0000_0000  # fake, 2 MiB-aligned device addresses: never dereferenced on the host
    t = lambda n, off=0: (A + off, A + (1 << 32), A + (2 << 32), A + (3 << 32) + off, 0, n)  # noqa: E731
    old = {k: _cabi.get_option(k) for k in ("mid_tiles",)}
    try:
        _cabi.set_option("mid_tiles", 0)  # two classes: shared descriptors from 131072 elements, one per tile below
        lay, cls, vec = layout([t(0), t(1), t(255), t(256), t(257), t(131071), t(131072), t(131073), t(1 << 20)], _cabi.FULL_PRECISION)
        assert lay["tile_elems"] == 256  # 64 lanes x 4 fp32
        assert cls == [0, 1, 1, 1, 1, 1, 2, 2, 2]
        assert lay["n_empty_tensors"] == 1 and lay["n_small_tensors"] == 5 and lay["n_large_tensors"] == 3
        # smallest large tensor has 131072 elements: chunk = 65536 (two chunks each at least)
        assert lay["large_chunk_elems"] == 65536
        assert lay["n_small_descriptors"] == 1 + 1 + 1 + 2 + 512
        assert lay["n_large_descriptors"] == 2 + 3 + 16
        assert lay["grid_large"] == lay["n_large_descriptors"] * (65536 // 256)
        assert lay["grid_small"] == lay["n_small_descriptors"]
        assert (lay["mid_chunk_elems"], lay["n_mid_tensors"], lay["n_mid_descriptors"], lay["grid_mid"]) == (0, 0, 0, 0)
        assert vec == [0, 1, 1, 1, 1, 1, 1, 1, 1]
        # three classes (the default): 16 tiles = 4096 elements share a descriptor from 4096 elements on
        _cabi.set_option("mid_tiles", 16)
        lay, cls, _ = layout([t(0), t(1), t(4095), t(4096), t(4097), t(131071), t(131072)], _cabi.FULL_PRECISION)
        assert cls == [0, 1, 1, 3, 3, 3, 2] and lay["mid_chunk_elems"] == 4096
        assert (lay["n_small_tensors"], lay["n_mid_tensors"], lay["n_large_tensors"]) == (2, 3, 1)
        assert lay["n_small_descriptors"] == 1 + 16 and lay["n_mid_descriptors"] == 1 + 2 + 32 and lay["n_large_descriptors"] == 2
        assert lay["grid_mid"] == 35 * 16 and lay["grid_small"] == 17 and lay["grid_large"] == 2 * 256
        _cabi.set_option("mid_tiles", 64)  # 16384 elements
        lay, cls, _ = layout([t(16383), t(16384), t(100000)], _cabi.FULL_PRECISION)
        assert cls == [1, 3, 3] and lay["mid_chunk_elems"] == 16384 and lay["n_mid_descriptors"] == 1 + 7 and lay["grid_mid"] == 8 * 64
        _cabi.set_option("mid_tiles", 0)
        # one 1.63e9-element tensor: chunk capped at 2^24, 98 descriptors
        lay, cls, _ = layout([t(1_630_000_000)], _cabi.MEMORY_EFFICIENT_MIXED_PRECISION)
        assert lay["large_chunk_elems"] == 1 << 24 and lay["n_large_descriptors"] == 98 and cls == [2]
        # PURE_FP16 moves 8 halves per lane
        lay, _, _ = layout([t(5000)], _cabi.PURE_FP16)
        assert lay["tile_elems"] == 512 and lay["n_small_descriptors"] == 10
    finally:
        for k, v in old.items():
            _cabi.set_option(k, v)


@pytest.fixture
def two_classes():
    """No middle class for one test: every tile of a tensor under 131072 elements has its own descriptor."""
    old = _cabi.get_option("mid_tiles")
    _cabi.set_option("mid_tiles", 0)
    yield
    _cabi.set_option("mid_tiles", old)


def head_of(t, mode):
    out = ctypes.c_int64(-1)
    _cabi.check(_cabi.lib().fsadam_head_elems(rows(t), mode, ctypes.byref(out)))
    return out.value


def test_heads_bring_the_tiles_onto_line_boundaries():
    """The first elements of a tensor whose streams start off a cache line go to a descriptor of their own
    (fake addresses, host-side planning only)."""
    A = 0x7000_0000_0000
    same = lambda off, n, mode: tuple(A + (k << 34) + off * (2 if half else 4) for k, half in enumerate(_halves(mode))) + (0, n)  # noqa: E731
    F, MX, ME, P16 = _cabi.FULL_PRECISION, _cabi.MIXED_PRECISION, _cabi.MEMORY_EFFICIENT_MIXED_PRECISION, _cabi.PURE_FP16
    # aligned streams, short tensors: nothing to do
    assert head_of(same(0, 1 << 20, F), F) == 0
    assert head_of(same(256, 1 << 20, F), F) == 0  # fp32 streams 1 KiB in: aligned as well
    assert head_of(same(3, 8191, F), F) == 0
    # fp32 streams all 3 elements (12 bytes) past a 1 KiB boundary: 253 elements reach the next one
    assert head_of(same(3, 8192, F), F) == 253
    assert head_of(same(255, 8192, F), F) == 1
    # fp16 p and g at 2 bytes an element, fp32 state at 4: a head that is a multiple of 512 elements away suits both
    assert head_of(same(5, 100000, ME), ME) == 507
    assert head_of(same(300, 100000, ME), ME) == 212
    assert head_of(same(7, 100000, P16), P16) == 505
    # MIXED_PRECISION: fp32 p, m, v, fp16 g and fp16 copy
    t = same(9, 100000, MX)
    t = t[:4] + (A + (5 << 34) + 9 * 2, t[5])
    assert head_of(t, MX) == 503
    # state allocated on its own (aligned), parameters and gradients 4 elements into a flat buffer: moving
    # the tiles would take m and v off their lines, which costs more than it gains
    assert head_of((A + 16, A + (1 << 34), A + (2 << 34), A + (3 << 34) + 16, 0, 100000), F) == 0
    # the same with fp16 parameters and gradients (8 bytes in): the fp32 state carries more bytes per element
    assert head_of((A + 8, A + (1 << 34), A + (2 << 34), A + (3 << 34) + 8, 0, 100000), ME) == 0
    # only the gradient off its line: it follows the others
    assert head_of((A, A + (1 << 34), A + (2 << 34), A + (3 << 34) + 16, 0, 100000), F) == 0
    # the other way round, p, m, v 64 bytes in and the gradient aligned: the three heavier streams win
    assert head_of((A + 64, A + (1 << 34) + 64, A + (2 << 34) + 64, A + (3 << 34), 0, 100000), F) == 240
    old = _cabi.get_option("align_heads")
    try:
        _cabi.set_option("align_heads", 0)
        assert head_of(same(3, 8192, F), F) == 0
    finally:
        _cabi.set_option("align_heads", old)


def _halves(mode):
    """which of p, m, v, g are fp16 in a mode"""
    return {_cabi.FULL_PRECISION: (0, 0, 0, 0), _cabi.MIXED_PRECISION: (0, 0, 0, 1), _cabi.MEMORY_EFFICIENT_MIXED_PRECISION: (1, 0, 0, 1),
            _cabi.PURE_FP16: (1, 1, 1, 1)}[mode]


def test_no_other_head_would_align_better():
    """The head is chosen among a handful of candidates (the counts that bring one stream onto a line or a
    1 KiB boundary).  An exhaustive search over every count below 1024 with the same weights (bytes a
    stream moves per element x 0 / 1 / 5 / 6 for 1 KiB-, line-, 16-byte- or element-aligned) must not find
    a cheaper one, nor an equally cheap shorter one."""
    rng = np.random.default_rng(77)
    A = 0x7000_0000_0000
    for case in range(300):
        mode = [_cabi.FULL_PRECISION, _cabi.MIXED_PRECISION, _cabi.MEMORY_EFFICIENT_MIXED_PRECISION, _cabi.PURE_FP16][case % 4]
        sizes = [2 if h else 4 for h in _halves(mode)]
        streams = [(A + (k << 34) + int(rng.integers(0, 512)) * sz * int(rng.choice([1, 1, 4, 32])), sz, (1 if k == 3 else 2) * sz)
                   for k, sz in enumerate(sizes)]
        copy = A + (5 << 34) + int(rng.integers(0, 512)) * 2 if mode == _cabi.MIXED_PRECISION else 0
        if copy:
            streams.append((copy, 2, 2))

        def cost(head):
            total = 0
            for addr, sz, moved in streams:
                a = addr + head * sz
                total += moved * (0 if a % 1024 == 0 else 1 if a % 128 == 0 else 5 if a % 16 == 0 else 6)
            return total

        got = head_of((streams[0][0], streams[1][0], streams[2][0], streams[3][0], copy, 50000), mode)
        best = min(range(1024), key=lambda h: (cost(h), h))
        assert (cost(got), got) == (cost(best), best), (case, mode, [hex(s[0]) for s in streams], got, best)


def test_rows_that_continue_each_other_are_laid_out_as_one_run():
    """Back-to-back views of flat buffers (every stream of row t+1 starts where row t's ended) become one run; a
    stream that breaks the sequence, in any of the lists, starts a new one (fake addresses, host-side planning)."""
    A = 0x7000_0000_0000
    sizes = [1000, 3, 70000, 0, 5000, 140000, 9]

    def packed(mode, breaks=(), sizes=sizes):
        """Rows packed into four (five) flat buffers; `breaks`: (row, stream) pairs where that stream skips 64 bytes."""
        ps, ss, gs = (2 if mode in (_cabi.MEMORY_EFFICIENT_MIXED_PRECISION, _cabi.PURE_FP16) else 4,
                      2 if mode == _cabi.PURE_FP16 else 4, 4 if mode == _cabi.FULL_PRECISION else 2)
        at = [A, A + (1 << 36), A + (2 << 36), A + (3 << 36), A + (4 << 36)]
        width = [ps, ss, ss, gs, 2]
        out = []
        for t, n in enumerate(sizes):
            for k in range(5):
                if (t, k) in breaks:
                    at[k] += 64
            out.append((at[0], at[1], at[2], at[3], at[4] if mode == _cabi.MIXED_PRECISION else 0, n))
            for k in range(5):
                at[k] += n * width[k]
        return out

    total = sum(sizes)
    for mode in (_cabi.FULL_PRECISION, _cabi.MIXED_PRECISION, _cabi.MEMORY_EFFICIENT_MIXED_PRECISION, _cabi.PURE_FP16):
        tile = 512 if mode == _cabi.PURE_FP16 else 256
        lay, cls, vec = layout(packed(mode), mode)
        assert lay["n_runs"] == 1 and lay["n_empty_tensors"] == 1, mode
        assert cls == [2, 2, 2, 0, 2, 2, 2] and vec == [1, 1, 1, 0, 1, 1, 1]
        assert lay["n_large_tensors"] == 1 and lay["n_small_tensors"] == 0 and lay["n_mid_tensors"] == 0
        assert lay["n_large_descriptors"] == -(-total // lay["large_chunk_elems"]) and lay["n_small_descriptors"] == 0
        assert lay["grid_large"] * tile >= total
        # the same rows one by one
        old = _cabi.get_option("merge_runs")
        try:
            _cabi.set_option("merge_runs", 0)
            lay0, cls0, _ = layout(packed(mode), mode)
        finally:
            _cabi.set_option("merge_runs", old)
        assert lay0["n_runs"] == 6 and cls0[3] == 0 and cls0[1] == 1 and cls0[5] == 2
        # a break in one stream only: p (0), v (2), g (3), and in MIXED the fp16 copy (4)
        for stream in (0, 2, 3) + ((4,) if mode == _cabi.MIXED_PRECISION else ()):
            lay, cls, _ = layout(packed(mode, breaks={(4, stream)}), mode)
            assert lay["n_runs"] == 2, (mode, stream)
            assert cls[:3] == [3, 3, 3] and cls[4:] == [2, 2, 2]  # 71003 elements in front, 145009 behind
        # a break at every row: nothing to merge
        lay, _, _ = layout(packed(mode, breaks={(t, 1) for t in range(1, 7)}), mode)
        assert lay["n_runs"] == 6
    # the copy stream of the 4-list modes is not looked at
    rows4 = packed(_cabi.FULL_PRECISION)
    rows4 = [r[:4] + (0x1234560 + 8 * i,) + r[5:] for i, r in enumerate(rows4)]
    assert layout(rows4, _cabi.FULL_PRECISION)[0]["n_runs"] == 1


def test_shared_chunks_shrink_until_they_divide_the_tensors_well():
    """The chunk a shared descriptor covers starts at half the smallest large tensor and is halved while the tiles behind
    the tensors' ends (workgroups that are launched and find nothing to do) exceed 1 % of the elements."""
    import _cases as C

    A = 0x7000_0000_0000
    row = lambda n: (A, A + (1 << 40), A + (2 << 40), A + (3 << 40), A + (4 << 40), n)  # noqa: E731
    old = _cabi.get_option("merge_runs")
    _cabi.set_option("merge_runs", 0)  # every row has the same fake address: keep them apart
    try:
        # Llama-7B: 2^23 would leave the last chunk of every 4096 x 11008 matrix 5/8 empty; 2^20 divides every matrix
        sizes = [C.numel(sh) for sh in C.llama7b_shapes()]
        lay, _, _ = layout([row(n) for n in sizes], _cabi.PURE_FP16)
        assert lay["large_chunk_elems"] == 1 << 20
        large = [n for n in sizes if n >= 131072]
        assert lay["grid_large"] * lay["tile_elems"] == sum(large)  # not one tile behind an end
        # GPT-2 small: every matrix is a multiple of 65536 elements except the embedding
        sizes = [C.numel(sh) for sh in C.gpt2_small_shapes()]
        lay, _, _ = layout([row(n) for n in sizes], _cabi.MIXED_PRECISION)
        large = [n for n in sizes if n >= 131072]
        assert lay["large_chunk_elems"] == 65536 and lay["grid_large"] * lay["tile_elems"] - sum(large) < 0.01 * sum(large)
        # the flat shard keeps the largest chunk: 98 x 2^24 is 0.87 % more than 1.63e9
        lay, _, _ = layout([row(1_630_000_000)], _cabi.MEMORY_EFFICIENT_MIXED_PRECISION)
        assert lay["large_chunk_elems"] == 1 << 24 and lay["n_large_descriptors"] == 98
        # one tensor just over a power of two: 2^24 + 2^20 elements would need two chunks of 2^23... halved down to 2^20
        lay, _, _ = layout([row((1 << 24) + (1 << 20))], _cabi.FULL_PRECISION)
        assert lay["large_chunk_elems"] == 1 << 20 and lay["n_large_descriptors"] == 17
    finally:
        _cabi.set_option("merge_runs", old)


def test_layout_counts_heads_among_the_small_descriptors(two_classes):
    A = 0x7000_0000_0000
    t = lambda n, off: (A + off, A + (1 << 34) + off, A + (2 << 34) + off, A + (3 << 34) + off, 0, n)  # noqa: E731
    # 100 elements short of a 1 KiB boundary: head 100, then exactly two shared chunks
    lay, cls, vec = layout([t(131072 + 100, 1024 - 400)], _cabi.FULL_PRECISION)
    assert cls == [2] and vec == [1]
    assert lay["n_large_descriptors"] == 2 and lay["n_small_descriptors"] == 1
    # without the head the same tensor needs a third chunk
    old = _cabi.get_option("align_heads")
    try:
        _cabi.set_option("align_heads", 0)
        lay0, cls0, vec0 = layout([t(131072 + 100, 1024 - 400)], _cabi.FULL_PRECISION)
        assert cls0 == [2] and vec0 == [1] and lay0["n_large_descriptors"] == 3 and lay0["n_small_descriptors"] == 0
    finally:
        _cabi.set_option("align_heads", old)
    # a head can take a tensor below the size that shares descriptors, and can be longer than a tile
    lay, cls, vec = layout([t(131072 + 10, 4)], _cabi.FULL_PRECISION)  # head 255, 130827 left
    assert cls == [1] and vec == [1] and lay["n_large_descriptors"] == 0 and lay["n_small_descriptors"] == 1 + -(-130827 // 256)
    half = lambda n, off: (A + off, A + (1 << 34) + off, A + (2 << 34) + off, A + (3 << 34) + off, 0, n)  # noqa: E731
    lay, cls, vec = layout([half(9000, 2)], _cabi.PURE_FP16)  # 2 bytes in: head 511 halves, under one 512-element tile
    assert lay["n_small_descriptors"] == 1 + -(-(9000 - 511) // 512) and vec == [1]
    # vector_ok describes what follows the head: 3 elements in, the tiles start aligned
    lay, cls, vec = layout([t(10000, 12), t(5000, 12)], _cabi.FULL_PRECISION)
    assert vec == [1, 0]


def test_layout_matches_a_python_model_on_drawn_lists():
    """Descriptor and workgroup counts for drawn lists, modes and options against ten lines of Python."""
    import random

    rng = random.Random(42)
    A = 0x7000_0000_0000
    names = ("mid_tiles",)
    old = {k: _cabi.get_option(k) for k in names}
    try:
        for _ in range(120):
            block, groups, cap = 64, 1, 1 << 24
            mid_tiles = rng.choice([0, 1, 2, 16, 16, 64])
            _cabi.set_option("mid_tiles", mid_tiles)
            mode = rng.choice([_cabi.FULL_PRECISION, _cabi.MIXED_PRECISION, _cabi.MEMORY_EFFICIENT_MIXED_PRECISION, _cabi.PURE_FP16])
            sizes = [rng.choice([0, 1, rng.randrange(2, 5000), rng.randrange(5000, 131072), 131072, rng.randrange(131072, 1 << 22),
                                 rng.randrange(1 << 22, 1 << 31)]) for _ in range(rng.randrange(1, 30))]
            tile = block * (8 if mode == _cabi.PURE_FP16 else 4) * groups
            large = [n for n in sizes if n >= 131072]
            chunk = 65536
            if large:
                chunk = 1 << ((min(large) // 2).bit_length() - 1)
            chunk = min(cap, max(65536, min(1 << 24, chunk)))
            # halved until the tiles behind the tensors' ends are at most 1 % of the large tensors' elements
            while chunk > 65536 and (sum(-(-n // chunk) * chunk for n in large) - sum(large)) * 100 > sum(large):
                chunk //= 2
            want_large = sum(-(-n // chunk) for n in large)
            # a middle class only for 2..64 tiles per descriptor and chunks of at most half the large threshold
            mid_chunk = tile * mid_tiles if mid_tiles > 1 and 2 * tile * mid_tiles <= 131072 else 0
            is_mid = lambda n: mid_chunk and mid_chunk <= n < 131072  # noqa: E731
            want_mid = sum(-(-n // mid_chunk) for n in sizes if is_mid(n))
            want_small = sum(-(-n // tile) for n in sizes if 0 < n < 131072 and not is_mid(n))
            rows_ = [(A, A + (1 << 40), A + (2 << 40), A + (3 << 40), A + (4 << 40) if mode == _cabi.MIXED_PRECISION else 0, n) for n in sizes]
            lay, cls, _ = layout(rows_, mode)
            what = f"block {block} groups {groups} cap {cap} mode {mode} sizes {sizes}"
            assert lay["tile_elems"] == tile and lay["large_chunk_elems"] == chunk, what
            assert lay["n_large_descriptors"] == want_large and lay["n_small_descriptors"] == want_small, what
            assert lay["grid_large"] == want_large * (chunk // tile) and lay["grid_small"] == want_small, what
            assert lay["mid_chunk_elems"] == mid_chunk and lay["n_mid_descriptors"] == want_mid and lay["grid_mid"] == want_mid * mid_tiles, what
            assert cls == [0 if n == 0 else (2 if n >= 131072 else 3 if is_mid(n) else 1) for n in sizes], what
    finally:
        for k, v in old.items():
            _cabi.set_option(k, v)


def test_layout_alignment_rule_per_mode():
    A = 0x7000_0000_0000
    n = 1000

    def vec_ok(mode, p=0, m=0, v=0, g=0, pc=0):
        _, _, vec = layout([(A + p, A + (1 << 32) + m, A + (2 << 32) + v, A + (3 << 32) + g, A + (4 << 32) + pc, n)], mode)
        return vec[0]

    # fp32 streams need 16 bytes; fp16 streams need 8 bytes in the 4-element modes and 16 in PURE_FP16
    assert vec_ok(_cabi.FULL_PRECISION) == 1
    for k in ("p", "m", "v", "g"):
        assert vec_ok(_cabi.FULL_PRECISION, **{k: 4}) == 0 and vec_ok(_cabi.FULL_PRECISION, **{k: 16}) == 1
    assert vec_ok(_cabi.MIXED_PRECISION, g=8) == 1 and vec_ok(_cabi.MIXED_PRECISION, g=2) == 0
    assert vec_ok(_cabi.MIXED_PRECISION, pc=8) == 1 and vec_ok(_cabi.MIXED_PRECISION, pc=6) == 0 and vec_ok(_cabi.MIXED_PRECISION, p=8) == 0
    assert vec_ok(_cabi.MEMORY_EFFICIENT_MIXED_PRECISION, p=8, g=8) == 1 and vec_ok(_cabi.MEMORY_EFFICIENT_MIXED_PRECISION, m=8) == 0
    assert vec_ok(_cabi.PURE_FP16, p=8) == 0 and vec_ok(_cabi.PURE_FP16, p=16, m=16, v=16, g=16) == 1


def test_bad_arguments_return_einval_before_touching_a_device():
    L = _cabi.lib()
    A = 0x7000_0000_0000
    good = (A, A + 4096, A + 8192, A + 12288, 0, 16)
    args = (1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, 0.0, 1, 1, 1, None, None)
    EINVAL = header_define("FSADAM_EINVAL")
    cases = [
        (rows(good), 0, _cabi.FULL_PRECISION, "empty"),               # multi_tensor_apply.cuh:51
        (rows(good), 1, 7, "unknown precision mode"),
        (rows(good), 1, _cabi.FULL_PRECISION_FP16_COPY, "needs p_copy"),
        (None, 1, _cabi.FULL_PRECISION, "NULL"),
        (rows((A, A, A, A, 0, -5)), 1, _cabi.FULL_PRECISION, "negative numel"),
        (rows((0, A, A, A, 0, 16)), 1, _cabi.FULL_PRECISION, "NULL p/m/v/g"),
        (rows((A, A, A, A + 2, 0, 16)), 1, _cabi.FULL_PRECISION, "not aligned to its element size"),
        (rows((A, A, A, A + 1, 0, 16)), 1, _cabi.PURE_FP16, "not aligned to its element size"),
        (rows(good), 1, _cabi.MIXED_PRECISION, "needs p_copy"),
    ]
    for arr, n, mode, needle in cases:
        rc = L.fsadam_step(arr, n, mode, *args)
        assert rc == EINVAL, needle
        assert needle in last_error()
    out = _cabi.FsAdamLayout()
    assert L.fsadam_layout(rows(good), 1, 9, ctypes.byref(out), None, None) == EINVAL
    assert L.fsadam_layout(rows(good), 1, 0, None, None, None) == EINVAL


def test_plan_lifecycle_without_a_device():
    L = _cabi.lib()
    EINVAL = header_define("FSADAM_EINVAL")
    handle = ctypes.c_void_p()
    assert L.fsadam_plan_create(5, ctypes.byref(handle)) == EINVAL
    assert L.fsadam_plan_create(_cabi.PURE_FP16, None) == EINVAL
    _cabi.check(L.fsadam_plan_create(_cabi.PURE_FP16, ctypes.byref(handle)))
    info = _cabi.FsAdamPlanInfo()
    _cabi.check(L.fsadam_plan_info(handle, ctypes.byref(info)))
    assert info.mode == _cabi.PURE_FP16 and info.n_tensors == 0 and info.uploads == 0 and info.n_launches == 0
    # stepping a plan that has no tensors is an argument error, not a crash
    assert L.fsadam_plan_step(handle, 1e-3, 0.9, 0.999, 1e-8, 1.0, 65536.0, 0.0, 1, 1, 1, None, None) == EINVAL
    assert "no tensors" in last_error()
    assert L.fsadam_plan_set_tensors(handle, None, 1, None) == EINVAL
    # the variant with the gradient scale on the device insists on a pointer
    assert L.fsadam_plan_step_dev_scale(handle, 1e-3, 0.9, 0.999, 1e-8, None, 65536.0, 0.0, 1, 1, 1, None, None) == EINVAL
    assert "grad_scale_dev" in last_error()
    assert L.fsadam_plan_step_dev_scale(None, 1e-3, 0.9, 0.999, 1e-8, ctypes.c_void_p(4096), 65536.0, 0.0, 1, 1, 1, None, None) == EINVAL
    _cabi.check(L.fsadam_plan_destroy(handle))
    _cabi.check(L.fsadam_plan_destroy(None))
    _cabi.check(L.fsadam_clear_cache())


# ---- the Python face of the native call (validation of multi_tensor_apply.cuh:49-67, dispatch of kernel.cu:165-263)

def _lists(p_dtype, g_dtype, s_dtype, n=8, copy=False):
    mk = lambda dt: [torch.zeros(n, dtype=dt), torch.zeros(3, dtype=dt)]  # noqa: E731
    out = [mk(p_dtype), mk(s_dtype), mk(s_dtype), mk(g_dtype)]
    if copy:
        out.append(mk(torch.float16))
    return out


def test_mode_dispatch_follows_the_reference():
    f32, f16 = torch.float32, torch.float16
    assert fused_adam_hip.mode_of_lists(_lists(f32, f32, f32)) == _cabi.FULL_PRECISION
    assert fused_adam_hip.mode_of_lists(_lists(f32, f16, f32, copy=True)) == _cabi.MIXED_PRECISION
    assert fused_adam_hip.mode_of_lists(_lists(f16, f16, f32)) == _cabi.MEMORY_EFFICIENT_MIXED_PRECISION
    assert fused_adam_hip.mode_of_lists(_lists(f16, f16, f16)) == _cabi.PURE_FP16
    assert fused_adam_hip.mode_of_lists(_lists(f32, f32, f32, copy=True)) == _cabi.FULL_PRECISION_FP16_COPY  # extension
    for bad in (_lists(f32, f16, f32), _lists(f32, f32, f16), _lists(torch.bfloat16, torch.bfloat16, f32),
                _lists(f16, f16, torch.float64), _lists(f16, f16, f32, copy=True), _lists(f32, f32, f32)[:3], [[], [], [], []]):
        with pytest.raises(RuntimeError):
            fused_adam_hip.mode_of_lists(bad)


def test_list_validation_raises_runtime_error_like_torch_check():
    flag = torch.zeros(1)
    call = lambda lists: fused_adam_hip.adam(65536, None, lists, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 1, 1, 0.0)  # noqa: E731
    with pytest.raises(RuntimeError, match="not cuda"):
        call(_lists(torch.float32, torch.float32, torch.float32))
    # same order as the reference: contiguity is checked before the device (multi_tensor_apply.cuh:59-64)
    lists = _lists(torch.float32, torch.float32, torch.float32)
    lists[0][0] = torch.zeros(16)[::2]
    with pytest.raises(RuntimeError, match="not contiguous"):
        call(lists)


def test_rows_of_lists_matches_the_struct_layout():
    lists = _lists(torch.float32, torch.float16, torch.float32, copy=True)
    arr = fused_adam_hip.rows_of_lists(lists)
    assert arr.shape == (2, 6) and arr.dtype == np.int64 and arr.flags["C_CONTIGUOUS"]
    view = ctypes.cast(arr.ctypes.data, ctypes.POINTER(_cabi.FsAdamTensor))
    for t in range(2):
        assert view[t].p == lists[0][t].data_ptr() and view[t].m == lists[1][t].data_ptr()
        assert view[t].v == lists[2][t].data_ptr() and view[t].g == lists[3][t].data_ptr()
        assert view[t].p_copy == lists[4][t].data_ptr() and view[t].numel == lists[0][t].numel()


def test_optimizer_module_imports_and_exposes_the_reference_names():
    import fairscale_amd.optim as fo

    assert [p.name for p in fo.Precision] == ["FULL_PRECISION", "MIXED_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION", "PURE_FP16"]
    assert [p.value for p in fo.Precision] == [1, 2, 3, 4]  # auto() values of adam.py:19-23
    assert issubclass(fo.Adam, torch.optim.Optimizer)
    assert issubclass(fo.GradScaler, torch.amp.GradScaler)


def test_versioned_state_map_counts_what_changes_the_key_set():
    """``optimizer.state`` of Adam: the steady-state step trusts its cached per-parameter state dicts only
    while this counter stands still."""
    import copy
    import pickle

    from fairscale_amd.optim.adam import _VersionedState

    st = _VersionedState(dict)
    v0 = st.version
    a = st["a"]           # created on first access (torch's defaultdict(dict) behaviour)
    assert a == {} and st.version > v0
    v1 = st.version
    st["a"]["step"] = 1   # changing a state dict in place is not a change of the map
    assert st["a"] is a and st.version == v1
    for change in (lambda: st.__setitem__("b", {}), lambda: st.pop("b"), lambda: st.setdefault("c", {}), lambda: st.update(d={}),
                   lambda: st.__delitem__("c"), lambda: st.popitem(), lambda: st.clear()):
        before = st.version
        change()
        assert st.version > before
    st["x"]["step"] = 7
    for clone in (pickle.loads(pickle.dumps(st)), copy.deepcopy(st)):
        assert type(clone) is _VersionedState and clone["x"] == {"step": 7} and clone["fresh"] == {}


def test_wide_assembly_stores_carry_their_wait_states():
    """The write-through store comes from inline assembly, so the compiler does not keep vector instructions away from the
    store's data registers for the two wait states a store of more than 64 bits needs on gfx950: the assembly text has to.
    (What happens without them: a parameter per lane comes out wrong in FULL_PRECISION with fp16 copies, which the GPU suite
    shows.)  Every 128-bit store in an asm statement of the library's sources is followed by `s_nop 1` in the same statement."""
    import glob
    import re

    src_dir = os.path.join(REPO, "fairscale_amd", "csrc")
    wide = 0
    sources = (glob.glob(os.path.join(src_dir, "fsadam*.h")) + glob.glob(os.path.join(src_dir, "*_kernels.h"))
               + [os.path.join(src_dir, "fsadam.hip"), os.path.join(src_dir, "membench.hip")])  # the microbenchmarks too: their figures decide shapes
    for path in sources:
        text = open(path).read()
        for statement in re.findall(r'asm volatile\((.*?)\);', text, flags=re.S):
            if "global_store_dwordx4" in statement or "global_store_dwordx3" in statement:
                wide += 1
                after = statement[re.search(r'global_store_dwordx[34]', statement).end():]
                assert re.search(r'\\n\\ts_nop 1"', after), f"{path}: a wide store without its wait states"
    assert wide >= 2


def test_assembly_loads_wait_in_their_own_statement():
    """A load issued from inline assembly is not counted by the compiler, which may therefore read (copy, spill) the
    result register before the data has arrived unless the statement that issues the load also waits for it."""
    import re

    for name in ("membench.hip", "fsadam.hip", "fsadam_common.h", "adam_kernels.h", "grad_kernels.h"):
        text = open(os.path.join(REPO, "fairscale_amd", "csrc", name)).read()
        for statement in re.findall(r'asm volatile\((.*?)\);', text, flags=re.S):
            if "global_load" in statement:
                assert "s_waitcnt vmcnt(0)" in statement, f"{name}: a load from assembly without its wait"
