"""The C++ list walk (csrc/tensor_rows.cpp) against the Python walk it replaces, on host tensors.

The helper reads pointers and metadata only, so everything but the "is on a GPU" check can be
exercised without one (device index -1 = host tensors).
"""
from __future__ import annotations

import numpy as np
import pytest
import torch

from fairscale_amd import _rows
from fairscale_amd.fused_adam_hip import rows_of_lists

native = _rows.native
pytestmark = pytest.mark.skipif(native is None, reason="csrc/_tensor_rows is not built")

F32, F16 = 0, 1


def make_lists(sizes, depth=4, p_dtype=torch.float32, s_dtype=torch.float32, g_dtype=torch.float32):
    p = [torch.zeros(n, dtype=p_dtype) for n in sizes]
    m = [torch.zeros(n, dtype=s_dtype) for n in sizes]
    v = [torch.zeros(n, dtype=s_dtype) for n in sizes]
    g = [torch.zeros(n, dtype=g_dtype) for n in sizes]
    lists = [p, m, v, g]
    if depth == 5:
        lists.append([torch.zeros(n, dtype=torch.float16) for n in sizes])
    return lists


def fill(lists, codes, rows, device=-1):
    return native.fill_rows(lists, codes, device, rows.ctypes.data, len(lists[0]))


def test_module_exports_the_status_names():
    names = ["UNCHANGED", "CHANGED", "NOT_TENSOR", "NOT_CONTIGUOUS", "NOT_CUDA", "NUMEL", "DTYPE", "DEVICE", "LENGTH",
             "NO_GRAD", "SPARSE", "NO_STATE", "ERROR", "STALE"]
    values = [getattr(native, n) for n in names]
    assert len(set(values)) == len(values)
    assert native.UNCHANGED == 0 and native.CHANGED == 1 and all(v < 0 for v in values[2:])
    assert _rows.describe(native.NUMEL) == "NUMEL"


@pytest.mark.parametrize("depth", [4, 5])
def test_fill_rows_equals_the_python_walk(depth):
    sizes = [5, 0, 1, 4097, 33]
    lists = make_lists(sizes, depth, g_dtype=torch.float16 if depth == 5 else torch.float32)
    codes = (F32, F32, F32, F16, F16) if depth == 5 else (F32, F32, F32, F32)
    rows = np.zeros((len(sizes), 6), np.int64)
    status, lst, idx, extra = fill(lists, codes, rows)
    assert (status, lst, idx, extra) == (native.CHANGED, -1, -1, None)
    assert np.array_equal(rows, rows_of_lists(lists))
    assert fill(lists, codes, rows)[0] == native.UNCHANGED
    lists[3][2] = torch.zeros(1, dtype=lists[3][2].dtype)  # one gradient moved
    assert fill(lists, codes, rows)[0] == native.CHANGED
    assert np.array_equal(rows, rows_of_lists(lists))


def test_fill_rows_clears_the_copy_column_when_there_are_four_lists():
    lists = make_lists([3, 4])
    rows = np.full((2, 6), 7, np.int64)
    assert fill(lists, (F32,) * 4, rows)[0] == native.CHANGED
    assert (rows[:, 4] == 0).all()


def test_fill_rows_reports_the_first_offence_in_the_reference_order():
    """multi_tensor_apply.cuh:55-65: per list, per tensor: contiguous, cuda, numel."""
    codes = (F32,) * 4
    rows = np.zeros((3, 6), np.int64)

    lists = make_lists([4, 6, 8])
    lists[1][1] = torch.zeros(12)[::2]  # right numel, not contiguous
    lists[2][0] = torch.zeros(5)        # wrong numel, in a later list
    assert fill(lists, codes, rows)[:3] == (native.NOT_CONTIGUOUS, 1, 1)

    lists = make_lists([4, 6, 8])
    lists[2][2] = torch.zeros(9)
    assert fill(lists, codes, rows)[:3] == (native.NUMEL, 2, 2)

    lists = make_lists([4, 6, 8])
    lists[3][0] = torch.zeros(4, dtype=torch.float16)
    assert fill(lists, codes, rows)[:3] == (native.DTYPE, 3, 0)

    lists = make_lists([4, 6, 8])
    lists[1] = lists[1][:2]
    assert fill(lists, codes, rows)[:2] == (native.LENGTH, 1)

    lists = make_lists([4, 6, 8])
    lists[0][1] = "not a tensor"
    assert fill(lists, codes, rows)[:3] == (native.NOT_TENSOR, 0, 1)

    lists = make_lists([4, 6, 8])
    lists[3][1] = torch.zeros(6).to_sparse()
    assert fill(lists, codes, rows)[:3] == (native.SPARSE, 3, 1)

    # with a GPU index, host tensors are refused where the reference says "not cuda"
    assert fill(make_lists([4, 6, 8]), codes, rows, device=0)[:3] == (native.NOT_CUDA, 0, 0)
    # depth and code count must agree
    assert native.fill_rows(make_lists([4]), (F32,) * 5, -1, rows.ctypes.data, 1)[0] == native.LENGTH
    assert native.fill_rows(make_lists([4])[:3], (F32,) * 3, -1, rows.ctypes.data, 1)[0] == native.LENGTH


class Group:
    """Parameters with gradients and the states an optimizer would hold for them."""

    def __init__(self, sizes, p_dtype=torch.float32, s_dtype=torch.float32, with_masters=False, with_outs=False):
        self.params = [torch.nn.Parameter(torch.zeros(n, dtype=p_dtype)) for n in sizes]
        for p in self.params:
            p.grad = torch.zeros_like(p)
        self.states = [{"step": 3, "exp_avg": torch.zeros(n, dtype=s_dtype), "exp_avg_sq": torch.zeros(n, dtype=s_dtype)}
                       for n in sizes]
        self.masters = [torch.nn.Parameter(torch.zeros(n)) for n in sizes] if with_masters else None
        self.outs = [torch.zeros(n, dtype=torch.float16) for n in sizes] if with_outs else None
        self.rows = np.zeros((len(sizes), 6), np.int64)
        self.codes = (F32 if (with_masters or p_dtype == torch.float32) else F16, F16 if s_dtype == torch.float16 else F32,
                      F16 if p_dtype == torch.float16 else F32)

    def gather(self, snapshot=None, device=-1):
        return native.gather(self.params, tuple(self.params) if snapshot is None else snapshot, self.masters, self.states,
                             self.outs, self.codes, device, self.rows.ctypes.data)

    def expected_rows(self):
        lists = [self.masters or self.params, [s["exp_avg"] for s in self.states], [s["exp_avg_sq"] for s in self.states],
                 [p.grad for p in self.params]]
        if self.masters is not None:
            lists.append(self.params)
        elif self.outs is not None:
            lists.append(self.outs)
        return rows_of_lists(lists)


def test_gather_writes_the_rows_and_advances_every_step_counter():
    g = Group([7, 1, 300])
    assert g.gather() == (native.CHANGED, -1, -1, 4)
    assert np.array_equal(g.rows, g.expected_rows())
    assert [s["step"] for s in g.states] == [4, 4, 4]
    assert g.gather() == (native.UNCHANGED, -1, -1, 5)
    g.params[1].grad = torch.zeros(1)  # backward allocated a new gradient
    assert g.gather() == (native.CHANGED, -1, -1, 6)
    assert np.array_equal(g.rows, g.expected_rows())
    g.states[2]["step"] = 40  # the call reports the last parameter's counter (adam.py:272)
    assert g.gather()[3] == 41


def test_gather_memory_efficient_and_pure_fp16_dtypes():
    g = Group([8, 9], p_dtype=torch.float16)
    assert g.gather()[0] == native.CHANGED
    assert np.array_equal(g.rows, g.expected_rows())
    g = Group([8, 9], p_dtype=torch.float16, s_dtype=torch.float16)
    assert g.gather()[0] == native.CHANGED
    g.states[1]["exp_avg_sq"] = torch.zeros(9)  # fp32 state in a PURE_FP16 group
    assert g.gather()[:3] == (native.DTYPE, 2, 1)


def test_gather_mixed_precision_takes_p_from_the_masters_and_writes_the_params_as_copies():
    g = Group([8, 9], p_dtype=torch.float16, with_masters=True)
    assert g.gather()[0] == native.CHANGED
    assert np.array_equal(g.rows, g.expected_rows())
    assert g.rows[0, 0] == g.masters[0].data_ptr() and g.rows[0, 4] == g.params[0].data_ptr()
    assert g.rows[0, 3] == g.params[0].grad.data_ptr()


def test_gather_with_attached_copies():
    g = Group([8, 9], with_outs=True)
    assert g.gather()[0] == native.CHANGED
    assert np.array_equal(g.rows, g.expected_rows())
    g.outs[1] = torch.zeros(9)
    assert g.gather()[:3] == (native.DTYPE, 4, 1)


def test_gather_refuses_without_touching_a_counter():
    g = Group([7, 1, 300])
    g.params[2].grad = None
    assert g.gather()[:3] == (native.NO_GRAD, 3, 2)
    g.params[2].grad = torch.zeros(300).to_sparse()
    assert g.gather()[:3] == (native.SPARSE, 3, 2)
    g.params[2].grad = torch.zeros(300)
    g.states[0]["exp_avg"] = torch.zeros(8)  # torch itself refuses a gradient of another size; a state can differ
    assert g.gather()[:3] == (native.NUMEL, 1, 0)
    g.states[0]["exp_avg"] = torch.zeros(7)
    g.params[2].grad = torch.zeros(600)[::2]
    assert g.gather()[:3] == (native.NOT_CONTIGUOUS, 3, 2)
    g.params[2].grad = torch.zeros(300)
    del g.states[1]["exp_avg_sq"]
    assert g.gather()[:3] == (native.NO_STATE, 1, 1)
    g.states[1] = {}
    assert g.gather()[:3] == (native.NO_STATE, 1, 1)
    assert [s.get("step") for s in g.states] == [3, None, 3]
    assert g.gather(device=0)[0] == native.NOT_CUDA


def test_gather_notices_a_parameter_list_edited_in_place():
    g = Group([7, 1, 300])
    snapshot = tuple(g.params)
    assert g.gather(snapshot)[0] == native.CHANGED
    replacement = torch.nn.Parameter(torch.zeros(1))
    replacement.grad = torch.zeros(1)
    g.params[1] = replacement
    assert g.gather(snapshot)[:3] == (native.STALE, 0, 1)
    assert g.gather(snapshot[:2])[0] == native.STALE
    assert [s["step"] for s in g.states] == [4, 4, 4]


def test_tensor_subclasses_are_left_to_the_python_walk():
    class Tagged(torch.Tensor):
        pass

    lists = make_lists([4, 4])
    lists[0][1] = torch.zeros(4).as_subclass(Tagged)
    rows = np.zeros((2, 6), np.int64)
    assert fill(lists, (F32,) * 4, rows)[:3] == (native.NOT_TENSOR, 0, 1)


def test_fill_grad_rows():
    grads = [torch.zeros(n, dtype=torch.float16) for n in (5, 0, 70001)]
    rows = np.zeros((3, 2), np.int64)
    assert native.fill_grad_rows(grads, F16, -1, rows.ctypes.data) == (native.UNCHANGED, 3, -1, None)
    assert rows[:, 0].tolist() == [g.data_ptr() for g in grads] and rows[:, 1].tolist() == [5, 0, 70001]
    assert native.fill_grad_rows(grads, F32, -1, rows.ctypes.data)[:3] == (native.DTYPE, 3, 0)
    grads[2] = torch.zeros(140002, dtype=torch.float16)[::2]
    assert native.fill_grad_rows(grads, F16, -1, rows.ctypes.data)[:3] == (native.NOT_CONTIGUOUS, 3, 2)
    grads[2] = torch.zeros(4, dtype=torch.float16).to_sparse()
    assert native.fill_grad_rows(grads, F16, -1, rows.ctypes.data)[:3] == (native.SPARSE, 3, 2)
    assert native.fill_grad_rows(grads[:2], F16, 0, rows.ctypes.data)[:3] == (native.NOT_CUDA, 3, 0)
    assert native.fill_grad_rows([], F16, -1, rows.ctypes.data)[0] == native.LENGTH


def test_gather_with_parameters_that_sit_out():
    """A state of None marks a parameter that had no gradient when the lists were collected: it must still
    have none; rows are written for the others only."""
    g = Group([7, 1, 300, 12])
    g.params[1].grad = None
    g.states[1] = None
    g.rows = np.zeros((3, 6), np.int64)
    assert g.gather() == (native.CHANGED, -1, -1, 4)
    active = [0, 2, 3]
    assert g.rows[:, 0].tolist() == [g.params[t].data_ptr() for t in active]
    assert g.rows[:, 3].tolist() == [g.params[t].grad.data_ptr() for t in active]
    assert g.rows[:, 5].tolist() == [7, 300, 12]
    assert [s["step"] if s else None for s in g.states] == [4, None, 4, 4]
    assert g.gather()[0] == native.UNCHANGED
    g.params[1].grad = torch.zeros(1)  # it takes part from now on: the lists must be collected again
    assert g.gather()[:3] == (native.STALE, 3, 1)
    assert [s["step"] if s else None for s in g.states] == [5, None, 5, 5]
    g.params[1].grad = None
    g.params[3].grad = None  # one that used to take part lost its gradient
    assert g.gather()[:3] == (native.NO_GRAD, 3, 3)
    for t in (0, 2, 3):
        g.states[t] = None
        g.params[t].grad = None
    assert g.gather()[0] == native.NO_GRAD  # nobody takes part
