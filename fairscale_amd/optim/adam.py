"""``Adam`` / ``Precision``: the interface of ``fairscale/optim/adam.py`` over the gfx950 kernels.

Same constructor, attributes, ``state_dict`` keys, exceptions and optimizer-state-scale behaviour as
the reference class (``fairscale/optim/adam.py:42-297``); the native call it makes per (param group,
device) goes to ``libfsadam.so`` instead of ``fairscale.fused_adam_cuda``.

Deliberate differences, all supersets of the reference behaviour:

* ``step(closure=None, *, scale=1.0)``: the gradient scale the kernel divides by is reachable through
  the class (the reference hard-codes 1.0, adam.py:238, although its docstring lists ``scale``).
* ``lr``/``eps``/``betas``/``weight_decay`` are range-checked (``ValueError``), which is what
  ``tests/optim/test_adam.py:357-370`` expects.
* The device flag is only allocated, cleared and read back in PURE_FP16: the other three modes cannot
  raise it (fused_adam_cuda_kernel.cu:94-105 is the only writer), so they step without a host sync.
  In PURE_FP16 it is cleared only after a step that raised it (a flag read back as 0 is still 0).
  The scale bookkeeping they do every step (adam.py:289-295) is kept.
* After an overflow m and v are zeroed in place rather than re-allocated (adam.py:285-288).  Parameters that
  never had a gradient get zero ``exp_avg``/``exp_avg_sq`` without a ``"step"`` there, as in the reference; should
  such a parameter receive a gradient later, its counter starts at 0 (the reference raises ``KeyError``).
* ``load_state_dict`` keeps fp32 ``exp_avg``/``exp_avg_sq`` exact for fp16 parameters (the reference
  round-trips them through fp16, adam.py:176-182).
* The fp32 master copies of MIXED_PRECISION carry no ``.grad`` (the reference allocates a zero one per
  copy, adam.py:128, and never reads it).
* ``exp_avg``/``exp_avg_sq`` are laid out like the parameters (``zeros_like`` per parameter in the reference,
  adam.py:226-228): parameters that are back-to-back views of one buffer (OSS's buckets, oss.py:630-659) get
  state that is back-to-back views of one buffer too, and so do the fp32 master copies of MIXED_PRECISION; the
  state of a run of 8192 elements or more starts as many elements past a 1 KiB boundary as the run does.  The native
  layout then treats each run as one tensor.  The placement is re-established (one copy of the state) after
  ``load_state_dict`` and after ``optimizer.state[p]`` has been assigned directly, as
  ``OSS.load_state_dict`` does (oss.py:453-461).
"""
from __future__ import annotations

from collections import defaultdict
from enum import Enum, auto
from typing import Any, Callable, Dict, List, Optional, Tuple, Union

import torch

from .. import _cabi, _rows
from ..fused_adam_hip import TensorListPlan, mode_codes

_cabi.lib()  # loading the kernels is part of importing the optimizer: no library, no Adam

__all__ = ["Adam", "Precision"]


class Precision(Enum):
    """Where parameters, gradients and optimizer state live (adam.py:19-23)."""

    FULL_PRECISION = auto()
    MIXED_PRECISION = auto()
    MEMORY_EFFICIENT_MIXED_PRECISION = auto()
    PURE_FP16 = auto()


_NATIVE_MODE = {
    Precision.FULL_PRECISION: _cabi.FULL_PRECISION,
    Precision.MIXED_PRECISION: _cabi.MIXED_PRECISION,
    Precision.MEMORY_EFFICIENT_MIXED_PRECISION: _cabi.MEMORY_EFFICIENT_MIXED_PRECISION,
    Precision.PURE_FP16: _cabi.PURE_FP16,
}

_MAX_OPTIM_SCALE = 2 ** 16


_PLACE_MIN = 8192  # shorter runs are left where the allocator puts them (the native layout gives them no head either)


def _adjacent_runs(tensors: List[torch.Tensor]) -> List[List[int]]:
    """Indices of ``tensors`` grouped into maximal runs of consecutive entries that lie back to back in
    memory (entry k+1 starts at the byte behind entry k's last element)."""
    runs: List[List[int]] = []
    end = None
    last = None  # the last non-empty tensor of the current run
    for k, t in enumerate(tensors):
        if t.numel() == 0 and runs:
            runs[-1].append(k)  # nothing to place: it rides along (the native layout skips empty rows as well)
            continue
        ptr = t.data_ptr()
        if end is not None and ptr == end and t.is_contiguous() and t.dtype == last.dtype and t.device == last.device:
            runs[-1].append(k)
        else:
            runs.append([k])
        end = ptr + t.numel() * t.element_size() if t.is_contiguous() else None
        last = t
    return runs


def _phase(t: torch.Tensor) -> int:
    """Where a tensor starts, in elements past a boundary of 512 elements (1 KiB of fp16, 2 KiB of fp32)."""
    return (t.data_ptr() // t.element_size()) % 512


def _needs_placing(total: int) -> bool:
    """A run of ``total`` elements is long enough for the native layout to split off a head, so that the tiles behind it
    start on 1 KiB boundaries: the streams that accompany the run must then share its phase.  A wave moves 512 or 1024
    contiguous bytes of a stream per instruction, and a stream that is on a 128-byte line but off a 1 KiB boundary costs
    1.5 % of the step's rate (all four: 5 %); the allocator hands out 512-byte granules, so without this every stream of a
    separately allocated tensor has even odds of being off."""
    return total >= _PLACE_MIN


def _buffer_placed_like(first: torch.Tensor, total: int, dtype: torch.dtype, zero: bool) -> torch.Tensor:
    """``total`` elements of ``dtype`` for a stream that accompanies a run starting at ``first``.  For a run long enough to
    be given a head, the stream starts as many elements past a boundary of 512 elements as the run does (which may be
    none): the native layout then finds ONE head length that puts the tiles of both on 1 KiB boundaries, wherever the
    allocator put the run.  Taken from a plain allocation when that happens to have the right phase, else from one 512
    elements longer."""
    make = torch.zeros if zero else torch.empty
    if not _needs_placing(total):
        return make(total, dtype=dtype, device=first.device)
    want = _phase(first)
    buf = torch.empty(total, dtype=dtype, device=first.device)
    if _phase(buf) == want:
        return buf.zero_() if zero else buf
    del buf
    buf = make(total + 512, dtype=dtype, device=first.device)
    start = (want - _phase(buf)) % 512
    return buf[start:start + total]


def _placed(streams: List[torch.Tensor], likes: List[torch.Tensor]) -> bool:
    """Do ``streams`` (one per entry of the run ``likes``) already lie back to back, at the run's phase?"""
    first, total = likes[0], sum(t.numel() for t in likes)
    end = None
    for st, like in zip(streams, likes):
        if not st.is_contiguous() or st.numel() != like.numel() or st.device != like.device:
            return False
        if like.numel() == 0:
            continue  # nothing to lie anywhere
        if end is not None and st.data_ptr() != end:
            return False
        end = st.data_ptr() + st.numel() * st.element_size()
    if _needs_placing(total):
        return _phase(streams[0]) == _phase(first)
    return True


class _VersionedState(defaultdict):
    """``optimizer.state`` that counts its own insertions and removals, so that the step can tell in
    O(1) whether the per-parameter state dicts it collected earlier are still the ones in the map."""

    version = 0

    def __setitem__(self, key, value):
        self.version += 1
        super().__setitem__(key, value)

    def __delitem__(self, key):
        self.version += 1
        super().__delitem__(key)

    def pop(self, *args):
        self.version += 1
        return super().pop(*args)

    def popitem(self):
        self.version += 1
        return super().popitem()

    def clear(self):
        self.version += 1
        super().clear()

    def update(self, *args, **kwargs):
        self.version += 1
        super().update(*args, **kwargs)

    def setdefault(self, key, default=None):
        self.version += 1
        return super().setdefault(key, default)


class Adam(torch.optim.Optimizer):
    """Fused Adam on MI355X. GPU-only.

    Arguments (as ``fairscale.optim.Adam``, adam.py:76-88):
        params: iterable of parameters (a flat list; the precision is read off the first one).
        lr: learning rate (default 1e-3).
        bias_correction: apply the ``sqrt(1-beta2^t)/(1-beta1^t)`` factor to the step (default True).
        betas: running-average coefficients (default (0.9, 0.999)).
        eps: denominator term (default 1e-8); it is NOT rescaled by the bias correction.
        eps_inside_sqrt: ``sqrt(v + eps)`` instead of ``sqrt(v) + eps`` (default False).
        weight_decay: ``p -= step_size * weight_decay * p`` (default 0).
        max_grad_norm: stored in ``defaults`` and unused, as in the reference.
        amsgrad: not supported (``RuntimeError``).
        precision: a ``Precision``; inferred from the first parameter when None (fp32 ->
            FULL_PRECISION, otherwise MIXED_PRECISION).
    """

    state: dict
    defaults: dict
    # Lay ``exp_avg`` / ``exp_avg_sq`` (and the fp32 master copies) out like the parameters: see ``_place_state``.  With
    # False (set it on the class before constructing an optimizer, or on an instance before its first step) every
    # parameter gets state from an allocation of its own, as ``zeros_like`` gives it in the reference (adam.py:226-228):
    # for code that pickles, frees or replaces the state of single parameters and counts on each tensor owning its storage.
    place_state: bool = True

    def __init__(
        self,
        params: Any,
        lr: Optional[float] = 1e-3,
        bias_correction: Optional[bool] = True,
        betas: Optional[Tuple[float, float]] = (0.9, 0.999),
        eps: Optional[float] = 1e-8,
        eps_inside_sqrt: Optional[bool] = False,
        weight_decay: Optional[float] = 0.0,
        max_grad_norm: Optional[float] = 0.0,
        amsgrad: Optional[bool] = False,
        precision: Optional[Precision] = None,
    ):
        parameters: List[Any] = list(params)
        first_dtype = parameters[0].dtype
        if precision is None:  # adam.py:92-95
            precision = Precision.FULL_PRECISION if first_dtype == torch.float32 else Precision.MIXED_PRECISION
        self.precision = precision
        if precision is not Precision.FULL_PRECISION:  # adam.py:97-98
            assert first_dtype == torch.float16

        pure_fp16 = precision is Precision.PURE_FP16
        self.optim_type = torch.float16 if pure_fp16 else torch.float32  # adam.py:100
        self._optim_scale = float(_MAX_OPTIM_SCALE) if pure_fp16 else 1.0  # adam.py:101
        self._steps_since_optim_scale_change = 0
        self._optim_scale_update_freq = 2000  # GradScaler's default growth interval (adam.py:103)
        # kept for interface parity; the native step never reads it (fused_adam_cuda_kernel.cu:26)
        self._overflow_buf = torch.zeros(1, dtype=torch.int32, device="cuda")

        if amsgrad:
            raise RuntimeError("FusedAdam does not support the AMSGrad variant.")
        if lr is not None and not 0.0 <= lr:
            raise ValueError(f"Invalid learning rate: {lr}")
        if eps is not None and not 0.0 <= eps:
            raise ValueError(f"Invalid epsilon value: {eps}")
        if betas is not None:
            for k, beta in enumerate(betas):
                if not 0.0 <= beta < 1.0:
                    raise ValueError(f"Invalid beta parameter at index {k}: {beta}")
        if weight_decay is not None and not 0.0 <= weight_decay:
            raise ValueError(f"Invalid weight_decay value: {weight_decay}")

        super().__init__(
            parameters,
            dict(lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay,
                 max_grad_norm=max_grad_norm),
        )
        self.eps_mode = 0 if eps_inside_sqrt else 1  # adam.py:117
        self.state = _VersionedState(dict, self.state)

        self.fp32_param_groups: List[Any] = []
        if self.mixed_precision:
            self._build_fp32_params(parameters)

        self._plans: Dict[Tuple[int, torch.device], TensorListPlan] = {}
        self._flags: Dict[torch.device, torch.Tensor] = {}

    # ------------------------------------------------------------------ interface of the reference

    def _build_fp32_params(self, params: Any) -> None:
        """fp32 master copies of fp16 parameters, one group (adam.py:123-153)."""
        # The reference also gives every copy a zero .grad (adam.py:128) that nothing ever reads: 4 bytes per
        # parameter (6.5 GB on a 1.63e9 shard) that are not spent here.  Parameters that lie back to back in
        # one buffer get master copies that do too, so that the native layout can treat the run as one tensor.
        params = list(params)
        masters: List[Any] = [None] * len(params)
        datas = [p.data for p in params]
        for run in (_adjacent_runs(datas) if self.place_state else [[k] for k in range(len(datas))]):
            likes = [datas[k] for k in run]
            flat = self._stream_for(likes[0], sum(t.numel() for t in likes), torch.float32, zero=False)
            at = 0
            for k, like in zip(run, likes):
                view = flat[at:at + like.numel()].view(like.shape)
                view.copy_(like)
                masters[k] = torch.nn.Parameter(view)
                at += like.numel()
        group: Dict[str, Any] = {"params": masters}
        for name, default in self.defaults.items():
            group.setdefault(name, default)
        self.fp32_param_groups = [group]

    def _stream_for(self, first: torch.Tensor, total: int, dtype: torch.dtype, zero: bool) -> torch.Tensor:
        if not self.place_state:
            return (torch.zeros if zero else torch.empty)(total, dtype=dtype, device=first.device)
        return _buffer_placed_like(first, total, dtype, zero)

    @property
    def supports_memory_efficient_fp16(self) -> bool:
        return True

    @property
    def _step_supports_amp_scaling(self) -> bool:
        return False

    @property
    def mixed_precision(self) -> bool:
        return self.precision is Precision.MIXED_PRECISION

    def state_dict(self) -> Dict[str, Any]:
        out = super().state_dict()
        out["optim_scale"] = self._optim_scale  # adam.py:169
        return out

    def load_state_dict(self, state_dict: Dict[str, Any]) -> None:
        super().load_state_dict(state_dict)
        self._optim_scale = state_dict["optim_scale"]  # adam.py:174
        # torch casts floating state to the parameter dtype; take m and v from the saved tensors instead
        # so that fp32 state of fp16 parameters is restored bit for bit, and lay them out like the parameters
        # (one copy, straight into place).
        saved_ids = [[pid for pid in g["params"]] for g in state_dict["param_groups"]]
        saved_state = state_dict["state"]
        for gi, (group, ids) in enumerate(zip(self.param_groups, saved_ids)):
            masters = self.fp32_param_groups[gi]["params"] if self.mixed_precision else None
            states, likes = [], []
            for pj, (pid, p) in enumerate(zip(ids, group["params"])):
                if pid not in saved_state or p not in self.state:
                    continue
                like = masters[pj] if masters is not None else p
                state = self.state[p]
                for key in ("exp_avg", "exp_avg_sq"):
                    if key in saved_state[pid]:
                        state[key] = saved_state[pid][key].detach().to(device=like.device, dtype=self.optim_type)
                states.append(state)
                likes.append(like)
            self._place_state(states, likes, fresh_copy=True)
        self._plans_invalidate()

    # ------------------------------------------------------------------ the step

    def _plans_invalidate(self) -> None:
        for plan in self.__dict__.get("_plans", {}).values():
            plan.close()
        self._plans = {}
        self._group_cache = {}

    def _flag_for(self, device: torch.device) -> torch.Tensor:
        """The overflow flag of a device, holding 0.  The kernel only ever raises it, so it is cleared
        again only after a step that raised it (or whose result was never read): a step that read back 0
        leaves it ready for the next one.  (The reference allocates a fresh zero flag per group and
        step, adam.py:256.)"""
        unread = self.__dict__.setdefault("_flags_unread", set())
        flag = self._flags.get(device)
        if flag is None:
            flag = torch.zeros(1, dtype=torch.float32, device=device)
            self._flags[device] = flag
        elif device in unread:
            flag.zero_()
        unread.add(device)
        return flag

    def _read_flags(self, flags: List[torch.Tensor]) -> bool:
        """adam.py:278: did any device raise its flag?  One blocking read per flag, as in the reference."""
        raised = False
        for flag in flags:
            if flag.item() != 0.0:
                raised = True
            else:
                self._flags_unread.discard(flag.device)
        return raised

    def attach_fp16_copies(self, copies: Optional[Dict[torch.Tensor, torch.Tensor]]) -> None:
        """FULL_PRECISION only.  ``copies`` maps parameters to fp16 tensors of the same shape that the
        step then overwrites with ``half(p)`` in the same pass (None detaches).  This is the cast FSDP
        redoes before every forward (``_cast_fp32_param_shards_to_fp16``,
        ``fully_sharded_data_parallel.py:2253-2267``); fused, it costs 2 written bytes per parameter
        instead of a separate 4-byte read and 2-byte write.  Every parameter that gets a gradient must
        have a copy attached."""
        if copies is not None:
            if self.precision is not Precision.FULL_PRECISION:
                raise RuntimeError("fp16 copies can only be attached in FULL_PRECISION (MIXED_PRECISION already writes them)")
            for p, c in copies.items():
                if c.dtype != torch.float16 or c.numel() != p.numel() or c.device != p.device or not c.is_contiguous():
                    raise RuntimeError("an fp16 copy must be a contiguous float16 tensor with the parameter's numel and device")
        self._fp16_copies = dict(copies) if copies is not None else None
        self._plans_invalidate()

    def _gather(self, gi: int, group: Dict[str, Any]):
        """The per-parameter walk of adam.py:207-254: lazy state, step counters, tensor lists per device.
        Also (re)builds the group's fast-path cache when every parameter took part and shares one device."""
        mixed = self.mixed_precision
        copies = self.__dict__.get("_fp16_copies")
        if type(self.state) is not _VersionedState:  # torch's load_state_dict / __setstate__ put a plain map back
            self.state = _VersionedState(dict, self.state)
        state_map, optim_type = self.state, self.optim_type
        masters = self.fp32_param_groups[gi]["params"] if mixed else None
        batches: Dict[torch.device, List[List[torch.Tensor]]] = {}
        states: List[Optional[dict]] = []  # one entry per parameter; None for those that sit this step out
        outs: List[Optional[torch.Tensor]] = []
        step_no = None
        params = group["params"]
        depth = 5 if (mixed or copies is not None) else 4
        # first pass: who takes part, lazy state (adam.py:223-228; the tensors come from _place_state), counters
        active: List[int] = []
        for pj, p in enumerate(params):
            grad = p.grad
            if grad is None:
                states.append(None)
                continue
            if grad.is_sparse:
                raise RuntimeError("FusedAdam does not support sparse gradients, please consider SparseAdam instead")
            state = state_map[p]
            if "step" not in state:  # empty, or zeroed by an overflow before its first gradient
                state["step"] = 0
            states.append(state)
            active.append(pj)
        likes = [masters[pj] if mixed else params[pj] for pj in active]
        self._place_state([states[pj] for pj in active], likes)
        for pj, like in zip(active, likes):
            p, state = params[pj], states[pj]
            step_no = state["step"] = state["step"] + 1  # the call uses the last parameter's counter (adam.py:272)
            lists = batches.get(p.device)
            if lists is None:
                lists = batches[p.device] = [[] for _ in range(depth)]
            lists[0].append(like)
            lists[1].append(state["exp_avg"])
            lists[2].append(state["exp_avg_sq"])
            lists[3].append(p.grad)
            if mixed:
                lists[4].append(p)
            elif copies is not None:
                if p not in copies:
                    raise RuntimeError("a parameter with a gradient has no fp16 copy attached")
                lists[4].append(copies[p])
        outs = [copies.get(p) if (copies is not None and not mixed and st is not None) else None for p, st in zip(params, states)]
        caches = self.__dict__.setdefault("_group_cache", {})
        if len(batches) == 1:  # one device: the steady-state walks can take over from the next step on
            device = next(iter(batches))
            n_active = len(batches[device][0])
            caches[gi] = (params, tuple(params), states, masters, outs if (copies is not None and not mixed) else None, device, state_map,
                          state_map.version, n_active)
        else:
            caches.pop(gi, None)
        return batches, step_no

    def _place_state(self, states: List[dict], likes: List[torch.Tensor], fresh_copy: bool = False) -> None:
        """Give every state dict its ``exp_avg``/``exp_avg_sq``, laid out like the parameters: each run of
        parameters that lie back to back in memory gets state that lies back to back, starting as many
        elements past a 1 KiB boundary as the run does.  Missing tensors are created as zeros (adam.py:226-228);
        tensors that are there but lie elsewhere (restored from a checkpoint, or assigned to
        ``optimizer.state[p]`` directly) are copied into place once.  State of another dtype, shape or device
        is left alone: the checks of the step name it.  ``fresh_copy``: the tensors in ``states`` belong to
        somebody else (a checkpoint): copy them even where they already lie right."""
        optim_type = self.optim_type
        runs = _adjacent_runs(likes) if self.place_state else [[k] for k in range(len(likes))]
        # All first moments are allocated before the first second moment, so that exp_avg and exp_avg_sq of one
        # parameter do not end up exactly one tensor apart: a model's matrices tend to be powers of two in size
        # (4096 x 4096 halves = 32 MiB), and two streams of one tile a power of two apart fall onto the same DRAM
        # channel and bank at every instant (measured: 2-3 points of bandwidth on such tensors).
        for key in ("exp_avg", "exp_avg_sq"):
            for run in runs:
                run_likes = [likes[k] for k in run]
                total = sum(t.numel() for t in run_likes)
                have = [states[k].get(key) for k in run]
                there = [t for t in have if t is not None]
                if any(t.dtype != optim_type or t.numel() != like.numel() or t.device != like.device
                       for t, like in zip(have, run_likes) if t is not None):
                    for k, like in zip(run, run_likes):  # foreign state: only fill the gaps
                        if states[k].get(key) is None:
                            states[k][key] = self._stream_for(like, like.numel(), optim_type, zero=True).view(like.shape)
                        elif fresh_copy:
                            states[k][key] = states[k][key].clone()
                    continue
                if len(there) == len(have) and not fresh_copy and (not self.place_state or _placed(have, run_likes)):
                    continue
                flat = self._stream_for(run_likes[0], total, optim_type, zero=len(there) < len(have))
                at = 0
                for k, like, old in zip(run, run_likes, have):
                    view = flat[at:at + like.numel()].view(like.shape)
                    if old is not None:
                        view.copy_(old.view(like.shape) if old.is_contiguous() else old.reshape(like.shape))
                    states[k][key] = view
                    at += like.numel()

    def _steady_group(self, gi: int, group: Dict[str, Any]):
        """The cached view of a group whose every parameter took part in the last general walk, or None
        when the parameter list, the state map or the fp32 master copies were replaced or edited since."""
        cache = self.__dict__.get("_group_cache", {}).get(gi)
        if cache is None:
            return None
        params, snapshot, states, masters, outs, device, state_map, version, _ = cache
        if group["params"] is not params or len(params) != len(snapshot) or len(snapshot) == 0:
            return None
        if self.state is not state_map or state_map.version != version:
            return None
        if masters is not None and (self.fp32_param_groups[gi]["params"] is not masters or len(masters) != len(snapshot)):
            return None
        return cache

    def _gather_native(self, gi: int, group: Dict[str, Any], native_mode: int):
        """The steady-state walk in one C++ loop (csrc/tensor_rows.cpp): gradients, state tensors,
        checks, pointers and step counters.  Returns (plan, table_changed, step) or None when the
        helper is not built or anything is out of the ordinary; the general walk (``_gather``) then decides."""
        native = _rows.native
        if native is None:
            return None
        cache = self._steady_group(gi, group)
        if cache is None:
            return None
        params, snapshot, states, masters, outs, device, _, _, n_active = cache
        if device.type != "cuda":
            return None
        plan = self._plan_for(gi, device, native_mode)
        codes = mode_codes(native_mode)
        buf = plan.rows_buffer(n_active)
        status, _, _, step_no = native.gather(params, snapshot, masters, states, None if masters is not None else outs,
                                               (codes[0], codes[1], codes[3]), device.index, buf.ctypes.data)
        if status < 0:
            plan.mark_dirty()
            return None
        return plan, status == native.CHANGED, step_no

    def _plan_for(self, gi: int, device: torch.device, native_mode: int) -> TensorListPlan:
        plan = self._plans.get((gi, device))
        if plan is None:
            plan = self._plans[(gi, device)] = TensorListPlan(native_mode, device)
        return plan

    def _launch_group(self, gi: int, group: Dict[str, Any], native_mode: int, watch_overflow: bool, scale, flags: List[torch.Tensor]) -> None:
        """Walk one parameter group and enqueue its step (adam.py:202-276); the flags to read back are appended to ``flags``."""
        beta1, beta2 = group["betas"]
        bias_correction = 1 if group["bias_correction"] else 0
        ready = self._gather_native(gi, group, native_mode)
        if ready is not None:
            plan, table_changed, step_no = ready
            flag = None
            if watch_overflow:
                flag = self._flag_for(plan.device)
                flags.append(flag)
            plan.step_rows(table_changed, group["lr"], beta1, beta2, group["eps"], scale, self._optim_scale, flag,
                           step_no, self.eps_mode, bias_correction, group["weight_decay"])
            return
        batches, step_no = self._gather(gi, group)
        if not batches:
            # adam.py:256 indexes the first device of an empty dict
            raise IndexError("list index out of range")
        for device, lists in batches.items():
            flag = None
            if watch_overflow:
                flag = self._flag_for(device)
                flags.append(flag)
            self._plan_for(gi, device, native_mode).step(
                lists, group["lr"], beta1, beta2, group["eps"], scale, self._optim_scale, flag, step_no, self.eps_mode,
                bias_correction, group["weight_decay"])

    def step(self, closure: Optional[Callable[[], float]] = None, *, scale: Union[float, torch.Tensor] = 1.0) -> Optional[float]:
        """One optimization step (adam.py:184-297).

        Arguments:
            closure: re-evaluates the model and returns the loss.
            scale: gradients are divided by this inside the kernel (loss scale or clip factor folded
                into the step).  A Python float, or a one-element float32 tensor on the parameters'
                device that the kernel reads when it runs, so that a factor computed on the device
                (``clip_grad_norm_(..., fold="device")``) costs no host synchronisation.
        """
        loss = closure() if closure is not None else None
        # What the native call would refuse is checked before the walk touches a step counter, so that a refused
        # step leaves the optimizer as it was.  (The reference counts first too, adam.py:234, but its native call
        # has no such refusals.)
        if isinstance(scale, torch.Tensor) and (scale.dtype != torch.float32 or scale.numel() != 1 or not scale.is_cuda):
            raise RuntimeError("a tensor scale must be float32 with one element on the parameters' device")
        if torch.cuda.is_current_stream_capturing():
            raise RuntimeError("Adam.step() cannot be captured into a graph: the step size depends on the step count and "
                               "travels by value, so every replay would repeat this step's bias correction")
        self.__dict__.setdefault("_plans", {})  # absent after unpickling
        self.__dict__.setdefault("_flags", {})
        native_mode = _NATIVE_MODE[self.precision]
        if self.__dict__.get("_fp16_copies") is not None:
            native_mode = _cabi.FULL_PRECISION_FP16_COPY
        watch_overflow = self.precision is Precision.PURE_FP16

        for gi, group in enumerate(self.param_groups):
            flags: List[torch.Tensor] = []
            if torch.autograd._profiler_enabled():
                # a named range around the walk and the launch, as OSS puts one around its optimizer step (oss.py:230)
                with torch.autograd.profiler.record_function("fairscale_amd::adam::fused_step"):
                    self._launch_group(gi, group, native_mode, watch_overflow, scale, flags)
            else:
                self._launch_group(gi, group, native_mode, watch_overflow, scale, flags)

            overflowed = self._read_flags(flags) if flags else False  # adam.py:278
            if overflowed:
                self._steps_since_optim_scale_change = 0
                self._optim_scale /= 2
                if self._optim_scale < 1.0:
                    raise RuntimeError("Optimizer state scale < 1. This may mean that gradients are exploding")
                self._zero_all_state()
            else:
                self._steps_since_optim_scale_change += 1

            if self._steps_since_optim_scale_change == self._optim_scale_update_freq:  # adam.py:292-295
                self._steps_since_optim_scale_change = 0
                if self._optim_scale < _MAX_OPTIM_SCALE:
                    self._optim_scale *= 2

        return loss

    def _zero_all_state(self) -> None:
        """m = v = 0 for every parameter of every group (adam.py:285-288): in place where the tensors are
        there (their layout stays), fresh zeros where they are not -- also for parameters that have not had a
        gradient yet, which the reference gives state here as well."""
        stale: List[torch.Tensor] = []
        created = False
        # The parameters of the step that has just run are zeroed through its own table, one launch per group and
        # device: the state tensors the table points at are the ones the step checked and used.
        done = set()
        for gi, group in enumerate(self.param_groups):
            cache = self._steady_group(gi, group)  # None when the list, the state map or the master copies changed since
            if cache is None:
                continue
            states, device = cache[2], cache[5]
            plan = self._plans.get((gi, device))
            active = [st for st in states if st is not None]
            if plan is None or not plan.current() or len(states) != len(group["params"]):
                continue
            # the table must still point at these very tensors (a group that has not stepped yet in this call was
            # gathered a step ago): compare the pointers it was built from with the state tensors of now
            try:
                now = [[st["exp_avg"].data_ptr() for st in active], [st["exp_avg_sq"].data_ptr() for st in active]]
            except KeyError:
                continue
            if not plan.holds_state(now[0], now[1]):
                continue
            plan.zero_state()
            done.update(id(st) for st in active)
        for group in self.param_groups:
            for p in group["params"]:
                state = self.state[p]
                if id(state) in done:
                    continue
                for key in ("exp_avg", "exp_avg_sq"):
                    t = state.get(key)
                    if t is not None and t.dtype == self.optim_type and t.shape == p.shape and t.device == p.device:
                        stale.append(t)
                    else:
                        state[key] = torch.zeros_like(p, dtype=self.optim_type)
                        created = True
        if stale:
            torch._foreach_zero_(stale)
        if created:
            self._group_cache = {}  # the next step walks the list again and lays the new tensors out with the rest
