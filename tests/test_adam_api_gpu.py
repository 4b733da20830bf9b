"""GPU tests of ``fairscale_amd.optim.Adam``: the behaviours ``tests/optim/test_adam.py`` of the
reference pins (precision inference, state dtypes, state_dict round trips, optimizer-state-scale
transitions, error types), plus whole trajectories against the oracle's host state machine."""
from __future__ import annotations

import copy
import io

import numpy as np
import pytest
import torch

import _cases as C
from _cases import FULL, MEMEFF, MIXED, PURE16

pytestmark = pytest.mark.gpu


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(1)
    yield


@pytest.fixture(scope="module")
def api(cuda_device):
    from fairscale_amd.optim import Adam, GradScaler, Precision

    return Adam, GradScaler, Precision


def tiny_problem(dtype, device):
    """loss = sum((W x + b)^2) for a 2x1 weight, like the reference's tests."""
    weight = torch.randn(2, 1).to(device=device, dtype=dtype).requires_grad_()
    bias = torch.randn(2).to(device=device, dtype=dtype).requires_grad_()
    x = torch.randn(1).to(device=device, dtype=dtype)
    return weight, bias, x


def closure_for(opt, weight, bias, x):
    def fn():
        opt.zero_grad()
        loss = (weight.mv(x) + bias).pow(2).sum()
        loss.backward()
        return loss

    return fn


def loss_goes_down(opt, weight, bias, x, steps=5):
    repr(opt)
    fn = closure_for(opt, weight, bias, x)
    first = fn().item()
    for _ in range(steps):
        opt.step(fn)
    return fn().item() < first


def state_dtypes(opt, params):
    return {opt.state[p][k].dtype for p in params for k in ("exp_avg", "exp_avg_sq")}


# ---- precision modes (test_adam.py:111-195)

def test_full_precision_is_inferred_from_fp32_parameters(api, cuda_device):
    Adam, _, Precision = api
    w, b, x = tiny_problem(torch.float32, cuda_device)
    opt = Adam([w, b], lr=1e-3)
    assert opt.precision is Precision.FULL_PRECISION and opt.optim_type == torch.float32
    assert loss_goes_down(opt, w, b, x)
    assert not opt.fp32_param_groups and not opt.mixed_precision
    assert state_dtypes(opt, [w, b]) == {torch.float32}
    assert w.dtype == torch.float32


def test_mixed_precision_is_inferred_from_fp16_parameters(api, cuda_device):
    Adam, _, Precision = api
    w, b, x = tiny_problem(torch.float16, cuda_device)
    opt = Adam([w, b], lr=1e-3)
    assert opt.precision is Precision.MIXED_PRECISION and opt.mixed_precision
    assert loss_goes_down(opt, w, b, x)
    assert len(opt.fp32_param_groups) == len(opt.param_groups) == 1
    for master, half in zip(opt.fp32_param_groups[0]["params"], opt.param_groups[0]["params"]):
        assert master.dtype == torch.float32 and half.dtype == torch.float16
        assert (master.detach() - half.detach().float()).abs().max().item() < 1e-3
        assert torch.equal(master.detach().half(), half.detach())  # the copy-out is half(master), exactly
    assert state_dtypes(opt, [w, b]) == {torch.float32}


def test_memory_efficient_keeps_fp16_params_and_fp32_state(api, cuda_device):
    Adam, _, Precision = api
    w, b, x = tiny_problem(torch.float16, cuda_device)
    opt = Adam([w, b], lr=1e-3, precision=Precision.MEMORY_EFFICIENT_MIXED_PRECISION)
    assert loss_goes_down(opt, w, b, x)
    assert w.dtype == torch.float16 and not opt.fp32_param_groups
    assert state_dtypes(opt, [w, b]) == {torch.float32}


def test_pure_fp16_keeps_everything_in_fp16(api, cuda_device):
    Adam, _, Precision = api
    w, b, x = tiny_problem(torch.float16, cuda_device)
    opt = Adam([w, b], lr=1e-3, precision=Precision.PURE_FP16)
    assert opt.optim_type == torch.float16 and opt._optim_scale == 2.0 ** 16
    assert loss_goes_down(opt, w, b, x)
    assert w.dtype == torch.float16 and not opt.fp32_param_groups
    assert state_dtypes(opt, [w, b]) == {torch.float16}


def test_properties_and_defaults(api, cuda_device):
    Adam, _, _ = api
    w, b, _ = tiny_problem(torch.float32, cuda_device)
    opt = Adam([w, b])
    assert opt.supports_memory_efficient_fp16 is True and opt._step_supports_amp_scaling is False
    assert opt.defaults == {"lr": 1e-3, "bias_correction": True, "betas": (0.9, 0.999), "eps": 1e-8, "weight_decay": 0.0, "max_grad_norm": 0.0}
    assert opt.eps_mode == 1 and Adam([w, b], eps_inside_sqrt=True).eps_mode == 0
    assert opt._optim_scale == 1.0 and opt._optim_scale_update_freq == 2000 and opt._steps_since_optim_scale_change == 0
    assert opt._overflow_buf.dtype == torch.int32 and opt._overflow_buf.is_cuda


def test_works_with_grad_scaler(api, cuda_device):  # test_adam.py:242-259
    Adam, GradScaler, Precision = api
    w, b, x = tiny_problem(torch.float16, cuda_device)
    opt = Adam([w, b], lr=1e-3, precision=Precision.PURE_FP16)
    scaler = GradScaler()
    first = None
    for i in range(5):
        opt.zero_grad()
        loss = (w.mv(x) + b).pow(2).sum()
        if i == 0:
            first = loss.item()
        scaler.scale(loss).backward()
        scaler.step(opt)
        scaler.update()
    assert loss.item() < first


# ---- state_dict (test_adam.py:64-103, 262-305)

@pytest.mark.parametrize("precision_name", ["FULL_PRECISION", "PURE_FP16", "MIXED_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION"])
def test_state_dict_round_trip_keeps_lock_step(api, cuda_device, precision_name):
    """Save after 5 steps, load into a fresh optimizer on cloned weights: m and v are equal and five
    more steps side by side stay bitwise equal.  The two mixed modes are expected failures in the
    reference (its load casts fp32 state through fp16); here the state is restored exactly."""
    Adam, _, Precision = api
    precision = getattr(Precision, precision_name)
    dtype = torch.float32 if precision is Precision.FULL_PRECISION else torch.float16
    w, b, x = tiny_problem(dtype, cuda_device)
    opt = Adam([w, b], lr=1e-3, precision=precision)
    fn = closure_for(opt, w, b, x)
    for _ in range(5):
        opt.step(fn)
    w2 = w.data.clone().requires_grad_()
    b2 = b.data.clone().requires_grad_()
    opt2 = Adam([w2, b2], lr=1e-3, precision=precision)
    # through a file, with the loader that executes nothing: tensors, ints, floats and lists only
    buffer = io.BytesIO()
    torch.save(opt.state_dict(), buffer)
    buffer.seek(0)
    sd = torch.load(buffer, weights_only=True)
    assert sd["optim_scale"] == opt._optim_scale
    assert set(sd) == {"state", "param_groups", "optim_scale"}
    assert set(sd["state"][0]) == {"step", "exp_avg", "exp_avg_sq"}  # the reference's keys (adam.py:223-228)
    opt2.load_state_dict(sd)
    for p, q in ((w, w2), (b, b2)):
        for key in ("exp_avg", "exp_avg_sq"):
            assert opt2.state[q][key].dtype == opt.optim_type
            assert torch.equal(opt.state[p][key], opt2.state[q][key])
        assert opt2.state[q]["step"] == opt.state[p]["step"] == 5
    if opt.fp32_param_groups:  # masters are rebuilt from fp16, not saved (test_adam.py:90-95)
        opt2.fp32_param_groups = copy.deepcopy(opt.fp32_param_groups)
    fn2 = closure_for(opt2, w2, b2, x)
    for _ in range(5):
        opt.step(fn)
        opt2.step(fn2)
        assert torch.equal(w, w2) and torch.equal(b, b2)


# ---- optimizer-state scale (test_adam.py:308-337)

def test_optim_scale_grows_after_a_clean_interval(api, cuda_device):
    Adam, _, Precision = api
    w, b, x = tiny_problem(torch.float16, cuda_device)
    opt = Adam([w, b], lr=1e-3, precision=Precision.PURE_FP16)
    opt._optim_scale_update_freq = 1
    opt._optim_scale = 2 ** 15
    closure_for(opt, w, b, x)()
    opt.step()
    assert opt._optim_scale == 2 ** 16
    closure_for(opt, w, b, x)()
    opt.step()
    assert opt._optim_scale == 2 ** 16  # capped


def test_exploding_state_raises_when_scale_drops_below_one(api, cuda_device):
    Adam, _, Precision = api
    w = torch.tensor([[float("inf")]]).half().to(cuda_device).requires_grad_()
    x = torch.tensor([1.0]).half().to(cuda_device).requires_grad_()
    opt = Adam([w], lr=1e-3, precision=Precision.PURE_FP16)
    opt._optim_scale = 1.0
    opt.zero_grad()
    w.mv(x).pow(2).sum().backward()
    with pytest.raises(RuntimeError, match="Optimizer state scale < 1"):
        opt.step()


def test_build_fp32_params_can_be_called_again(api, cuda_device):
    Adam, _, _ = api
    w = torch.randn(10, 5).to(cuda_device).half().requires_grad_()
    b = torch.randn(10).to(cuda_device).half().requires_grad_()
    opt = Adam([w, b], lr=1e-3)
    opt._build_fp32_params([w, b])
    assert len(opt.fp32_param_groups) == 1
    for master, half in zip(opt.fp32_param_groups[0]["params"], [w, b]):
        assert master.dtype == torch.float32 and master.grad is None  # no unused zero gradient (4 B per parameter saved)
        assert torch.equal(master.detach(), half.detach().float())


# ---- constructor errors (test_adam.py:355-406)

def test_constructor_errors(api, cuda_device):
    Adam, _, Precision = api
    w = torch.randn(10, 5, device=cuda_device, requires_grad=True)
    b = torch.randn(10, device=cuda_device, requires_grad=True)
    with pytest.raises(ValueError):
        Adam([w, b], lr=1e-2, betas=(1.0, 0.0))
    with pytest.raises(ValueError):
        Adam([w, b], lr=1e-2, weight_decay=-1)
    with pytest.raises(RuntimeError, match="AMSGrad"):
        Adam([w, b], lr=1e-2, amsgrad=True)
    for precision in (Precision.MIXED_PRECISION, Precision.MEMORY_EFFICIENT_MIXED_PRECISION, Precision.PURE_FP16):
        with pytest.raises(AssertionError):
            Adam([w, b], lr=1e-2, precision=precision)


def test_step_without_any_gradient_raises_index_error(api, cuda_device):
    Adam, _, _ = api
    w, b, _ = tiny_problem(torch.float32, cuda_device)
    with pytest.raises(IndexError):  # adam.py:256 indexes an empty dict's first key
        Adam([w, b]).step()


def test_sparse_gradients_are_refused(api, cuda_device):
    Adam, _, _ = api
    w = torch.randn(4, 3, device=cuda_device, requires_grad=True)
    w.grad = torch.zeros(4, 3, device=cuda_device).to_sparse()
    with pytest.raises(RuntimeError, match="sparse"):
        Adam([w]).step()


# ---- whole trajectories against the oracle's host state machine

MODE_OF = {"FULL_PRECISION": FULL, "MIXED_PRECISION": MIXED, "MEMORY_EFFICIENT_MIXED_PRECISION": MEMEFF, "PURE_FP16": PURE16}


@pytest.mark.parametrize("precision_name", list(MODE_OF))
def test_trajectory_matches_oracle_state_machine(oracle, api, cuda_device, precision_name):
    """8 steps over a ragged list with weight decay, a parameter that never gets a gradient, a
    parameter whose gradient is missing on some steps and (PURE_FP16) an overflow on step 4: params,
    m, v, step counters and the optimizer-state scale must follow the oracle exactly."""
    Adam, _, Precision = api
    mode = MODE_OF[precision_name]
    pd, gd, _ = C.MODE_DTYPES[mode]
    host_dtype = np.float16 if mode != FULL else np.float32
    sizes = [3, 1000, 4097, 70000, 150001]
    rng = np.random.default_rng(80 + mode)
    host = [(rng.standard_normal(n).astype(np.float32) * 0.02).astype(host_dtype) for n in sizes]
    params = [torch.from_numpy(h.copy()).to(cuda_device).requires_grad_() for h in host]
    opt = Adam(params, lr=2e-3, betas=(0.8, 0.99), eps=1e-6, weight_decay=0.02, precision=getattr(Precision, precision_name))
    ref = oracle.OracleAdam([h.copy() for h in host], mode, lr=2e-3, betas=(0.8, 0.99), eps=1e-6, weight_decay=0.02)
    opt._optim_scale_update_freq = ref.optim_scale_update_freq = 3
    for step in range(1, 9):
        grads = []
        for j, n in enumerate(sizes):
            if j == 0 or (j == 2 and step % 3 == 0):
                grads.append(None)  # never / sometimes without a gradient (adam.py:212)
                continue
            g = (rng.standard_normal(n).astype(np.float32) * 1e-3).astype(gd)
            if mode == PURE16 and step == 4 and j == 3:
                g[12345] = np.float16(6e4)
            grads.append(g)
        for p, g in zip(params, grads):
            p.grad = None if g is None else torch.from_numpy(g).to(cuda_device)
        opt.step()
        ref.step(grads)
        assert opt._optim_scale == ref.optim_scale, f"step {step}"
        assert opt._steps_since_optim_scale_change == ref.steps_since_optim_scale_change
        for j, p in enumerate(params):
            assert np.array_equal(p.detach().cpu().numpy().view(np.uint8), ref.params[j].view(np.uint8)), f"step {step} param {j}"
            if ref.state[j].get("step") is not None:
                st = opt.state[p]
                assert st["step"] == ref.state[j]["step"]
                for key in ("exp_avg", "exp_avg_sq"):
                    assert np.array_equal(st[key].cpu().numpy().view(np.uint8), ref.state[j][key].view(np.uint8)), f"step {step} {key}[{j}]"
        if mode == MIXED:
            for j, master in enumerate(opt.fp32_param_groups[0]["params"]):
                assert np.array_equal(master.detach().cpu().numpy(), ref.fp32_params[j])
    if mode == PURE16:
        assert opt._optim_scale < 2.0 ** 16 or ref.optim_scale == 2.0 ** 16  # it backed off at step 4 (and may have regrown)
    never = opt.state[params[0]]  # a parameter that never had a gradient
    if mode == PURE16:  # the overflow of step 4 gave it zero state without a counter, as adam.py:285-288 does
        assert set(never) == {"exp_avg", "exp_avg_sq"}
        assert all(not t.any() and t.dtype == torch.float16 and t.shape == params[0].shape for t in never.values())
    else:
        assert len(never) == 0


@pytest.mark.parametrize("seed", range(10))
def test_random_trajectories_match_the_oracle_state_machine(oracle, api, cuda_device, seed):
    """Drawn trajectories through the optimizer class: precision, list, hyper-parameters, a growth
    interval of a few steps, gradients that go missing, a ``scale`` keyword, and (PURE_FP16) overflows
    planted on drawn steps, so that backoff, zeroing and regrowth interleave.  Parameters, m, v, step
    counters and the scale bookkeeping must follow ``OracleAdam`` bit for bit after every step."""
    import random

    Adam, _, Precision = api
    rng = random.Random(6000 + seed)
    precision_name = rng.choice(list(MODE_OF))
    mode = MODE_OF[precision_name]
    pd, gd, _ = C.MODE_DTYPES[mode]
    host_dtype = np.float16 if mode != FULL else np.float32
    sizes = [rng.choice([1, 5, 255, 256, 513, 4097, 20000, 131072, 200001]) for _ in range(rng.randrange(2, 9))]
    nrng = np.random.default_rng(6100 + seed)
    host = [(nrng.standard_normal(n).astype(np.float32) * 0.02).astype(host_dtype) for n in sizes]
    hyper = dict(lr=rng.choice([1e-3, 1e-2]), betas=rng.choice([(0.9, 0.999), (0.8, 0.99)]), eps=rng.choice([1e-8, 1e-5]),
                 weight_decay=rng.choice([0.0, 0.05]), bias_correction=rng.random() < 0.7, eps_inside_sqrt=rng.random() < 0.5)
    scale = rng.choice([1.0, 64.0]) if mode != FULL else 1.0
    params = [torch.from_numpy(h.copy()).to(cuda_device).requires_grad_() for h in host]
    opt = Adam(params, precision=getattr(Precision, precision_name), **hyper)
    ref = oracle.OracleAdam([h.copy() for h in host], mode, **hyper)
    opt._optim_scale_update_freq = ref.optim_scale_update_freq = rng.choice([2, 3, 5])
    overflow_steps = set(rng.sample(range(2, 13), 3)) if mode == PURE16 else set()
    print(f"seed {seed}: {precision_name}, sizes {sizes}, {hyper}, scale {scale}, overflow on {sorted(overflow_steps)}", flush=True)
    for step in range(1, 13):
        grads = []
        for j, n in enumerate(sizes):
            if step > 1 and rng.random() < 0.1:
                grads.append(None)
                continue
            g = (nrng.standard_normal(n).astype(np.float32) * np.float32(1e-3 * scale)).astype(gd)
            if step in overflow_steps and j == len(sizes) - 1:
                g[rng.randrange(n)] = np.float16(6e4)
            grads.append(g)
        if all(g is None for g in grads):
            grads[0] = (nrng.standard_normal(sizes[0]).astype(np.float32) * np.float32(1e-3 * scale)).astype(gd)
        for p, g in zip(params, grads):
            p.grad = None if g is None else torch.from_numpy(g).to(cuda_device)
        opt.step(scale=scale)
        ref.step(grads, scale=scale)
        assert opt._optim_scale == ref.optim_scale, f"step {step}"
        assert opt._steps_since_optim_scale_change == ref.steps_since_optim_scale_change, f"step {step}"
        for j, p in enumerate(params):
            assert np.array_equal(p.detach().cpu().numpy().view(np.uint8), ref.params[j].view(np.uint8)), f"step {step} param {j}"
            if ref.state[j].get("step") is not None:
                st = opt.state[p]
                assert st["step"] == ref.state[j]["step"], f"step {step} counter {j}"
                for key in ("exp_avg", "exp_avg_sq"):
                    assert np.array_equal(st[key].cpu().numpy().view(np.uint8), ref.state[j][key].view(np.uint8)), f"step {step} {key}[{j}]"
        if mode == MIXED:
            for j, master in enumerate(opt.fp32_param_groups[0]["params"]):
                assert np.array_equal(master.detach().cpu().numpy(), ref.fp32_params[j]), f"step {step} master {j}"


def test_scale_keyword_divides_the_gradients(oracle, api, cuda_device):
    """step(scale=s) on gradients multiplied by s gives the bits of step() on the plain gradients."""
    Adam, _, Precision = api
    rng = np.random.default_rng(90)
    h = (rng.standard_normal(5000).astype(np.float32) * 0.02).astype(np.float16)
    g = (rng.standard_normal(5000).astype(np.float32) * 1e-3).astype(np.float16)
    g = np.where(np.abs(g.astype(np.float32)) < 1e-4, np.float16(1e-3), g)  # keep halves normal at both scales
    outs = []
    for s in (1.0, 1024.0):
        p = torch.from_numpy(h.copy()).to(cuda_device).requires_grad_()
        opt = Adam([p], precision=Precision.MEMORY_EFFICIENT_MIXED_PRECISION)
        p.grad = torch.from_numpy((g.astype(np.float32) * s).astype(np.float16)).to(cuda_device)
        opt.step(scale=s)
        outs.append((p.detach().clone(), opt.state[p]["exp_avg"].clone(), opt.state[p]["exp_avg_sq"].clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)


@pytest.mark.parametrize("precision_name", ["FULL_PRECISION", "MIXED_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION", "PURE_FP16"])
@pytest.mark.parametrize("scale", [64.0, 3.0])
def test_scale_as_a_device_tensor_gives_the_bits_of_a_host_scale(api, cuda_device, precision_name, scale):
    """step(scale=tensor): the kernel reads the value when it runs and divides by it; a power of two or not,
    the results are those of step(scale=float)."""
    Adam, _, Precision = api
    results = []
    for on_device in (False, True):
        params = _random_problem(precision_name, cuda_device, sizes=(10, 3000, 200001), seed=9)
        opt = Adam(params, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name])
        holder = torch.zeros(1, device=cuda_device)
        for step in range(1, 4):
            _set_grads(params, step, seed=9)
            holder.fill_(scale)  # written on the stream just before the step: nothing waits on the host
            opt.step(scale=holder if on_device else scale)
        results.append([p.detach().clone() for p in params] + [opt.state[p][k].clone() for p in params for k in ("exp_avg", "exp_avg_sq")])
    for a, b in zip(*results):
        assert torch.equal(a, b)
    with pytest.raises(RuntimeError, match="float32"):
        opt.step(scale=torch.ones(1, dtype=torch.float64, device=cuda_device))


def test_attached_fp16_copies_follow_the_fp32_parameters(api, cuda_device):
    """attach_fp16_copies: the step leaves half(p) in the attached tensors, parameters and state are those
    of a plain FULL_PRECISION optimizer bit for bit; detaching stops the writes."""
    Adam, _, Precision = api
    torch.manual_seed(7)
    base = [torch.randn(n, device=cuda_device) * 0.02 for n in (10, 3000, 150000)]
    grads = [[torch.randn_like(b) * 1e-3 for b in base] for _ in range(3)]
    plain = [b.clone().requires_grad_() for b in base]
    fused = [b.clone().requires_grad_() for b in base]
    copies = {p: torch.zeros(p.numel(), dtype=torch.float16, device=cuda_device) for p in fused}
    opt_a, opt_b = Adam(plain, weight_decay=0.01), Adam(fused, weight_decay=0.01)
    opt_b.attach_fp16_copies(copies)
    for step_grads in grads:
        for p, q, g in zip(plain, fused, step_grads):
            p.grad, q.grad = g.clone(), g.clone()
        opt_a.step()
        opt_b.step()
        for p, q in zip(plain, fused):
            assert torch.equal(p, q) and torch.equal(copies[q], q.detach().half())
            assert torch.equal(opt_a.state[p]["exp_avg_sq"], opt_b.state[q]["exp_avg_sq"])
    opt_b.attach_fp16_copies(None)
    snapshot = {q: copies[q].clone() for q in fused}
    opt_b.step()
    assert all(torch.equal(copies[q], snapshot[q]) for q in fused)
    w16 = torch.zeros(4, device=cuda_device).half().requires_grad_()
    with pytest.raises(RuntimeError, match="FULL_PRECISION"):
        Adam([w16], precision=Precision.PURE_FP16).attach_fp16_copies({w16: torch.zeros(4, dtype=torch.float16, device=cuda_device)})
    with pytest.raises(RuntimeError, match="float16"):
        opt_b.attach_fp16_copies({fused[0]: torch.zeros(10, device=cuda_device)})


def test_table_is_sent_again_only_when_a_pointer_moves(api, cuda_device):
    Adam, _, _ = api
    params = [torch.randn(n, device=cuda_device).requires_grad_() for n in (10, 3000, 200000)]
    opt = Adam(params)
    grads = [torch.randn_like(p) * 1e-3 for p in params]
    for p, g in zip(params, grads):
        p.grad = g
    for _ in range(3):
        opt.step()
    plan = next(iter(opt._plans.values()))
    info = plan.info()
    assert info["uploads"] == 1 and info["n_tensors"] == 3 and info["n_launches"] == 1 and info["n_vector_tensors"] == 3
    params[1].grad = torch.randn_like(params[1]) * 1e-3  # a fresh gradient tensor: its pointer moves
    opt.step()
    assert plan.info()["uploads"] == 2
    opt.step()
    assert plan.info()["uploads"] == 2


def test_native_call_checks_list_shapes_on_device(cuda_device):
    from fairscale_amd import fused_adam_hip

    mk = lambda *ns: [torch.zeros(n, device=cuda_device) for n in ns]  # noqa: E731
    flag = torch.zeros(1, device=cuda_device)
    call = lambda lists: fused_adam_hip.adam(65536, None, lists, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, flag, 1, 1, 1, 0.0)  # noqa: E731
    with pytest.raises(RuntimeError, match="Size mismatch among tensor lists"):
        call([mk(4, 5), mk(4), mk(4, 5), mk(4, 5)])
    with pytest.raises(RuntimeError, match="Size mismatch"):
        call([mk(4, 5), mk(4, 6), mk(4, 5), mk(4, 5)])
    with pytest.raises(RuntimeError, match="found_inf"):
        fused_adam_hip.adam(65536, None, [mk(4)] * 4, 1e-3, 0.9, 0.999, 1e-8, 1.0, 1.0, torch.zeros(1), 1, 1, 1, 0.0)
    call([mk(4, 5), mk(4, 5), mk(4, 5), mk(4, 5)])  # and a well-formed call goes through
    torch.cuda.synchronize()


# ---- the per-step walk over the parameters: C++ helper and Python walk

def _random_problem(precision_name, device, sizes=(10, 3000, 70001), seed=5):
    gen = torch.Generator().manual_seed(seed)
    dtype = torch.float32 if precision_name == "FULL_PRECISION" else torch.float16
    return [(torch.randn(n, generator=gen) * 0.02).to(device=device, dtype=dtype).requires_grad_() for n in sizes]


def _set_grads(params, step, seed=5):
    gen = torch.Generator().manual_seed(seed * 1000 + step)
    for p in params:
        p.grad = (torch.randn(p.numel(), generator=gen) * 1e-3).to(device=p.device, dtype=p.dtype)


@pytest.mark.parametrize("precision_name", ["FULL_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION", "PURE_FP16", "MIXED_PRECISION"])
def test_parameters_packed_into_a_flat_buffer_step_like_separate_ones(api, cuda_device, precision_name):
    """Parameters (and gradients) that are views packed back to back into one buffer start between cache
    lines.  Their state is allocated the same number of elements past a 1 KiB boundary (modulo 512), so one
    head aligns every stream; the values must be those of the same parameters allocated one by one, and
    saving and loading the state must keep them."""
    Adam, _, Precision = api
    sizes = (9001, 33, 0, 8192, 140003, 20000)  # an empty parameter rides along in the run
    separate = _random_problem(precision_name, cuda_device, sizes)
    dtype = separate[0].dtype
    flat = torch.empty(sum(sizes) + 3, device=cuda_device, dtype=dtype)
    flat_grad = torch.empty_like(flat)
    packed, at = [], 3
    for p in separate:
        view = flat[at:at + p.numel()]
        view.copy_(p.detach())
        packed.append(view.requires_grad_())
        at += p.numel()
    opts = [Adam(ps, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name]) for ps in (separate, packed)]
    for step in range(1, 4):
        _set_grads(separate, step)
        at = 3
        for p, q in zip(separate, packed):
            q.grad = flat_grad[at:at + p.numel()].copy_(p.grad)
            at += p.numel()
        for opt in opts:
            opt.step(scale=2.0)
    # the packed list is ONE run for the native layout (parameters, gradients, state and in MIXED_PRECISION the fp32
    # master copies all lie back to back); the separately allocated one is five
    infos = [next(iter(opt._plans.values())).info() for opt in opts]
    assert 1 < infos[0]["n_runs"] <= len(sizes) and infos[1]["n_runs"] == 1
    assert infos[1]["n_descriptors"] < infos[0]["n_descriptors"]
    for p, q in zip(separate, packed):
        assert torch.equal(p.detach(), q.detach())
        for key in ("exp_avg", "exp_avg_sq"):
            a, b = opts[0].state[p][key], opts[1].state[q][key]
            assert torch.equal(a, b)
            if precision_name != "MIXED_PRECISION" and q.numel() >= 8192 and q.data_ptr() % 128:
                assert (b.data_ptr() // b.element_size() - q.data_ptr() // q.element_size()) % 512 == 0, "state not placed like its parameter"
                assert b.is_contiguous() and b.shape == q.shape
    blob = io.BytesIO()
    torch.save(opts[1].state_dict(), blob)
    blob.seek(0)
    fresh = Adam(packed, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name])
    fresh.load_state_dict(torch.load(blob, weights_only=True))
    for q in packed:
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(fresh.state[q][key], opts[1].state[q][key])


@pytest.mark.parametrize("precision_name", ["FULL_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION", "PURE_FP16", "MIXED_PRECISION"])
def test_state_of_separately_allocated_parameters_shares_their_phase_unless_switched_off(api, cuda_device, precision_name):
    """The allocator hands out 512-byte granules, so a parameter of its own starts on a 1 KiB boundary or half a
    kilobyte past one: its state (and fp32 master copy) starts the same number of elements past a boundary of 512
    elements, so that ONE head puts every stream the optimizer owns on 1 KiB boundaries.  With ``place_state`` off every
    state tensor owns an allocation of exactly its size, as ``zeros_like`` gives it in the reference
    (adam.py:226-228), and a single parameter's state pickles to its own size.  Same values either way."""
    Adam, _, Precision = api
    sizes = (8192, 70001, 9000, 33, 20480, 131072 + 128)
    keep = [torch.empty(128, device=cuda_device) for _ in range(3)]  # shift the allocator's phase between the lists
    a = _random_problem(precision_name, cuda_device, sizes)
    b = [p.detach().clone().requires_grad_() for p in a]
    placed = Adam(a, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name])
    plain = Adam(b, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name])
    plain.place_state = False
    if precision_name == "MIXED_PRECISION":  # the master copies were made by the constructor: make them again, unplaced
        plain._build_fp32_params(b)
    for step in range(1, 4):
        _set_grads(a, step)
        for p, q in zip(a, b):
            q.grad = p.grad.clone()
        placed.step()
        plain.step()
    phase = lambda t: (t.data_ptr() // t.element_size()) % 512  # noqa: E731
    for j, (p, q) in enumerate(zip(a, b)):
        assert torch.equal(p.detach(), q.detach())
        like = placed.fp32_param_groups[0]["params"][j] if precision_name == "MIXED_PRECISION" else p
        if precision_name == "MIXED_PRECISION" and p.numel() >= 8192:
            assert phase(like) == phase(p)
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(placed.state[p][key], plain.state[q][key])
            if p.numel() >= 8192:
                assert phase(placed.state[p][key]) == phase(like), (j, key)
            own = plain.state[q][key]
            assert own.untyped_storage().nbytes() == own.numel() * own.element_size() and own.storage_offset() == 0
        blob = io.BytesIO()
        torch.save(plain.state[q], blob)
        assert blob.getbuffer().nbytes < 2 * q.numel() * plain.state[q]["exp_avg"].element_size() + 4096
    del keep


# ---- runs: parameters that are back-to-back views of one buffer (oss.py:630-659, param_bucket.py:62-90)

def _packed_problem(precision_name, device, sizes, lead=3, seed=5):
    """The parameters of ``_random_problem`` once separately allocated and once as views packed back to back into a
    flat buffer that starts ``lead`` elements in, with a flat gradient buffer of the same layout."""
    separate = _random_problem(precision_name, device, sizes, seed)
    dtype = separate[0].dtype
    flat = torch.empty(sum(sizes) + lead, device=device, dtype=dtype)
    flat_grad = torch.zeros_like(flat)
    packed, grad_views, at = [], [], lead
    for p in separate:
        view = flat[at:at + p.numel()]
        view.copy_(p.detach())
        packed.append(view.requires_grad_())
        grad_views.append(flat_grad[at:at + p.numel()])
        at += p.numel()
    return separate, packed, grad_views


def _runs(opt):
    return next(iter(opt._plans.values())).info()["n_runs"]


ALL_PRECISIONS = ["FULL_PRECISION", "MIXED_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION", "PURE_FP16"]


@pytest.mark.parametrize("precision_name", ALL_PRECISIONS)
def test_a_stream_that_breaks_the_sequence_splits_the_run(api, cuda_device, precision_name):
    """Packed parameters whose gradients are NOT all packed: the gradient of the third parameter lives in an
    allocation of its own, so the list is three runs (before, the odd one, after); a parameter in the middle that
    gets no gradient (frozen) splits its run as well.  Values as for separately allocated parameters throughout."""
    Adam, _, Precision = api
    sizes = (9001, 33, 8192, 140003, 20000, 7)
    separate, packed, grad_views = _packed_problem(precision_name, cuda_device, sizes)
    opts = [Adam(ps, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name]) for ps in (separate, packed)]
    odd = torch.empty(sizes[2], device=cuda_device, dtype=packed[0].dtype)
    for step in range(1, 7):
        _set_grads(separate, step)
        frozen = 4 if step >= 4 else None  # from step 4 on the fifth parameter sits out
        for j, (p, q, gv) in enumerate(zip(separate, packed, grad_views)):
            if j == frozen:
                p.grad = q.grad = None
            else:
                q.grad = (odd if j == 2 else gv).copy_(p.grad)
        for opt in opts:
            opt.step()
        # (separately allocated tensors may merge as well, where the allocator happens to put them back to back)
        assert _runs(opts[0]) <= (len(sizes) if frozen is None else len(sizes) - 1)
        assert _runs(opts[1]) == (3 if frozen is None else 4), step
    for p, q in zip(separate, packed):
        assert torch.equal(p.detach(), q.detach())
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(opts[0].state[p][key], opts[1].state[q][key])


@pytest.mark.parametrize("precision_name", ALL_PRECISIONS)
def test_state_that_does_not_follow_the_parameters_is_put_in_place(api, cuda_device, precision_name):
    """Gradients and parameters packed, the state not: ``optimizer.state[p]`` assigned directly with tensors
    allocated one by one (what ``OSS.load_state_dict`` does, oss.py:453-461).  The step after that lays the state
    out with the parameters again (one copy), the list is one run, and the values go on as if nothing had happened."""
    Adam, _, Precision = api
    sizes = (9001, 33, 8192, 140003, 20000)
    separate, packed, grad_views = _packed_problem(precision_name, cuda_device, sizes)
    opts = [Adam(ps, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name]) for ps in (separate, packed)]

    def both_step(step):
        _set_grads(separate, step)
        for p, q, gv in zip(separate, packed, grad_views):
            q.grad = gv.copy_(p.grad)
        for opt in opts:
            opt.step()

    for step in (1, 2):
        both_step(step)
    assert _runs(opts[1]) == 1
    for q in packed:
        old = opts[1].state[q]
        opts[1].state[q] = {"step": old["step"], "exp_avg": old["exp_avg"].clone(), "exp_avg_sq": old["exp_avg_sq"].clone()}
    strays = [opts[1].state[q]["exp_avg"] for q in packed]
    for step in (3, 4):
        both_step(step)
    assert _runs(opts[1]) == 1
    assert all(opts[1].state[q]["exp_avg"] is not t for q, t in zip(packed, strays))
    for p, q in zip(separate, packed):
        assert torch.equal(p.detach(), q.detach())
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(opts[0].state[p][key], opts[1].state[q][key])


# ---- what the callers' checkpoint flows do to this optimizer (done by hand: the callers themselves are out of scope)

def _copy_to_device(value, device):
    """fairscale.internal.params.recursive_copy_to_device (params.py:29-56) in four lines."""
    if isinstance(value, torch.Tensor):
        return value.to(device)
    if isinstance(value, (list, tuple)):
        return type(value)(_copy_to_device(v, device) for v in value)
    if isinstance(value, dict):
        return {k: _copy_to_device(v, device) for k, v in value.items()}
    return value


def _lock_step(opt_a, params_a, opt_b, params_b, first_step, steps=3, overflow_at=None):
    for step in range(first_step, first_step + steps):
        _set_grads(params_a, step)
        if overflow_at == step:
            params_a[-1].grad[5] = 6e4
        for p, q in zip(params_a, params_b):
            q.grad = p.grad.clone() if q.grad is None or q.grad.data_ptr() == p.grad.data_ptr() else q.grad.copy_(p.grad)
        opt_a.step()
        opt_b.step()
        assert opt_a._optim_scale == opt_b._optim_scale
        for p, q in zip(params_a, params_b):
            assert torch.equal(p.detach(), q.detach()), f"step {step}"
            for key in ("exp_avg", "exp_avg_sq"):
                assert torch.equal(opt_a.state[p][key], opt_b.state[q][key]), f"step {step} {key}"
            assert opt_a.state[p]["step"] == opt_b.state[q]["step"]


def _clone_problem(params, opt, Adam, precision, packed):
    """Parameters with the values ``params`` hold now (packed into one buffer or one by one) and a fresh optimizer;
    in MIXED_PRECISION the fp32 master copies are carried over, as the reference's tests do (test_adam.py:90-95)."""
    if packed:
        flat = torch.empty(sum(p.numel() for p in params) + 3, device=params[0].device, dtype=params[0].dtype)
        flat_grad = torch.zeros_like(flat)
        clones, at = [], 3
        for p in params:
            view = flat[at:at + p.numel()]
            view.copy_(p.detach())
            clones.append(view.requires_grad_())
            clones[-1].grad = flat_grad[at:at + p.numel()]
            at += p.numel()
    else:
        clones = [p.detach().clone().requires_grad_() for p in params]
    fresh = Adam(clones, lr=1e-2, weight_decay=0.01, precision=precision)
    if opt.fp32_param_groups:
        for mine, theirs in zip(fresh.fp32_param_groups[0]["params"], opt.fp32_param_groups[0]["params"]):
            mine.data.copy_(theirs.data)
    return clones, fresh


@pytest.mark.parametrize("precision_name", ALL_PRECISIONS)
@pytest.mark.parametrize("packed", [False, True])
def test_state_moved_to_the_cpu_and_assigned_back_directly_as_oss_does(api, cuda_device, precision_name, packed):
    """``OSS.consolidate_state_dict`` copies ``optim.state_dict()`` to the CPU recursively (oss.py:333-336);
    ``OSS.load_state_dict`` copies each parameter's entry back to the device and assigns it to
    ``optim.state[param]`` directly (oss.py:453-461) -- ``Adam.load_state_dict`` never runs and ``optim_scale``
    is not part of what OSS saves (oss.py:413).  After that the two optimizers must stay in lock step; in
    PURE_FP16 that needs the scale the state was stored with, which the caller has to carry over."""
    Adam, _, Precision = api
    precision = Precision[precision_name]
    sizes = (9001, 33, 8192, 140003)
    params = _random_problem(precision_name, cuda_device, sizes)
    opt = Adam(params, lr=1e-2, weight_decay=0.01, precision=precision)
    opt._optim_scale_update_freq = 2  # PURE_FP16: the scale moves during the test
    for step in range(1, 5):
        _set_grads(params, step)
        if precision_name == "PURE_FP16" and step == 3:
            params[-1].grad[7] = 6e4  # an overflow: the saved scale is not the constructor's
        opt.step()
    saved = _copy_to_device(opt.state_dict(), torch.device("cpu"))
    assert all(t.device.type == "cpu" for st in saved["state"].values() for t in st.values() if isinstance(t, torch.Tensor))
    clones, fresh = _clone_problem(params, opt, Adam, precision, packed)
    fresh._optim_scale_update_freq = 2
    for pid, q in zip(saved["param_groups"][0]["params"], clones):
        fresh.state[q] = _copy_to_device(saved["state"][pid], q.device)
    if precision_name == "PURE_FP16":
        assert saved["optim_scale"] != fresh._optim_scale
    fresh._optim_scale = saved["optim_scale"]
    fresh._steps_since_optim_scale_change = opt._steps_since_optim_scale_change
    _lock_step(opt, params, fresh, clones, first_step=5, steps=4, overflow_at=7 if precision_name == "PURE_FP16" else None)
    if packed:
        assert _runs(fresh) == 1  # the directly assigned state was laid out with the packed parameters


@pytest.mark.parametrize("precision_name", ALL_PRECISIONS)
def test_state_of_a_flat_parameter_cut_into_slices_and_flattened_again_as_fsdp_does(api, cuda_device, precision_name):
    """FSDP's full optimizer state dict holds, per original parameter, the slice of the flat parameter's state
    viewed in that parameter's shape (``_unflatten_optim_state``, fsdp_optim_utils.py:120-200) and ``step`` once;
    loading flattens again with ``torch.cat`` of the reshaped slices (``flatten_optim_state_dict``, :38-52) and
    hands the result to ``optim.load_state_dict``."""
    Adam, _, Precision = api
    precision = Precision[precision_name]
    shapes = [(50, 100), (4000,), (3, 7, 11), (130000,)]
    numels = [int(np.prod(sh)) for sh in shapes]
    flat = _random_problem(precision_name, cuda_device, (sum(numels),))
    opt = Adam(flat, lr=1e-2, weight_decay=0.01, precision=precision)
    for step in range(1, 4):
        _set_grads(flat, step)
        opt.step()
    sd = _copy_to_device(opt.state_dict(), torch.device("cpu"))
    # unflatten: one entry per original parameter
    unflat = {}
    for gid, (n, sh, start) in enumerate(zip(numels, shapes, np.cumsum([0] + numels[:-1]))):
        unflat[gid] = {key: sd["state"][0][key][start:start + n].clone().view(sh) for key in ("exp_avg", "exp_avg_sq")}
        unflat[gid]["step"] = sd["state"][0]["step"]
    assert [tuple(unflat[g]["exp_avg"].shape) for g in unflat] == shapes
    # flatten again
    again = {"state": {0: {key: torch.cat([unflat[g][key].reshape(-1) for g in sorted(unflat)]) for key in ("exp_avg", "exp_avg_sq")}},
             "param_groups": sd["param_groups"], "optim_scale": sd["optim_scale"]}
    again["state"][0]["step"] = unflat[0]["step"]
    clones, fresh = _clone_problem(flat, opt, Adam, precision, packed=False)
    fresh.load_state_dict(again)
    assert fresh.state[clones[0]]["exp_avg"].dtype == opt.optim_type and fresh.state[clones[0]]["exp_avg"].is_cuda
    _lock_step(opt, flat, fresh, clones, first_step=4)


@pytest.mark.parametrize("precision_name", ALL_PRECISIONS)
def test_load_state_dict_lays_the_state_out_with_packed_parameters(api, cuda_device, precision_name):
    """A checkpoint written by an optimizer over separately allocated parameters, loaded by one over packed
    views: the restored state is packed like the parameters (the list is one run from the first step on, without
    a second copy), bit for bit what was saved, and the two stay in lock step."""
    Adam, _, Precision = api
    precision = Precision[precision_name]
    params = _random_problem(precision_name, cuda_device, (9001, 33, 8192, 140003))
    opt = Adam(params, lr=1e-2, weight_decay=0.01, precision=precision)
    for step in range(1, 4):
        _set_grads(params, step)
        opt.step()
    blob = io.BytesIO()
    torch.save(opt.state_dict(), blob)
    blob.seek(0)
    clones, fresh = _clone_problem(params, opt, Adam, precision, packed=True)
    fresh.load_state_dict(torch.load(blob, weights_only=True))
    states = [fresh.state[q]["exp_avg"] for q in clones]
    for a, b in zip(states, states[1:]):
        assert b.data_ptr() == a.data_ptr() + a.numel() * a.element_size()
    _lock_step(opt, params, fresh, clones, first_step=4)
    assert _runs(fresh) == 1
    assert all(fresh.state[q]["exp_avg"] is t for q, t in zip(clones, states)), "the loaded state was copied a second time"


def test_a_table_the_library_refused_is_sent_again(api, cuda_device, monkeypatch):
    """When ``fsadam_plan_set_tensors`` fails after the gradients have moved (out of memory for the table, a HIP
    error), the row buffer already holds the new pointers.  The next step must not take 'nothing changed' for
    'the device table is current': it sends the table again and the results are those of an undisturbed run."""
    from fairscale_amd import _cabi

    Adam, _, _ = api
    a = _random_problem("FULL_PRECISION", cuda_device, sizes=(1000, 70001), seed=21)
    b = [p.detach().clone().requires_grad_() for p in a]
    opt_a, opt_b = Adam(a, lr=1e-2), Adam(b, lr=1e-2)
    for step in (1, 2):
        _set_grads(a, step, seed=21)
        _set_grads(b, step, seed=21)
        opt_a.step()
        opt_b.step()
    plan = next(iter(opt_b._plans.values()))
    assert plan.info()["uploads"] == 2  # _set_grads makes new tensors: the pointers move every step
    L = _cabi.lib()
    real = L.fsadam_plan_set_tensors
    calls = []

    class Once:
        def __call__(self, *args):
            calls.append(1)
            if len(calls) == 1:
                return -3  # FSADAM_ENOMEM, nothing was done
            return real(*args)

    _set_grads(a, 3, seed=21)
    _set_grads(b, 3, seed=21)
    monkeypatch.setattr(L, "fsadam_plan_set_tensors", Once())
    with pytest.raises(_cabi.FsAdamError):
        opt_b.step()
    # The training loop catches the error and steps again with the same gradients (which have not moved this time).
    # The refused step had advanced b's counters (the walk runs before the native call); a is put in the same place.
    for p in a:
        opt_a.state[p]["step"] += 1
    opt_a.step()
    opt_b.step()
    monkeypatch.undo()
    assert len(calls) == 3 and plan.info()["uploads"] == 3  # refused for b, then a, then b again: the table was re-sent
    for step in (4, 5):
        _set_grads(a, step, seed=21)
        _set_grads(b, step, seed=21)
        opt_a.step()
        opt_b.step()
    torch.cuda.synchronize(cuda_device)
    for p, q in zip(a, b):
        assert opt_a.state[p]["step"] == opt_b.state[q]["step"] == 6
        assert torch.equal(p.detach(), q.detach())
        for key in ("exp_avg", "exp_avg_sq"):
            assert torch.equal(opt_a.state[p][key], opt_b.state[q][key])


def test_hyperparameters_left_as_numpy_scalars_or_tensors_are_accepted(api, cuda_device):
    """A scheduler may leave ``np.float32`` or a one-element tensor in ``group["lr"]``; the reference's binding
    converts anything with ``__float__`` (fused_adam_cuda.cpp:4-8), and the result is that of the plain float."""
    Adam, _, _ = api
    outs = []
    for lr, wd in ((1e-2, 0.01), (np.float32(1e-2), np.float64(0.01)), (torch.tensor(1e-2), torch.tensor(0.01, dtype=torch.float64))):
        params = _random_problem("FULL_PRECISION", cuda_device)
        opt = Adam(params, lr=1e-2, weight_decay=0.01)
        opt.param_groups[0]["lr"], opt.param_groups[0]["weight_decay"] = lr, wd
        for step in range(1, 4):
            _set_grads(params, step)
            opt.step()
        outs.append([p.detach().clone() for p in params])
    for other in outs[1:]:
        for a, b in zip(outs[0], other):
            assert torch.equal(a, b)


def test_list_walk_helper_is_loaded():
    from fairscale_amd import _rows

    assert _rows.native is not None, "fairscale_amd/csrc/_tensor_rows*.so is not built"


@pytest.mark.parametrize("precision_name", ["FULL_PRECISION", "MIXED_PRECISION", "MEMORY_EFFICIENT_MIXED_PRECISION", "PURE_FP16"])
def test_helper_and_python_walks_step_identically(api, cuda_device, precision_name, monkeypatch):
    from fairscale_amd import _rows

    Adam, _, Precision = api
    results = []
    for use_helper in (True, False):
        if not use_helper:
            monkeypatch.setattr(_rows, "native", None)
        params = _random_problem(precision_name, cuda_device)
        opt = Adam(params, lr=1e-2, weight_decay=0.01, precision=Precision[precision_name])
        for step in range(1, 6):
            _set_grads(params, step)
            opt.step(scale=2.0)
        results.append(([p.detach().clone() for p in params],
                        [opt.state[p][k].clone() for p in params for k in ("exp_avg", "exp_avg_sq")],
                        [opt.state[p]["step"] for p in params],
                        [m.detach().clone() for g in opt.fp32_param_groups for m in g["params"]]))
    with_helper, without = results
    assert with_helper[2] == without[2] == [5, 5, 5]
    for a, b in zip(with_helper[0] + with_helper[1] + with_helper[3], without[0] + without[1] + without[3]):
        assert torch.equal(a, b)


def test_parameter_list_edited_in_place_is_noticed(api, cuda_device):
    Adam, _, _ = api
    params = _random_problem("FULL_PRECISION", cuda_device)
    opt = Adam(params, lr=1e-2)
    for step in (1, 2, 3):
        _set_grads(params, step)
        opt.step()
    old = params[1]
    old_value = old.detach().clone()
    new = torch.full((3000,), 0.5, device=cuda_device).requires_grad_()
    opt.param_groups[0]["params"][1] = new
    _set_grads(params, 4)
    new.grad = torch.full_like(new, 1e-3)
    opt.step()
    assert torch.equal(old, old_value), "the parameter that left the list must not be stepped"
    assert opt.state[new]["step"] == 1 and opt.state[params[0]]["step"] == 4
    # fresh state (m = 0.1 g, v = 0.001 g^2), but the bias correction of the call is that of the last
    # parameter's counter, 4 (adam.py:272)
    g = 1e-3
    delta = 1e-2 * (1 - 0.999 ** 4) ** 0.5 / (1 - 0.9 ** 4) * (0.1 * g) / ((0.001 * g * g) ** 0.5 + 1e-8)
    assert torch.allclose(new.detach(), torch.full_like(new, 0.5 - delta), rtol=0, atol=1e-6)


def test_replaced_or_missing_state_and_gradients_are_noticed(api, cuda_device):
    Adam, _, _ = api
    params = _random_problem("FULL_PRECISION", cuda_device)
    opt = Adam(params, lr=1e-2)
    for step in (1, 2, 3):
        _set_grads(params, step)
        opt.step()
    opt.state[params[2]] = {}  # dropped state: re-initialised by the next step
    _set_grads(params, 4)
    opt.step()
    assert opt.state[params[2]]["step"] == 1 and opt.state[params[0]]["step"] == 4
    # a parameter without a gradient sits the step out (adam.py:214-215)
    _set_grads(params, 5)
    params[0].grad = None
    before = params[0].detach().clone()
    opt.step()
    assert torch.equal(params[0], before) and opt.state[params[0]]["step"] == 4 and opt.state[params[1]]["step"] == 5
    # and joins again afterwards
    _set_grads(params, 6)
    opt.step()
    assert opt.state[params[0]]["step"] == 5 and not torch.equal(params[0], before)
    # a state tensor replaced under the same key is picked up (pointers are read every step)
    opt.state[params[1]]["exp_avg"] = torch.zeros_like(params[1])
    kept = opt.state[params[1]]["exp_avg"]
    _set_grads(params, 7)
    opt.step()
    assert kept.abs().sum().item() > 0
    # a sparse gradient is refused with the reference's message (adam.py:218)
    params[1].grad = torch.zeros_like(params[1]).to_sparse()
    with pytest.raises(RuntimeError, match="sparse"):
        opt.step()


def test_walk_cost_for_four_thousand_tensors(api, cuda_device):
    """Not a timing assertion against the clock of a shared box: the steady-state step of a long list must
    not re-send its table and must stay well under the general walk."""
    import time

    Adam, _, _ = api
    params = [torch.zeros(16, device=cuda_device).requires_grad_() for _ in range(4096)]
    for p in params:
        p.grad = torch.zeros_like(p)
    opt = Adam(params)
    opt.step()
    opt.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(20):
        opt.step()
    steady = (time.perf_counter() - t0) / 20
    torch.cuda.synchronize()
    assert next(iter(opt._plans.values())).info()["uploads"] == 1
    assert opt.state[params[-1]]["step"] == 22
    print(f"steady-state host time per step, 4096 tensors: {steady * 1e3:.3f} ms")
    assert steady < 0.02  # generous: the Python walk took about 2 ms, the helper about 0.3 ms


def test_added_param_group_steps_with_its_own_hyperparameters(api, cuda_device):
    """``add_param_group`` after construction (the constructor itself takes a flat list, adam.py:90-91):
    each group is one native call with its own lr / betas / weight decay, so two groups in one optimizer
    give the same bits as two optimizers."""
    Adam, _, _ = api
    a = _random_problem("FULL_PRECISION", cuda_device, sizes=(100, 5000), seed=7)
    b = _random_problem("FULL_PRECISION", cuda_device, sizes=(33, 140000), seed=8)
    a2 = [p.detach().clone().requires_grad_() for p in a]
    b2 = [p.detach().clone().requires_grad_() for p in b]
    both = Adam(a, lr=1e-2)
    both.add_param_group({"params": b, "lr": 3e-3, "betas": (0.8, 0.99), "weight_decay": 0.1})
    one, two = Adam(a2, lr=1e-2), Adam(b2, lr=3e-3, betas=(0.8, 0.99), weight_decay=0.1)
    for step in range(1, 5):
        _set_grads(a, step, seed=7)
        _set_grads(b, step, seed=8)
        for src, dst in ((a, a2), (b, b2)):
            for p, q in zip(src, dst):
                q.grad = p.grad.clone()
        both.step()
        one.step()
        two.step()
    assert len(both._plans) == 2
    for p, q in zip(a + b, a2 + b2):
        assert torch.equal(p, q)


def test_a_step_on_a_capturing_stream_is_refused(api, cuda_device):
    """Recorded into a graph the step would replay one step's bias correction for ever: the library says no,
    enqueues nothing, and the optimizer works on afterwards."""
    Adam, _, _ = api
    params = _random_problem("FULL_PRECISION", cuda_device, sizes=(1000, 70001), seed=11)
    opt = Adam(params, lr=1e-2)
    _set_grads(params, 1, seed=11)
    opt.step()
    torch.cuda.synchronize(cuda_device)
    before = [p.detach().clone() for p in params]
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="captured"):  # raised by Adam.step before anything is touched
        with torch.cuda.graph(graph):
            opt.step()
    torch.cuda.synchronize(cuda_device)
    for p, b in zip(params, before):
        assert torch.equal(p, b)
    assert opt.state[params[0]]["step"] == 1  # refused before the walk: no counter moved
    opt.step()
    torch.cuda.synchronize(cuda_device)
    assert not torch.equal(params[1], before[1])


@pytest.mark.parametrize("use_helper", [True, False])
def test_frozen_parameters_do_not_disable_the_steady_state_walk(api, cuda_device, use_helper, monkeypatch):
    """A parameter that never gets a gradient (a frozen layer left in the list) is skipped as in
    adam.py:214-215, and the others still go through the cached walk: one table upload, right results;
    when it starts to get gradients it joins with a fresh state."""
    from fairscale_amd import _rows

    if not use_helper:
        monkeypatch.setattr(_rows, "native", None)
    Adam, _, _ = api
    params = _random_problem("FULL_PRECISION", cuda_device, sizes=(500, 3000, 70001), seed=13)
    twin = [p.detach().clone().requires_grad_() for p in params]
    opt, ref = Adam(params, lr=1e-2), Adam([twin[0], twin[2]], lr=1e-2)
    grads = [torch.randn_like(p) * 1e-3 for p in params]
    frozen = params[1].detach().clone()
    for step in range(1, 6):
        for p, q, g in zip(params, twin, grads):
            p.grad, q.grad = g, g
        params[1].grad = None
        opt.step()
        ref.step()
    assert torch.equal(params[1], frozen) and len(opt.state[params[1]]) == 0
    assert torch.equal(params[0], twin[0]) and torch.equal(params[2], twin[2])
    assert next(iter(opt._plans.values())).info()["uploads"] == 1
    params[1].grad = grads[1]
    opt.step()
    assert opt.state[params[1]]["step"] == 1 and opt.state[params[0]]["step"] == 6
    assert not torch.equal(params[1], frozen)


@pytest.mark.parametrize("seed", range(30))
def test_drawn_list_defects_are_refused_by_both_walks(cuda_device, seed, monkeypatch):
    """One defect planted at a drawn place of a drawn list (stride, dtype, numel, a host tensor, a missing entry,
    a sparse tensor): ``adam`` raises ``RuntimeError`` with the C++ helper and without it, and the same list
    without the defect goes through."""
    import random

    from fairscale_amd import _rows, fused_adam_hip

    rng = random.Random(31000 + seed)
    mode_name = rng.choice(["FULL", "MIXED", "MEMEFF", "PURE16"])
    dts = {"FULL": (torch.float32,) * 4, "MIXED": (torch.float32, torch.float32, torch.float32, torch.float16, torch.float16),
           "MEMEFF": (torch.float16, torch.float32, torch.float32, torch.float16), "PURE16": (torch.float16,) * 4}[mode_name]
    sizes = [rng.choice([1, 5, 300, 4097]) for _ in range(rng.randrange(1, 6))]
    make = lambda: [[torch.zeros(n, dtype=dt, device=cuda_device) for n in sizes] for dt in dts]  # noqa: E731
    flag = torch.zeros(1, device=cuda_device)
    call = lambda lists: fused_adam_hip.adam(0, None, lists, 1e-3, 0.9, 0.999, 1e-8, 1.0, 65536.0 if mode_name == "PURE16" else 1.0,  # noqa: E731
                                             flag, 1, 1, 1, 0.0)
    d, t = rng.randrange(len(dts)), rng.randrange(len(sizes))
    n, dt = sizes[t], dts[d]
    defect = rng.choice(["stride", "dtype", "numel", "host", "length", "sparse"])
    if defect == "stride" and n == 1:
        defect = "numel"  # a one-element tensor is contiguous whatever its stride
    for use_helper in (True, False):
        if not use_helper:
            monkeypatch.setattr(_rows, "native", None)
        call(make())
        lists = make()
        if defect == "stride":
            lists[d][t] = torch.zeros(2 * n, dtype=dt, device=cuda_device)[::2]
        elif defect == "dtype":
            lists[d][t] = torch.zeros(n, dtype=torch.float64, device=cuda_device)
        elif defect == "numel":
            lists[d][t] = torch.zeros(n + 1, dtype=dt, device=cuda_device)
        elif defect == "host":
            lists[d][t] = torch.zeros(n, dtype=dt)
        elif defect == "length":
            lists[d] = lists[d][:-1] if d > 0 else lists[d] + [torch.zeros(3, dtype=dt, device=cuda_device)]
        else:
            lists[d][t] = torch.zeros(n, dtype=dt, device=cuda_device).to_sparse()
        with pytest.raises((RuntimeError, NotImplementedError)):
            call(lists)
    torch.cuda.synchronize(cuda_device)
