#!/usr/bin/env python3
"""Benchmark of the fused Adam step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the configuration the headline metric is quoted on): a single rank's OSS shard of a
13B model -- one contiguous buffer of 1.63e9 parameters, MEMORY_EFFICIENT_MIXED_PRECISION (fp16
params and grads, fp32 m/v, grads scaled by 1024).  A "step" is one ``Adam.step()`` over that shard
with everything resident in HBM.  Prints ONE JSON line; under "also": the same number of parameters
stepped in the other three dtype combinations (MIXED_PRECISION = fp32 master + fp16 grads + fp16
copy-out, 28 B/param; FULL_PRECISION 28; PURE_FP16 14), the pre-step gradient pass over the shard's
fp16 gradients, a list of 4096 ragged fp32 tensors (host time and device time per step; separately
allocated, packed into flat buffers, with gradients that move every step), and the other benchmark
configurations at their real sizes: "c1_..." (one fp32 tensor of 2^20, 10 steps with fresh gradients, on
the host cores and on the GPU), "c2_..." (the 148-tensor GPT-2-small list, MIXED_PRECISION, gradients
scaled by 65536) and "c5_..." (the 291-tensor Llama-7B list, PURE_FP16 with optimizer-state scaling,
including one step whose gradients overflow the state: flag read-back, scale halved, state zeroed).

"roofline" prices the dominant kernel against 8 TB/s of HBM: algorithmic bytes per launch (22 B per
parameter in this mode: reads p16,g16,m32,v32, writes p16,m32,v32) over the kernel's average duration
measured with HIP events on the launch stream over K back-to-back launches through the plan call of the
C ABI ("kernel_ms_min/median/max": the spread over those launches, one event between every two;
"ms_per_step" and "step_ms_median" are the same steps through ``Adam.step()``, which is what "value" counts).  "achieved" is therefore algorithmic bytes over event time; "traffic" is
NOT measured by this run: it is the HBM byte count rocprofv3's counters gave for this workload at default
options, read from the summary named in "traffic_source" (left out when options were changed).
"cpu_baseline" times the same math as in-place torch CPU ops on the host cores for a bounded sample.

    python bench.py --micro     the microbenchmarks the kernel's shape rests on (see run_micro)
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
if REPO not in sys.path:
    sys.path.insert(0, REPO)

HBM_PEAK_GBS = 8000.0
BYTES_PER_PARAM = {"FULL_PRECISION": 28, "MIXED_PRECISION": 28, "MEMORY_EFFICIENT_MIXED_PRECISION": 22, "PURE_FP16": 14}
SHARD_NUMEL = 1_630_000_000


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--numel", type=int, default=SHARD_NUMEL, help="parameters in the flat shard")
    ap.add_argument("--mode", default="MEMORY_EFFICIENT_MIXED_PRECISION", choices=list(BYTES_PER_PARAM))
    ap.add_argument("--no-also", action="store_true", help="skip the secondary measurements (other dtype combinations, gradient pass, ragged list)")
    ap.add_argument("--also-only", action="append", default=[], metavar="KEY",
                    help="of the secondary measurements run only those whose key under \"also\" starts with KEY (may be repeated)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-numel", type=int, default=1 << 26, help="sample size of the CPU baseline")
    ap.add_argument("--calib-copy-bytes", type=int, default=0,
                    help="first run the microbenchmark library's plain copy kernel over this many bytes three times (a dispatch of "
                         "known traffic, for scaling the profiler's FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--micro", action="store_true", help="run the structure microbenchmarks instead (libfsadam_membench.so, built on demand) and print a table")
    ap.add_argument("--micro-numel", type=int, default=SHARD_NUMEL)
    ap.add_argument("--micro-data", default="random", choices=["random", "zeros"],
                    help="what the microbenchmark's buffers hold and its write-only kernels store (the bandwidth of this part depends on it)")
    ap.add_argument("--lds-sweep", default="", metavar="BYTES,BYTES,...",
                    help="instead of the benchmark: the kernel's rate on --numel parameters in --mode for each of these LDS ballasts "
                         "(library option lds_throttle), one line each")
    ap.add_argument("--opt", action="append", default=[], metavar="NAME=VALUE", help="library tuning option (lds_throttle, merge_runs, align_heads, mid_tiles, ...)")
    return ap.parse_args()


def make_shard(torch, precision_name, numel, device):
    """Flat parameter + gradient of the mode's dtypes, generated on the device (synthetic)."""
    gen = torch.Generator(device=device).manual_seed(4000)
    scale = 1024.0
    if precision_name == "FULL_PRECISION":
        p = torch.empty(numel, device=device, dtype=torch.float32).normal_(0, 0.02, generator=gen)
        g = torch.empty(numel, device=device, dtype=torch.float32).normal_(0, 1e-3, generator=gen)
        scale = 1.0
    else:
        p = torch.empty(numel, device=device, dtype=torch.float16).normal_(0, 0.02, generator=gen)
        g = torch.empty(numel, device=device, dtype=torch.float16).normal_(0, 1e-3 * scale, generator=gen)
    p.requires_grad_()
    p.grad = g
    return p, scale


def spread(values):
    """min / median / max of a list of per-step times."""
    ordered = sorted(values)
    n = len(ordered)
    median = ordered[n // 2] if n % 2 else 0.5 * (ordered[n // 2 - 1] + ordered[n // 2])
    return {"min": ordered[0], "median": median, "max": ordered[-1]}


def time_loop(torch, one_step, steps, warmup):
    """W untimed steps, then K steps between synchronisations.  Returns (wall seconds until the device is idle,
    host seconds until the last call returned, per-step device milliseconds).  The events sit on torch's current
    stream, which is the stream the optimizer hands to the library; one event between every two steps."""
    for i in range(warmup):
        one_step(i)
    torch.cuda.synchronize()
    events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    events[0].record()
    for i in range(steps):
        one_step(warmup + i)
        events[i + 1].record()
    host = time.perf_counter() - t0
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, host, [events[i].elapsed_time(events[i + 1]) for i in range(steps)]


def measure_gpu(torch, precision_name, numel, steps, warmup, device):
    from fairscale_amd.optim import Adam, Precision

    p, scale = make_shard(torch, precision_name, numel, device)
    opt = Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, precision=getattr(Precision, precision_name))
    wall, _, per_step = time_loop(torch, lambda i: opt.step(scale=scale), steps, warmup)
    plan_obj = next(iter(opt._plans.values()))
    plan = plan_obj.info()
    assert torch.isfinite(p.detach()[:4096].float()).all()
    bpp = BYTES_PER_PARAM[precision_name]
    sp = spread(per_step)
    # The kernel on its own: the same launches through the plan call of the C ABI, back to back without the host in
    # between.  In PURE_FP16 Adam.step() reads the overflow flag back after every launch (as the reference does,
    # adam.py:278), which leaves the GPU idle until the host has seen the flag and queued the next step; the other
    # modes never wait, and the two figures agree.
    flag = opt._flags.get(device)
    done = opt.state[p]["step"]
    group = opt.param_groups[0]

    def launch_only(i):
        plan_obj.step_rows(False, group["lr"], group["betas"][0], group["betas"][1], group["eps"], scale, opt._optim_scale, flag,
                           done + 1 + i, opt.eps_mode, 1, group["weight_decay"])

    _, _, raw = time_loop(torch, launch_only, steps, 2)
    kernel_ms = sum(raw) / steps  # one launch per step: plan["n_launches"] == 1
    raw_sp = spread(raw)
    out = {
        "params_per_s": numel * steps / wall,
        "ms_per_step": wall / steps * 1e3,
        "step_ms_min": sp["min"], "step_ms_median": sp["median"], "step_ms_max": sp["max"],
        "kernel_ms": kernel_ms,
        "kernel_ms_min": raw_sp["min"], "kernel_ms_median": raw_sp["median"], "kernel_ms_max": raw_sp["max"],
        "bytes_per_param": bpp,
        "achieved_gbs": numel * bpp / kernel_ms / 1e6,
        "plan": {k: plan[k] for k in ("n_launches", "grid", "block", "tile_elems", "n_descriptors", "lds_throttle", "n_vector_tensors")},
    }
    del opt, p
    torch.cuda.empty_cache()
    return out


def measure_ragged(torch, steps, warmup, device, count=4096, seed=3000, packed=False, moving=False):
    """4096 fp32 tensors of log-uniform sizes (numel = max(1, round(2**U(0, 20)))), FULL_PRECISION with weight
    decay and eps inside the square root: the list-handling case.  Host time per step in the back-to-back loop,
    host time of ``step()`` alone with the device idle (``host_work_ms_per_step``), device time per step, and wall
    time of back-to-back steps.  ``packed``: the
    parameters are views laid back to back into one flat buffer that starts one element in (so nearly every
    tensor starts between cache lines), the gradients likewise.  ``moving``: every step finds the gradients in
    other tensors than the step before (two sets taking turns, as when ``zero_grad(set_to_none=True)`` lets the
    allocator hand out other blocks), so the descriptor table is rebuilt and sent again every step."""
    import random

    from fairscale_amd import _rows
    from fairscale_amd.optim import Adam, Precision

    rng = random.Random(seed)
    sizes = [max(1, round(2 ** rng.uniform(0.0, 20.0))) for _ in range(count)]
    if packed:
        flat = torch.empty(sum(sizes) + 1, device=device).normal_(0, 0.02)
        flat_grad = torch.empty_like(flat).normal_(0, 1e-3)
        params, at = [], 1
        for n in sizes:
            params.append(flat[at:at + n].requires_grad_())
            params[-1].grad = flat_grad[at:at + n]
            at += n
    else:
        params = [torch.empty(n, device=device).normal_(0, 0.02).requires_grad_() for n in sizes]
        for p in params:
            p.grad = torch.empty_like(p).normal_(0, 1e-3)
    opt = Adam(params, lr=1e-3, weight_decay=0.01, eps_inside_sqrt=True, precision=Precision.FULL_PRECISION)
    sets = [[p.grad for p in params], [torch.empty_like(p).normal_(0, 1e-3) for p in params]] if moving else None

    def one_step(i):
        if moving:
            for p, g in zip(params, sets[i % 2]):
                p.grad = g
        opt.step()

    harness_ms = None
    if moving:  # what the loop around the step costs on its own: 4096 assignments to .grad per step
        t0 = time.perf_counter()
        for i in range(steps):
            for p, g in zip(params, sets[i % 2]):
                p.grad = g
        harness_ms = (time.perf_counter() - t0) / steps * 1e3
    wall, host, per_step = time_loop(torch, one_step, steps, warmup)
    # what the host does per step when it never has to wait for the device (in the loop above it runs ahead until the
    # library's ring of descriptor tables is in use and then waits for a step to finish, which is device time)
    host_work = 0.0
    for i in range(steps):
        if moving:
            for p, g in zip(params, sets[i % 2]):
                p.grad = g
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        opt.step()
        host_work += time.perf_counter() - t0
    torch.cuda.synchronize()
    total = sum(sizes)
    plan = next(iter(opt._plans.values())).info()
    sp = spread(per_step)
    out = {"tensors": count, "numel": total, "steps": steps, "host_ms_per_step": host / steps * 1e3, "host_work_ms_per_step": host_work / steps * 1e3,
           "device_ms_per_step": sum(per_step) / steps,
           "device_ms_min": sp["min"], "device_ms_median": sp["median"], "device_ms_max": sp["max"],
           "ms_per_step": wall / steps * 1e3, "params_per_s": total * steps / wall, "bytes_per_param": 28,
           "achieved_gbs": total * 28 * steps / wall / 1e9, "frac_of_hbm_peak": total * 28 * steps / wall / 1e9 / HBM_PEAK_GBS,
           "frac_of_hbm_peak_at_median": total * 28 / sp["median"] / 1e6 / HBM_PEAK_GBS,
           "n_launches": plan["n_launches"], "n_descriptors": plan["n_descriptors"], "n_runs": plan["n_runs"], "uploads": plan["uploads"],
           "list_walk": "c++" if _rows.native is not None else "python"}
    if harness_ms is not None:
        out["harness_ms_per_step"] = harness_ms  # part of host_ms_per_step that is this benchmark's own loop, not the optimizer
    del opt, params, sets
    torch.cuda.empty_cache()
    return out


def measure_grad_pass(torch, numel, steps, warmup, device):
    """The pre-step gradient pass over the same shard's fp16 gradients: norms + overflow check only
    (2 B/param read) and with the unscale written back (2 B read + 2 B written)."""
    from fairscale_amd.grad_pass import grad_pass

    g = torch.empty(numel, device=device, dtype=torch.float16).normal_(0, 1.0)
    out = {}
    for name, write_back, bpp in (("norm_and_check", False, 2), ("unscale_norm_and_check", True, 4)):
        inv = 1.0 / 1024 if not write_back else 1.0 - 2.0 ** -12  # written back every step: keep the values in range
        for _ in range(warmup):
            grad_pass([g], inv, write_back=write_back)
        torch.cuda.synchronize()
        # K passes between two events for the rate (a pass is three launches and takes 0.5-1 ms: an event behind every one
        # would be part of what is timed), then K more with an event behind each for the spread
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            grad_pass([g], inv, write_back=write_back)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        events[0].record()
        for i in range(steps):
            grad_pass([g], inv, write_back=write_back)
            events[i + 1].record()
        torch.cuda.synchronize()
        median = spread([events[i].elapsed_time(events[i + 1]) for i in range(steps)])["median"]
        out[name] = {"ms": ms, "ms_median": median, "bytes_per_param": bpp, "achieved_gbs": numel * bpp / ms / 1e6,
                     "frac_of_hbm_peak": numel * bpp / ms / 1e6 / HBM_PEAK_GBS, "frac_at_median": numel * bpp / median / 1e6 / HBM_PEAK_GBS}
    del g
    torch.cuda.empty_cache()
    return out


def measure_c1(torch, device):
    """Benchmark configuration 1 exactly, on the host cores and on the GPU: ONE fp32 tensor of 2^20 parameters
    ~N(0, 0.02) (seed 1000), m = v = 0, lr 1e-3, betas (0.9, 0.999), eps 1e-8 outside the square root, no weight decay,
    10 steps with fresh gradients ~N(0, 1e-3) (seed 1000 + step), all drawn on the CPU in float32.  The CPU leg is the
    same math as in-place torch CPU ops on all host cores; the GPU leg is ``Adam.step()`` (the working set, 16 MiB, sits
    in the caches: its rate says nothing about HBM).  The two results are compared (they differ by the order of
    torch's CPU loops, so to a tolerance)."""
    from fairscale_amd.optim import Adam, Precision
    from oracle import adam_oracle as O
    from oracle.adam_torch_cpu import step_torch_cpu

    n, steps = 1 << 20, 10
    p0 = torch.randn(n, generator=torch.Generator().manual_seed(1000)) * 0.02
    grads = [torch.randn(n, generator=torch.Generator().manual_seed(1000 + step)) * 1e-3 for step in range(1, steps + 1)]
    kw = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)
    times = []
    for rep in range(3):  # the third repetition is the one reported (threads and pages warm)
        p, m, v = p0.clone(), torch.zeros(n), torch.zeros(n)
        t0 = time.perf_counter()
        for step, g in enumerate(grads, 1):
            step_torch_cpu(O.FULL_PRECISION, p, m, v, g, None, step=step, **kw)
        times.append(time.perf_counter() - t0)
    cpu_s = times[-1]
    q = p0.to(device).requires_grad_()
    dev_grads = [g.to(device) for g in grads]
    opt = Adam([q], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, precision=Precision.FULL_PRECISION)
    torch.cuda.synchronize()
    events = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    events[0].record()
    for i, g in enumerate(dev_grads):
        q.grad = g  # another tensor every step, as after zero_grad(set_to_none=True)
        opt.step()
        events[i + 1].record()
    torch.cuda.synchronize()
    gpu_s = time.perf_counter() - t0
    per_step = [events[i].elapsed_time(events[i + 1]) for i in range(steps)]
    diff = (q.detach().cpu() - p).abs().max().item() / p.abs().max().item()
    assert diff < 1e-6, f"C1: GPU and CPU results differ by {diff}"
    sp = spread(per_step[1:])  # the first step creates the state and the plan
    return {"numel": n, "steps": steps, "cpu": {"params_per_s": n * steps / cpu_s, "ms_per_step": cpu_s / steps * 1e3, "cores": int(torch.get_num_threads()),
                                                 "kind": "port (oracle/adam_torch_cpu.py, in-place torch CPU ops)"},
            "gpu": {"params_per_s": n * steps / gpu_s, "ms_per_step": gpu_s / steps * 1e3, "device_ms_min": sp["min"], "device_ms_median": sp["median"],
                    "device_ms_max": sp["max"], "note": "10 steps from a cold optimizer, wall time; 16 MiB working set, cache-resident"},
            "max_abs_diff_over_max_abs": diff}


def measure_c2(torch, steps, warmup, device):
    """Benchmark configuration 2: the GPT-2-small list (148 tensors, 124 439 808 parameters) in MIXED_PRECISION -- fp32
    master copies, m and v; fp16 gradients pre-scaled by 65536 and the same number passed as ``scale``; fp16 parameters
    written in the same pass -- through ``Adam.step()``.  28 bytes per parameter."""
    from fairscale_amd.optim import Adam, Precision

    shapes = [(50257, 768), (1024, 768)]
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]
    shapes += [(768,), (768,)]
    gen = torch.Generator(device=device).manual_seed(2000)
    params = [torch.empty(sh, device=device, dtype=torch.float16).normal_(0, 0.02, generator=gen).requires_grad_() for sh in shapes]
    for p in params:
        p.grad = torch.empty_like(p).normal_(0, 1e-3 * 65536, generator=gen)
    opt = Adam(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, precision=Precision.MIXED_PRECISION)
    wall, host, per_step = time_loop(torch, lambda i: opt.step(scale=65536.0), steps, warmup)
    total = sum(p.numel() for p in params)
    assert len(params) == 148 and total == 124_439_808
    plan = next(iter(opt._plans.values())).info()
    sp = spread(per_step)
    assert all(torch.isfinite(p.detach()[..., :64].float()).all() for p in params[:3])
    out = {"tensors": 148, "numel": total, "steps": steps, "ms_per_step": wall / steps * 1e3, "host_ms_per_step": host / steps * 1e3,
           "device_ms_min": sp["min"], "device_ms_median": sp["median"], "device_ms_max": sp["max"], "params_per_s": total * steps / wall,
           "bytes_per_param": 28, "achieved_gbs": total * 28 * steps / wall / 1e9, "frac_of_hbm_peak": total * 28 * steps / wall / 1e9 / HBM_PEAK_GBS,
           "frac_of_hbm_peak_at_median": total * 28 / sp["median"] / 1e6 / HBM_PEAK_GBS,
           "n_launches": plan["n_launches"], "n_descriptors": plan["n_descriptors"], "n_runs": plan["n_runs"], "grad_scale": 65536.0,
           "note": "3.5 GB working set"}
    del opt, params
    torch.cuda.empty_cache()
    return out


def measure_c5(torch, steps, warmup, device):
    """Benchmark configuration 5: the Llama-7B list (291 tensors, 6 738 415 616 parameters; 32 layers, hidden 4096, FFN
    11008, vocabulary 32000) in PURE_FP16 -- fp16 parameters, gradients, m and v, optimizer-state scale 2^16 -- through
    ``Adam.step()``, which reads the overflow flag back every step as the reference does.  After the clean steps one step
    runs with 1 gradient element in 10^6 set to 6e4: the stored second moment overflows, the flag comes back raised, the
    scale is halved and all of m and v is zeroed (27 GB); that step is timed on its own and its effects are asserted,
    then one more clean step runs at the halved scale.  14 bytes per parameter."""
    from fairscale_amd.optim import Adam, Precision

    h, f, vocab = 4096, 11008, 32000
    shapes = [(vocab, h)]
    for _ in range(32):
        shapes += [(h, h)] * 4 + [(f, h), (h, f), (f, h), (h,), (h,)]
    shapes += [(h,), (vocab, h)]
    total = sum(a * (b[0] if b else 1) for a, *b in shapes)
    assert len(shapes) == 291 and total == 6_738_415_616
    free, _ = torch.cuda.mem_get_info(device)
    if free < total * 8 + (8 << 30):
        return {"skipped": f"needs {(total * 8 >> 30) + 8} GiB of device memory, {free >> 30} GiB free"}
    gen = torch.Generator(device=device).manual_seed(5000)
    params = [torch.empty(sh, device=device, dtype=torch.float16).normal_(0, 0.02, generator=gen).requires_grad_() for sh in shapes]
    for p in params:
        p.grad = torch.empty_like(p).normal_(0, 1e-3, generator=gen)
    opt = Adam(params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, precision=Precision.PURE_FP16)
    wall, host, per_step = time_loop(torch, lambda i: opt.step(), steps, warmup)
    assert opt._optim_scale == 65536.0 and opt._steps_since_optim_scale_change == steps + warmup
    sp = spread(per_step)
    # one step on its own behind 20 ms of an idle GPU, timed like the two single steps below (wall clock around the call
    # and a synchronisation): what a step costs when the device has to come back from idling, with nothing else changed
    torch.cuda.synchronize()
    time.sleep(0.02)
    t0 = time.perf_counter()
    opt.step()
    torch.cuda.synchronize()
    after_idle_ms = (time.perf_counter() - t0) * 1e3
    # the overflow step
    cpu_gen = torch.Generator().manual_seed(5002)
    saved = []
    for p in params:
        k = p.numel() // 1_000_000
        if k:
            idx = torch.randint(0, p.numel(), (k,), generator=cpu_gen).to(device)
            flat = p.grad.view(-1)
            saved.append((flat, idx, flat[idx].clone()))
            flat[idx] = 6e4
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    opt.step()
    torch.cuda.synchronize()
    overflow_ms = (time.perf_counter() - t0) * 1e3
    assert opt._optim_scale == 32768.0 and opt._steps_since_optim_scale_change == 0, "the overflow was not acted upon"
    zeroed = all(not bool(opt.state[p][key].any()) for p in params for key in ("exp_avg", "exp_avg_sq"))
    assert zeroed, "m and v were not zeroed after the overflow"
    for flat, idx, old in saved:
        flat[idx] = old
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    opt.step()
    torch.cuda.synchronize()
    after_ms = (time.perf_counter() - t0) * 1e3
    assert opt._optim_scale == 32768.0 and opt._steps_since_optim_scale_change == 1
    plan = next(iter(opt._plans.values())).info()
    out = {"tensors": 291, "numel": total, "ms_per_step": wall / steps * 1e3, "host_ms_per_step": host / steps * 1e3,
           "device_ms_min": sp["min"], "device_ms_median": sp["median"], "device_ms_max": sp["max"], "params_per_s": total * steps / wall,
           "bytes_per_param": 14, "achieved_gbs": total * 14 * steps / wall / 1e9, "frac_of_hbm_peak": total * 14 * steps / wall / 1e9 / HBM_PEAK_GBS,
           "frac_of_hbm_peak_at_median": total * 14 / sp["median"] / 1e6 / HBM_PEAK_GBS,
           "n_launches": plan["n_launches"], "n_descriptors": plan["n_descriptors"], "n_runs": plan["n_runs"],
           "overflow_step": {"ms": overflow_ms, "injected": "1 gradient element in 10^6 set to 6e4", "optim_scale_before": 65536.0,
                             "optim_scale_after": opt._optim_scale, "state_zeroed": zeroed,
                             "note": "step + blocking flag read-back + scale halved + m, v of all 291 tensors zeroed in place by one launch (27 GB written)"},
           "clean_step_after_backoff_ms": after_ms, "single_step_after_20ms_idle_ms": after_idle_ms,
           "note": "every step includes the blocking read-back of the overflow flag, as in the reference (adam.py:278)"}
    del opt, params, saved
    torch.cuda.empty_cache()
    return out


def measure_cpu(torch, precision_name, numel, budget_s=15.0):
    """The same math as in-place torch CPU ops on `numel` parameters; stops after ~budget_s."""
    from oracle import adam_oracle as O
    from oracle.adam_torch_cpu import step_torch_cpu

    mode = {"FULL_PRECISION": O.FULL_PRECISION, "MIXED_PRECISION": O.MIXED_PRECISION,
            "MEMORY_EFFICIENT_MIXED_PRECISION": O.MEMORY_EFFICIENT_MIXED_PRECISION, "PURE_FP16": O.PURE_FP16}[precision_name]
    pd = torch.float32 if mode in (O.FULL_PRECISION, O.MIXED_PRECISION) else torch.float16
    gd = torch.float32 if mode == O.FULL_PRECISION else torch.float16
    sd = torch.float16 if mode == O.PURE_FP16 else torch.float32
    gen = torch.Generator().manual_seed(4000)
    scale = 1.0 if mode == O.FULL_PRECISION else 1024.0
    p = (torch.randn(numel, generator=gen) * 0.02).to(pd)
    g = (torch.randn(numel, generator=gen) * (1e-3 * scale)).to(gd)
    m, v = torch.zeros(numel, dtype=sd), torch.zeros(numel, dtype=sd)
    pc = torch.zeros(numel, dtype=torch.float16) if mode == O.MIXED_PRECISION else None
    kw = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, grad_scale=scale, optim_scale=65536.0 if mode == O.PURE_FP16 else 1.0)
    step_torch_cpu(mode, p, m, v, g, pc, step=1, **kw)  # warm-up
    done, t0 = 0, time.perf_counter()
    while True:
        step_torch_cpu(mode, p, m, v, g, pc, step=2 + done, **kw)
        done += 1
        el = time.perf_counter() - t0
        if el > budget_s or done >= 2000:
            break
    return {"value": numel * done / el, "unit": "params/s", "cores": int(torch.get_num_threads()), "kind": "port",
            "sample": f"{done} steps of the same {precision_name} math (in-place torch CPU ops, oracle/adam_torch_cpu.py) on a flat {numel}-parameter buffer, {el:.1f} s"}


# counter summaries under profiles/ that hold "traffic = <bytes> bytes per launch" for a workload
TRAFFIC_SUMMARIES = {"flat_shard_1630000000_MEMORY_EFFICIENT_MIXED_PRECISION": "fsadam_tiles_flat_shard_1p63e9_hbm_counters.txt"}


def load_traffic(workload_key):
    """HBM bytes per launch from the committed counter summary, if there is one for this workload."""
    import re

    name = TRAFFIC_SUMMARIES.get(workload_key)
    if name is None:
        return None
    try:
        with open(os.path.join(REPO, "profiles", name)) as fh:
            found = re.search(r"traffic = (\d+) bytes per launch", fh.read())
    except OSError:
        return None
    return int(found.group(1)) if found else None


def run_lds_sweep(torch, args, device):
    """The kernel's rate on ONE set of tensors (a flat shard of --numel parameters in --mode, state allocated once by the
    optimizer) for each LDS ballast of --lds-sweep: between two values only the plan is made anew, so that where the
    allocator put the tensors does not enter the comparison.  Three series of back-to-back launches per value (K launches
    between two events, K sized to about 100 ms), the best of them printed.  LDS is handed out in granules of 1280 bytes:
    a ballast of B bytes allows floor(128 / ceil(B / 1280)) waves per compute unit."""
    from fairscale_amd import _cabi
    from fairscale_amd.optim import Adam, Precision

    p, scale = make_shard(torch, args.mode, args.numel, device)
    opt = Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, precision=getattr(Precision, args.mode))
    opt.step(scale=scale)
    bpp = BYTES_PER_PARAM[args.mode]
    launches = max(10, min(2000, int(0.1 * 6.7e12 / (args.numel * bpp))))
    group = opt.param_groups[0]
    for lds in (int(x) for x in args.lds_sweep.split(",")):
        _cabi.set_option("lds_throttle", lds)
        opt._plans_invalidate()
        for _ in range(3):
            opt.step(scale=scale)  # the first one makes the plan and sends the table
        plan_obj = next(iter(opt._plans.values()))
        flag = opt._flags.get(device)
        done = opt.state[p]["step"]
        best = None
        for _ in range(3):
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(launches):
                plan_obj.step_rows(False, group["lr"], group["betas"][0], group["betas"][1], group["eps"], scale, opt._optim_scale, flag,
                                   done + 1 + i, opt.eps_mode, 1, group["weight_decay"])
            e1.record()
            torch.cuda.synchronize()
            ms = e0.elapsed_time(e1) / launches
            best = ms if best is None else min(best, ms)
        waves = 128 // -(-lds // 1280) if lds > 0 else 0
        print(f"{args.mode} numel {args.numel:>11d} ballast {lds:6d} B ({waves:2d} waves per CU): {best:9.4f} ms per launch "
              f"= {args.numel * bpp / best / 1e6 / HBM_PEAK_GBS * 100:5.2f} % of the HBM peak", flush=True)


def load_membench():
    """The microbenchmark library (fairscale_amd/csrc/membench.hip), compiled first when it is missing or older than its
    source: nothing in the product loads it, so the ordinary build leaves it out."""
    import ctypes

    from fairscale_amd.csrc import build as csrc_build

    if not csrc_build.membench_is_current():
        print(f"building {csrc_build.MEMBENCH_LIBRARY} ...", file=sys.stderr, flush=True)
        csrc_build.build_membench()
    return ctypes.CDLL(csrc_build.MEMBENCH_LIBRARY)


def run_micro(torch, args, device):
    """The measurements the kernel's shape rests on, from kernels the tree builds (fairscale_amd/csrc/membench.hip):
    one-shot tiles against a grid-stride loop, residency (LDS ballast) sweep, temporal against non-temporal accesses,
    the descriptor read with one scalar load against a descriptor staged in LDS, tiles in an XCD-aware order, reads and
    writes in device-wide phases, the cache-policy bits of loads and stores, and the ceilings of this part for reads only,
    writes only and the step's mix.  Prints one line per variant and one JSON line at the end."""
    import ctypes

    L = load_membench()
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.fsadam_membench_launch.restype = i32
    L.fsadam_membench_launch.argtypes = [i32, vp, vp, vp, vp, i64, i32, i32, vp, vp, vp]
    L.fsadam_membench_table_bytes.restype = i64
    L.fsadam_membench_table_bytes.argtypes = [i64]
    L.fsadam_membench_set_pattern.restype = None
    L.fsadam_membench_set_pattern.argtypes = [i32]
    L.fsadam_membench_set_pattern(1 if args.micro_data == "random" else 0)
    n = args.micro_numel // 4 * 4
    bufs = [torch.zeros(n, device=device, dtype=torch.float32) for _ in range(4)]
    if args.micro_data == "random":  # values like a step's: every mantissa bit in use (the update keeps them bounded)
        for b in bufs:
            b.normal_(0, 1.0)
    table = torch.zeros(L.fsadam_membench_table_bytes(n), device=device, dtype=torch.uint8)
    sink = torch.zeros(1, device=device)
    stream = torch.cuda.current_stream().cuda_stream

    def launch(kind, lds=0, param=0):
        rc = L.fsadam_membench_launch(kind, *(b.data_ptr() for b in bufs), n, lds, param, table.data_ptr(), sink.data_ptr(), stream)
        assert rc == 0, f"membench variant {kind} returned {rc}"

    launch(-1)
    results = []

    def measure(name, kind, bytes_per_elt, lds=0, param=0, iters=10):
        for _ in range(3):
            launch(kind, lds, param)
        torch.cuda.synchronize()
        events = [torch.cuda.Event(enable_timing=True) for _ in range(iters + 1)]
        events[0].record()
        for i in range(iters):
            launch(kind, lds, param)
            events[i + 1].record()
        torch.cuda.synchronize()
        times = [events[i].elapsed_time(events[i + 1]) for i in range(iters)]
        sp = spread(times)
        gbs = n * bytes_per_elt / sp["median"] / 1e6
        results.append({"variant": name, "kind": kind, "lds_bytes": lds, "param": param, "bytes_per_element": bytes_per_elt,
                        "ms_median": sp["median"], "ms_min": sp["min"], "gbs_at_median": gbs, "frac_of_hbm_peak": gbs / HBM_PEAK_GBS})
        print(f"{name:<78s} {sp['median']:8.3f} ms  {gbs:7.0f} GB/s  {gbs / HBM_PEAK_GBS * 100:5.1f} %", flush=True)

    print(f"# {n} elements per stream; GB/s of algorithmic bytes at the median of 10 launches; peak {HBM_PEAK_GBS:.0f} GB/s; data: {args.micro_data}")
    print("# fp32 shape: p, m, v, g read, p, m, v written (28 B/element)")
    for wg in (4, 8, 16):
        measure(f"grid-stride loop, 256 threads, {wg} workgroups per CU, non-temporal", 1, 28, param=wg)
    measure("one-shot tiles (one wave64 each), full residency, non-temporal", 0, 28)
    measure("one-shot tiles, full residency, plain (temporal) loads and stores", 2, 28)
    for lds in (5120, 8192, 10240, 12288, 13312, 16384, 20480, 26624, 32768, 65536):
        measure(f"one-shot tiles, LDS ballast {lds:5d} B (at most {163840 // lds:2d} waves per CU), non-temporal", 0, 28, lds=lds)
    measure("one-shot tiles, ballast 16384 B, plain (temporal) loads and stores", 2, 28, lds=16384)
    measure("table of descriptors, ONE scalar load per wave, ballast 16384 B", 4, 28, lds=16384)
    measure("table of descriptors staged in LDS + barrier, ballast 16384 B (incl. the 64 B staged)", 3, 28, lds=16384 - 64)
    measure("table of descriptors staged in LDS + barrier, no ballast", 3, 28)
    print("# the same two ways to the descriptor with the stores written through (sc1 nt), each over its own range of ballasts")
    for lds in (8960, 11520, 14080, 16640, 19200):
        measure(f"28 B shape, table, ONE scalar load per wave, stores [sc1 nt], ballast {lds:5d} B", 30, 28, lds=lds)
        measure(f"28 B shape, table staged in LDS + barrier, stores [sc1 nt], ballast {lds:5d} B (incl. the 64 B staged)", 31, 28, lds=lds - 64)
    launch(-2)  # the table again, for p and g as fp16 streams
    for lds in (6400, 8960, 10240, 11520, 12800, 14080):
        measure(f"22 B shape, table, ONE scalar load per wave, stores [sc1 nt], ballast {lds:5d} B", 32, 22, lds=lds)
        measure(f"22 B shape, table staged in LDS + barrier, stores [sc1 nt], ballast {lds:5d} B (incl. the 64 B staged)", 33, 22, lds=lds - 64)
    launch(-1)
    measure("reads only, four fp32 streams (16 B/element), ballast 16384 B", 5, 16, lds=16384)
    measure("writes only, three fp32 streams (12 B/element), ballast 16384 B", 6, 12, lds=16384)
    print("# the write side on its own (fp32 streams)")
    for lds in (0, 8192, 12288, 20480, 32768):
        measure(f"writes only, three streams, ballast {lds:5d} B", 6, 12, lds=lds)
    measure("writes only, three streams, plain (temporal) stores, ballast 16384 B", 11, 12, lds=16384)
    measure("writes only, three streams, 4 KiB per wave and stream, ballast 32768 B", 12, 12, lds=32768)
    measure("writes only, ONE stream (a fill), ballast 16384 B", 10, 4, lds=16384)
    measure("writes only, ONE stream (a fill), no ballast", 10, 4)
    for lds in (32768, 53248, 81920):
        measure(f"28 B shape, four vectors per lane: 16 loads, then 12 stores, ballast {lds:5d} B", 13, 28, lds=lds)
    print("# tiles in an XCD-aware order: each of the eight XCDs works through runs of consecutive tiles (1 KiB per stream and tile)")
    for lg in (2, 5, 10, 16):
        measure(f"28 B shape, runs of {1 << lg:5d} tiles per XCD, ballast 16384 B", 14, 28, lds=16384, param=lg)
    for lg in (2, 10):
        measure(f"writes only, three streams, runs of {1 << lg:5d} tiles per XCD, ballast 16384 B", 16, 12, lds=16384, param=lg)
    print("# MEMORY_EFFICIENT shape: p, g fp16 and m, v fp32 read (12 B/element), p, m, v written (10 B/element)")
    measure("reads only (12 B/element), ballast 12288 B", 7, 12, lds=12288)
    measure("writes only (10 B/element), ballast 12288 B", 8, 10, lds=12288)
    measure("reads and writes (22 B/element), ballast 12288 B", 9, 22, lds=12288)
    for lg in (2, 10):
        measure(f"reads and writes (22 B/element), runs of {1 << lg:5d} tiles per XCD, ballast 12288 B", 15, 22, lds=12288, param=lg)
    print("# reads and writes in device-wide phases set by the real-time counter: every wave loads only in the first 12/22 of a period, stores only in the rest")
    for lds, period in ((0, 50), (0, 200), (8192, 50), (8192, 200), (12288, 50), (12288, 200)):
        measure(f"reads and writes (22 B/element), phases of {period / 100:.1f} us, ballast {lds:5d} B", 19, 22, lds=lds, param=period)
    bits = lambda k: " ".join(b for b, m in (("sc0", 1), ("sc1", 2), ("nt", 4)) if k & m) or "none"  # noqa: E731
    print("# the cache-policy bits of the memory instructions (sc0, sc1: the scope an access is coherent at; nt: non-temporal; the compiler's")
    print("# non-temporal builtins, used by every line above, set nt alone).  MEMORY_EFFICIENT shape, ballast 12288 B")
    for k in range(8):
        measure(f"reads and writes (22 B/element), stores [{bits(k)}], loads [nt]", 20, 22, lds=12288, param=k)
    for k in range(8):
        measure(f"reads and writes (22 B/element), loads [{bits(k)}], stores [nt]", 21, 22, lds=12288, param=k)
    print("# stores written through the L2 (sc1 nt), as the Adam kernels issue them")
    for lds in (8192, 10240, 11264, 12288, 13312, 14336, 16384):
        measure(f"reads and writes (22 B/element), stores [sc1 nt], ballast {lds:5d} B", 20, 22, lds=lds, param=6)
    for lds in (12288, 14336, 15360, 16384, 18432, 20480):
        measure(f"28 B shape, stores [sc1 nt], ballast {lds:5d} B", 24, 28, lds=lds, param=6)
    for lds in (0, 12288, 16384, 20480, 24576, 32768):
        measure(f"writes only (10 B/element), stores [nt], ballast {lds:5d} B", 23, 10, lds=lds, param=4)
        measure(f"writes only (10 B/element), stores [sc1 nt], ballast {lds:5d} B", 23, 10, lds=lds, param=6)
    lab = lambda run=0, tiles=0, wide=0: 6 | (run << 4) | (tiles << 8) | (wide << 12)  # noqa: E731
    measure("reads and writes (22 B/element), stores [sc1 nt], two tiles per wave, ballast 20480 B", 26, 22, lds=20480, param=lab(tiles=1))
    measure("reads and writes (22 B/element), stores [sc1 nt], four tiles per wave, ballast 40960 B", 26, 22, lds=40960, param=lab(tiles=2))
    measure("reads and writes (22 B/element), stores [sc1 nt], workgroups of 256 threads, ballast 32768 B", 26, 22, lds=32768, param=lab(wide=1))
    measure("reads and writes (22 B/element), stores [sc1 nt], runs of 4 tiles per XCD, ballast 10240 B", 26, 22, lds=10240, param=lab(run=2))
    measure("reads and writes (22 B/element), stores [sc1 nt], half a tile per wave (8 and 4 bytes per lane), ballast 7168 B", 29, 22, lds=7168)
    by = {r["variant"]: r for r in results}
    r_gbs = by["reads only (12 B/element), ballast 12288 B"]["gbs_at_median"]
    w_gbs = by["writes only (10 B/element), ballast 12288 B"]["gbs_at_median"]
    w_best = max(r["gbs_at_median"] for r in results if r["variant"].startswith("writes only (10 B/element), stores [sc1 nt]"))
    serial = 22.0 / (12.0 / r_gbs + 10.0 / w_gbs)
    serial_best = 22.0 / (12.0 / r_gbs + 10.0 / w_best)
    print(f"# 12 B read at {r_gbs:.0f} GB/s + 10 B written at {w_gbs:.0f} GB/s (stores [nt], same residency), one after the other: {serial:.0f} GB/s = "
          f"{serial / HBM_PEAK_GBS * 100:.1f} % of peak")
    print(f"# 12 B read at {r_gbs:.0f} GB/s + 10 B written at {w_best:.0f} GB/s (stores [sc1 nt], their best residency), one after the other: "
          f"{serial_best:.0f} GB/s = {serial_best / HBM_PEAK_GBS * 100:.1f} % of peak")
    print(json.dumps({"micro": results, "numel": n, "data": args.micro_data, "memeff_mix_ceiling_gbs": serial_best,
                      "memeff_mix_ceiling_nt_stores_gbs": serial}))


def main():
    args = parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU: the Adam step of one rank's shard needs no communication, so "
              f"--gpus {args.gpus} is not supported (every rank would run this same kernel on its own shard).", file=sys.stderr)
        sys.exit(2)
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    from fairscale_amd import _cabi

    for item in args.opt:
        name, value = item.split("=")
        _cabi.set_option(name, int(value))
    device = torch.device("cuda", 0)
    torch.cuda.set_device(device)

    if args.micro:
        run_micro(torch, args, device)
        return
    if args.lds_sweep:
        run_lds_sweep(torch, args, device)
        return
    if args.calib_copy_bytes > 0:
        import ctypes

        M = load_membench()
        M.fsadam_membench_copy.restype = ctypes.c_int
        M.fsadam_membench_copy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        n = args.calib_copy_bytes // 16 * 16
        src = torch.zeros(n, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            rc = M.fsadam_membench_copy(dst.data_ptr(), src.data_ptr(), n, torch.cuda.current_stream().cuda_stream)
            assert rc == 0, f"fsadam_membench_copy returned {rc}"
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    main_res = measure_gpu(torch, args.mode, args.numel, args.steps, args.warmup, device)
    also = {}
    wanted = lambda key: not args.no_also and (not args.also_only or any(key.startswith(k) for k in args.also_only))  # noqa: E731
    # the other three dtype combinations on the same number of parameters
    for mode in ("MIXED_PRECISION", "FULL_PRECISION", "PURE_FP16", "MEMORY_EFFICIENT_MIXED_PRECISION"):
        if mode == args.mode or not wanted(mode):
            continue
        r = measure_gpu(torch, mode, args.numel, args.steps, args.warmup, device)
        also[mode] = {"params_per_s": r["params_per_s"], "ms_per_step": r["ms_per_step"], "step_ms_median": r["step_ms_median"],
                      "kernel_ms": r["kernel_ms"], "kernel_ms_min": r["kernel_ms_min"], "kernel_ms_median": r["kernel_ms_median"],
                      "kernel_ms_max": r["kernel_ms_max"], "bytes_per_param": r["bytes_per_param"], "achieved_gbs": r["achieved_gbs"],
                      "frac_of_hbm_peak": r["achieved_gbs"] / HBM_PEAK_GBS,
                      "frac_of_hbm_peak_through_adam_step": args.numel * r["bytes_per_param"] / r["ms_per_step"] / 1e6 / HBM_PEAK_GBS}
    # steps of 0.5-1.5 ms: at least 100 of them, so that one slow step does not make the wall-clock figure
    short_steps = max(args.steps, 100)
    legs = [("grad_pass_fp16", lambda: measure_grad_pass(torch, args.numel, args.steps, args.warmup, device)),
            ("ragged_4096_FULL_PRECISION", lambda: measure_ragged(torch, short_steps, args.warmup, device)),
            ("ragged_4096_packed_views_FULL_PRECISION", lambda: measure_ragged(torch, short_steps, args.warmup, device, packed=True)),
            ("ragged_4096_moving_gradients_FULL_PRECISION", lambda: measure_ragged(torch, short_steps, args.warmup, device, moving=True)),
            ("c2_gpt2_small_148_tensors_MIXED_PRECISION", lambda: measure_c2(torch, short_steps, args.warmup, device)),
            ("c5_llama7b_291_tensors_PURE_FP16", lambda: measure_c5(torch, min(args.steps, 10), min(args.warmup, 3), device))]
    if not args.no_cpu:
        legs.append(("c1_flat_2pow20_FULL_PRECISION_10_steps", lambda: measure_c1(torch, device)))
    for key, leg in legs:
        if wanted(key):
            also[key] = leg()
    cpu = None if args.no_cpu else measure_cpu(torch, args.mode, args.cpu_numel)

    workload = f"flat_shard_{args.numel}_{args.mode}"
    # every measured configuration in a few numbers each, under a key of its own next to the headline's roofline:
    # ms per step (kernel time for the flat shard, device time per step for the lists), the fraction of the HBM peak that
    # gives over the run, and the fraction at the median step
    frac_of = lambda numel, bpp, ms: numel * bpp / ms / 1e6 / HBM_PEAK_GBS  # noqa: E731
    configs = {workload: {"ms": main_res["kernel_ms"], "frac": frac_of(args.numel, main_res["bytes_per_param"], main_res["kernel_ms"]),
                          "frac_at_median": frac_of(args.numel, main_res["bytes_per_param"], main_res["kernel_ms_median"])}}
    for key, r in also.items():
        if key in BYTES_PER_PARAM:
            configs[f"flat_shard_{args.numel}_{key}"] = {"ms": r["kernel_ms"], "frac": r["frac_of_hbm_peak"],
                                                         "frac_at_median": frac_of(args.numel, r["bytes_per_param"], r["kernel_ms_median"])}
        elif key == "grad_pass_fp16":
            for name, g in r.items():
                configs[f"grad_pass_fp16_{name}_{args.numel}"] = {"ms": g["ms"], "frac": g["frac_of_hbm_peak"], "frac_at_median": g["frac_at_median"]}
        elif key.startswith("c1_"):
            configs[key] = {"ms": r["gpu"]["device_ms_median"], "frac": None, "frac_at_median": None,
                            "cpu_ms": r["cpu"]["ms_per_step"], "note": "cache-resident: no HBM statement"}
        elif "skipped" not in r:
            configs[key] = {"ms": r["ms_per_step"], "frac": r["frac_of_hbm_peak"], "frac_at_median": r["frac_of_hbm_peak_at_median"]}
            if "overflow_step" in r:
                configs[key]["overflow_step_ms"] = r["overflow_step"]["ms"]
                configs[key]["clean_step_after_backoff_ms"] = r["clean_step_after_backoff_ms"]
                configs[key]["single_step_after_20ms_idle_ms"] = r["single_step_after_20ms_idle_ms"]
    # the committed counter summary speaks for default options only
    traffic = load_traffic(workload) if not args.opt else None
    traffic_source = (f"profiles/{TRAFFIC_SUMMARIES[workload]} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this workload at default options; "
                      "not measured by this run)") if traffic is not None else None
    line = {
        "metric": "params updated/sec + HBM GB/s (% of peak), 1.6B-param shard, mixed precision",
        "value": main_res["params_per_s"],
        "unit": "params/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": workload, "numel": args.numel, "precision": args.mode, "tensors": 1,
                   "storage": {"FULL_PRECISION": "p,g,m,v fp32", "MIXED_PRECISION": "p,m,v fp32; g, copy-out fp16",
                               "MEMORY_EFFICIENT_MIXED_PRECISION": "p,g fp16; m,v fp32", "PURE_FP16": "p,g,m,v fp16"}[args.mode], "grad_scale": 1024.0 if args.mode != "FULL_PRECISION" else 1.0,
                   "entry": "fairscale_amd.optim.Adam.step", "library": os.path.relpath(_cabi.library_path(), REPO), "abi": _cabi.ABI_VERSION,
                   **main_res["plan"],
                   "options": {k: _cabi.get_option(k) for k in ("lds_throttle", "merge_runs", "align_heads", "mid_tiles")}},
        "roofline": {"bound": "hbm", "achieved": main_res["achieved_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": main_res["achieved_gbs"] / HBM_PEAK_GBS, "traffic": traffic, "traffic_source": traffic_source,
                     "kernel": "fsadam_tiles", "kernel_ms": main_res["kernel_ms"], "step_ms_median": main_res["step_ms_median"],
                     "kernel_ms_min": main_res["kernel_ms_min"],
                     "kernel_ms_median": main_res["kernel_ms_median"], "kernel_ms_max": main_res["kernel_ms_max"],
                     "frac_at_median": args.numel * main_res["bytes_per_param"] / main_res["kernel_ms_median"] / 1e6 / HBM_PEAK_GBS,
                     "bytes_per_param": main_res["bytes_per_param"], "configs": configs},
        "cpu_baseline": cpu,
        "also": also,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
