#!/usr/bin/env python3
"""Benchmark of the fused Adam step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the configuration the headline metric is quoted on): a single rank's OSS shard of a
13B model -- one contiguous buffer of 1.63e9 parameters, MEMORY_EFFICIENT_MIXED_PRECISION (fp16
params and grads, fp32 m/v, grads scaled by 1024).  A "step" is one ``Adam.step()`` over that shard
with everything resident in HBM.  Prints ONE JSON line; under "also": the same number of parameters
stepped in the other three dtype combinations (MIXED_PRECISION = fp32 master + fp16 grads + fp16
copy-out, 28 B/param; FULL_PRECISION 28; PURE_FP16 14), the pre-step gradient pass over the shard's
fp16 gradients, and a list of 4096 ragged fp32 tensors (host time and device time per step).

"roofline" prices the dominant kernel against 8 TB/s of HBM: algorithmic bytes per launch (22 B per
parameter in this mode: reads p16,g16,m32,v32, writes p16,m32,v32) over the kernel's average duration
measured with HIP events on the launch stream.  "cpu_baseline" times the same math as in-place torch
CPU ops on the host cores for a bounded sample.
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
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--cpu-numel", type=int, default=1 << 26, help="sample size of the CPU baseline")
    ap.add_argument("--calib-copy-bytes", type=int, default=0,
                    help="first run the library's plain copy kernel over this many bytes three times (a dispatch of known "
                         "traffic, for scaling the profiler's FETCH_SIZE / WRITE_SIZE counters)")
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


def time_steps(torch, opt, scale, steps, warmup):
    """W untimed steps, then K steps between synchronisations; wall time and HIP-event time (events sit
    on torch's current stream, which is the stream the optimizer hands to the library)."""
    for _ in range(warmup):
        opt.step(scale=scale)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        opt.step(scale=scale)
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) / 1e3


def measure_gpu(torch, precision_name, numel, steps, warmup, device):
    from fairscale_amd.optim import Adam, Precision

    p, scale = make_shard(torch, precision_name, numel, device)
    opt = Adam([p], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=0.0, precision=getattr(Precision, precision_name))
    wall, dev_s = time_steps(torch, opt, scale, steps, warmup)
    plan = next(iter(opt._plans.values())).info()
    assert torch.isfinite(p.detach()[:4096].float()).all()
    bpp = BYTES_PER_PARAM[precision_name]
    kernel_s = dev_s / steps  # one launch per step: plan["n_launches"] == 1
    out = {
        "params_per_s": numel * steps / wall,
        "ms_per_step": wall / steps * 1e3,
        "kernel_ms": kernel_s * 1e3,
        "bytes_per_param": bpp,
        "achieved_gbs": numel * bpp / kernel_s / 1e9,
        "plan": {k: plan[k] for k in ("n_launches", "grid", "block", "tile_elems", "n_descriptors", "lds_throttle", "n_vector_tensors")},
    }
    del opt, p
    torch.cuda.empty_cache()
    return out


def measure_ragged(torch, steps, warmup, device, count=4096, seed=3000, packed=False, moving=False):
    """4096 fp32 tensors of log-uniform sizes (numel = max(1, round(2**U(0, 20)))), FULL_PRECISION with weight
    decay and eps inside the square root: the list-handling case.  Host time per step (the calls return
    without waiting), device time per step, and wall time of back-to-back steps.  ``packed``: the
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

    for i in range(warmup):
        one_step(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for i in range(steps):
        one_step(warmup + i)
    e1.record()
    host = time.perf_counter() - t0
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    total = sum(sizes)
    plan = next(iter(opt._plans.values())).info()
    out = {"tensors": count, "numel": total, "host_ms_per_step": host / steps * 1e3, "device_ms_per_step": e0.elapsed_time(e1) / steps,
           "ms_per_step": wall / steps * 1e3, "params_per_s": total * steps / wall, "bytes_per_param": 28,
           "achieved_gbs": total * 28 * steps / wall / 1e9, "frac_of_hbm_peak": total * 28 * steps / wall / 1e9 / HBM_PEAK_GBS,
           "n_launches": plan["n_launches"], "n_descriptors": plan["n_descriptors"], "uploads": plan["uploads"],
           "list_walk": "c++" if _rows.native is not None else "python"}
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
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            grad_pass([g], inv, write_back=write_back)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / steps
        out[name] = {"ms": ms, "bytes_per_param": bpp, "achieved_gbs": numel * bpp / ms / 1e6, "frac_of_hbm_peak": numel * bpp / ms / 1e6 / HBM_PEAK_GBS}
    del g
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

    if args.calib_copy_bytes > 0:
        n = args.calib_copy_bytes // 16 * 16
        src = torch.zeros(n, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        for _ in range(3):
            _cabi.check(_cabi.lib().fsadam_calib_copy(dst.data_ptr(), src.data_ptr(), n, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    main_res = measure_gpu(torch, args.mode, args.numel, args.steps, args.warmup, device)
    also = {}
    if not args.no_also:
        # the other three dtype combinations on the same number of parameters
        for mode in ("MIXED_PRECISION", "FULL_PRECISION", "PURE_FP16", "MEMORY_EFFICIENT_MIXED_PRECISION"):
            if mode == args.mode:
                continue
            r = measure_gpu(torch, mode, args.numel, args.steps, args.warmup, device)
            also[mode] = {"params_per_s": r["params_per_s"], "ms_per_step": r["ms_per_step"], "kernel_ms": r["kernel_ms"],
                          "bytes_per_param": r["bytes_per_param"], "achieved_gbs": r["achieved_gbs"],
                          "frac_of_hbm_peak": r["achieved_gbs"] / HBM_PEAK_GBS}
    if not args.no_also:
        also["grad_pass_fp16"] = measure_grad_pass(torch, args.numel, args.steps, args.warmup, device)
        also["ragged_4096_FULL_PRECISION"] = measure_ragged(torch, args.steps, args.warmup, device)
        also["ragged_4096_packed_views_FULL_PRECISION"] = measure_ragged(torch, args.steps, args.warmup, device, packed=True)
        also["ragged_4096_moving_gradients_FULL_PRECISION"] = measure_ragged(torch, args.steps, args.warmup, device, moving=True)
    cpu = None if args.no_cpu else measure_cpu(torch, args.mode, args.cpu_numel)

    workload = f"flat_shard_{args.numel}_{args.mode}"
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
                   "entry": "fairscale_amd.optim.Adam.step", **main_res["plan"],
                   "options": {k: _cabi.get_option(k) for k in ("lds_throttle", "merge_runs", "align_heads", "mid_tiles")}},
        "roofline": {"bound": "hbm", "achieved": main_res["achieved_gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": main_res["achieved_gbs"] / HBM_PEAK_GBS, "traffic": load_traffic(workload),
                     "kernel": "fsadam_tiles", "kernel_ms": main_res["kernel_ms"], "bytes_per_param": main_res["bytes_per_param"]},
        "cpu_baseline": cpu,
        "also": also,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
