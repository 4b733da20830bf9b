"""What can be said about bench.py without a GPU: it refuses more than one GPU with a message, its
HBM-traffic figure comes out of the committed counter summary, and its byte counts per parameter are the
ones the update equations imply."""
from __future__ import annotations

import os
import subprocess
import sys

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    proc = subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE, stderr=subprocess.PIPE,
                          text=True, timeout=120)
    assert proc.returncode == 2
    assert "one GPU" in proc.stderr and proc.stdout.strip() == ""


def test_traffic_figure_comes_from_the_counter_summary():
    import bench

    got = bench.load_traffic("flat_shard_1630000000_MEMORY_EFFICIENT_MIXED_PRECISION")
    algorithmic = 22 * 1_630_000_000
    assert isinstance(got, int) and abs(got - algorithmic) < 0.01 * algorithmic  # measured traffic = algorithmic bytes within 1 %
    assert bench.load_traffic("some other workload") is None
    for name in os.listdir(os.path.join(REPO, "profiles")):
        assert name.endswith((".txt", ".md")), f"profiles/ holds text summaries only, found {name}"


def test_bytes_per_parameter_follow_from_the_streams():
    import bench

    # reads p, m, v, g + writes p, m, v (+ the fp16 copy in MIXED_PRECISION); fused_adam_cuda_kernel.cu:77-80,100-101,113-114,120-121,128-129
    want = {"FULL_PRECISION": 4 * 4 + 3 * 4, "MIXED_PRECISION": (4 + 4 + 4 + 2) + (4 + 4 + 4 + 2),
            "MEMORY_EFFICIENT_MIXED_PRECISION": (2 + 4 + 4 + 2) + (2 + 4 + 4), "PURE_FP16": 4 * 2 + 3 * 2}
    assert bench.BYTES_PER_PARAM == want
    assert bench.HBM_PEAK_GBS == 8000.0


def test_spread_is_min_median_max():
    import bench

    assert bench.spread([3.0, 1.0, 2.0]) == {"min": 1.0, "median": 2.0, "max": 3.0}
    assert bench.spread([4.0, 1.0, 2.0, 3.0]) == {"min": 1.0, "median": 2.5, "max": 4.0}


def test_benchmark_configurations_have_the_sizes_the_baseline_names():
    """The lists bench.py builds for configurations 2 and 5 are the ones the parity tests use."""
    import inspect

    import bench
    import _cases as C

    src = inspect.getsource(bench.measure_c2) + inspect.getsource(bench.measure_c5)
    assert "124_439_808" in src and "6_738_415_616" in src and "== 148" in src and "== 291" in src
    assert sum(C.numel(s) for s in C.gpt2_small_shapes()) == 124_439_808 and len(C.gpt2_small_shapes()) == 148
    assert sum(C.numel(s) for s in C.llama7b_shapes()) == 6_738_415_616 and len(C.llama7b_shapes()) == 291


def test_measurement_selectors_are_options_of_the_benchmark(monkeypatch):
    """--also-only picks secondary measurements by the start of their key, --lds-sweep takes a list of ballasts; both are
    what the commands in profiles/ use, so they must stay spelled this way."""
    import bench

    monkeypatch.setattr(sys, "argv", ["bench.py", "--also-only", "grad_pass", "--also-only", "c5_", "--lds-sweep", "8960,12288", "--steps", "3"])
    args = bench.parse_args()
    assert args.also_only == ["grad_pass", "c5_"] and args.lds_sweep == "8960,12288" and args.steps == 3
    for name in os.listdir(os.path.join(REPO, "profiles")):
        text = open(os.path.join(REPO, "profiles", name)).read()
        for flag in ("--also-only", "--lds-sweep", "--micro", "--calib-copy-bytes", "--no-also", "--no-cpu"):
            if flag in text:
                assert flag in open(os.path.join(REPO, "bench.py")).read(), f"profiles/{name} uses {flag}, which bench.py no longer has"
