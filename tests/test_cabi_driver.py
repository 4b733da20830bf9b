"""The C ABI driven from plain C, without torch in the process (tests/cabi_driver/cabi_driver.c).

The program is built beforehand (``__graft_entry__.build()`` or ``make -C tests/cabi_driver``); here it
is only started as a child process.
"""
from __future__ import annotations

import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
DRIVER = os.path.join(HERE, "cabi_driver", "_build", "cabi_driver")


def run_driver():
    assert os.path.exists(DRIVER), "tests/cabi_driver/_build/cabi_driver is not built (make -C tests/cabi_driver)"
    return subprocess.run([DRIVER], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)


def test_driver_links_and_reports_a_missing_gpu_cleanly():
    """Loads libfsadam.so and the HIP runtime outside Python; without a GPU it must say so and exit 2."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present: the GPU test runs the program for real")
    proc = run_driver()
    assert proc.returncode == 2 and "no GPU" in proc.stdout, proc.stdout


@pytest.mark.gpu
def test_every_mode_matches_the_oracle_from_plain_c(cuda_device):
    proc = run_driver()
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout
    assert "all modes bit-identical to the oracle" in proc.stdout
    assert proc.stdout.count(" 0 differ") == 5
    assert proc.stdout.count("ok") >= 3 and "WRONG" not in proc.stdout  # the gradient pass lines
