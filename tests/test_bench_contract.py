"""bench.py's contract where no GPU is: more than one GPU is refused with a message (this build shards nothing), and
without a GPU the benchmark fails loudly - there is no CPU path behind any workload for it to fall back to."""

from __future__ import annotations

import subprocess
import sys

import torch

from .helpers import ROOT


def _bench(*args: str) -> subprocess.CompletedProcess:
    return subprocess.run([sys.executable, "bench.py", *args], cwd=ROOT, capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused():
    r = _bench("--gpus", "2")
    assert r.returncode == 2 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_gpu_no_number():
    if torch.cuda.is_available():
        return  # on a GPU box the benchmark runs; the GPU suite covers it
    for args in (("--steps", "1", "--warmup", "0", "--no-cpu"), ("--workload", "gemv_bf16", "--no-cpu"),
                 ("--workload", "moe_mxfp4", "--no-cpu")):
        r = _bench(*args)
        assert r.returncode != 0 and "no GPU is visible" in r.stderr, args
        assert not any(line.startswith("{") for line in r.stdout.splitlines()), args   # no JSON line: nothing measured
