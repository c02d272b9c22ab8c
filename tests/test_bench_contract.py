"""The benchmark's command-line contract, checked without a GPU: more than one GPU is refused with a message, a run
without a GPU says so instead of measuring a fallback, and the product sources never reach into the oracle."""
import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=300, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    done = _run("--gpus", "2")
    assert done.returncode != 0
    assert "one GPU" in done.stderr and done.stdout.strip() == ""


def test_without_a_gpu_the_benchmark_says_so():
    import torch
    if torch.cuda.is_available():
        return      # on a GPU box the real run is the driver's business
    done = _run("--steps", "1", "--warmup", "0")
    assert done.returncode != 0 and "needs a GPU" in done.stderr and done.stdout.strip() == ""


def test_only_tests_the_smoke_check_and_the_cpu_baseline_use_the_oracle():
    uses = re.compile(r"^\s*(from|import)\s+oracle\b", re.M)
    for folder, _, files in os.walk(os.path.join(ROOT, "crit_amd")):
        for name in files:
            if name.endswith((".py", ".hip", ".hpp", ".h")):
                text = open(os.path.join(folder, name), errors="replace").read()
                assert not uses.search(text) and "oracle/" not in text, os.path.join(folder, name)
    bench = open(os.path.join(ROOT, "bench.py")).read()
    inside = bench[bench.index("def cpu_baseline"):bench.index("def append_sweep")]
    outside = bench.replace(inside, "")
    assert uses.search(inside) and not uses.search(outside)
