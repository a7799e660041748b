"""bench.py's command-line contract, as far as it can be checked without a GPU: more than one GPU is refused with a
message (this build runs the whole model on one), and the flags the driver passes are accepted."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0
    assert "one gpu" in (r.stderr + r.stdout).lower()
    assert r.stdout.strip() == ""  # no JSON line for a run that did not happen


def test_help_lists_the_contract_flags():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--sweep", "--config4", "--traffic-probe", "--gemm-probe"):
        assert flag in r.stdout
