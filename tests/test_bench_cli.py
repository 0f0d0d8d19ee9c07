"""bench.py contract checks that need no GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode != 0
    assert "one GPU" in p.stderr and p.stdout.strip() == ""


def test_help_names_the_contract_flags():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True,
                       timeout=120)
    assert p.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--config"):
        assert flag in p.stdout
