"""bench.py's command line: one GPU only, and the flags the driver passes are accepted."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1", "--warmup", "0"],
                       capture_output=True, text=True, timeout=300)
    text = r.stdout + r.stderr
    assert "one GPU" in text and "--gpus 2" in text
    assert not text.strip().startswith("{")   # no result line


def test_help_lists_the_contract_flags():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--M"):
        assert flag in r.stdout
