"""bench.py's command line, as far as it can be checked without a GPU: more than one GPU is refused with a message
(this build runs on one GPU), and the workload list is what the documentation names."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused_with_a_message():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode != 0
    assert "ONE GPU" in out.stderr and not out.stdout.strip()


def test_workloads_named_in_the_help():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--help"], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 0
    for w in ("C2", "C3", "C4", "C5", "ENDS", "MIGRATE", "LAYERS", "RAWK", "MFMA_CEILING"):
        assert w in out.stdout
