"""The module-level sweep is a user-facing script: it must import without a GPU and refuse to run."""
import subprocess
import sys
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_perf_sweep_imports_and_needs_a_gpu():
    import torch
    from permutohedral_encoding_amd import perf_sweep
    assert callable(perf_sweep.measure) and callable(perf_sweep.main)
    if torch.cuda.is_available():
        return
    r = subprocess.run([sys.executable, "-m", "permutohedral_encoding_amd.perf_sweep", "--dims", "3", "--iters", "12"],
                       cwd=ROOT, capture_output=True, text=True)
    assert r.returncode != 0 and "no GPU" in (r.stderr + r.stdout)
