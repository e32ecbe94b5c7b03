"""The measuring command refuses to run without a GPU instead of timing a fallback."""
import subprocess
import sys

import torch

from conftest import ROOT


def test_measure_needs_a_gpu():
    if torch.cuda.is_available():
        return
    r = subprocess.run([sys.executable, "-m", "sonicboom_amd.ops.measure", "product", "--rows", "8"], cwd=ROOT,
                       capture_output=True, text=True)
    assert r.returncode == 2 and "no GPU" in r.stderr
