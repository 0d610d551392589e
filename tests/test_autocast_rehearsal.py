"""The autocast (fp16) training path, rehearsed on the CPU in a separate
process (tests/autocast_rehearsal.py explains how); the GPU run of the same
path is tests/test_zz_half_layers.py::test_training_step_under_autocast."""
import os
import subprocess
import sys


def test_autocast_training_steps_on_the_emulated_back_end():
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "autocast_rehearsal.py")
    res = subprocess.run([sys.executable, script], capture_output=True, text=True, timeout=900)
    assert res.returncode == 0, res.stdout + res.stderr
    lines = res.stdout.strip().splitlines()
    assert lines[-1] == "ok" and len(lines) == 4, res.stdout
    assert all("torch.float16" in ln for ln in lines[:3])
