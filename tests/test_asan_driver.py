"""Builds tests/emu/emu_check (the kernels compiled as host C++ with
AddressSanitizer, every entry point on exactly sized heap buffers) and runs
its `quick` mode.  Takes several minutes, so it only runs on request:

    EXACT_RUN_ASAN=1 python -m pytest tests/test_asan_driver.py
"""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.skipif(os.environ.get("EXACT_RUN_ASAN") != "1", reason="set EXACT_RUN_ASAN=1 (several minutes)")
def test_every_entry_point_is_clean_under_address_sanitizer():
    build = subprocess.run([sys.executable, os.path.join(HERE, "emu", "build_emu.py"), "--asan"],
                           capture_output=True, text=True, timeout=900)
    assert build.returncode == 0, build.stdout + build.stderr
    exe = build.stdout.strip().splitlines()[-1]
    run = subprocess.run([exe, os.environ.get("EXACT_ASAN_MODE", "quick")], capture_output=True, text=True,
                         timeout=3600, env={**os.environ, "ASAN_OPTIONS": "detect_leaks=0"})
    assert run.returncode == 0 and "all checks passed" in run.stdout, run.stdout[-2000:] + run.stderr[-2000:]
