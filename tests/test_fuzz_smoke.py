"""A few seconds of tests/fuzz_emulated.py (a fresh seed per day keeps widening
what has been tried; a failure prints the shape)."""
import time

import fuzz_emulated


def test_randomised_differential_run():
    seed = int(time.time() // 86400)
    assert fuzz_emulated.run(seed, 8.0) > 20
