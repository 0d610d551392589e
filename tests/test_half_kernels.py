"""The fp16 entry points on the SIMT emulator against oracle/exact_oracle_half.py
(bit-exact: packed bytes, fp16 scale / min, fp16 dequantised values, masks)."""
import numpy as np
import pytest

import emu_util as e
import exact_oracle as o
import exact_oracle_half as oh

F16, F32 = np.float16, np.float32
SHAPES = [(1, 1), (5, 3), (37, 25), (64, 32), (100, 76), (33, 40), (129, 100), (203, 256), (61, 602), (16, 1024),
          (19, 520), (8, 8), (300, 128)]


def u16(a):
    return np.ascontiguousarray(a).view(np.uint16)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", SHAPES)
@pytest.mark.parametrize("supplied", [True, False])
def test_pack_and_unpack_f16(N, G, bits, supplied):
    rng = np.random.default_rng(N * 31 + G + bits)
    x = (rng.standard_normal((N, G)) * 3).astype(F16)
    if N > 2:
        x[1] = x[1, 0]                                   # constant row
        x[2] = (rng.standard_normal(G) * 2e-6).astype(F16)   # a spread whose reciprocal overflows fp16: scale = inf (G > 1)
    noise = rng.random((N, G), dtype=F32) if supplied else o.philox_noise_rows(0xFEED, (2 << 32) + 8, N, G)
    packed, sc, mn = e.minmax_pack_f16(x, bits, noise if supplied else None, 0xFEED, (2 << 32) + 8)
    wp, ws, wm = oh.quantize_activation(x, bits, noise)
    assert np.array_equal(packed, wp)
    assert np.array_equal(u16(sc), u16(ws)) and np.array_equal(u16(mn), u16(wm))
    out = e.unpack_f16(packed, bits, sc, mn, N, G)
    assert np.array_equal(u16(out), u16(oh.unpack(wp, bits, ws, wm, N, G)))


def test_pack_f16_limits():
    assert e.minmax_pack_f16(np.zeros((2, 1032), F16), 2, expect_rc=-3) is None     # G > 1024
    assert e.minmax_pack_f16(np.zeros((2, 8), F16), 3, expect_rc=-2) is None
    packed, sc, mn = e.minmax_pack_f16(np.zeros((0, 8), F16), 2)
    assert packed.tolist() == [0]


@pytest.mark.parametrize("n", [1, 3, 4, 7, 33, 257, 2049, 10007])
def test_mask_kernels_f16(n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 4).astype(F16)
    g = (rng.standard_normal(n) * 4).astype(F16)
    u = rng.random(n, dtype=F32)
    y, m = e.relu_fwd_f16(x)
    wy, wm = oh.relu_fwd(x)
    assert np.array_equal(u16(y), u16(wy)) and np.array_equal(m, wm)
    assert np.array_equal(u16(e.mask_bwd_f16("relu", g, m)), u16(oh.relu_bwd(g, wm)))
    y, m = e.leaky_relu_fwd_f16(x, 0.2)
    wy, wm = oh.leaky_relu_fwd(x, 0.2)
    assert np.array_equal(u16(y), u16(wy)) and np.array_equal(m, wm)
    assert np.array_equal(u16(e.mask_bwd_f16("leaky", g, m, 0.2)), u16(oh.leaky_relu_bwd(g, wm, 0.2)))
    for relu in (False, True):
        for noise in (u, None):
            un = u if noise is not None else o.philox_noise_flat(9, 12, n)
            y, m = e.dropout_fwd_f16(x, 0.3, noise, 9, 12, relu=relu)
            wy, wm = oh.dropout_fwd(x, 0.3, un, relu=relu)
            assert np.array_equal(u16(y), u16(wy)) and np.array_equal(m, wm)
            assert np.array_equal(u16(e.mask_bwd_f16("dropout", g, m, 0.3)), u16(oh.dropout_bwd(g, wm, 0.3)))


def test_mask_kernels_f16_round_twice_on_every_operand():
    """All finite fp16 values through the scaling kernels, at constants for which
    rounding once and rounding twice differ (tests/test_oracle_half.py)."""
    from gpu_util import all_finite_halves
    x = all_finite_halves()
    ones = np.ones(x.size, F32)
    y, m = e.leaky_relu_fwd_f16(x, 0.1)
    wy, wm = oh.leaky_relu_fwd(x, 0.1)
    assert np.array_equal(u16(y), u16(wy)) and np.array_equal(m, wm)
    assert np.array_equal(u16(e.mask_bwd_f16("leaky", x, np.zeros_like(m), 0.1)),
                          u16(oh.leaky_relu_bwd(x, np.zeros_like(wm), 0.1)))
    y, m = e.dropout_fwd_f16(x, 0.4, ones, 0, 0)
    wy, wm = oh.dropout_fwd(x, 0.4, ones)
    assert np.array_equal(u16(y), u16(wy)) and np.array_equal(m, wm)
    assert np.array_equal(u16(e.mask_bwd_f16("dropout", x, m, 0.4)), u16(oh.dropout_bwd(x, wm, 0.4)))
