"""Pins oracle/exact_oracle_half.py against torch's CPU fp16 tensor arithmetic
(every torch op on an fp16 CPU tensor evaluates in fp32 and rounds to fp16, the
behaviour of at::Half's operators that the reference's fp16 kernels rely on)."""
import numpy as np
import pytest
import torch

import exact_oracle as o
import exact_oracle_half as oh

F16, F32 = np.float16, np.float32


def rows(N, G, seed, spread=3.0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((N, G)) * spread).astype(F16)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_scale_matches_torch_half_arithmetic(bits):
    x = torch.from_numpy(rows(300, 40, bits))
    mn, mx = x.min(1).values, x.max(1).values
    want = (2 ** bits - 1) / (mx - mn)              # reciprocal() * int on an fp16 tensor, as ops.py:39 does
    got = oh.compute_scale(mn.float().numpy(), mx.float().numpy(), bits)
    assert want.dtype == torch.float16 and np.array_equal(got.astype(F16).view(np.uint16), want.numpy().view(np.uint16))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_quantised_values_match_torch_half_arithmetic(bits):
    xn = rows(257, 24, 10 + bits)
    xn[3] = xn[3, 0]                                  # constant row
    noise = np.random.default_rng(bits).random(xn.shape, dtype=F32)
    x = torch.from_numpy(xn)
    mn, mx = x.min(1).values, x.max(1).values
    scale = (2 ** bits - 1) / (mx - mn)
    t = (x - mn[:, None]) * scale[:, None]            # two fp16 roundings
    t = t.float() + torch.from_numpy(noise) - 0.5     # Half + float -> float
    q = torch.clamp(torch.nan_to_num(t, nan=0.0), min=0).round().to(torch.int64).numpy()
    packed, sc, m = oh.quantize_activation(xn, bits, noise)
    assert np.array_equal(sc.view(np.uint16), scale.numpy().view(np.uint16)) and np.array_equal(m, mn.numpy())
    # unpack the oracle's bytes with the fp32 oracle's layout code and compare the codes
    wpt = 8 // bits
    N, G = xn.shape
    n_round = N + (wpt - N % wpt) % wpt
    p = packed[:(n_round // wpt) * G].reshape(n_round // wpt, 1, G).astype(np.int64)
    codes = ((p >> (np.arange(wpt) * bits).reshape(1, wpt, 1)) & (2 ** bits - 1)).reshape(n_round, G)[:N]
    keep = q <= 2 ** bits - 1                          # a spill into the next field is not a code of its own
    assert np.array_equal(codes[keep], q[keep]) and keep.mean() > 0.999
    assert packed.size == o.packed_nbytes(N, G, bits) and packed[-1] == 0


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_unpack_matches_torch_half_arithmetic(bits):
    xn = rows(130, 16, 20 + bits)
    noise = np.full(xn.shape, 0.5, F32)
    packed, sc, mn = oh.quantize_activation(xn, bits, noise)
    out = oh.unpack(packed, bits, sc, mn, *xn.shape)
    wpt = 8 // bits
    N, G = xn.shape
    n_round = N + (wpt - N % wpt) % wpt
    p = packed[:(n_round // wpt) * G].reshape(n_round // wpt, 1, G).astype(np.int64)
    codes = ((p >> (np.arange(wpt) * bits).reshape(1, wpt, 1)) & (2 ** bits - 1)).reshape(n_round, G)[:N]
    q = torch.from_numpy(codes).to(torch.float16)
    want = q / torch.from_numpy(sc)[:, None] + torch.from_numpy(mn)[:, None]
    assert out.dtype == F16 and np.array_equal(out.view(np.uint16), want.numpy().view(np.uint16))
    # and the round trip stays within one quantisation step (+ fp16 rounding of the result)
    step = 1.0 / sc.astype(F32)
    err = np.abs(out.astype(F32) - xn.astype(F32))
    ok = np.isfinite(step)
    assert (err[ok] <= (step[ok, None] * 1.0 + np.abs(xn[ok].astype(F32)) * 2e-3 + 1e-3)).all()


def test_overflowing_half_scale_saturates_like_the_conversion():
    """A row whose spread is so small that its reciprocal overflows fp16: the scale is inf, the minimum
    gives 0 * inf = NaN -> code 0, every other element +inf, which __float2int_rn
    (cvt.rni.s32.f32, clamped to the int32 range) turns into INT_MAX; the uint8
    accumulator keeps its low bits shifted by the row's position in the byte."""
    x = np.array([[0.0, 5e-6, 0.0, 1e-5], [1.5e-5, 5e-6, 1.5e-5, 1e-5]], np.float16)      # spreads of 1e-5: 1 / spread > 65504
    for bits, want in ((8, [0, 0xFF, 0, 0xFF, 0xFF, 0, 0xFF, 0xFF]), (2, [0xFC, 0xFF, 0xFC, 0xFF]), (1, [0xFE, 0xFF, 0xFE, 0xFF])):
        packed, scale, mn = oh.quantize_activation(x, bits, np.full(x.shape, 0.25, np.float32))
        assert np.isinf(scale.astype(np.float32)).all()
        assert packed[:-1].tolist() == want and packed[-1] == 0


def test_mask_ops_match_torch_half():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(1000) * 4).astype(F16)
    g = (rng.standard_normal(1000) * 4).astype(F16)
    u = rng.random(1000, dtype=F32)
    xt, gt = torch.from_numpy(x), torch.from_numpy(g)
    y, m = oh.relu_fwd(x)
    assert np.array_equal(y, torch.relu(xt).numpy()) and np.array_equal(oh.relu_bwd(g, m), torch.where(xt > 0, gt, torch.zeros_like(gt)).numpy())
    y, m = oh.leaky_relu_fwd(x, 0.2)
    want = torch.where(xt > 0, xt, (xt.float() * 0.2).half())
    assert np.array_equal(y.view(np.uint16), want.numpy().view(np.uint16))
    keep = torch.from_numpy(u) > 0.3
    pinv = np.float32(1.0 / (1.0 - float(np.float32(0.3))))
    want = (xt.float() * keep.float() * float(pinv)).half()
    y, m = oh.dropout_fwd(x, 0.3, u)
    assert np.array_equal(y.view(np.uint16), want.numpy().view(np.uint16)) and np.array_equal(m, o._pack_bits(keep.numpy()))
    p1m = np.float32(1.0 - float(np.float32(0.3)))
    want = torch.where(keep, (gt.float() / float(p1m)).half(), torch.zeros_like(gt))
    assert np.array_equal(oh.dropout_bwd(g, m, 0.3).view(np.uint16), want.numpy().view(np.uint16))
    y2, m2 = oh.dropout_fwd(x, 0.3, u, relu=True)
    y1, m1 = oh.relu_fwd(x)
    y3, m3 = oh.dropout_fwd(y1, 0.3, u)
    assert np.array_equal(y2.view(np.uint16), y3.view(np.uint16)) and np.array_equal(m2, m1 & m3)


def _once(exact64):
    """fp64 (exact or correctly rounded) result -> fp16 in ONE rounding."""
    with np.errstate(over="ignore"):
        return np.asarray(exact64, np.float64).astype(F16)


def test_dropout_rounds_twice_and_the_layer_test_inputs_tell_the_difference():
    """at::Half arithmetic rounds the fp32 product and then converts it to
    fp16.  A kernel that rounds the exact product once (what a fused
    multiply-and-convert instruction does) differs on inputs whose fp32 result
    is a tie of the fp16 grid.  The inputs of the layer test (seed 0, 100 x 48,
    p = 0.4) must contain such elements, so that test can tell the two apart."""
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((100, 48)) * 3).astype(F16).reshape(-1)
    rng.standard_normal((100, 48))
    u = rng.random((100, 48), dtype=F32).reshape(-1)
    y, _ = oh.dropout_fwd(x, 0.4, u)
    pinv = F32(1.0 / (1.0 - float(F32(0.4))))
    keep = u > F32(0.4)
    once = _once(x.astype(np.float64) * keep * float(pinv))        # 11-bit x 24-bit: exact in fp64
    differ = (y.view(np.uint16) != once.view(np.uint16)) & (y != 0)
    assert differ.sum() == 185
    # and torch's fp16 CPU arithmetic agrees with the oracle on every one of them
    want = (torch.from_numpy(x).float() * torch.from_numpy(keep).float() * float(pinv)).half().numpy()
    assert np.array_equal(y.view(np.uint16), want.view(np.uint16))


def test_every_half_operand_separates_one_rounding_from_two():
    """The exhaustive operand (all finite fp16 values) used by the kernel tests
    contains double-rounding cases for each element-wise fp16 operation -- at
    the constants those tests use (slope 0.1, p = 0.4).  Slope 0.2 and p = 0.3
    have no such case over the whole fp16 range, so passing with them shows
    nothing about the rounding."""
    from gpu_util import all_finite_halves
    x = all_finite_halves()
    ones = np.ones(x.size, F32)
    neg = ~(x > 0)

    def leaky_cases(slope):
        y, _ = oh.leaky_relu_fwd(x, slope)
        return (y[neg].view(np.uint16) != _once(x[neg].astype(np.float64) * float(F32(slope))).view(np.uint16)).sum()

    def dropout_cases(p):
        y, m = oh.dropout_fwd(x, p, ones)
        pinv = F32(1.0 / (1.0 - float(F32(p))))
        p1m = F32(1.0 - float(F32(p)))
        fwd = (y.view(np.uint16) != _once(x.astype(np.float64) * float(pinv)).view(np.uint16)).sum()
        bwd = (oh.dropout_bwd(x, m, p).view(np.uint16) != _once(x.astype(np.float64) / float(p1m)).view(np.uint16)).sum()
        return fwd, bwd

    assert leaky_cases(0.1) > 50 and leaky_cases(0.2) == 0
    fwd, bwd = dropout_cases(0.4)
    assert fwd > 1000 and bwd > 1000
    assert dropout_cases(0.3) == (0, 0)
