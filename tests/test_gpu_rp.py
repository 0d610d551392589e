"""GPU parity of the random-projection GEMMs against the oracle within 1e-5
relative, with the projection matrix passed in, on every matrix-core path:
the fp32 instruction, the bf16 instruction on operands split in three (any
matrix), and the bf16 instruction on the signs of a +-c matrix."""
import numpy as np
import pytest
import torch

import exact_oracle as o
from exact_amd import ops
from exact_amd.conf import config
from gpu_util import dev, host_randn

pytestmark = pytest.mark.gpu


def close(got, want, rtol=1e-5):
    scale = np.abs(want).max()
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=rtol, atol=rtol * scale)


def _matrix_on_device(R, path):
    """The projection matrix as the given path wants it: config.matrix_cores
    set, and for "signs" the mark that ops._projection_matrix puts on a +-c
    matrix it drew itself."""
    config.matrix_cores = "fp32" if path == "fp32" else "bf16"
    r = dev(R)
    if path == "signs":
        assert (np.abs(R) == np.abs(R).max()).all()
        r._exact_sign_matrix = True
    return r


PATHS = [("rademacher", "fp32"), ("rademacher", "split"), ("rademacher", "signs"), ("gaussian", "fp32"), ("gaussian", "split")]


@pytest.mark.parametrize("dist,path", PATHS)
@pytest.mark.parametrize("N,D,frac", [(1, 256, 0.125), (31, 256, 0.125), (1000, 256, 0.125), (257, 602, 0.125),
                                      (500, 100, 0.25), (129, 256, 0.25), (64, 128, 0.5), (77, 50, 0.3),
                                      (130, 7, 0.5), (4099, 256, 0.125), (300, 256, 0.49), (333, 256, 0.25),
                                      (70, 1024, 0.125), (2000, 602, 0.2)])
def test_rp_forward_backward(cuda, N, D, frac, dist, path):
    print(f"case rp N={N} D={D} frac={frac} {dist} {path}", flush=True)
    k = o.kept_acts(frac, D)
    rng = np.random.default_rng(N + D)
    R = o.rademacher_matrix(D, k, rng) if dist == "rademacher" else o.gaussian_matrix(D, k, rng)
    X = host_randn((N, D), D)
    r = _matrix_on_device(R, path)
    config.rp_matrix_source = lambda D_, k_, device: r
    xr, Rdev = ops.input2rp(dev(X), k)
    assert xr.shape == (N, k) and torch.equal(Rdev.cpu(), torch.from_numpy(R))
    close(xr, o.input2rp(X, R))
    back = ops.rp2input(xr, (N, D), Rdev)
    assert back.shape == (N, D)
    close(back, o.rp2input(xr.cpu().numpy(), R))


def test_generated_matrices(cuda):
    x = torch.randn(64, 256, device=cuda)
    xr, R = ops.input2rp(x, 32)
    assert set(R.unique().tolist()) == {float(np.float32(-1 / 32 ** 0.5)), float(np.float32(1 / 32 ** 0.5))}
    config.rp_distribution = "gaussian"
    xr, R = ops.input2rp(torch.randn(64, 4096, device=cuda), 64)
    assert abs(R.var().item() - 1 / 64) < 1e-3
    # E[x R R^T] = x: the decompressed tensor is an unbiased estimate
    acc = torch.zeros_like(x)
    config.rp_distribution = "rademacher"
    for _ in range(200):
        xr, R = ops.input2rp(x, 32)
        acc += ops.rp2input(xr, x.shape, R)
    assert ((acc / 200 - x).abs().mean() / x.abs().mean()).item() < 0.25


def _table(r, mode):
    """exact_rp_prepare_bf16 through the C ABI into a buffer of exactly the documented size plus guard bytes."""
    from exact_amd import _lib
    L = _lib.lib()
    D, k = r.shape
    nb = int(L.exact_rp_table_nbytes(D, k, mode))
    assert nb > 0
    t = torch.full((nb + 64,), 0x5C, dtype=torch.uint8, device=r.device)
    assert L.exact_rp_prepare_bf16(r.data_ptr(), D, k, mode, t.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    assert (t[nb:] == 0x5C).all()
    return t


def _shape_cases():
    small = [(300, 256, 0.125), (1001, 602, 0.125), (515, 100, 0.25), (130, 256, 0.25), (77, 50, 0.3), (64, 256, 0.5),
             (20011, 256, 0.125)]
    cases = [(N, D, frac, bits) for (N, D, frac) in small for bits in (1, 2, 4, 8)]
    # the first-layer shapes of the three benchmark configurations at full size, at their own bit width
    return cases + [(169343, 256, 0.125, 2), (232965, 602, 0.125, 2), (2449029, 100, 0.25, 1)]


@pytest.mark.parametrize("N,D,k", [(70, 256, 32), (33, 100, 25), (40, 602, 76), (64, 48, 128), (5000, 256, 64)])
def test_bf16_paths_on_integers_are_exact(cuda, N, D, k):
    """Small integers: every term and every partial sum is exact whatever the
    order, so the signs path must return c * (integer sum) rounded once and the
    general path the integer product itself -- a k-slot paired with the wrong
    feature, a wrong fragment or a missed tail shows as a wrong integer."""
    from exact_amd import _lib
    L = _lib.lib()
    sp = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(N + D + k)
    S = (2.0 * rng.integers(0, 2, (D, k)) - 1).astype(np.float32)
    c = np.float32(1.0 / np.sqrt(k))
    R = (S * c).astype(np.float32)
    X = rng.integers(-9, 10, (N, D)).astype(np.float32) * np.float32(0.25)
    Xr = rng.integers(-9, 10, (N, k)).astype(np.float32)
    Ri = rng.integers(-5, 6, (D, k)).astype(np.float32)
    x, xr = dev(X), dev(Xr)
    r, ri = _table(dev(R), 2), _table(dev(Ri), 1)
    out = torch.empty((N, k), device=cuda)
    back = torch.empty((N, D), device=cuda)
    assert L.exact_rp_fwd_bf16_f32(x.data_ptr(), r.data_ptr(), N, D, k, 2, out.data_ptr(), sp) == 0
    want = ((X.astype(np.float64) @ S.astype(np.float64)).astype(np.float32) * c).astype(np.float32)
    assert np.array_equal(out.cpu().numpy(), want)
    assert L.exact_rp_bwd_bf16_f32(xr.data_ptr(), r.data_ptr(), N, D, k, 2, back.data_ptr(), sp) == 0
    want = ((Xr.astype(np.float64) @ S.astype(np.float64).T).astype(np.float32) * c).astype(np.float32)
    assert np.array_equal(back.cpu().numpy(), want)
    assert L.exact_rp_fwd_bf16_f32(x.data_ptr(), ri.data_ptr(), N, D, k, 1, out.data_ptr(), sp) == 0
    assert np.array_equal(out.cpu().numpy(), (X.astype(np.float64) @ Ri.astype(np.float64)).astype(np.float32))
    assert L.exact_rp_bwd_bf16_f32(xr.data_ptr(), ri.data_ptr(), N, D, k, 1, back.data_ptr(), sp) == 0
    assert np.array_equal(back.cpu().numpy(), (Xr.astype(np.float64) @ Ri.astype(np.float64).T).astype(np.float32))


@pytest.mark.parametrize("path", ["fp32", "split", "signs"])
@pytest.mark.parametrize("N,D,frac,bits", _shape_cases())
def test_projection_and_quantisation_in_one_launch_against_the_oracle(cuda, N, D, frac, bits, path):
    """exact_rp_minmax_pack_f32 / exact_rp_minmax_pack_bf16_f32 through the C ABI
    (input2rp -> quantize_activation, ops.py:141-149): packed bytes, scale and min equal
    the ORACLE's quantiser applied to the product the library's own projection kernel of
    the same matrix-core path returns, for a supplied noise tensor and for the internal
    Philox stream; the product itself is within 1e-5 of the oracle's."""
    from exact_amd import _lib
    print(f"case rp+pack N={N} D={D} frac={frac} bits={bits} {path}", flush=True)
    L = _lib.lib()
    mode = {"fp32": 0, "split": 1, "signs": 2}[path]
    k = o.kept_acts(frac, D)
    rng = np.random.default_rng(N + D + bits)
    R = o.rademacher_matrix(D, k, rng)
    X = host_randn((N, D), N)
    u = rng.random((N, k), dtype=np.float32)
    x, r, noise = dev(X), dev(R), dev(u)
    sp = torch.cuda.current_stream().cuda_stream
    xr = torch.empty((N, k), device=cuda)
    if mode == 0:
        assert L.exact_rp_fwd_f32(x.data_ptr(), r.data_ptr(), N, D, k, xr.data_ptr(), sp) == 0
    else:
        table = _table(r, mode)
        assert L.exact_rp_fwd_bf16_f32(x.data_ptr(), table.data_ptr(), N, D, k, mode, xr.data_ptr(), sp) == 0
    close(xr, o.input2rp(X, R))
    product = xr.cpu().numpy()
    nb = int(L.exact_packed_nbytes(N, k, bits))
    seed, off = 0x1234ABCD5678, (3 << 32) + 40
    for un, nptr in ((u, noise.data_ptr()), (o.philox_noise_rows(seed, off, N, k), None)):
        want = o.quantize_activation(product, bits, un)
        packed = torch.full((nb + 64,), -91, dtype=torch.int8, device=cuda)
        s32, m32 = torch.empty(N, device=cuda), torch.empty(N, device=cuda)
        sbf = torch.empty(N, dtype=torch.bfloat16, device=cuda)
        mbf = torch.empty(N, dtype=torch.bfloat16, device=cuda)
        if mode == 0:
            rc = L.exact_rp_minmax_pack_f32(x.data_ptr(), r.data_ptr(), nptr, seed, off, N, D, k, bits, packed.data_ptr(),
                                            s32.data_ptr(), m32.data_ptr(), sbf.data_ptr(), mbf.data_ptr(), sp)
        else:
            rc = L.exact_rp_minmax_pack_bf16_f32(x.data_ptr(), table.data_ptr(), mode, nptr, seed, off, N, D, k, bits,
                                                 packed.data_ptr(), s32.data_ptr(), m32.data_ptr(), sbf.data_ptr(),
                                                 mbf.data_ptr(), sp)
        assert rc == 0
        got = packed.cpu().numpy().view(np.uint8)
        assert np.array_equal(got[:nb], want[0]) and (got[nb:] == np.uint8(256 - 91)).all()
        assert np.array_equal(s32.cpu().numpy().view(np.uint32), want[4].view(np.uint32))
        assert np.array_equal(m32.cpu().numpy(), want[5])
        assert np.array_equal(sbf.view(torch.int16).cpu().numpy().view(np.uint16), want[2])
        assert np.array_equal(mbf.view(torch.int16).cpu().numpy().view(np.uint16), want[3])
