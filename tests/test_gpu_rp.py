"""GPU parity of the random-projection GEMMs (MFMA fp32) against the oracle
within 1e-5 relative, with the projection matrix passed in."""
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


@pytest.mark.parametrize("dist", ["rademacher", "gaussian"])
@pytest.mark.parametrize("N,D,frac", [(1, 256, 0.125), (31, 256, 0.125), (1000, 256, 0.125), (257, 602, 0.125),
                                      (500, 100, 0.25), (129, 256, 0.25), (64, 128, 0.5), (77, 50, 0.3),
                                      (130, 7, 0.5), (4099, 256, 0.125), (300, 256, 0.49)])
def test_rp_forward_backward(cuda, N, D, frac, dist):
    print(f"case rp N={N} D={D} frac={frac} {dist}", flush=True)
    k = o.kept_acts(frac, D)
    rng = np.random.default_rng(N + D)
    R = o.rademacher_matrix(D, k, rng) if dist == "rademacher" else o.gaussian_matrix(D, k, rng)
    X = host_randn((N, D), D)
    config.rp_matrix_source = lambda D_, k_, device: dev(R)
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


def _shape_cases():
    small = [(300, 256, 0.125), (1001, 602, 0.125), (515, 100, 0.25), (130, 256, 0.25), (77, 50, 0.3), (64, 256, 0.5),
             (20011, 256, 0.125)]
    cases = [(N, D, frac, bits) for (N, D, frac) in small for bits in (1, 2, 4, 8)]
    # the first-layer shapes of the three benchmark configurations at full size, at their own bit width
    return cases + [(169343, 256, 0.125, 2), (232965, 602, 0.125, 2), (2449029, 100, 0.25, 1)]


@pytest.mark.parametrize("N,D,frac,bits", _shape_cases())
def test_projection_and_quantisation_in_one_launch_against_the_oracle(cuda, N, D, frac, bits):
    """exact_rp_minmax_pack_f32 through the C ABI (input2rp -> quantize_activation,
    ops.py:141-149): packed bytes, scale and min equal the ORACLE's quantiser applied to
    the product the library's own projection kernel returns, for a supplied noise tensor
    and for the internal Philox stream; the product itself is within 1e-5 of the oracle's."""
    from exact_amd import _lib
    print(f"case rp+pack N={N} D={D} frac={frac} bits={bits}", flush=True)
    L = _lib.lib()
    k = o.kept_acts(frac, D)
    rng = np.random.default_rng(N + D + bits)
    R = o.rademacher_matrix(D, k, rng)
    X = host_randn((N, D), N)
    u = rng.random((N, k), dtype=np.float32)
    x, r, noise = dev(X), dev(R), dev(u)
    sp = torch.cuda.current_stream().cuda_stream
    xr = torch.empty((N, k), device=cuda)
    assert L.exact_rp_fwd_f32(x.data_ptr(), r.data_ptr(), N, D, k, xr.data_ptr(), sp) == 0
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
        rc = L.exact_rp_minmax_pack_f32(x.data_ptr(), r.data_ptr(), nptr, seed, off, N, D, k, bits, packed.data_ptr(),
                                        s32.data_ptr(), m32.data_ptr(), sbf.data_ptr(), mbf.data_ptr(), sp)
        assert rc == 0
        got = packed.cpu().numpy().view(np.uint8)
        assert np.array_equal(got[:nb], want[0]) and (got[nb:] == np.uint8(256 - 91)).all()
        assert np.array_equal(s32.cpu().numpy().view(np.uint32), want[4].view(np.uint32))
        assert np.array_equal(m32.cpu().numpy(), want[5])
        assert np.array_equal(sbf.view(torch.int16).cpu().numpy().view(np.uint16), want[2])
        assert np.array_equal(mbf.view(torch.int16).cpu().numpy().view(np.uint16), want[3])
