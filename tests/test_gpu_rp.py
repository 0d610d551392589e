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
