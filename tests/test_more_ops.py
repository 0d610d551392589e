"""The remaining operators of the reference's extension modules -- LeakyReLU
mask, ELU, max / min aggregation, edge-value gradients -- against
oracle/exact_oracle_extra.py: kernels on the SIMT emulator (always) and the
Python layers on both back ends (the GPU ones marked gpu)."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

import emu_util as e
import exact_amd as exact
import exact_oracle as o
import exact_oracle_extra as ox
from exact_amd.cpp_extension import quantization as extq
from exact_amd.cpp_extension import spmm as ext_spmm
from exact_amd.conf import config
from exact_amd.sparse import SparseTensor
from exact_amd.spmm import QMatmul, qmatmul

F32 = np.float32


def csr(M, N, nnz, seed, empty_rows=True):
    rng = np.random.default_rng(seed)
    r = rng.integers(0, M, nnz)
    if empty_rows:
        r[r % 7 == 3] = 0
    A = sp.coo_matrix((rng.standard_normal(nnz).astype(F32), (r, rng.integers(0, N, nnz))), shape=(M, N)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    return A


# ------------------------------------------------------------ kernels (emulated)
@pytest.mark.parametrize("n", [1, 5, 33, 257, 2049, 10007])
def test_leaky_relu_kernel(n):
    rng = np.random.default_rng(n)
    x, g = rng.standard_normal(n).astype(F32), rng.standard_normal(n).astype(F32)
    for slope in (0.2, 0.01):
        y, mask = e.leaky_relu_fwd(x, slope)
        wy, wm = ox.leaky_relu_fwd(x, slope)
        assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mask, wm)
        assert np.array_equal(e.leaky_relu_bwd(g, mask, slope).view(np.uint32), ox.leaky_relu_bwd(g, wm, slope).view(np.uint32))


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("valued", [True, False])
@pytest.mark.parametrize("is_max", [True, False])
@pytest.mark.parametrize("M,N,K", [(60, 40, 256), (33, 50, 40), (20, 20, 602), (45, 30, 7), (9, 12, 1)])
def test_minmax_kernel(M, N, K, is_max, valued, idx):
    A = csr(M, N, M * 6, M + K)
    X = np.random.default_rng(K).standard_normal((N, K)).astype(F32)
    X[1] = X[2]
    val = A.data if valued else None
    out, arg = e.spmm_minmax(A.indptr, A.indices, val, X, is_max, idx)
    wout, warg = ox.spmm_minmax(A.indptr, A.indices, val, X, is_max)
    assert np.array_equal(out.view(np.uint32), wout.view(np.uint32)) and np.array_equal(arg.astype(np.int64), warg)


@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("M,N,K", [(60, 40, 256), (33, 50, 40), (20, 20, 602), (45, 30, 7), (9, 12, 1), (30, 30, 1000)])
def test_sddmm_kernel(M, N, K, reduce):
    A = csr(M, N, M * 5, M * 3 + K)
    rng = np.random.default_rng(K)
    mat, grad = rng.standard_normal((N, K)).astype(F32), rng.standard_normal((M, K)).astype(F32)
    row = np.repeat(np.arange(M), np.diff(A.indptr))
    for idx in (np.int64, np.int32):
        got = e.sddmm(row, A.indptr, A.indices, mat, grad, reduce, idx)
        want = ox.sddmm(row, A.indptr, A.indices, mat, grad, reduce)
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * np.abs(want).max())


# ------------------------------------------------------------ layers (both back ends)
def test_leaky_relu_and_elu_layers(backend):
    x = torch.randn(300, 47, device=backend, requires_grad=True)
    xr = x.detach().clone().requires_grad_()
    g = torch.randn(300, 47, device=backend)
    y = exact.QLeakyReLU(0.2)(x)
    y.backward(g)
    yr = F.leaky_relu(xr, 0.2)
    yr.backward(g)
    assert torch.equal(y, yr) and torch.equal(x.grad, xr.grad)
    assert torch.equal(extq.act_quantized_leaky_relu(x.detach(), 0.01), F.leaky_relu(x.detach(), 0.01))
    # ELU: forward is the stock op; backward uses the DEQUANTISED input (8 bits: close to exact)
    config.activation_compression_bits = [8]
    layer = exact.QELU(1.0).train()
    x2 = torch.randn(200, 32, device=backend, requires_grad=True)
    x2r = x2.detach().clone().requires_grad_()
    g2 = torch.randn(200, 32, device=backend)
    y2 = layer(x2)
    y2.backward(g2)
    F.elu(x2r, 1.0).backward(g2)
    assert torch.equal(y2, F.elu(x2.detach(), 1.0))
    assert (x2.grad - x2r.grad).abs().max() < 0.05 and not torch.equal(x2.grad, x2r.grad)
    assert torch.equal(layer.eval()(x2.detach()), F.elu(x2.detach(), 1.0))


@pytest.mark.parametrize("reduce", ["max", "min"])
@pytest.mark.parametrize("valued", [True, False])
def test_max_min_aggregation_forward_and_backward(backend, reduce, valued):
    A = csr(120, 120, 700, 5)
    K = 24
    g = torch.Generator().manual_seed(1)
    X = torch.randn(120, K, generator=g)
    dY = torch.randn(120, K, generator=g)
    adj = SparseTensor.from_scipy(A, backend)
    if not valued:
        adj = adj.set_value(None)
    val = A.data if valued else None
    wout, warg = ox.spmm_minmax(A.indptr, A.indices, val, X.numpy(), reduce == "max")
    _, wgm = ox.spmm_minmax_bw(A.indices, val, X.numpy(), warg, dY.numpy(), A.nnz)
    x = X.clone().to(backend).requires_grad_()
    y = QMatmul(reduce)(adj, x)
    assert np.array_equal(y.detach().cpu().numpy().view(np.uint32), wout.view(np.uint32))
    y.backward(dY.to(backend))
    np.testing.assert_allclose(x.grad.cpu().numpy(), wgm, rtol=1e-5, atol=1e-6)
    out, arg = (ext_spmm.spmm_max_fw if reduce == "max" else ext_spmm.spmm_min_fw)(*adj.csr()[:2], adj.csr()[2], x.detach())
    assert np.array_equal(arg.cpu().numpy(), warg) and torch.equal(out, y.detach())


@pytest.mark.parametrize("reduce", ["sum", "mean", "max"])
def test_edge_value_gradient(backend, reduce):
    """value.requires_grad: the dense operand is kept compressed and restored
    for the value gradient (8 bits here, so the result is close to the exact
    gradient; with compression off it is the exact one)."""
    A = csr(90, 90, 500, 6)
    K = 16
    g = torch.Generator().manual_seed(2)
    X, dY = torch.randn(90, K, generator=g), torch.randn(90, K, generator=g)
    row = np.repeat(np.arange(90), np.diff(A.indptr))
    if reduce == "max":
        _, warg = ox.spmm_minmax(A.indptr, A.indices, A.data, X.numpy(), True)
        want, _ = ox.spmm_minmax_bw(A.indices, A.data, X.numpy(), warg, dY.numpy(), A.nnz)
    else:
        want = ox.sddmm(row, A.indptr, A.indices, X.numpy(), dY.numpy(), reduce)
    for compress, tol in ((False, 1e-5), (True, 0.05)):
        config.compress_activation = compress
        config.activation_compression_bits = [8]
        adj = SparseTensor.from_scipy(A, backend)
        value = adj.storage._value.clone().requires_grad_()
        adj = adj.set_value(value)
        x = X.clone().to(backend).requires_grad_()
        y = qmatmul(adj, x, reduce)
        y.backward(dY.to(backend))
        got = value.grad.cpu().numpy()
        assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max()), (compress, np.abs(got - want).max())
        assert x.grad is not None
