"""Pins for oracle/exact_oracle_extra.py without the reference: torch autograd
for LeakyReLU, dense brute force for max / min aggregation and its scatter
backward, dense products for the edge-value gradient."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

import exact_oracle_extra as ox

F32 = np.float32


def small_csr(M, N, nnz, seed):
    rng = np.random.default_rng(seed)
    A = sp.coo_matrix((rng.standard_normal(nnz).astype(F32), (rng.integers(0, M, nnz), rng.integers(0, N, nnz))),
                      shape=(M, N)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    return A


@pytest.mark.parametrize("slope", [0.2, 0.01, 0.0, 1.5])
def test_leaky_relu_matches_torch_autograd(slope):
    rng = np.random.default_rng(0)
    x = rng.standard_normal(1003).astype(F32)
    x[:2] = [0.0, -0.0]
    g = rng.standard_normal(1003).astype(F32)
    y, mask = ox.leaky_relu_fwd(x, slope)
    t = torch.from_numpy(x.copy()).requires_grad_()
    ty = F.leaky_relu(t, slope)
    ty.backward(torch.from_numpy(g))
    assert np.array_equal(y, ty.detach().numpy())
    assert np.array_equal(ox.leaky_relu_bwd(g, mask, slope), t.grad.numpy())


@pytest.mark.parametrize("is_max", [True, False])
@pytest.mark.parametrize("valued", [True, False])
def test_minmax_matches_dense_brute_force(is_max, valued):
    A = small_csr(40, 30, 200, 1)
    X = np.random.default_rng(2).standard_normal((30, 7)).astype(F32)
    X[3] = X[5]                                              # ties: the first entry in CSR order must win
    val = A.data if valued else None
    out, arg = ox.spmm_minmax(A.indptr, A.indices, val, X, is_max)
    nnz = A.nnz
    for r in range(40):
        es = list(range(A.indptr[r], A.indptr[r + 1]))
        for k in range(7):
            if not es:
                assert out[r, k] == 0 and arg[r, k] == nnz
                continue
            vals = [F32(A.data[e] if valued else 1) * X[A.indices[e], k] if valued else X[A.indices[e], k] for e in es]
            best = max(vals) if is_max else min(vals)
            assert out[r, k] == best and arg[r, k] == es[vals.index(best)]
    # backward == autograd through a dense gather of the arg entries
    dY = np.random.default_rng(3).standard_normal(out.shape).astype(F32)
    gv, gm = ox.spmm_minmax_bw(A.indices, val, X, arg, dY, nnz)
    Xt = torch.from_numpy(X).double().requires_grad_()
    vt = torch.from_numpy(A.data).double().requires_grad_()
    a = torch.from_numpy(np.where(arg == nnz, 0, arg))
    src = torch.from_numpy(A.indices.astype(np.int64))[a]
    picked = Xt[src, torch.arange(7).expand_as(src)]
    o_t = (vt[a] * picked if valued else picked) * torch.from_numpy((arg != nnz).astype(np.float64))
    o_t.backward(torch.from_numpy(dY).double())
    np.testing.assert_allclose(gm, Xt.grad.numpy(), rtol=1e-5, atol=1e-6)
    if valued:
        np.testing.assert_allclose(gv, vt.grad.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("reduce", ["sum", "mean"])
def test_sddmm_is_the_gradient_of_spmm_wrt_values(reduce):
    A = small_csr(50, 35, 300, 4)
    X = np.random.default_rng(5).standard_normal((35, 9))
    dY = np.random.default_rng(6).standard_normal((50, 9))
    row = np.repeat(np.arange(50), np.diff(A.indptr))
    got = ox.sddmm(row, A.indptr, A.indices, X, dY, reduce)
    # d/dval[e] of sum(dY * (A @ X)) = dY[row[e]] . X[col[e]]   (/ deg for mean)
    want = np.array([dY[row[e]] @ X[A.indices[e]] for e in range(A.nnz)])
    if reduce == "mean":
        want = want / np.maximum(np.diff(A.indptr), 1)[row]
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-6)
