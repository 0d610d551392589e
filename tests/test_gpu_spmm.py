"""GPU parity of CSR SpMM (sum / mean, valued / unvalued, int32 / int64
indices) and of its transpose-backward against the oracle, within 1e-5
relative (fp32), plus the torch_sparse-style container."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import exact_oracle as o
from exact_amd.cpp_extension import spmm as ext_spmm
from exact_amd.nn import matmul
from exact_amd.ops import qspmm_mean, qspmm_sum
from exact_amd.sparse import SparseTensor, gcn_norm
from exact_amd.spmm import QMatmul, qmatmul
from gpu_util import dev, host_randn

pytestmark = pytest.mark.gpu
RTOL = 1e-5


def powerlaw_csr(M, avg_deg, seed, n_cols=None, hub=0):
    rng = np.random.default_rng(seed)
    n_cols = n_cols or M
    deg = np.minimum((rng.zipf(2.1, M) * avg_deg / 2.5).astype(np.int64), n_cols)
    deg[rng.integers(0, M, max(1, M // 50))] = 0        # some empty rows
    if hub:
        deg[rng.integers(0, M, 3)] = hub                # rows far longer than one 64-entry chunk
    rows = np.repeat(np.arange(M), deg)
    cols = rng.integers(0, n_cols, rows.size)
    A = sp.coo_matrix((rng.standard_normal(rows.size).astype(np.float32), (rows, cols)), shape=(M, n_cols)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    return A


def close(got, want):
    want = np.asarray(want)
    scale = np.abs(want).max() + 1e-30
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=RTOL, atol=RTOL * scale)


@pytest.mark.parametrize("idx", [torch.int64, torch.int32])
@pytest.mark.parametrize("valued", [True, False])
@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("M,K,avg,hub", [(1000, 256, 8, 700), (513, 40, 5, 0), (300, 602, 20, 3000),
                                         (2000, 100, 10, 0), (64, 1, 3, 0), (200, 47, 4, 150), (10, 128, 2, 0)])
def test_forward(cuda, M, K, avg, hub, reduce, valued, idx):
    print(f"case spmm M={M} K={K} reduce={reduce} valued={valued} idx={idx}", flush=True)
    A = powerlaw_csr(M, avg, M + K, hub=min(hub, M))
    X = host_randn((M, K), K)
    val = A.data if valued else None
    want = o.spmm_csr(A.indptr, A.indices, val, X, reduce)
    got = ext_spmm.spmm_csr(dev(A.indptr.astype(np.int64)).to(idx), dev(A.indices.astype(np.int64)).to(idx),
                            dev(val) if valued else None, dev(X), reduce)
    close(got, want)
    empty = np.diff(A.indptr) == 0
    assert (got.cpu().numpy()[empty] == 0).all()


def test_rectangular_and_empty(cuda):
    A = powerlaw_csr(300, 6, 1, n_cols=120)
    X = host_randn((120, 64), 2)
    got = ext_spmm.spmm_csr(dev(A.indptr.astype(np.int64)), dev(A.indices.astype(np.int64)), dev(A.data), dev(X), "sum")
    close(got, o.spmm_csr(A.indptr, A.indices, A.data, X, "sum"))
    z = ext_spmm.spmm_csr(torch.zeros(5, dtype=torch.long, device=cuda), torch.zeros(0, dtype=torch.long, device=cuda),
                          None, dev(X), "mean")
    assert z.shape == (4, 64) and (z == 0).all()


def test_forward_equals_dense_like_reference_test(cuda):
    """test/test_op.py:505-554 compares with torch_sparse.matmul on N=10000,
    nnz=50000; here the dense product is the stand-in."""
    rng = np.random.default_rng(0)
    N, nnz = 10000, 50000
    A = sp.coo_matrix((rng.random(nnz).astype(np.float32), (rng.integers(0, N, nnz), rng.integers(0, N, nnz))),
                      shape=(N, N)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    adj = SparseTensor.from_scipy(A, "cuda")
    X = torch.randn(N, 64, device=cuda)
    dense = torch.from_numpy(A.toarray()).cuda()
    for reduce in ("sum", "mean"):
        for valued in (True, False):
            a = adj if valued else adj.set_value(None)
            d = dense if valued else (dense != 0).float()
            want = d.double() @ X.double()
            if reduce == "mean":
                want = want / torch.from_numpy(np.maximum(np.diff(A.indptr), 1)).cuda().view(-1, 1)
            got = qmatmul(a, X, reduce)
            torch.testing.assert_close(got.double(), want, rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("valued", [True, False])
def test_backward_is_transpose_product(cuda, reduce, valued):
    A = powerlaw_csr(800, 7, 9, hub=500)
    K = 96
    X = host_randn((800, K), 3)
    dY = host_randn((800, K), 4)
    val = A.data if valued else None
    row, colptr, csr2csc = o.csr_transpose(A.indptr, A.indices, 800)
    if reduce == "sum":
        want = o.spmm_sum_bw(row, colptr, csr2csc, val, dY)
    else:
        want = o.spmm_mean_bw(row, np.diff(A.indptr), colptr, csr2csc, val, dY)
    adj = SparseTensor.from_scipy(A, "cuda")
    if not valued:
        adj = adj.set_value(None)
    st = adj.storage
    assert np.array_equal(st.colptr().cpu().numpy(), colptr) and np.array_equal(st.csr2csc().cpu().numpy(), csr2csc)
    assert np.array_equal(st.row().cpu().numpy(), row)
    x = dev(X).requires_grad_()
    y = QMatmul(reduce)(adj, x)
    close(y.detach(), o.spmm_csr(A.indptr, A.indices, val, X, reduce))
    y.backward(dev(dY))
    close(x.grad, want)
    # the uncompressed layer product gives the same gradient
    x2 = dev(X).requires_grad_()
    matmul(adj, x2, reduce).backward(dev(dY))
    close(x2.grad, want)
    # direct Function call with the reference's positional signature
    rowptr, col, value = adj.csr()
    x3 = dev(X).requires_grad_()
    if reduce == "sum":
        y3 = qspmm_sum.apply(st.row(), rowptr, col, value, st.colptr(), st.csr2csc(), valued, x3, None, None, None)
    else:
        y3 = qspmm_mean.apply(st.row(), rowptr, col, value, st.rowcount(), st.colptr(), st.csr2csc(), valued, x3,
                              None, None, None)
    y3.backward(dev(dY))
    close(x3.grad, want)


def test_gcn_norm_and_errors(cuda):
    A = powerlaw_csr(500, 5, 11)
    A = ((A + A.T) != 0).astype(np.float32).tocsr()
    adj = gcn_norm(SparseTensor.from_scipy(A, "cuda").set_value(None), add_self_loops=True)
    At = (A.tolil())
    At.setdiag(1.0)
    At = At.tocsr()
    d = np.asarray(At.sum(1)).reshape(-1) ** -0.5
    want = sp.diags(d) @ At @ sp.diags(d)
    np.testing.assert_allclose(adj.to_dense().cpu().numpy(), want.toarray(), rtol=1e-6, atol=1e-7)
    rowptr, col, value = adj.csr()
    with pytest.raises(RuntimeError, match="`row` is missing"):
        ext_spmm.spmm_sum_fw(None, rowptr, col, value, None, None, torch.randn(500, 8, device=cuda, requires_grad=True))
    with pytest.raises(RuntimeError, match="Input mismatch"):
        ext_spmm.spmm_csr(rowptr, col, value[:-1], torch.randn(500, 8, device=cuda), "sum")
    with pytest.raises(ValueError):
        qmatmul(adj, torch.randn(500, 8, device=cuda), "mul")
