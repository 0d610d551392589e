"""The sparse product at the sizes the benchmark runs it (the three full-batch
graph configurations), where a dense or scipy restatement no longer fits a
test: properties that hold at any size, the reproducible row-wise kernel as a
second implementation, and a sample of rows against the CPU oracle.

The reference pins its kernel against torch_sparse.matmul on N = 10,000
(test/test_op.py:529-554); sum and mean, forward and the transpose used by
backward (spmm.cc:57-79, 115-139)."""
import numpy as np
import pytest
import torch

import exact_oracle as o
from exact_amd.benchmarks import EPOCH_CONFIGS, powerlaw_graph
from exact_amd.conf import config
from exact_amd.cpp_extension import spmm as ext_spmm
from exact_amd.sparse import gcn_norm

pytestmark = pytest.mark.gpu

# (benchmark configuration, feature widths the model aggregates at)
CASES = [("cfg3_gcn_int2", (256, 40)), ("cfg4_sage_int2_rp0.125", (602, 256)), ("cfg5_sage_int1_rp0.25", (100, 256))]


def _graph(name, cuda):
    kind, n, edges = EPOCH_CONFIGS[name][:3]
    adj = powerlaw_graph(n, edges, seed=1, device=cuda)
    if kind == "gcn":
        adj = gcn_norm(adj, add_self_loops=True)
    return adj.to_int32_().fill_cache_(), ("sum" if kind == "gcn" else "mean")


def _close(got, want, scale, tol=1e-5):
    """|got - want| <= tol * (sum of |terms| of that output element): the bound
    that any order of fp32 summation of the same terms satisfies with room."""
    return bool(((got - want).abs() <= tol * scale + 1e-30).all())


@pytest.mark.parametrize("name,widths", CASES)
def test_spmm_at_benchmark_size(cuda, name, widths):
    adj, reduce = _graph(name, cuda)
    rowptr, col, value = adj.csr()
    st = adj.storage
    M, nnz = adj.sparse_size(0), col.numel()
    deg = (rowptr[1:] - rowptr[:-1]).float()
    # A @ 1: row sums.  Unvalued sum -> the degree, exactly (small integers); mean -> 1 on non-empty rows
    ones = torch.ones(M, 8, device=cuda)
    if value is None:
        assert torch.equal(ext_spmm.spmm_csr(rowptr, col, None, ones, "sum"), deg[:, None].expand(M, 8))
        # the mean of ones: rows inside one chunk and hub rows (divided once at the end) give exactly 1; a row
        # of up to 2048 entries cut by chunk boundaries adds at most 33 rounded quotients count / length
        got = ext_spmm.spmm_csr(rowptr, col, None, ones, "mean")
        assert torch.allclose(got, (deg > 0).float()[:, None].expand(M, 8), rtol=0, atol=2e-6)
        hubs = deg > 2048
        assert bool(hubs.any()) and torch.equal(got[hubs], torch.ones_like(got[hubs]))
    else:
        want = torch.zeros(M, device=cuda, dtype=torch.float64).index_add_(0, st.row().long(), value.double())
        got = ext_spmm.spmm_csr(rowptr, col, value, ones, "sum")
        assert torch.allclose(got[:, 0].double(), want, rtol=1e-5, atol=1e-6)
    gen = torch.Generator(device=cuda).manual_seed(5)
    for K in widths:
        X = torch.randn(M, K, generator=gen, device=cuda)
        out = ext_spmm.spmm_csr(rowptr, col, value, X, reduce)
        assert out.shape == (M, K) and torch.isfinite(out).all()
        # the reproducible kernel (one wavefront per row, entries in CSR order) as a second implementation
        config.deterministic_spmm = True
        ref = ext_spmm.spmm_csr(rowptr, col, value, X, reduce)
        absum = ext_spmm.spmm_csr(rowptr, col, None if value is None else value.abs(), X.abs(), reduce)
        config.deterministic_spmm = False
        assert _close(out, ref, absum)
        # a sample of rows against the CPU oracle (sequential fp32 accumulation in CSR order, reducer.cuh:43-85)
        pick = torch.randperm(M, generator=torch.Generator().manual_seed(K))[:128]
        hubs = torch.topk(deg, 2).indices.cpu()
        rows = torch.cat([pick, hubs]).tolist()
        for r in rows[:130] if K == widths[0] else rows[:16]:
            s, e = int(rowptr[r]), int(rowptr[r + 1])
            cols = col[s:e].long()
            xr = X[cols].cpu().numpy()
            w = np.ones(e - s, np.float32) if value is None else value[s:e].cpu().numpy()
            want = o.spmm_csr(np.array([0, e - s]), np.arange(e - s), w, xr, reduce)[0]
            assert np.array_equal(ref[r].cpu().numpy(), want)                     # row-wise kernel: bit for bit
            assert _close(out[r].cpu(), torch.from_numpy(want), absum[r].cpu())
        # transpose identity <A X, Y> = <X, A^T Y> with the operands backward uses
        Y = torch.randn(M, K, generator=gen, device=cuda)
        if reduce == "sum":
            _, At_Y = ext_spmm.spmm_sum_bw(st.row(), rowptr, col, value, st.colptr(), st.csr2csc(), None, Y,
                                           value is not None, False, True)
        else:
            _, At_Y = ext_spmm.spmm_mean_bw(st.row(), rowptr, col, value, st.rowcount(), st.colptr(), st.csr2csc(),
                                            None, Y, value is not None, False, True)
        lhs = (out.double() * Y.double()).sum().item()
        rhs = (X.double() * At_Y.double()).sum().item()
        norm = (absum.double() * Y.double().abs()).sum().item()
        assert abs(lhs - rhs) <= 1e-6 * norm, (lhs, rhs, norm)
        del X, Y, out, ref, absum, At_Y
    ext_spmm.clear_csc_cache()
