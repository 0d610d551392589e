"""GPU parity at the shapes the three full-batch benchmark configurations
launch (N = 169,343 / 232,965 / 2,449,029): the weight-gradient and
column-sum kernels of the linear backward (backward_func.cc:83-93), the
decompressing projection (ops.py:121-125), the remaining sparse and mask
kernels at kernel level, and one full-size training step of the 3-layer GCN
against the oracle model."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

import exact_oracle as o
import exact_oracle_extra as ox
import oracle_model as om
from exact_amd import _lib
from exact_amd.conf import config
from exact_amd.cpp_extension import backward_func as bf
from exact_amd.cpp_extension import spmm as ext_spmm
from gpu_util import SeededNoise, dev, powerlaw_csr

pytestmark = pytest.mark.gpu

BIG = (169343, 2449029)


def _ints(shape, device, seed, lo=-3, hi=4):
    g = torch.Generator(device=device).manual_seed(seed)
    return torch.randint(lo, hi, shape, generator=g, device=device).float()


# (K, D) of dW = dY^T . X in the benchmark models (with and without projection), plus shapes that
# reach every work split of the kernel (1 or 2 column blocks per wavefront either way, 1 / 2 / 4 row slabs)
DW_SHAPES = [(256, 256), (256, 128), (40, 256), (256, 64), (47, 64), (256, 25), (41, 32), (256, 76),
             (16, 64), (24, 300), (64, 256), (256, 32), (300, 64), (256, 602)]


@pytest.mark.parametrize("cores", ["bf16", "fp32"])
@pytest.mark.parametrize("N", BIG)
@pytest.mark.parametrize("K,D", DW_SHAPES)
def test_weight_gradient_is_the_integer_product_at_benchmark_size(cuda, N, K, D, cores):
    """exact_linear_dw_f32 on small integers: every product and every partial
    sum is an integer below 2^24, so fp32 is exact whatever the order and the
    result must equal the float64 product bit for bit -- a wrong fragment, a
    row counted twice or missed, or a lost atomic shows.  Contiguous and with
    row strides longer than the width (NaN in the padding)."""
    print(f"case dW N={N} K={K} D={D} {cores}", flush=True)
    config.matrix_cores = cores
    dy, x = _ints((N, K), cuda, N + K), _ints((N, D), cuda, N + D + 1)
    want = (dy.double().t() @ x.double()).float()
    got = bf.weight_gradient(dy, x)
    assert got.shape == (K, D) and torch.equal(got, want)
    wide_dy = torch.full((N, K + 3), float("nan"), device=cuda)
    wide_x = torch.full((N, D + 9), float("nan"), device=cuda)
    wide_dy[:, 2:2 + K], wide_x[:, 5:5 + D] = dy, x
    assert torch.equal(bf.weight_gradient(wide_dy[:, 2:2 + K], wide_x[:, 5:5 + D]), want)


# (D, K) of the dense products x . M of the benchmark models: F.linear with M = W^T, the input gradient with M = W,
# and the first SAGE layer's x [R | W_l^T]; plus widths that cut the 256-column slabs and the 32-column tiles unevenly
GEMM_SHAPES = [(256, 256), (128, 256), (256, 40), (100, 256), (256, 47), (604, 332), (256, 300), (64, 1024), (1024, 64), (8, 8), (602, 256), (50, 121)]


@pytest.mark.parametrize("N", BIG)
@pytest.mark.parametrize("D,K", GEMM_SHAPES)
def test_tall_gemm_is_the_integer_product_at_benchmark_size(cuda, N, D, K):
    """exact_tall_gemm_bf16_f32 through the shim on small integers: every bf16
    piece, product and partial sum is exact, so the result equals the float64
    product bit for bit -- a wrong fragment, slab or tile offset, or a row missed,
    shows.  With the matrix direct and transposed (a weight as F.linear holds
    it), a bias, an addend and accumulation in place."""
    if N * max(D, K) > 700_000_000:
        pytest.skip("operands beyond what this test allocates")
    print(f"case gemm N={N} D={D} K={K}", flush=True)
    config.matrix_cores, config.tall_gemm_min_depth, config.tall_gemm_max_rows_wide = "bf16", 1, 10 ** 9
    x = _ints((N, D), cuda, N + D, -5, 6)
    m = _ints((D, K), cuda, D + K, -5, 6)
    bias = _ints((K,), cuda, K, -9, 10)
    want = (x.double() @ m.double())
    got = bf.tall_matmul(x, m)
    assert got.shape == (N, K) and torch.equal(got, want.float())
    assert hasattr(m, "_exact_gemm_table")                      # the library kernel ran, not the framework's GEMM
    weight = m.t().contiguous()                                 # [K, D]
    assert torch.equal(bf.tall_matmul(x, weight, transposed=True, bias=bias), (want + bias.double()).float())
    wide = torch.full((N, K + 6), float("nan"), device=cuda)
    add = _ints((N, K), cuda, 5, -9, 10)
    wide[:, 3:3 + K] = add
    view = wide[:, 3:3 + K]
    out = bf.tall_matmul(x, m, addend=view, into=view)          # accumulate into a strided view
    assert out is view and torch.equal(view, (want + add.double()).float())
    assert torch.isnan(wide[:, :3]).all() and torch.isnan(wide[:, 3 + K:]).all()


@pytest.mark.parametrize("N,D,K", [(169343, 256, 256), (50000, 604, 332), (20000, 1024, 1024), (16384, 4096, 32), (16385, 32, 4096)])
def test_tall_gemm_accuracy_and_the_framework_gemm(cuda, N, D, K):
    """Random operands with rows and columns of very different size: within 1e-6
    of the sum of the absolute terms of the float64 product (a dropped low-order
    bf16 piece would miss that by far), and as close to it as the framework's
    fp32 GEMM is."""
    print(f"case gemm accuracy N={N} D={D} K={K}", flush=True)
    config.matrix_cores, config.tall_gemm_min_depth, config.tall_gemm_max_rows_wide = "bf16", 1, 10 ** 9
    g = torch.Generator(device=cuda).manual_seed(N + D)
    x = torch.randn(N, D, generator=g, device=cuda) * torch.exp(8 * torch.rand(N, 1, generator=g, device=cuda) - 4)
    m = torch.randn(D, K, generator=g, device=cuda) * torch.exp(8 * torch.rand(1, K, generator=g, device=cuda) - 4)
    got = bf.tall_matmul(x, m)
    assert hasattr(m, "_exact_gemm_table")
    rows = torch.arange(0, N, max(1, N // 4096), device=cuda)
    want = x[rows].double() @ m.double()
    bound = x[rows].abs().double() @ m.abs().double()
    mine = (got[rows].double() - want).abs()
    assert (mine <= 1e-6 * bound + 1e-30).all()
    theirs = (x[rows].mm(m).double() - want).abs()
    assert (mine / (bound + 1e-30)).max().item() <= 4 * max((theirs / (bound + 1e-30)).max().item(), 2.0 ** -24)


def test_tall_gemm_takes_rows_aligned_to_eight_bytes(cuda):
    """An operand that starts 8 bytes into a 16-byte line (a view into a larger
    buffer), with a feature count that is and is not a multiple of 4: the kernel
    reads it with 8-byte loads; integer operands, exact result."""
    config.matrix_cores, config.tall_gemm_min_depth = "bf16", 1
    for D, K in ((256, 256), (602, 40), (50, 300)):
        print(f"case gemm 8-byte aligned D={D} K={K}", flush=True)
        N = 40001
        flat = _ints((N * D + 2,), cuda, D + K, -5, 6)
        x = flat[2:].view(N, D)
        assert x.data_ptr() % 16 == 8 and x.is_contiguous()
        m = _ints((D, K), cuda, D, -5, 6)
        with torch.no_grad():
            got = bf.tall_matmul(x, m)
        assert hasattr(m, "_exact_gemm_table")
        assert torch.equal(got.double(), x.double() @ m.double())


def test_tall_gemm_reprepares_a_changed_matrix(cuda):
    """The fragment table is remembered on the matrix and rebuilt when it changes in place (an optimiser step)."""
    config.matrix_cores = "bf16"
    x = _ints((20000, 64), cuda, 1)
    w = torch.nn.Parameter(_ints((48, 64), cuda, 2))
    with torch.no_grad():
        first = bf.tall_matmul(x, w, transposed=True)
        assert torch.equal(first, x.mm(w.t()))
        w.add_(1.0)
        assert torch.equal(bf.tall_matmul(x, w, transposed=True), x.mm(w.t()))
    config.matrix_cores = "fp32"
    with torch.no_grad():
        assert torch.equal(bf.tall_matmul(x, w, transposed=True), x.mm(w.t()))   # the framework's GEMM


@pytest.mark.parametrize("cores", ["bf16", "fp32"])
@pytest.mark.parametrize("N,K,D", [(20000, 1024, 1024), (16384, 1000, 513), (50000, 1, 1), (30011, 7, 1024), (169343, 256, 256)])
def test_weight_gradient_limits_of_the_wrapper(cuda, N, K, D, cores):
    """The widest operands the wrapper hands to the kernel, and the narrowest;
    random operands with rows of very different size within 1e-5 of the sum of
    the absolute terms."""
    print(f"case dW N={N} K={K} D={D} {cores}", flush=True)
    config.matrix_cores = cores
    dy, x = _ints((N, K), cuda, 1), _ints((N, D), cuda, 2)
    assert torch.equal(bf.weight_gradient(dy, x), (dy.double().t() @ x.double()).float())
    g = torch.Generator(device=cuda).manual_seed(3)
    spread = torch.exp(8 * torch.rand(N, 1, generator=g, device=cuda) - 4)
    dy, x = torch.randn(N, K, generator=g, device=cuda) * spread, torch.randn(N, D, generator=g, device=cuda) * spread
    want = dy.double().t() @ x.double()
    bound = dy.abs().double().t() @ x.abs().double()
    assert ((bf.weight_gradient(dy, x).double() - want).abs() <= 1e-5 * bound + 1e-30).all()


@pytest.mark.parametrize("N,K", [(2449029, 47), (2449029, 256), (169343, 40), (232965, 41), (169343, 256)])
def test_column_sums_at_benchmark_size(cuda, N, K):
    """exact_colsum_f32 (the bias gradient, backward_func.cc:90-91): exact on
    small integers, within fp32 summation error of float64 on random data."""
    print(f"case colsum N={N} K={K}", flush=True)
    x = _ints((N, K), cuda, N + K, -8, 9)
    assert torch.equal(bf.column_sums(x), x.double().sum(0).float())
    g = torch.Generator(device=cuda).manual_seed(K)
    y = torch.randn(N, K, generator=g, device=cuda)
    err = (bf.column_sums(y).double() - y.double().sum(0)).abs().max().item()
    assert err <= 1e-6 * y.abs().double().sum(0).max().item()


@pytest.mark.parametrize("N,K", [(20000, 602), (169343, 300), (5000, 8192), (4099, 257)])
def test_column_sums_wider_than_256_through_the_c_abi(cuda, N, K):
    """The wide form of the column-sum kernel (more than 256 columns), which
    the Python wrapper does not use: straight through the C ABI."""
    print(f"case colsum wide N={N} K={K}", flush=True)
    x = _ints((N, K), cuda, N + K, -8, 9)
    out = torch.full((K + 8,), -77.0, device=cuda)
    rc = _lib.lib().exact_colsum_f32(x.data_ptr(), N, K, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    assert torch.equal(out[:K], x.double().sum(0).float()) and (out[K:] == -77.0).all()


@pytest.mark.parametrize("path", ["fp32", "split", "signs"])
@pytest.mark.parametrize("N,k,D", [(169343, 32, 256), (232965, 76, 602), (232965, 32, 256), (2449029, 25, 100),
                                   (2449029, 64, 256)])
def test_rp2input_at_benchmark_size(cuda, N, k, D, path):
    """rp2input (ops.py:121-125) = X_r . R^T through exact_rp_bwd_f32 /
    exact_rp_bwd_bf16_f32 at the shapes of the three configurations, on every
    matrix-core path: every element within 1e-5 of a float64 product, and
    sampled rows against the oracle's own routine."""
    from exact_amd import ops
    print(f"case rp2input N={N} k={k} D={D} {path}", flush=True)
    rng = np.random.default_rng(N + k)
    R = o.rademacher_matrix(D, k, rng)
    g = torch.Generator(device=cuda).manual_seed(N + D)
    xr = torch.randn(N, k, generator=g, device=cuda)
    r = dev(R)
    config.matrix_cores = "fp32" if path == "fp32" else "bf16"
    if path == "signs":
        r._exact_sign_matrix = True
    got = ops.rp2input(xr, (N, D), r)
    assert got.shape == (N, D)
    want = xr.double() @ r.double().t()
    scale = want.abs().max().item()
    assert (got.double() - want).abs().max().item() <= 1e-5 * scale
    rows = torch.arange(0, N, max(1, N // 2048), device=cuda)
    want_rows = o.rp2input(xr[rows].cpu().numpy(), R)
    np.testing.assert_allclose(got[rows].cpu().numpy(), want_rows, rtol=1e-5, atol=1e-5 * np.abs(want_rows).max())


# ---- the remaining kernels at kernel level ---------------------------------------------------------
def _csr(M, N, nnz, seed, empty_rows=True):
    rng = np.random.default_rng(seed)
    r = rng.integers(0, M, nnz)
    if empty_rows:
        r[r % 7 == 3] = 0
    A = sp.coo_matrix((rng.standard_normal(nnz).astype(np.float32), (r, rng.integers(0, N, nnz))), shape=(M, N)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    return A


def _minmax_vectorised(rowptr, col, val, X, is_max):
    """Second restatement of max / min aggregation for graphs too large for the
    oracle's entry-by-entry loop: segment extreme with reduceat, arg = the
    smallest entry index that attains it (the first extreme entry in CSR
    order, reducer.cuh:62-66).  Held to the oracle's loop in the test below."""
    rowptr, col = np.asarray(rowptr, np.int64), np.asarray(col, np.int64)
    M, K, nnz = rowptr.size - 1, X.shape[1], col.size
    T = X[col] if val is None else (np.asarray(val, np.float32)[:, None] * X[col]).astype(np.float32)
    deg = np.diff(rowptr)
    rows = np.nonzero(deg > 0)[0]
    out = np.zeros((M, K), np.float32)
    arg = np.full((M, K), nnz, np.int64)
    if rows.size:
        red = np.maximum if is_max else np.minimum
        ext = red.reduceat(T, rowptr[rows], axis=0)          # rows.size x K (segments end at the next start)
        # reduceat runs a segment to the next listed start; rows without entries between two listed rows own no entry
        out[rows] = ext
        row_of = np.repeat(np.arange(M), deg)
        hit = T == out[row_of]
        idx = np.where(hit, np.arange(nnz)[:, None], nnz)
        arg[rows] = np.minimum.reduceat(idx, rowptr[rows], axis=0)
    return out, arg


@pytest.mark.parametrize("idx", [torch.int64, torch.int32])
@pytest.mark.parametrize("valued", [True, False])
@pytest.mark.parametrize("is_max", [True, False])
@pytest.mark.parametrize("M,N,K", [(60, 40, 256), (33, 50, 40), (20, 20, 602), (45, 30, 7), (9, 12, 1)])
def test_minmax_kernel_against_the_oracle(cuda, M, N, K, is_max, valued, idx):
    A = _csr(M, N, M * 6, M + K)
    X = np.random.default_rng(K).standard_normal((N, K)).astype(np.float32)
    X[1] = X[2]
    val = A.data if valued else None
    fw = ext_spmm.spmm_max_fw if is_max else ext_spmm.spmm_min_fw
    out, arg = fw(dev(A.indptr).to(idx), dev(A.indices).to(idx), None if val is None else dev(val), dev(X))
    wout, warg = ox.spmm_minmax(A.indptr, A.indices, val, X, is_max)
    assert np.array_equal(out.cpu().numpy().view(np.uint32), wout.view(np.uint32))
    assert arg.dtype == idx and np.array_equal(arg.cpu().numpy().astype(np.int64), warg)
    vout, varg = _minmax_vectorised(A.indptr, A.indices, val, X, is_max)
    assert np.array_equal(vout.view(np.uint32), wout.view(np.uint32)) and np.array_equal(varg, warg)


@pytest.mark.parametrize("is_max", [True, False])
def test_minmax_kernel_on_a_100k_row_graph(cuda, is_max):
    n, K = 100_000, 24
    A = powerlaw_csr(n, int(n * 5), 11)
    rng = np.random.default_rng(5)
    A.data[:] = rng.standard_normal(A.nnz).astype(np.float32)
    X = rng.standard_normal((n, K)).astype(np.float32)
    fw = ext_spmm.spmm_max_fw if is_max else ext_spmm.spmm_min_fw
    for val in (A.data, None):
        out, arg = fw(dev(A.indptr.astype(np.int32)), dev(A.indices.astype(np.int32)), None if val is None else dev(val),
                      dev(X))
        wout, warg = _minmax_vectorised(A.indptr, A.indices, val, X, is_max)
        assert np.array_equal(out.cpu().numpy().view(np.uint32), wout.view(np.uint32))
        assert np.array_equal(arg.cpu().numpy().astype(np.int64), warg)


@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("M,N,K", [(60, 40, 256), (33, 50, 40), (20, 20, 602), (45, 30, 7), (9, 12, 1), (30, 30, 1000),
                                   (100_000, 100_000, 40)])
def test_sddmm_kernel_against_the_oracle(cuda, M, N, K, reduce):
    A = _csr(M, N, M * 5, M * 3 + K) if M < 1000 else powerlaw_csr(M, M * 5, 12)
    rng = np.random.default_rng(K)
    mat, grad = rng.standard_normal((N, K)).astype(np.float32), rng.standard_normal((M, K)).astype(np.float32)
    row = np.repeat(np.arange(M), np.diff(A.indptr))
    want = ox.sddmm(row, A.indptr, A.indices, mat, grad, reduce)
    for idx in (torch.int64, torch.int32):
        got = ext_spmm.spmm_value_bw(dev(row).to(idx), dev(A.indptr).to(idx), dev(A.indices).to(idx), dev(mat), dev(grad),
                                     reduce)
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=1e-5, atol=1e-5 * np.abs(want).max())


@pytest.mark.parametrize("n", [1, 5, 33, 257, 2049, 10007, 169343 * 256])
def test_leaky_relu_kernel_against_the_oracle(cuda, n):
    L = _lib.lib()
    sp_ = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(n % 1000)
    x, gy = torch.randn(n, generator=g), torch.randn(n, generator=g)
    xd, gd = x.to(cuda), gy.to(cuda)
    words = (n + 31) // 32
    for slope in (0.2, 0.01):
        y = torch.empty_like(xd)
        mask = torch.full((words + 4,), 0x5A5A5A5A, dtype=torch.int32, device=cuda)
        assert L.exact_leaky_relu_fwd_f32(xd.data_ptr(), n, slope, y.data_ptr(), mask.data_ptr(), sp_) == 0
        wy, wm = ox.leaky_relu_fwd(x.numpy(), slope)
        got_mask = mask.cpu().numpy().view(np.uint32)
        assert np.array_equal(y.cpu().numpy().view(np.uint32), wy.view(np.uint32))
        assert np.array_equal(got_mask[:words], wm) and (got_mask[words:] == 0x5A5A5A5A).all()
        dx = torch.empty_like(gd)
        assert L.exact_leaky_relu_bwd_f32(gd.data_ptr(), mask.data_ptr(), n, slope, dx.data_ptr(), sp_) == 0
        assert np.array_equal(dx.cpu().numpy().view(np.uint32), ox.leaky_relu_bwd(gy.numpy(), wm, slope).view(np.uint32))


# ---- one training step of the 3-layer GCN configuration at full size -------------------------------
def test_one_full_size_step_of_the_deep_gcn_against_the_oracle_model(cuda):
    """Configuration 3 at its full size (169,343 nodes, 3 layers 128 -> 256 ->
    256 -> 40, batch norm, ReLU, dropout 0.5, INT2): one forward + backward of
    the reference's loop (arxiv/train_full_batch.py:256-266) with the noise
    supplied to both sides; loss within 1e-3 of the oracle model's and every
    parameter gradient within 1e-3 of its norm."""
    import exact_amd as exact
    from exact_amd.models import GCN
    from exact_amd.sparse import SparseTensor, gcn_norm
    from test_layers import _flat, _params_of_gcn, wire_noise
    n, feat, hidden, classes = 169343, 128, 256, 40
    A = powerlaw_csr(n, 1_160_000, 1)
    adj = gcn_norm(SparseTensor.from_scipy(A).set_value(None), add_self_loops=True)
    rowptr, col, value = adj.csr()
    graph = om.Graph(rowptr.numpy(), col.numpy(), value.numpy())
    adj = adj.to(cuda).fill_cache_()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(n, feat, generator=g)
    labels = torch.randint(0, classes, (n,), generator=g)
    train_idx = torch.randperm(n, generator=g)[: n // 2]
    torch.manual_seed(7)
    model = exact.QModule(GCN(feat, hidden, classes, 3, dropout=0.5, batch_norm=True)).to(cuda).train()
    params = _params_of_gcn(model)
    other = wire_noise(29)
    print("case cfg3 full-size step: product", flush=True)
    loss = F.nll_loss(F.log_softmax(model(x.to(cuda), adj)[train_idx.to(cuda)], dim=-1), labels[train_idx].to(cuda))
    loss.backward()
    torch.cuda.synchronize()
    print("case cfg3 full-size step: oracle model", flush=True)
    om.use_native(True)
    try:
        c = om.Ctx(2, 1.0, other.noise, None)
        out_o = om.gcn_forward(c, params, graph, x, 0.5, True, None)
        loss_o = F.nll_loss(F.log_softmax(out_o[train_idx], dim=-1), labels[train_idx])
        loss_o.backward()
    finally:
        om.use_native(False)
    print(f"loss {loss.item():.6f} oracle {loss_o.item():.6f}", flush=True)
    assert abs(loss.item() - loss_o.item()) < 1e-3
    m = model.model
    names = [f"conv{i}.weight" for i in range(3)] + [f"conv{i}.bias" for i in range(3)] + \
            [f"bn{i}.weight" for i in range(2)] + [f"bn{i}.bias" for i in range(2)]
    mine = [c_.weight.grad for c_ in m.convs] + [c_.bias.grad for c_ in m.convs if c_.bias is not None] + \
           [b.weight.grad for b in m.bns] + [b.bias.grad for b in m.bns]
    for name, a, b in zip(names, mine, _flat(params)):
        diff, norm = (a.cpu() - b.grad).norm().item(), b.grad.norm().item()
        print(f"{name}: |grad| {norm:.3e} |diff| {diff:.3e}", flush=True)
        # a bias ahead of a batch norm reaches the loss only through the quantisation error of the norm's saved
        # input: its gradient is three orders of magnitude below the others, hence the absolute floor
        assert diff < 1e-3 * norm + 1e-6, (name, diff, norm)
