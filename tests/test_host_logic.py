"""Host-side logic that needs neither a GPU nor the kernels: the config
singleton, the CSR container against scipy, argument checks of the shims, the
`exact` alias, helpers."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import exact_amd
from exact_amd import ops, utils
from exact_amd.conf import QuantizationConfig, config
from exact_amd.cpp_extension import quantization as extq
from exact_amd.cpp_extension import spmm as ext_spmm
from exact_amd.qsheme import QScheme
from exact_amd.sparse import SparseTensor, gcn_norm


def test_config_has_the_reference_fields_and_defaults():
    c = QuantizationConfig()
    want = dict(compress_activation=True, activation_compression_bits=[2], initial_bits=8, stochastic=True,
                use_gradient=False, simulate=False, enable_quantized_bn=True, kept_frac=1.0, single_precision=True,
                dropout2=False, empty_cache_threshold=None, swap=False, amp=False, debug_memory_op_forward=False,
                debug_memory_op_backward=False, debug_remove_bn=False, debug_remove_relu=False,
                debug_remove_dropout=False)
    for k, v in want.items():
        assert getattr(c, k) == v, k
    c.activation_compression_bits.append(4)                 # defaults are not shared between instances
    assert QuantizationConfig().activation_compression_bits == [2]
    assert config is exact_amd.config


def test_install_as_exact_aliases_the_package():
    exact_amd.install_as_exact()
    import exact
    import exact.cpp_extension.quantization as q
    from exact import QModule, config as cfg       # noqa: F401
    from exact.ops import quantize_activation    # noqa: F401
    assert exact is exact_amd and q is extq and cfg is config


def test_compression_off_passes_the_activation_through():
    x = torch.zeros(4, 4)
    config.compress_activation = False
    assert ops.quantize_activation(x, None) == (x, None, None, None)
    assert ops.dequantize_activation((x, None, None, None), x.shape) is x


def test_shims_reject_host_tensors_with_the_reference_messages():
    x, v = torch.zeros(8, 8), torch.zeros(8)
    with pytest.raises(RuntimeError, match="data must be a CUDA tensor!"):
        extq.pack_single_precision(x, v, v, v, 2, True)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor!"):
        extq.act_quantized_relu(x)
    with pytest.raises(RuntimeError, match="input must be a CUDA tensor!"):
        ops.quantize_activation(x, None)
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ext_spmm.spmm_csr(torch.zeros(9, dtype=torch.long), torch.zeros(0, dtype=torch.long), None, x, "sum")
    with pytest.raises(NotImplementedError, match="spmm_max_fw"):
        ext_spmm.spmm_csr(torch.zeros(9, dtype=torch.long), torch.zeros(0, dtype=torch.long), None, x, "max")
    with pytest.raises(RuntimeError, match="must be CUDA tensor"):
        ext_spmm.spmm_max_fw(torch.zeros(9, dtype=torch.long), torch.zeros(0, dtype=torch.long), None, x)


def test_sparse_tensor_matches_scipy():
    rng = np.random.default_rng(0)
    A = sp.random(60, 45, density=0.1, random_state=1, format="csr", dtype=np.float32)
    A.sort_indices()
    t = SparseTensor.from_scipy(A)
    rowptr, col, val = t.csr()
    assert np.array_equal(rowptr.numpy(), A.indptr) and np.array_equal(col.numpy(), A.indices)
    st = t.fill_cache_().storage
    At = A.T.tocsr()
    At.sort_indices()
    assert np.array_equal(st.colptr().numpy(), At.indptr)
    assert np.array_equal(st.row()[st.csr2csc()].numpy(), At.indices)
    assert np.array_equal(val[st.csr2csc()].numpy(), At.data)
    assert np.array_equal(st.rowcount().numpy(), np.diff(A.indptr))
    assert np.allclose(t.to_dense().numpy(), A.toarray())
    coo = A.tocoo()
    perm = rng.permutation(coo.nnz)
    t2 = SparseTensor.from_edge_index(torch.from_numpy(coo.row[perm]).long(), torch.from_numpy(coo.col[perm]).long(),
                                      torch.from_numpy(coo.data[perm]), (60, 45))
    assert np.array_equal(t2.csr()[0].numpy(), A.indptr) and np.array_equal(t2.csr()[1].numpy(), A.indices)
    t32 = SparseTensor.from_scipy(A).fill_cache_().to_int32_()
    assert all(getattr(t32.storage, n).dtype == torch.int32 for n in ("_rowptr", "_col", "_row", "_colptr", "_csr2csc"))
    assert t.set_value(None).csr()[2] is None and t.nnz() == A.nnz and t.sparse_sizes() == (60, 45)


def test_gcn_norm_matches_closed_form():
    A = sp.random(40, 40, density=0.1, random_state=2, format="csr", dtype=np.float32)
    A = ((A + A.T) != 0).astype(np.float32).tolil()
    A.setdiag(0)
    A = A.tocsr()
    A.eliminate_zeros()
    adj = gcn_norm(SparseTensor.from_scipy(A).set_value(None), add_self_loops=True)
    At = A + sp.eye(40, dtype=np.float32)
    d = np.asarray(At.sum(1)).reshape(-1) ** -0.5
    np.testing.assert_allclose(adj.to_dense().numpy(), (sp.diags(d) @ At @ sp.diags(d)).toarray(), rtol=1e-6, atol=1e-7)


def test_helpers():
    assert utils.cast_low_bit_int(torch.arange(10)).dtype == torch.int32
    assert utils.cast_low_bit_int(torch.tensor([2 ** 40])).dtype == torch.int64
    assert utils.cast_low_bit_int(None) is None
    ts = [torch.zeros(3, 4), torch.zeros(5, dtype=torch.int8), torch.zeros(2, dtype=torch.bfloat16), torch.zeros(7, dtype=torch.long)]
    assert utils.compute_tensor_bytes(ts) == 48 + 5 + 4 + 56 and utils.compute_tensor_bytes(ts[0]) == 48
    rec = utils.GlobalExpRecorder()
    rec.record("a", np.float32(1.23456789))
    rec.record("b", np.int64(3))
    assert rec.val_dict == {"a": 1.234568, "b": 3}
    n0 = len(QScheme.layers)
    a, b = QScheme("linear"), QScheme("linear")
    assert int(b.name.split("_")[1]) == int(a.name.split("_")[1]) + 1 and len(QScheme.layers) == n0 + 2
    with pytest.raises(ValueError):
        QScheme("conv")
    assert ops.kept_columns(256) == 256
    config.kept_frac = 0.125
    assert ops.kept_columns(256) == 32 and ops.kept_columns(602) == 76
    config.kept_frac = 0.25
    assert ops.kept_columns(100) == 25


def test_transpose_operands_are_kept_per_graph_and_die_with_it():
    """The gathered CSC operands of backward are attached to the graph's own
    csr2csc tensor: a second call reuses them, new edge values replace the one
    slot, values that require grad are never kept, and a graph that goes away
    leaves nothing behind."""
    import gc

    import torch

    from exact_amd.cpp_extension import spmm as ext_spmm
    ext_spmm.clear_csc_cache()

    def graph(seed):
        g = torch.Generator().manual_seed(seed)
        row = torch.sort(torch.randint(0, 50, (400,), generator=g)).values
        csr2csc = torch.randperm(400, generator=g)
        rowcount = torch.bincount(row, minlength=50)
        return row, csr2csc, rowcount, torch.rand(400, generator=g)

    row, csr2csc, rowcount, value = graph(0)
    a = ext_spmm._csc_operands("sum", row, value, None, csr2csc, True, torch.float32)
    b = ext_spmm._csc_operands("sum", row, value, None, csr2csc, True, torch.float32)
    assert a[0] is b[0] and a[1] is b[1] and torch.equal(a[1], value[csr2csc]) and torch.equal(a[0], row[csr2csc])
    m = ext_spmm._csc_operands("mean", row, None, rowcount, csr2csc, False, torch.float32)
    assert m[0] is a[0] and torch.equal(m[1], 1.0 / rowcount[row[csr2csc]].clamp(min=1).float())
    value.mul_(2.0)                                           # same storage, new version: the slot is rebuilt
    c = ext_spmm._csc_operands("sum", row, value, None, csr2csc, True, torch.float32)
    assert c[1] is not a[1] and torch.equal(c[1], value[csr2csc]) and len(ext_spmm._CSC_CACHE) == 1
    # two different tensors of version 0 at the same address (what the caching allocator produces when edge
    # weights are recomputed every step): the address must not be taken for the tensor
    import numpy as np
    buf = np.random.default_rng(0).random(400, dtype=np.float32)
    first = torch.from_numpy(buf)
    f = ext_spmm._csc_operands("sum", row, first, None, csr2csc, True, torch.float32)
    assert torch.equal(f[1], first[csr2csc])
    assert ext_spmm._CSC_CACHE[csr2csc]["sum"][0] is first     # held: its block cannot be reused while the slot lives
    kept_first = first.clone()
    del first
    ext_spmm._CSC_CACHE[csr2csc]["sum"] = (kept_first, 0, f[1])         # the slot as the allocator would leave it
    buf[:] = np.random.default_rng(1).random(400, dtype=np.float32)
    second = torch.from_numpy(buf)
    assert second._version == 0
    s2 = ext_spmm._csc_operands("sum", row, second, None, csr2csc, True, torch.float32)
    assert torch.equal(s2[1], second[csr2csc]) and not torch.equal(s2[1], f[1])
    alias = second.detach()                                    # another wrapper of the same storage does hit
    s3 = ext_spmm._csc_operands("sum", row, alias, None, csr2csc, True, torch.float32)
    assert s3[1] is s2[1]
    del kept_first, second, alias, f, s2, s3
    learned = value.clone().requires_grad_()
    d = ext_spmm._csc_operands("sum", row, learned, None, csr2csc, True, torch.float32)
    e = ext_spmm._csc_operands("sum", row, learned, None, csr2csc, True, torch.float32)
    assert d[1] is not e[1] and not d[1].requires_grad
    for seed in range(1, 30):                                 # a graph rebuilt every step
        r2, p2, rc2, v2 = graph(seed)
        ext_spmm._csc_operands("mean", r2, v2, rc2, p2, True, torch.float32)
        del r2, p2, rc2, v2
    gc.collect()
    assert len(ext_spmm._CSC_CACHE) == 1
    del row, csr2csc, rowcount, value, a, b, c, m
    gc.collect()
    assert len(ext_spmm._CSC_CACHE) == 0
