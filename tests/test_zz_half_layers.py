"""fp16 activations through the Python layers (what the reference's Functions
see under autocast, ops.py:130, 260, 313): compress / restore against
oracle/exact_oracle_half.py, the mask layers, the linear and sparse products,
a GCN step in fp16, and -- GPU only -- a training step under torch.autocast."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

import exact_amd as exact
import exact_oracle_half as oh
from exact_amd import ops
from exact_amd.conf import config
from exact_amd.cpp_extension import quantization as extq
from exact_amd.cpp_extension import spmm as ext_spmm
from exact_amd.models import GCN
from exact_amd.sparse import SparseTensor, gcn_norm
from gpu_util import FixedNoise, all_finite_halves, bytes_equal

F16, F32 = np.float16, np.float32


def graph(n, m, seed, backend):
    rng = np.random.default_rng(seed)
    A = sp.coo_matrix((np.ones(m, F32), (rng.integers(0, n, m), rng.integers(0, n, m))), shape=(n, n)).tocsr()
    A.data[:] = 1.0
    A.sort_indices()
    return A, gcn_norm(SparseTensor.from_scipy(A).set_value(None), add_self_loops=True).to(backend)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", [(203, 256), (61, 602), (37, 25), (16, 1024)])
def test_compress_restore_fp16_matches_oracle(backend, N, G, bits):
    rng = np.random.default_rng(N + G + bits)
    x = (rng.standard_normal((N, G)) * 3).astype(F16)
    x[1] = x[1, 0]                                              # a constant row: scale inf, codes 0
    x[2] = (rng.standard_normal(G) * 2e-6).astype(F16)          # a spread whose reciprocal overflows fp16: scale inf, codes saturate
    noise = rng.random((N, G), dtype=F32)
    config.noise_source = FixedNoise([torch.from_numpy(noise)])
    config.activation_compression_bits = [bits]
    xt = torch.from_numpy(x).to(backend)
    packed, qbits, scale, mn = ops.quantize_activation(xt, None)
    wp, ws, wm = oh.quantize_activation(x, bits, noise)
    assert qbits == bits and scale.dtype == torch.float16 and mn.dtype == torch.float16     # reference ops.py:82-83
    assert bytes_equal(packed, wp) and bytes_equal(scale, ws) and bytes_equal(mn, wm)
    restored = ops.dequantize_activation((packed, qbits, scale, mn), xt.shape)
    assert restored.dtype == torch.float16 and restored.shape == xt.shape
    want = oh.unpack(wp, bits, ws, wm, N, G)
    finite = ~np.isnan(want)                                    # 0 / inf scale rows restore to min; nothing is NaN there, but stay safe
    assert np.array_equal(restored.cpu().numpy().view(np.uint16)[finite], want.view(np.uint16)[finite])
    out = extq.unpack_single_precision(packed, bits, scale, mn, N, G)
    assert np.array_equal(out.cpu().numpy().view(np.uint16)[finite], want.view(np.uint16)[finite])


def test_mask_layers_fp16(backend):
    rng = np.random.default_rng(0)
    x = (rng.standard_normal((100, 48)) * 3).astype(F16)
    g = (rng.standard_normal((100, 48)) * 3).astype(F16)
    u = rng.random((100, 48), dtype=F32)
    xt = torch.from_numpy(x).to(backend).requires_grad_()
    gt = torch.from_numpy(g).to(backend)
    y = exact.QReLU().train()(xt)
    y.backward(gt)
    wy, wm = oh.relu_fwd(x.reshape(-1))
    assert y.dtype == torch.float16 and bytes_equal(y, wy) and bytes_equal(xt.grad, oh.relu_bwd(g.reshape(-1), wm))
    xt.grad = None
    y = exact.QLeakyReLU(0.2).train()(xt)
    y.backward(gt)
    wy, wm = oh.leaky_relu_fwd(x.reshape(-1), 0.2)
    assert bytes_equal(y, wy) and bytes_equal(xt.grad, oh.leaky_relu_bwd(g.reshape(-1), wm, 0.2))
    for layer, relu in ((exact.QDropout(0.4), False), (exact.QReLUDropout(0.4), True)):
        xt.grad = None
        config.noise_source = FixedNoise([torch.from_numpy(u)])
        y = layer.train()(xt)
        y.backward(gt)
        wy, wm = oh.dropout_fwd(x.reshape(-1), 0.4, u.reshape(-1), relu=relu)
        assert y.dtype == torch.float16 and bytes_equal(y, wy)
        assert bytes_equal(xt.grad, oh.dropout_bwd(g.reshape(-1), wm, 0.4))
        assert ops.take_compressed(y) is None               # the one-pass quantiser is fp32 only


def test_mask_layers_fp16_round_twice_on_every_operand(backend):
    """Every finite fp16 value through LeakyReLU (slope 0.1) and dropout
    (p = 0.4), forward and backward: constants at which a kernel that rounds
    the exact product once differs from at::Half's two roundings in thousands
    of these operands (tests/test_oracle_half.py)."""
    x = all_finite_halves()
    ones = np.ones(x.size, F32)
    xt = torch.from_numpy(x).to(backend).requires_grad_()
    y = exact.QLeakyReLU(0.1).train()(xt)
    y.backward(torch.from_numpy(-np.abs(x)).to(backend))     # gradient operand on the scaled side as well
    wy, wm = oh.leaky_relu_fwd(x, 0.1)
    assert bytes_equal(y, wy) and bytes_equal(xt.grad, oh.leaky_relu_bwd(-np.abs(x), wm, 0.1))
    xt.grad = None
    config.noise_source = FixedNoise([torch.from_numpy(ones)])
    y = exact.QDropout(0.4).train()(xt)
    y.backward(xt.detach())
    wy, wm = oh.dropout_fwd(x, 0.4, ones)
    assert bytes_equal(y, wy) and bytes_equal(xt.grad, oh.dropout_bwd(x, wm, 0.4))


def test_linear_and_sparse_products_fp16(backend):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(300, 64, generator=g).half().to(backend)
    w = (torch.randn(16, 64, generator=g) * 0.2).half().to(backend).requires_grad_()
    dy = torch.randn(300, 16, generator=g).half().to(backend)
    # 4 bits: at 8 bits the fp16 rounding of the scale (relative error up to ~7e-4, i.e. 0.2 of a level at 255)
    # makes the unclamped 256 -> 0 wrap of a row's largest element (reference kernel, no upper clamp) frequent
    config.activation_compression_bits = [4]
    xq = x.clone().requires_grad_()
    y = ops.qlinear.apply(xq, w, None, None, None, None, True)
    assert y.dtype == torch.float16 and torch.equal(y, F.linear(x, w.detach()))
    y.backward(dy)
    want_w = dy.float().t().mm(x.float())
    assert w.grad.dtype == torch.float16
    assert (w.grad.float() - want_w).norm() / want_w.norm() < 0.3     # INT4 noise: ~0.2 expected
    assert (xq.grad.float() - dy.float().mm(w.detach().float())).abs().max() < 0.05
    # projected: the GEMMs with the projection matrix are library GEMMs in fp16
    config.kept_frac = 0.25
    w.grad = None
    ops.qlinear.apply(x.clone().requires_grad_(), w, None, None, None, None, True).backward(dy)
    assert torch.isfinite(w.grad).all() and w.grad.dtype == torch.float16
    config.kept_frac = 1.0
    # sparse product: gather and accumulate in fp32, one rounding of the result
    A, adj = graph(300, 2000, 1, backend)
    rowptr, col, value = adj.csr()
    out = ext_spmm.spmm_csr(rowptr, col, value, x, "sum")
    want = ext_spmm.spmm_csr(rowptr, col, value, x.float(), "sum").half()
    assert out.dtype == torch.float16 and torch.equal(out, want)


def test_gcn_step_in_fp16(backend):
    """The whole layer stack on fp16 tensors (weights included), without
    BatchNorm -- torch's CPU batch norm has no fp16 kernel for the emulated run."""
    _, adj = graph(200, 1500, 2, backend)
    torch.manual_seed(1)
    model = exact.QModule(GCN(32, 64, 5, 3, dropout=0.5, batch_norm=False)).to(backend).half().train()
    x = torch.randn(200, 32).half().to(backend)
    labels = torch.randint(0, 5, (200,)).to(backend)
    out = model(x, adj)
    assert out.dtype == torch.float16
    F.cross_entropy(out.float(), labels).backward()
    assert all(p.grad is not None and p.grad.dtype == torch.float16 and torch.isfinite(p.grad).all()
               for p in model.parameters())


@pytest.mark.gpu
def test_training_step_under_autocast(cuda):
    """torch.autocast: the Functions cast their inputs to fp16 (custom_fwd), the
    kept activations are the fp16 ones, parameters and their gradients stay fp32
    (the bias additions promote the layer outputs back to fp32)."""
    seen = []
    real = extq.minmax_pack
    import unittest.mock as mock
    _, adj = graph(500, 4000, 3, cuda)
    torch.manual_seed(2)
    model = exact.QModule(GCN(32, 64, 5, 3, dropout=0.5, batch_norm=True)).to(cuda).train()
    x = torch.randn(500, 32, device=cuda)
    labels = torch.randint(0, 5, (500,), device=cuda)
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    losses = []
    with mock.patch.object(extq, "minmax_pack", lambda data, bits, want_fp32=False: seen.append(data.dtype) or real(data, bits, want_fp32)):
        for _ in range(5):
            opt.zero_grad()
            with torch.autocast("cuda", dtype=torch.float16):
                out = model(x, adj)
                loss = F.cross_entropy(out.float(), labels)
            loss.backward()
            opt.step()
            losses.append(loss.item())
    assert torch.float16 in seen                     # the linear layers compressed fp16 copies of their inputs
    assert all(np.isfinite(l) for l in losses)
    assert all(p.grad is not None and p.grad.dtype == torch.float32 and torch.isfinite(p.grad).all()
               for p in model.parameters())
