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
    # |d/dx elu| differs by at most |g| * exp(max(x, x_hat)) * |x_hat - x| <= |g| * |x_hat - x|, and an 8-bit copy with
    # bf16 scale / min is within range / 255 + 2^-8 * (|min| + range) of x: below 0.08 for N(0, 1) rows of 32
    assert ((x2.grad - x2r.grad).abs() <= 0.08 * g2.abs() + 1e-6).all() and not torch.equal(x2.grad, x2r.grad)
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


# ------------------------------------------------------------ fused epilogues (emulated kernels)
def _chain(x, prob, bits, act_noise, noise):
    """The chain the fused kernels replace, from the oracle's separate ops."""
    N, G = x.shape
    y1, m1 = o.relu_fwd(x.reshape(-1))
    y2, m2 = o.dropout_fwd(y1, prob, act_noise.reshape(-1))
    y2 = y2.reshape(N, G)
    packed, _, sbf, mbf, scale, mn = o.quantize_activation(y2, bits, noise)
    return y2, m1 & m2, packed, scale, mn, sbf, mbf


@pytest.mark.parametrize("n", [1, 7, 33, 257, 2049, 10007])
@pytest.mark.parametrize("supplied", [True, False])
def test_relu_dropout_kernel_equals_the_two_kernels(n, supplied):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(F32)
    noise = rng.random(n, dtype=F32) if supplied else o.philox_noise_flat(77, 5, n)
    y, mask = e.relu_dropout_fwd(x, 0.4, noise if supplied else None, 77, 5)
    y1, m1 = o.relu_fwd(x)
    y2, m2 = o.dropout_fwd(y1, 0.4, noise)
    assert np.array_equal(y.view(np.uint32), y2.view(np.uint32)) and np.array_equal(mask, m1 & m2)
    # backward of the pair = dropout backward on the joint mask
    g = rng.standard_normal(n).astype(F32)
    want = o.relu_bwd(o.dropout_bwd(g, m2, 0.4), m1)
    assert np.array_equal(e.dropout_bwd(g, mask, 0.4).view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", [(1, 8), (5, 16), (37, 40), (64, 256), (203, 256), (100, 128), (33, 1024), (19, 520),
                                 (129, 104), (12, 768)])
@pytest.mark.parametrize("supplied", [True, False])
def test_relu_dropout_pack_kernel_equals_the_chain(N, G, bits, supplied):
    rng = np.random.default_rng(N * 1000 + G + bits)
    x = (rng.standard_normal((N, G)) * 2).astype(F32)
    if N > 3:
        x[2] = -np.abs(x[2])                      # a row that ReLU zeroes entirely -> constant row
    if supplied:
        act_noise, noise = rng.random((N, G), dtype=F32), rng.random((N, G), dtype=F32)
    else:
        act_noise = o.philox_noise_flat(11, 3, N * G).reshape(N, G)
        noise = o.philox_noise_rows(12, 4, N, G)
    got = e.relu_dropout_minmax_pack(x, 0.5, bits, act_noise if supplied else None, noise if supplied else None,
                                     11, 3, 12, 4)
    want = _chain(x, 0.5, bits, act_noise, noise)
    names = ("y", "mask", "packed", "scale", "min", "scale_bf16", "min_bf16")
    for name, g_, w_ in zip(names, got, want):
        g_, w_ = np.ascontiguousarray(g_), np.ascontiguousarray(w_)
        assert g_.shape == w_.shape or g_.size == w_.size, name
        assert g_.tobytes() == w_.tobytes(), name


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", [(1, 8), (37, 40), (64, 256), (203, 256), (33, 1024), (129, 104)])
@pytest.mark.parametrize("supplied", [True, False])
def test_bn_relu_dropout_pack_kernel_equals_the_chain_on_the_normalised_input(N, G, bits, supplied):
    rng = np.random.default_rng(N * 999 + G + bits)
    x = (rng.standard_normal((N, G)) * 3 + 1).astype(F32)
    mean = rng.standard_normal(G).astype(F32)
    mult = (rng.random(G, dtype=F32) + F32(0.5)) * np.where(rng.random(G) < 0.2, F32(-1), F32(1)).astype(F32)
    shift = rng.standard_normal(G).astype(F32)
    if supplied:
        act_noise, noise = rng.random((N, G), dtype=F32), rng.random((N, G), dtype=F32)
    else:
        act_noise = o.philox_noise_flat(21, 8, N * G).reshape(N, G)
        noise = o.philox_noise_rows(22, 12, N, G)
    got = e.relu_dropout_minmax_pack(x, 0.25, bits, act_noise if supplied else None, noise if supplied else None,
                                     21, 8, 22, 12, norm=(mean, mult, shift))
    normalised = ((x - mean[None, :]) * mult[None, :] + shift[None, :]).astype(F32)   # three fp32 roundings
    want = _chain(normalised, 0.25, bits, act_noise, noise)
    for name, g_, w_ in zip(("y", "mask", "packed", "scale", "min", "scale_bf16", "min_bf16"), got, want):
        assert np.ascontiguousarray(g_).tobytes() == np.ascontiguousarray(w_).tobytes(), name
    # the identity normalisation is the plain kernel
    plain = e.relu_dropout_minmax_pack(x, 0.25, bits, act_noise if supplied else None, noise if supplied else None,
                                       21, 8, 22, 12)
    ident = e.relu_dropout_minmax_pack(x, 0.25, bits, act_noise if supplied else None, noise if supplied else None,
                                       21, 8, 22, 12, norm=(np.zeros(G, F32), np.ones(G, F32), np.zeros(G, F32)))
    for a_, b_ in zip(plain, ident):
        assert np.ascontiguousarray(a_).tobytes() == np.ascontiguousarray(b_).tobytes()


def test_bn_relu_dropout_pack_kernel_rejects_missing_vectors():
    x = np.zeros((4, 16), F32)
    v = np.zeros(16, F32)
    assert e.relu_dropout_minmax_pack(x, 0.5, 2, norm=(v, None, v), expect_rc=-1) is None
    assert e.relu_dropout_minmax_pack(np.zeros((4, 12), F32), 0.5, 2, norm=(v, v, v), expect_rc=-3) is None


def test_relu_dropout_pack_kernel_rejects_what_it_cannot_do():
    x = np.zeros((4, 12), F32)
    assert e.relu_dropout_minmax_pack(x, 0.5, 2, expect_rc=-3) is None          # G % 8 != 0
    assert e.relu_dropout_minmax_pack(np.zeros((2, 1032), F32), 0.5, 2, expect_rc=-3) is None
    assert e.relu_dropout_minmax_pack(np.zeros((4, 16), F32), 1.0, 2, expect_rc=-5) is None
    assert e.relu_dropout_minmax_pack(np.zeros((4, 16), F32), 0.5, 3, expect_rc=-2) is None
    assert e.relu_dropout_minmax_pack(np.zeros((4, 16), F32), 0.5, 2, act_noise=np.zeros((4, 16), F32), expect_rc=-5) is None


# ------------------------------------------------------------ fused epilogue (layers, both back ends)
def _train_steps(backend, fuse, noise_seed, philox_seed, kept_frac=1.0, bits=2, steps=3, hidden=64, fold_bn=False):
    """A few SGD steps of a 3-layer GCN; -> (losses, final weights)."""
    from exact_amd.models import GCN
    from exact_amd.sparse import gcn_norm
    from gpu_util import SeededNoise
    config.fuse_epilogue = fuse
    config.fold_batch_norm = fold_bn
    config.kept_frac = kept_frac
    config.activation_compression_bits = [bits]
    if noise_seed is None:
        config.noise_source = None
        torch.manual_seed(philox_seed)
        if backend.type == "cuda":
            torch.cuda.manual_seed(philox_seed)
    else:
        s = SeededNoise(noise_seed)
        config.noise_source, config.rp_matrix_source = s.noise_source, s.rp_matrix_source
    A = csr(300, 300, 2400, 9, empty_rows=False)
    adj = gcn_norm(SparseTensor.from_scipy(A).set_value(None), add_self_loops=True).to(backend)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(300, 48, generator=g).to(backend)
    labels = torch.randint(0, 5, (300,), generator=g).to(backend)
    torch.manual_seed(11)
    net = GCN(48, hidden, 5, 3, dropout=0.5, batch_norm=True)
    model = exact.QModule(net).to(backend).train()
    opt = torch.optim.SGD(model.parameters(), lr=0.05)
    losses = []
    for _ in range(steps):
        opt.zero_grad()
        loss = F.cross_entropy(model(x, adj), labels)
        loss.backward()
        opt.step()
        losses.append(loss.item())
    return losses, [p.detach().cpu().clone() for p in model.parameters()]


def _same_training(backend, l_a, w_a, l_b, w_b):
    if backend.type == "cpu":
        assert l_a == l_b and all(torch.equal(a, b) for a, b in zip(w_a, w_b))
    else:
        # the GPU SpMM adds the partial sums of split rows with fp32 atomics, in no fixed
        # order, so two runs of the SAME configuration already differ in the last bits
        assert np.allclose(l_a, l_b, rtol=0, atol=1e-3)
        assert all(torch.allclose(a, b, rtol=1e-3, atol=1e-3) for a, b in zip(w_a, w_b))


@pytest.mark.parametrize("kept_frac,bits", [(1.0, 2), (1.0, 8), (0.25, 1)])
def test_fused_epilogue_is_bit_identical_to_separate_layers(backend, kept_frac, bits):
    """Same supplied noise in the same order: the fused ReLU -> dropout ->
    quantise pass and the three separate layers give identical training."""
    l_sep, w_sep = _train_steps(backend, False, 5, 0, kept_frac, bits)
    l_fus, w_fus = _train_steps(backend, True, 5, 0, kept_frac, bits)
    _same_training(backend, l_sep, w_sep, l_fus, w_fus)


def test_fused_epilogue_uses_the_handed_over_copy(backend, monkeypatch):
    """kept_frac 1: the consumer adopts the copy made by the fused pass (no
    second quantisation of that tensor); an in-place change voids it."""
    from exact_amd import ops
    config.noise_source = None
    x = torch.randn(64, 32, device=backend)
    layer = exact.QReLUDropout(0.5).train()
    y = layer(x)
    q = ops.take_compressed(y)
    assert q is not None and q[1] == 2 and ops.take_compressed(y) is None       # taken once
    restored = ops.dequantize_activation(q, y.shape)
    scale = q[2].float()
    assert ((restored - y).abs() <= (1.0 / scale + 0.01 * y.abs().amax(1)).unsqueeze(1) + 1e-6)[torch.isfinite(scale)].all()
    y2 = layer(x)
    y2.mul_(2.0)
    assert ops.take_compressed(y2) is None                                      # stale after an in-place op
    y3 = layer(x)
    config.activation_compression_bits = [4]
    assert ops.take_compressed(y3) is None                                      # made for another bit width
    config.activation_compression_bits = [2]
    # widths the fused kernel does not take fall back to the mask-only pass
    y4 = layer(torch.randn(10, 12, device=backend))
    assert ops.take_compressed(y4) is None
    # gradient of the pair
    xg = torch.randn(50, 40, device=backend, requires_grad=True)
    yg = layer(xg)
    yg.backward(torch.ones_like(yg))
    assert torch.equal(xg.grad, (yg.detach() != 0).float() * 2.0)
    calls = []
    real = ops.quantize_activation
    monkeypatch.setattr(ops, "quantize_activation", lambda *a, **k: calls.append(1) or real(*a, **k))
    lin = exact.QLinear(40, 8).to(backend).train()
    lin(layer(xg.detach())).sum().backward()
    assert calls == []                                                          # adopted, not re-quantised
    lin(xg.detach()).sum().backward()
    assert calls == [1]


def test_fused_epilogue_with_internal_philox_noise(backend, monkeypatch):
    """Internal noise: the fused pass draws (dropout, quantiser) in the order
    the separate layers do, so a seeded run is again identical."""
    import itertools

    def reseed():
        if backend.type == "cpu":   # the emulated back end numbers its draws itself: restart the numbering
            counter = itertools.count(1)
            monkeypatch.setattr(extq, "next_philox", lambda device: (0xC0FFEE, 4 * next(counter)))

    reseed()
    l_sep, w_sep = _train_steps(backend, False, None, 123)
    reseed()
    l_fus, w_fus = _train_steps(backend, True, None, 123)
    _same_training(backend, l_sep, w_sep, l_fus, w_fus)


@pytest.mark.parametrize("supplied", [True, False])
@pytest.mark.parametrize("N,G,bits", [(203, 256, 2), (64, 128, 1), (37, 40, 4), (33, 1024, 8), (1000, 64, 2)])
def test_fused_shims_match_the_oracle_chain(backend, monkeypatch, N, G, bits, supplied):
    """The two fused entry points through the Python shims, on both back ends,
    against relu -> dropout -> quantize_activation of the oracle (bytes)."""
    from gpu_util import FixedNoise, bytes_equal
    rng = np.random.default_rng(N + G + bits)
    x = (rng.standard_normal((N, G)) * 2).astype(F32)
    x[1] = -np.abs(x[1])
    if supplied:
        act_noise, noise = rng.random((N, G), dtype=F32), rng.random((N, G), dtype=F32)
        config.noise_source = FixedNoise([torch.from_numpy(act_noise), torch.from_numpy(noise), torch.from_numpy(act_noise)])
    else:
        draws = iter([(0xABCDEF12345, 8), (0xABCDEF12345, 12), (0xABCDEF12345, 8)])
        monkeypatch.setattr(extq, "next_philox", lambda device: next(draws))
        act_noise = o.philox_noise_flat(0xABCDEF12345, 8, N * G).reshape(N, G)
        noise = o.philox_noise_rows(0xABCDEF12345, 12, N, G)
    want = _chain(x, 0.3, bits, act_noise, noise)
    xt = torch.from_numpy(x).to(backend)
    y, mask, packed, sbf, mbf = extq.relu_dropout_minmax_pack(xt, 0.3, bits)
    assert bytes_equal(y, want[0]) and bytes_equal(mask, want[1]) and bytes_equal(packed, want[2])
    assert bytes_equal(sbf, want[5]) and bytes_equal(mbf, want[6])
    y2, mask2 = extq.relu_dropout_fwd(xt, 0.3)
    assert bytes_equal(y2, want[0]) and bytes_equal(mask2, want[1])
    g = torch.from_numpy(rng.standard_normal((N, G)).astype(F32)).to(backend)
    want_dx = o.dropout_bwd(g.cpu().numpy().reshape(-1), want[1], 0.3)
    assert bytes_equal(extq.dropout_bwd(g, mask, 0.3), want_dx)


def test_swap_keeps_the_packed_codes_on_the_host(backend):
    """config.swap (reference ops.py:41-42, 50-51): between forward and backward
    the packed codes live in (pinned) host memory; results do not change."""
    from exact_amd import ops
    from gpu_util import SeededNoise
    x = torch.randn(200, 64, device=backend)
    outs = []
    for swap in (False, True):
        config.swap = swap
        s = SeededNoise(3)
        config.noise_source = s.noise_source
        q = ops.quantize_activation(x, None)
        assert q[0].device.type == "cpu" if swap else q[0].device == x.device
        if swap and backend.type == "cuda":
            assert q[0].is_pinned()
        outs.append((q[0].cpu().clone(), ops.dequantize_activation(q, x.shape)))
        lin = exact.QLinear(64, 16).to(backend).train()
        y = lin(exact.QReLUDropout(0.5).train()(x))       # the handed-over copy is offloaded too
        y.sum().backward()
        assert torch.isfinite(lin.weight.grad).all()
        mn, mx = x.min(1).values, x.max(1).values
        packed2, _ = ops.quantize_and_pack(x, 2, mn, mx)
        assert (packed2.device.type == "cpu") == (swap or backend.type == "cpu")
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


def test_simulate_mode(backend):
    """config.simulate (reference ops.py:18-31, 47-48): unpacked int32 codes made
    with tensor ops; within one level of the input, unbiased, usable by the layers."""
    from exact_amd import ops
    config.simulate = True
    for bits in (2, 8):
        config.activation_compression_bits = [bits]
        x = torch.randn(300, 64, device=backend)
        codes, qbits, scale, mn = ops.quantize_activation(x, None)
        assert codes.dtype == torch.int32 and codes.shape == x.shape and qbits == bits
        assert scale.dtype == torch.bfloat16 and int(codes.min()) >= 0 and int(codes.max()) <= 2 ** bits - 1
        xh = ops.dequantize_activation((codes, qbits, scale, mn), x.shape)
        step = (x.max(1).values - x.min(1).values) / (2 ** bits - 1)
        assert ((xh - x).abs() <= 1.05 * step.unsqueeze(1) + 0.02 * x.abs().amax(1, keepdim=True)).all()
    config.activation_compression_bits = [2]
    draws = torch.stack([ops.dequantize_activation(ops.quantize_activation(x, None), x.shape) for _ in range(64)])
    assert (draws.mean(0) - x).abs().mean() < 0.3 * (draws[0] - x).abs().mean()
    packed, scale32 = ops.quantize_and_pack(x, 2, x.min(1).values, x.max(1).values)
    assert packed.dtype == torch.int32 and scale32.dtype == torch.float32
    lin = exact.QLinear(64, 8).to(backend).train()
    lin(x.requires_grad_()).sum().backward()
    assert torch.isfinite(lin.weight.grad).all() and torch.isfinite(x.grad).all()


def test_elu_backward_kernel(backend):
    """_elu_backward_cuda (backward_func_cuda_kernel.cu:6-36) as a kernel of the
    library, fp32 and fp16, against the formula (exp within 2 ulp)."""
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator().manual_seed(3)
    for n in (1, 7, 1000, 4099):
        x = (torch.randn(n, generator=g) * 2).to(backend)
        x[::5] = 0.0
        dy = torch.randn(n, generator=g).to(backend)
        got = bf._elu_backward_cuda(dy, x, 1.3)
        want = torch.where(x >= 0, dy, (1.3 * dy) * torch.exp(x))
        assert torch.equal(got[x >= 0], dy[x >= 0])
        assert torch.allclose(got, want, rtol=1e-6, atol=0)
        got_h = bf._elu_backward_cuda(dy.half(), x.half(), 1.3)
        want_h = torch.where(x.half() >= 0, dy.half(), ((1.3 * dy.half().float()) * torch.exp(x.half().float())).half())
        assert got_h.dtype == torch.float16 and (got_h.float() - want_h.float()).abs().max() <= 2e-3 * want_h.float().abs().max()
    with pytest.raises(RuntimeError):
        bf._elu_backward_cuda(dy, x[:-1], 1.0)


@pytest.mark.gpu
def test_pack_work_split_is_tuned_once_and_never_changes_the_result(cuda):
    """tune_pack_geometry times the 1 / 2 / 4 column-groups-per-lane forms of
    the fused pack kernel; minmax_pack then uses the remembered one.  Whatever
    it picks, the bytes are those of the oracle."""
    from gpu_util import FixedNoise, bytes_equal, dev, host_noise, host_randn
    N, G, bits = 8192, 256, 2
    x = host_randn((N, G), 11)
    u = host_noise((N, G), 12)
    xt = dev(x)
    extq._PACK_GEOMETRY.pop((G, bits), None)
    timings = extq.tune_pack_geometry(xt, bits)
    assert sorted(timings) == [1, 2, 4] and all(t > 0 for t in timings.values())
    assert extq._PACK_GEOMETRY[(G, bits)] == min(timings, key=timings.get)
    want = o.quantize_activation(x, bits, u)
    for forced in (1, 2, 4):
        extq._PACK_GEOMETRY[(G, bits)] = forced
        config.noise_source = FixedNoise([dev(u)])
        packed, sbf, mbf = extq.minmax_pack(xt, bits)
        assert bytes_equal(packed, want[0]) and bytes_equal(sbf, want[2]) and bytes_equal(mbf, want[3])
    extq._PACK_GEOMETRY.pop((G, bits), None)
    config.noise_source = FixedNoise([dev(u)])
    big = dev(host_randn((4096, 256), 13))                 # 2^20 elements: tuned on first use
    extq._PACK_GEOMETRY.pop((256, 4), None)
    config.noise_source = None
    extq.minmax_pack(big, 4)
    assert extq._PACK_GEOMETRY.get((256, 4)) in (1, 2, 4)


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("valued", [True, False])
@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("M,N,K", [(60, 40, 256), (33, 50, 40), (20, 20, 602), (45, 30, 7), (9, 12, 1), (300, 100, 100)])
def test_rowwise_spmm_kernel_is_bit_identical_to_the_oracle(M, N, K, reduce, valued, idx):
    """The reproducible kernel sums in CSR order with one multiply and one add
    per entry -- exactly what the oracle (and its C twin) do."""
    import c_oracle as co
    A = csr(M, N, M * 7, M + K)
    X = np.random.default_rng(K).standard_normal((N, K)).astype(F32)
    val = A.data if valued else None
    got = e.spmm_rowwise(A.indptr, A.indices, val, X, reduce, idx)
    want = o.spmm_csr(A.indptr, A.indices, val, X, reduce)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(co.spmm_csr(A.indptr, A.indices, val, X, reduce).view(np.uint32), want.view(np.uint32))


def test_deterministic_spmm_switch(backend):
    """config.deterministic_spmm / torch.use_deterministic_algorithms select the
    reproducible kernel for forward and backward; the result is the oracle's, bit for bit."""
    A = csr(400, 400, 6000, 3, empty_rows=True)
    g = torch.Generator().manual_seed(5)
    X, dY = torch.randn(400, 64, generator=g), torch.randn(400, 64, generator=g)
    adj = SparseTensor.from_scipy(A, backend)
    want = o.spmm_csr(A.indptr, A.indices, A.data, X.numpy(), "sum")
    At = A.T.tocsr()
    At.sort_indices()
    want_bw = o.spmm_csr(At.indptr, At.indices, At.data, dY.numpy(), "sum")
    for how in ("config", "torch"):
        if how == "config":
            config.deterministic_spmm = True
        else:
            config.deterministic_spmm = False
            torch.use_deterministic_algorithms(True)
        try:
            x = X.clone().to(backend).requires_grad_()
            y = qmatmul(adj, x, "sum")
            y.backward(dY.to(backend))
        finally:
            torch.use_deterministic_algorithms(False)
        assert np.array_equal(y.detach().cpu().numpy().view(np.uint32), want.view(np.uint32))
        assert np.array_equal(x.grad.cpu().numpy().view(np.uint32), want_bw.view(np.uint32))


@pytest.mark.parametrize("N,K", [(1, 1), (3, 5), (7, 47), (1000, 41), (4099, 47), (513, 256), (2050, 100), (33, 602),
                                 (5, 8192), (40000, 3)])
def test_column_sum_kernel_counts_every_element_once(N, K):
    """exact_colsum_f32 on small integers, whose fp32 sums are exact whatever the
    order: any element missed, counted twice or added to the wrong column shows."""
    rng = np.random.default_rng(N * 7 + K)
    x = rng.integers(-8, 9, (N, K)).astype(np.float32)
    got = e.colsum(x)
    assert np.array_equal(got, x.astype(np.float64).sum(0).astype(np.float32))
    y = rng.standard_normal((N, K)).astype(np.float32)
    want = y.astype(np.float64).sum(0)
    assert np.allclose(e.colsum(y), want, rtol=0, atol=1e-6 * np.abs(y).astype(np.float64).sum(0).max() + 1e-30)


def test_column_sum_limits():
    assert e.colsum(np.zeros((2, 8193), np.float32), expect_rc=-3) is None
    assert e.colsum(np.zeros((0, 5), np.float32)).tolist() == [0.0] * 5


def test_bias_gradient_goes_through_the_column_sum_kernel(backend):
    """linear_backward's grad_output.sum(0) (backward_func.cc:90-91) for a tall
    fp32 matrix: same numbers as the framework's reduction to rounding."""
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator().manual_seed(5)
    for N, K in ((5000, 47), (4096, 256), (6001, 41)):
        dy = torch.randn(N, K, generator=g).to(backend)
        got = bf.column_sums(dy)
        want = dy.double().sum(0)
        assert got.dtype == torch.float32 and got.shape == (K,)
        assert (got.double() - want).abs().max().item() <= 1e-6 * dy.abs().double().sum(0).max().item()
        ints = torch.randint(-8, 9, (N, K), generator=g).float().to(backend)
        assert torch.equal(bf.column_sums(ints), ints.sum(0))
    small = torch.randn(10, 3).to(backend)
    assert torch.equal(bf.column_sums(small), small.sum(0))       # short matrices keep the framework's reduction


@pytest.mark.parametrize("N,K", [(1, 1), (3, 5), (7, 47), (1000, 40), (4099, 64), (513, 256), (2050, 100), (40000, 3)])
def test_batch_norm_backward_reduction_kernel(N, K):
    """exact_bn_backward_reduce_f32: sum of dy and of dy * (x - mean) per column.
    Small integers make every product and sum exact, so a misplaced or repeated
    element shows; random data within fp32 summation error of float64."""
    rng = np.random.default_rng(N + 13 * K)
    dy = rng.integers(-4, 5, (N, K)).astype(np.float32)
    x = rng.integers(-4, 5, (N, K)).astype(np.float32)
    mean = rng.integers(-2, 3, K).astype(np.float32)
    a, b = e.bn_backward_reduce(dy, x, mean)
    assert np.array_equal(a, dy.astype(np.float64).sum(0).astype(np.float32))
    assert np.array_equal(b, (dy.astype(np.float64) * (x - mean)).sum(0).astype(np.float32))
    dy, x = rng.standard_normal((N, K)).astype(np.float32), rng.standard_normal((N, K)).astype(np.float32) * 2 + 1
    mean = x.mean(0)
    a, b = e.bn_backward_reduce(dy, x, mean)
    prod = dy.astype(np.float64) * (x.astype(np.float64) - mean)
    assert np.allclose(a, dy.astype(np.float64).sum(0), rtol=0, atol=1e-6 * np.abs(dy).astype(np.float64).sum(0).max())
    assert np.allclose(b, prod.sum(0), rtol=0, atol=2e-6 * np.abs(prod).sum(0).max())
    assert e.bn_backward_reduce(np.zeros((2, 257), np.float32), np.zeros((2, 257), np.float32), np.zeros(257, np.float32),
                                expect_rc=-3) is None


@pytest.mark.gpu
@pytest.mark.parametrize("N,K,affine", [(169343, 256, True), (5000, 64, True), (20000, 40, False), (4097, 100, True)])
def test_batch_norm_backward_with_the_one_pass_reduction(cuda, N, K, affine):
    """native_batch_norm_backward through the library's column reduction + the
    framework's element-wise half, against the framework's one-call routine
    (what qbatch_norm.backward calls, ops.py:228-254)."""
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator(device=cuda).manual_seed(N + K)
    x = torch.randn(N, K, generator=g, device=cuda) * 1.5 + 0.3
    dy = torch.randn(N, K, generator=g, device=cuda)
    w = torch.rand(K, generator=g, device=cuda) + 0.5 if affine else None
    var, mean = torch.var_mean(x, dim=0, unbiased=False)
    invstd = torch.rsqrt(var + 1e-5)
    for mask in ([True, True, True], [True, False, False], [False, True, True]):
        mask = [mask[0], mask[1] and affine, mask[2] and affine]
        want = torch.ops.aten.native_batch_norm_backward(dy, x, w, None, None, mean, invstd, True, 1e-5, mask)
        got = bf.native_batch_norm_backward(dy, x, w, None, None, mean, invstd, True, 1e-5, mask)
        for a, b, m in zip(got, want, mask):
            if not m:
                assert a is None
                continue
            scale = b.abs().max().item() + 1e-12
            assert (a - b).abs().max().item() <= 2e-5 * scale, (mask, (a - b).abs().max().item(), scale)


@pytest.mark.parametrize("N,K", [(1, 1), (3, 5), (7, 47), (1000, 40), (4099, 64), (513, 256), (2050, 100)])
def test_column_moments_kernel(N, K):
    """exact_col_moments_f32: exact on small integers; on data with a mean far
    from zero the variance formed from the centred moments keeps its digits."""
    rng = np.random.default_rng(N + 17 * K)
    x = rng.integers(-4, 5, (N, K)).astype(np.float32)
    c = x[0].copy()
    a, b = e.col_moments(x, c)
    d = x.astype(np.float64) - c
    assert np.array_equal(a, d.sum(0).astype(np.float32)) and np.array_equal(b, (d * d).sum(0).astype(np.float32))
    x = (rng.standard_normal((N, K)) * 0.5 + 100.0).astype(np.float32)      # mean 200 standard deviations from zero
    a, b = e.col_moments(x, x[0])
    shift = a.astype(np.float64) / N
    var = b.astype(np.float64) / N - shift * shift
    want = x.astype(np.float64).var(0)
    assert np.allclose(x[0] + shift, x.astype(np.float64).mean(0), rtol=1e-6)
    if N > 100:
        assert np.allclose(var, want, rtol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("N,K", [(169343, 256), (5000, 64), (20000, 40)])
def test_batch_statistics_match_var_mean(cuda, N, K):
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator(device=cuda).manual_seed(N)
    x = torch.randn(N, K, generator=g, device=cuda) * 1.5 + 3.0
    var, mean = bf.batch_statistics(x)
    want_var, want_mean = torch.var_mean(x.double(), dim=0, unbiased=False)
    assert (mean.double() - want_mean).abs().max().item() < 1e-5
    assert ((var.double() - want_var) / want_var).abs().max().item() < 1e-5


def test_batch_statistics_of_sorted_rows(backend):
    """Rows sorted by value, the first 256 of them many standard deviations from
    the column mean: the moments stay centred near the mean (a sample spread over
    all rows), so the variance keeps its digits."""
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(6000, 9, generator=g) * 0.01 + torch.linspace(-50.0, 50.0, 6000)[:, None]).sort(0).values.contiguous()
    var, mean = bf.batch_statistics(x.to(backend))
    want_var, want_mean = torch.var_mean(x.double(), dim=0, unbiased=False)
    assert (mean.cpu().double() - want_mean).abs().max().item() < 1e-4
    assert ((var.cpu().double() - want_var) / want_var).abs().max().item() < 1e-5


def test_reductions_keep_the_framework_routines_on_request(backend, monkeypatch):
    """config.deterministic_reductions = True: no atomics-combined kernel is
    called for column sums, weight gradients and batch statistics."""
    from exact_amd import _lib
    from exact_amd.conf import config
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator().manual_seed(12)
    dy, x = torch.randn(16500, 8, generator=g).to(backend), torch.randn(16500, 12, generator=g).to(backend)
    free = (bf.column_sums(dy), bf.weight_gradient(dy, x), bf.batch_statistics(x))
    monkeypatch.setattr(config, "deterministic_reductions", True)

    def no_library():
        raise AssertionError("a library kernel was asked for")
    monkeypatch.setattr(_lib, "lib", no_library)
    fixed = (bf.column_sums(dy), bf.weight_gradient(dy, x), bf.batch_statistics(x))
    assert torch.equal(fixed[0], dy.sum(0)) and torch.equal(fixed[1], dy.t().mm(x))
    assert torch.allclose(free[0], fixed[0], atol=1e-3) and torch.allclose(free[1], fixed[1], atol=1e-3)
    assert torch.allclose(free[2][0], fixed[2][0], atol=1e-5) and torch.allclose(free[2][1], fixed[2][1], atol=1e-5)


def test_batch_norm_backward_refuses_mismatched_statistics_for_the_fast_path(backend, monkeypatch):
    """Statistics of the wrong length, type or device never reach the kernel:
    the call falls through to the framework's routine (which raises or handles
    them by its own rules)."""
    from exact_amd import _lib
    from exact_amd.cpp_extension import backward_func as bf
    seen = []
    monkeypatch.setattr(torch.ops.aten, "native_batch_norm_backward", lambda *a: seen.append(a) or "framework")
    monkeypatch.setattr(_lib, "lib", lambda: (_ for _ in ()).throw(AssertionError("kernel reached")))
    dy, x = torch.zeros(5000, 8).to(backend), torch.zeros(5000, 8).to(backend)
    ok = torch.ones(8).to(backend)
    for mean, invstd, weight in ((ok[:7], ok, ok), (ok, ok.double(), ok), (ok, ok, torch.ones(9).to(backend)), (None, ok, ok),
                                 (ok, ok.cpu() if ok.is_cuda else ok[:3], ok)):
        assert bf.native_batch_norm_backward(dy, x, weight, None, None, mean, invstd, True, 1e-5, (True, True, True)) == "framework"
    assert len(seen) == 5


def test_sparse_product_with_row_strides(backend):
    """The dense operand as a column slice of a wider buffer (unit column
    stride, longer row stride) and the padded copy the shim makes of wide,
    unaligned rows on dense graphs: same product, nothing outside the slice is
    read into the result."""
    import scipy.sparse as sp
    from exact_amd.cpp_extension import spmm as ext_spmm
    rng = np.random.default_rng(3)
    n, K = 300, 130                                          # 130 columns: > 128 and not a multiple of 32
    A = sp.random(n, n, density=0.08, format="csr", random_state=4, dtype=np.float32)   # ~24 entries per row >= 16
    A.sort_indices()
    rowptr = torch.from_numpy(A.indptr.astype(np.int64)).to(backend)
    col = torch.from_numpy(A.indices.astype(np.int64)).to(backend)
    val = torch.from_numpy(A.data).to(backend)
    X = rng.standard_normal((n, K)).astype(np.float32)
    wide = torch.full((n, K + 37), float("nan"))
    wide[:, 5:5 + K] = torch.from_numpy(X)
    wide = wide.to(backend)
    for reduce in ("sum", "mean"):
        want = o.spmm_csr(A.indptr, A.indices, A.data, X, reduce)
        scale = np.abs(want).max()
        got_view = ext_spmm.spmm_csr(rowptr, col, val, wide[:, 5:5 + K], reduce)          # strided, no copy
        got_pad = ext_spmm.spmm_csr(rowptr, col, val, torch.from_numpy(X).to(backend), reduce)   # padded copy
        assert np.allclose(got_view.cpu().numpy(), want, rtol=0, atol=1e-5 * scale)
        assert np.allclose(got_pad.cpu().numpy(), want, rtol=0, atol=1e-5 * scale)
    padded = ext_spmm._aligned_rows(torch.from_numpy(X).to(backend), A.nnz)
    assert padded.shape == (n, K) and padded.stride(0) == 160 and padded.stride(1) == 1
    assert ext_spmm._aligned_rows(wide[:, 5:5 + K], A.nnz).data_ptr() == wide[:, 5:5 + K].data_ptr()


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("N,K,D", [(1, 1, 1), (7, 3, 5), (100, 40, 256), (515, 256, 128), (1030, 64, 64), (333, 47, 25),
                                   (1201, 256, 76), (600, 130, 70), (513, 32, 200), (2100, 256, 256)])
def test_weight_gradient_kernel(N, K, D, bf16):
    """exact_linear_dw_f32 = dY^T . X.  Small integers: every product and sum is
    exact in fp32, so the result must equal the integer GEMM bit for bit (a
    wrong fragment, a row counted twice or a column off by one shows); random
    data within fp32 accumulation error of float64; row strides longer than the
    used width with NaN in the padding."""
    rng = np.random.default_rng(N + K + D)
    dy = rng.integers(-3, 4, (N, K)).astype(np.float32)
    x = rng.integers(-3, 4, (N, D)).astype(np.float32)
    assert np.array_equal(e.linear_dw(dy, x, bf16=bf16), (dy.astype(np.float64).T @ x.astype(np.float64)).astype(np.float32))
    assert np.array_equal(e.linear_dw(dy, x, ldy=K + 3, ldx=D + 9, bf16=bf16),
                          (dy.astype(np.float64).T @ x.astype(np.float64)).astype(np.float32))
    # rows of very different size: a dropped low-order piece of the bf16 form would show
    dy = (rng.standard_normal((N, K)) * np.exp(rng.uniform(-4, 4, (N, 1)))).astype(np.float32)
    x = (rng.standard_normal((N, D)) * np.exp(rng.uniform(-4, 4, (N, 1)))).astype(np.float32)
    want = dy.astype(np.float64).T @ x.astype(np.float64)
    bound = np.abs(dy).astype(np.float64).T @ np.abs(x).astype(np.float64)
    assert (np.abs(e.linear_dw(dy, x, bf16=bf16) - want) <= 1e-5 * bound + 1e-30).all()


def test_weight_gradient_limits():
    assert e.linear_dw(np.zeros((0, 4), np.float32), np.zeros((0, 6), np.float32)).tolist() == [[0.0] * 6] * 4
    assert e.emu().exact_linear_dw_f32(None, 4, None, 3, 5, 4, 6, None, None) == -3      # ldx < D


def test_linear_backward_uses_the_weight_gradient_kernel(backend):
    from exact_amd.cpp_extension import backward_func as bf
    g = torch.Generator().manual_seed(9)
    N, K, D = 16500, 48, 100
    dy, x = torch.randn(N, K, generator=g).to(backend), torch.randn(N, D, generator=g).to(backend)
    got = bf.weight_gradient(dy, x)
    want = dy.double().t().mm(x.double())
    assert got.dtype == torch.float32 and (got.double() - want).abs().max().item() <= 1e-5 * dy.abs().double().t().mm(x.abs().double()).max().item()
    wide = torch.randn(N, D + 28, generator=g).to(backend)
    assert torch.allclose(bf.weight_gradient(dy, wide[:, 3:3 + D]), dy.t().mm(wide[:, 3:3 + D]), rtol=1e-4, atol=1e-2)
    small = torch.randn(100, 5).to(backend)
    assert torch.equal(bf.weight_gradient(small, small), small.t().mm(small))       # short batches keep the library GEMM


def _stream_probe_words(x):
    """What lane L of the probe folds: the XOR of the bit patterns of its four
    16-byte loads, quads tile * 1024 + u * 256 + t of the stream."""
    tiles = x.size // 4096
    q = x.view(np.uint32)[:tiles * 4096].reshape(tiles, 4, 256, 4)
    return np.bitwise_xor.reduce(np.bitwise_xor.reduce(q, axis=3), axis=1).reshape(-1)


@pytest.mark.parametrize("n", [4096, 3 * 4096 + 77, 10 * 4096])
def test_stream_probe_reads_every_quad_and_writes_its_share(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    w = _stream_probe_words(x)
    lanes = w.size
    for out_bytes in (2, 4, 8, 16):
        got = e.stream_probe(x, out_bytes)
        want = {2: w.astype(np.uint16), 4: w, 8: np.stack([w, ~w], 1), 16: np.stack([w, ~w, w + np.uint32(1), w - np.uint32(1)], 1)}[out_bytes]
        assert np.array_equal(got[:lanes * out_bytes], np.ascontiguousarray(want).view(np.uint8).reshape(-1)), out_bytes
        assert (got[lanes * out_bytes:] == 0xA5).all()          # the incomplete last tile writes nothing
    assert (e.stream_probe(x, 0) == 0xA5).all()                  # read-only form


def test_stream_probe_arguments():
    x = np.zeros(8192, np.float32)
    assert e.stream_probe(x, 3, expect_rc=-5) is None
    assert (e.stream_probe(np.zeros(100, np.float32), 4) == 0xA5).all()   # less than one tile: nothing to do


@pytest.mark.gpu
def test_stream_probe_gpu():
    from exact_amd import _lib
    dev = torch.device("cuda:0")
    n = 1000 * 4096 + 5
    x = torch.randn(n, device=dev)
    w = _stream_probe_words(x.cpu().numpy())
    for out_bytes in (0, 2, 4, 8, 16):
        out = torch.full((max(16, (n // 16) * out_bytes) + 64,), 0xA5, dtype=torch.uint8, device=dev)
        rc = _lib.lib().exact_stream_probe_f32(x.data_ptr(), n, out_bytes, out.data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0
        got = out.cpu().numpy()
        if out_bytes == 4:
            assert np.array_equal(got[:w.size * 4].view(np.uint32), w)
        if out_bytes == 2:
            assert np.array_equal(got[:w.size * 2].view(np.uint16), w.astype(np.uint16))
        assert (got[w.size * out_bytes:] == 0xA5).all()

