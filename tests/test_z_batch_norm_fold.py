"""QBatchNorm1d folded into the ReLU -> dropout -> quantise pass
(exact_bn_relu_dropout_minmax_pack_f32): the layers on both back ends against
the separate layers they replace (layers.py:340-369, 284-325 of the reference).
The kernel itself is pinned bit for bit in test_more_ops.py.

Tolerances: the folded form takes the batch statistics from torch.var_mean and
normalises as (x - mean) * (weight * invstd) + bias; the separate QBatchNorm1d
lets native_batch_norm do both.  The two differ by a few fp32 roundings, 1e-5
absolute on O(1) outputs; gradients pass through a 2-bit copy of the input that
is the SAME in both forms (same noise), so they agree as closely."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import exact_amd as exact
from exact_amd import ops
from exact_amd.conf import config
from exact_amd.cpp_extension import quantization as extq
from gpu_util import SeededNoise


def _seeded(seed):
    s = SeededNoise(seed)
    config.noise_source, config.rp_matrix_source = s.noise_source, s.rp_matrix_source


def _run(backend, fold, x0, g0, p=0.3, affine=True, momentum=0.1, track=True, steps=2, width=None):
    """-> per-step (y, dx, dweight, dbias), final (running_mean, running_var, batches), compressed copy of y."""
    config.fuse_epilogue, config.fold_batch_norm = True, fold
    config.activation_compression_bits = [2]
    _seeded(3)
    torch.manual_seed(1)
    G = x0.shape[1]
    bn = exact.QBatchNorm1d(G, momentum=momentum, affine=affine, track_running_stats=track).to(backend).train()
    if affine:
        with torch.no_grad():
            bn.weight.copy_(torch.linspace(-1.5, 2.0, G))
            bn.bias.copy_(torch.linspace(0.5, -0.5, G))
    act = exact.QReLUDropout(p).train()
    outs = []
    for step in range(steps):
        x = (x0 * (1 + step)).clone().to(backend).requires_grad_(True)
        y = act(x, norm=bn)
        copy = ops.take_compressed(y)
        y.backward(g0.to(backend))
        outs.append((y.detach().cpu(), x.grad.cpu(), bn.weight.grad.cpu().clone() if affine else None,
                     bn.bias.grad.cpu().clone() if affine else None))
        if affine:
            bn.weight.grad = bn.bias.grad = None
    stats = (bn.running_mean.cpu(), bn.running_var.cpu(), int(bn.num_batches_tracked)) if track else None
    return outs, stats, copy


@pytest.mark.parametrize("N,G", [(200, 64), (37, 256), (513, 40)])
@pytest.mark.parametrize("affine,momentum,track", [(True, 0.1, True), (False, None, True), (True, 0.1, False)])
def test_folded_batch_norm_matches_the_separate_layers(backend, N, G, affine, momentum, track):
    g = torch.Generator().manual_seed(N + G)
    x0 = torch.randn(N, G, generator=g) * 2 + 0.5
    g0 = torch.randn(N, G, generator=g)
    sep, sep_stats, sep_copy = _run(backend, False, x0, g0, affine=affine, momentum=momentum, track=track)
    calls = []
    real = extq.bn_relu_dropout_minmax_pack
    try:
        extq.bn_relu_dropout_minmax_pack = lambda *a: (calls.append(1), real(*a))[1]
        fus, fus_stats, fus_copy = _run(backend, True, x0, g0, affine=affine, momentum=momentum, track=track)
    finally:
        extq.bn_relu_dropout_minmax_pack = real
    assert len(calls) == 2                                   # the one-pass kernel ran, once per step
    assert sep_copy is not None and fus_copy is not None     # both hand a compressed copy to the next layer
    for (ys, dxs, dws, dbs), (yf, dxf, dwf, dbf) in zip(sep, fus):
        # elements within rounding of zero may land on either side of the ReLU: equal to 1e-5 all the same
        assert torch.allclose(ys, yf, rtol=1e-5, atol=2e-5)
        flipped = (ys != 0) != (yf != 0)
        assert flipped.float().mean().item() < 1e-3
        # a flipped element changes the gradients of its whole column (batch norm's backward sums over the
        # column); columns are independent, so the others must agree
        same = ~flipped.any(0)
        assert same.float().mean().item() > 0.9
        assert torch.allclose(dxs[:, same], dxf[:, same], rtol=1e-3, atol=1e-3 * dxs.abs().max().item())
        if affine:
            assert torch.allclose(dws[same], dwf[same], rtol=1e-3, atol=1e-3 * dws.abs().max().item())
            assert torch.allclose(dbs[same], dbf[same], rtol=1e-3, atol=1e-3 * dbs.abs().max().item())
    if track:
        assert torch.allclose(sep_stats[0], fus_stats[0], rtol=1e-5, atol=1e-6)
        assert torch.allclose(sep_stats[1], fus_stats[1], rtol=1e-5, atol=1e-6)
        assert sep_stats[2] == fus_stats[2] == 2


def test_folded_batch_norm_against_plain_float64_arithmetic(backend):
    """Independent of the separate layers: the output is dropout(relu(batch
    norm)) of the input as float64 numpy computes it, the running statistics
    follow torch's rule (unbiased variance, momentum)."""
    config.fuse_epilogue = config.fold_batch_norm = True
    config.activation_compression_bits = [4]
    _seeded(8)
    N, G, p = 120, 48, 0.25
    x = torch.randn(N, G, generator=torch.Generator().manual_seed(2)) * 3 - 1
    bn = exact.QBatchNorm1d(G, momentum=0.2).to(backend).train()
    with torch.no_grad():
        bn.weight.uniform_(0.5, 1.5, generator=None)
        bn.bias.uniform_(-0.3, 0.3)
    y = exact.QReLUDropout(p)(x.to(backend), norm=bn)
    xd = x.double().numpy()
    mean, var = xd.mean(0), xd.var(0)
    z = (xd - mean) / np.sqrt(var + bn.eps) * bn.weight.detach().cpu().double().numpy() + bn.bias.detach().cpu().double().numpy()
    # noise draws in call order: 1 = quantiser noise of the batch norm's saved input, 2 = dropout
    keep = SeededNoise(8)
    keep.noise((N, G))
    keep = keep.noise((N, G)).numpy() > p
    want = np.where((z > 0) & keep, z / (1 - p), 0.0)
    got = y.detach().cpu().double().numpy()
    near_zero = np.abs(z) < 1e-5
    assert np.allclose(got[~near_zero], want[~near_zero], rtol=1e-5, atol=1e-5)
    assert np.allclose(bn.running_mean.cpu().numpy(), 0.2 * mean, rtol=1e-5, atol=1e-6)
    assert np.allclose(bn.running_var.cpu().numpy(), 0.8 + 0.2 * xd.var(0, ddof=1), rtol=1e-5, atol=1e-6)


def test_what_is_not_folded_runs_as_separate_layers(backend):
    config.fuse_epilogue = config.fold_batch_norm = True
    config.activation_compression_bits = [2]
    config.noise_source = None
    calls = []
    real = extq.bn_relu_dropout_minmax_pack
    act = exact.QReLUDropout(0.5).train()
    try:
        extq.bn_relu_dropout_minmax_pack = lambda *a: (calls.append(1), real(*a))[1]
        # a width the kernel does not take
        bn12 = exact.QBatchNorm1d(12).to(backend).train()
        y = act(torch.randn(20, 12, device=backend), norm=bn12)
        assert y.shape == (20, 12) and int(bn12.num_batches_tracked) == 1
        # a stock BatchNorm1d (config.enable_quantized_bn = False leaves them in place): its exact gradient is kept
        plain = torch.nn.BatchNorm1d(16).to(backend).train()
        x = torch.randn(20, 16, device=backend, requires_grad=True)
        act(x, norm=plain).sum().backward()
        assert int(plain.num_batches_tracked) == 1 and x.grad is not None
        # projection in use: the consumer wants a projected copy, which this pass does not make
        config.kept_frac = 0.5
        bn16 = exact.QBatchNorm1d(16).to(backend).train()
        act(torch.randn(20, 16, device=backend), norm=bn16)
        config.kept_frac = 1.0
        # switched off
        config.fold_batch_norm = False
        act(torch.randn(20, 16, device=backend), norm=bn16)
        assert int(bn16.num_batches_tracked) == 2
        assert calls == []
        # and the case it takes
        config.fold_batch_norm = True
        act(torch.randn(20, 16, device=backend), norm=bn16)
        assert calls == [1] and int(bn16.num_batches_tracked) == 3
    finally:
        extq.bn_relu_dropout_minmax_pack = real


def test_evaluation_mode_is_the_stock_arithmetic(backend):
    bn = exact.QBatchNorm1d(16).to(backend)
    with torch.no_grad():
        bn.running_mean.normal_()
        bn.running_var.uniform_(0.5, 2.0)
    bn.eval()
    act = exact.QReLUDropout(0.5).eval()
    x = torch.randn(9, 16, device=backend)
    assert torch.equal(act(x, norm=bn), F.relu(F.batch_norm(x, bn.running_mean, bn.running_var, bn.weight, bn.bias,
                                                           False, 0.1, bn.eps)))


@pytest.mark.parametrize("bits", [2, 8])
def test_training_with_the_fold_tracks_training_without_it(backend, bits):
    from test_more_ops import _train_steps
    l_sep, w_sep = _train_steps(backend, True, 5, 0, 1.0, bits, fold_bn=False)
    l_fus, w_fus = _train_steps(backend, True, 5, 0, 1.0, bits, fold_bn=True)
    assert np.allclose(l_sep, l_fus, rtol=0, atol=1e-3)
    assert all(torch.allclose(a, b, rtol=1e-3, atol=1e-3) for a, b in zip(w_sep, w_fus))


def test_the_stock_pair_accepts_a_norm_layer():
    from exact_amd.nn import ReLUDropout
    bn = torch.nn.BatchNorm1d(8).eval()
    x = torch.randn(5, 8)
    assert torch.equal(ReLUDropout(0.5).eval()(x, norm=bn), F.relu(bn(x)))


def test_views_off_a_16_byte_boundary_are_taken(backend):
    """A bias that lives in the middle of a flat parameter buffer, an input that is a row slice: same results."""
    config.activation_compression_bits = [2]
    flat = torch.randn(3 * 16 + 1, device=backend)
    mean, mult, shift = (flat[1 + 16 * i:1 + 16 * (i + 1)] for i in range(3))
    assert mean.data_ptr() % 16 != 0
    big = torch.randn(9, 16, device=backend)
    x = big.view(-1)[1:1 + 8 * 16].view(8, 16)
    assert x.data_ptr() % 16 != 0 and x.is_contiguous()
    _seeded(6)
    a = extq.bn_relu_dropout_minmax_pack(x, mean, mult, shift, 0.5, 2)
    _seeded(6)
    b = extq.bn_relu_dropout_minmax_pack(x.clone(), mean.clone(), mult.clone(), shift.clone(), 0.5, 2)
    assert all(torch.equal(u, v) for u, v in zip(a, b))
    _seeded(6)
    c = extq.relu_dropout_minmax_pack(x, 0.5, 2)
    _seeded(6)
    d = extq.relu_dropout_minmax_pack(x.clone(), 0.5, 2)
    assert all(torch.equal(u, v) for u, v in zip(c, d))
