"""GPU parity of the 1-bit-mask ReLU / dropout against the oracle (bit-exact
outputs, masks and gradients) and against the stock torch ops, as the
reference's own tests assert (test/test_op.py:22-41, 463-480)."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import exact_oracle as o
from exact_amd import _lib
from exact_amd.conf import config
from exact_amd.cpp_extension import quantization as extq
from gpu_util import FixedNoise, bytes_equal, dev, host_noise, host_randn

pytestmark = pytest.mark.gpu
SIZES = [1, 7, 8, 31, 32, 33, 255, 256, 257, 1000, 4096 + 5, 100000, 10000 * 128]


@pytest.mark.parametrize("n", SIZES)
def test_relu_bit_exact(cuda, n):
    print(f"case relu n={n}", flush=True)
    x = host_randn((n,), n)
    x[: min(n, 3)] = [0.0, -0.0, np.nan][: min(n, 3)]
    g = host_randn((n,), n + 1)
    want_y, want_mask = o.relu_fwd(x)
    tx = dev(x)
    y = torch.empty_like(tx)
    guard = 4
    mask = torch.full((o.mask_nwords(n) + guard,), 0x5A5A5A5A, dtype=torch.int32, device=cuda)
    assert _lib.lib().exact_relu_fwd_f32(tx.data_ptr(), n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(y, want_y)
    assert bytes_equal(mask[:-guard], want_mask)
    assert (mask[-guard:] == 0x5A5A5A5A).all()          # nothing written past ceil(n/32) words
    dx = torch.empty_like(tx)
    tg = dev(g)
    assert _lib.lib().exact_relu_bwd_f32(tg.data_ptr(), mask.data_ptr(), n, dx.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(dx, o.relu_bwd(g, want_mask))


@pytest.mark.parametrize("shape", [(10000, 128), (333, 77), (5,)])
def test_relu_autograd_equals_stock(cuda, shape):
    x = torch.randn(shape, device=cuda, requires_grad=True)
    xr = x.detach().clone().requires_grad_()
    y = extq.act_quantized_relu(x)
    yr = F.relu(xr)
    g = torch.randn(shape, device=cuda)
    y.backward(g)
    yr.backward(g)
    assert torch.equal(y, yr) and torch.equal(x.grad, xr.grad)      # exact, as test_op.py:37-41


@pytest.mark.parametrize("p", [0.5, 0.1, 0.0, 0.9])
@pytest.mark.parametrize("n", [1, 33, 1000, 4096 + 5, 10000 * 128])
def test_dropout_bit_exact_supplied_noise(cuda, n, p):
    print(f"case dropout n={n} p={p}", flush=True)
    x = host_randn((n,), n + 11)
    u = host_noise((n,), n + 12)
    g = host_randn((n,), n + 13)
    want_y, want_mask = o.dropout_fwd(x, p, u)
    tx, tu = dev(x), dev(u)
    y = torch.empty_like(tx)
    mask = torch.full((o.mask_nwords(n) + 2,), -1, dtype=torch.int32, device=cuda)
    L = _lib.lib()
    assert L.exact_dropout_fwd_f32(tx.data_ptr(), tu.data_ptr(), 0, 0, p, n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(y, want_y) and bytes_equal(mask[:-2], want_mask) and (mask[-2:] == -1).all()
    dx = torch.empty_like(tx)
    tg = dev(g)
    assert L.exact_dropout_bwd_f32(tg.data_ptr(), mask.data_ptr(), p, n, dx.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(dx, o.dropout_bwd(g, want_mask, p))


def test_dropout_internal_philox_matches_oracle(cuda):
    n, p, seed, off = 100003, 0.5, 0xFEEDFACE12345678, (3 << 32) + 77
    x = host_randn((n,), 1)
    want_y, want_mask = o.dropout_fwd(x, p, o.philox_noise_flat(seed, off, n))
    tx = dev(x)
    y = torch.empty_like(tx)
    mask = torch.empty(o.mask_nwords(n), dtype=torch.int32, device=cuda)
    assert _lib.lib().exact_dropout_fwd_f32(tx.data_ptr(), None, seed, off, p, n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(y, want_y) and bytes_equal(mask, want_mask)


def test_dropout_structure_like_reference_test(cuda):
    """test/test_op.py:463-480: zero pattern of output == zero pattern of grad;
    max(out) == max(grad) == 1/(1-p) on an all-ones input; eval is identity."""
    p = 0.5
    x = torch.ones(232965, 602 // 7, device=cuda, requires_grad=True)
    y = extq.act_quantized_dropout(x, p, True)
    y.backward(torch.ones_like(y))
    assert torch.equal(y == 0, x.grad == 0)
    assert y.max().item() == x.grad.max().item() == 2.0
    assert abs((y != 0).float().mean().item() - (1 - p)) < 2e-3
    assert extq.act_quantized_dropout(x, p, False) is x
    y2 = extq.act_quantized_dropout(x.detach(), p, True)
    assert not torch.equal(y2, y.detach())             # fresh noise on every call
    config.noise_source = FixedNoise([torch.full((8,), 0.75), torch.full((8,), 0.25)])
    a = extq.act_quantized_dropout(torch.ones(8, device=cuda), 0.5, True)
    b = extq.act_quantized_dropout(torch.ones(8, device=cuda), 0.5, True)
    assert (a == 2).all() and (b == 0).all()            # keep = u > p


def test_masks_at_config_2_size(cuda):
    """ReLU, dropout (supplied noise and the internal Philox stream) and the fused pair on
    every element of a [169343, 256] activation, bit for bit against the oracle."""
    n, p = 169343 * 256, 0.5
    print(f"case masks n={n}", flush=True)
    L = _lib.lib()
    x = host_randn((n,), 77)
    tx = dev(x)
    y = torch.empty_like(tx)
    mask = torch.full((o.mask_nwords(n) + 4,), 0x5A5A5A5A, dtype=torch.int32, device=cuda)
    # ReLU forward / backward
    assert L.exact_relu_fwd_f32(tx.data_ptr(), n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    want_y, want_mask = o.relu_fwd(x)
    assert bytes_equal(y, want_y) and bytes_equal(mask[:-4], want_mask) and (mask[-4:] == 0x5A5A5A5A).all()
    assert L.exact_relu_bwd_f32(tx.data_ptr(), mask.data_ptr(), n, y.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(y, o.relu_bwd(x, want_mask))
    # dropout with the internal Philox stream, then with a supplied noise tensor
    seed, off = 0xFEEDFACE12345678, (5 << 32) + 12
    assert L.exact_dropout_fwd_f32(tx.data_ptr(), None, seed, off, p, n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    noise = o.philox_noise_flat(seed, off, n)
    want_y, want_mask = o.dropout_fwd(x, p, noise)
    assert bytes_equal(y, want_y) and bytes_equal(mask[:-4], want_mask)
    tn = dev(noise)
    assert L.exact_dropout_fwd_f32(tx.data_ptr(), tn.data_ptr(), 0, 0, p, n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(y, want_y) and bytes_equal(mask[:-4], want_mask)
    assert L.exact_dropout_bwd_f32(tx.data_ptr(), mask.data_ptr(), p, n, y.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bytes_equal(y, o.dropout_bwd(x, want_mask, p))
    # ReLU -> dropout in one pass = the two oracle operators in a row, one joint mask
    assert L.exact_relu_dropout_fwd_f32(tx.data_ptr(), tn.data_ptr(), 0, 0, p, n, y.data_ptr(), mask.data_ptr(), None) == 0
    torch.cuda.synchronize()
    y1, m1 = o.relu_fwd(x)
    y2, m2 = o.dropout_fwd(y1, p, noise)
    assert bytes_equal(y, y2) and bytes_equal(mask[:-4], m1 & m2) and (mask[-4:] == 0x5A5A5A5A).all()
