"""GPU parity of the fused epilogue kernels, called through the C ABI, against the
chain of the oracle's separate operators (reference layers.py:284-325 QReLU ->
QDropout, ops.py:149 the next layer's quantize_activation; with a batch norm ahead
of them, layers.py:340-369): every output bit for bit, supplied noise and the
internal Philox streams, guard bytes behind every buffer."""
import numpy as np
import pytest
import torch

import exact_oracle as o
from exact_amd import _lib
from gpu_util import dev

pytestmark = pytest.mark.gpu
F32 = np.float32
GUARD = 64


def _chain(x, prob, bits, act_noise, noise):
    N, G = x.shape
    y1, m1 = o.relu_fwd(x.reshape(-1))
    y2, m2 = o.dropout_fwd(y1, prob, act_noise.reshape(-1))
    y2 = y2.reshape(N, G)
    packed, _, sbf, mbf, scale, mn = o.quantize_activation(y2, bits, noise)
    return y2, m1 & m2, packed, scale, mn, sbf, mbf


def _launch(x, prob, bits, act_noise, noise, seeds, norm=None):
    """-> (y, mask words, packed, scale f32, min f32, scale bf16 bits, min bf16 bits) as numpy arrays."""
    L = _lib.lib()
    N, G = x.shape
    n = N * G
    nb = int(L.exact_packed_nbytes(N, G, bits))
    words = (n + 31) // 32
    cuda = torch.device("cuda:0")
    packed = torch.full((nb + GUARD,), 0xA5, dtype=torch.uint8, device=cuda)
    y = torch.full((n + GUARD,), 7.0, device=cuda)
    mask = torch.full((words + GUARD,), 0x5A5A5A5A, dtype=torch.int32, device=cuda)
    s32, m32 = torch.zeros(N, device=cuda), torch.zeros(N, device=cuda)
    sbf = torch.zeros(N, dtype=torch.int16, device=cuda)
    mbf = torch.zeros(N, dtype=torch.int16, device=cuda)
    xd = dev(x)
    an = None if act_noise is None else dev(act_noise)
    qn = None if noise is None else dev(noise)
    ptr = lambda t: None if t is None else t.data_ptr()
    sp = torch.cuda.current_stream().cuda_stream
    act_seed, act_off, seed, off = seeds
    if norm is None:
        rc = L.exact_relu_dropout_minmax_pack_f32(xd.data_ptr(), prob, ptr(an), act_seed, act_off, ptr(qn), seed, off, N, G,
                                                  bits, y.data_ptr(), mask.data_ptr(), packed.data_ptr(), s32.data_ptr(),
                                                  m32.data_ptr(), sbf.data_ptr(), mbf.data_ptr(), sp)
    else:
        mean, mult, shift = (dev(v) for v in norm)
        rc = L.exact_bn_relu_dropout_minmax_pack_f32(xd.data_ptr(), mean.data_ptr(), mult.data_ptr(), shift.data_ptr(), prob,
                                                     ptr(an), act_seed, act_off, ptr(qn), seed, off, N, G, bits, y.data_ptr(),
                                                     mask.data_ptr(), packed.data_ptr(), s32.data_ptr(), m32.data_ptr(),
                                                     sbf.data_ptr(), mbf.data_ptr(), sp)
    assert rc == 0, rc
    torch.cuda.synchronize()
    pk, yy, mk = packed.cpu().numpy(), y.cpu().numpy(), mask.cpu().numpy().view(np.uint32)
    assert (pk[nb:] == 0xA5).all() and (yy[n:] == 7.0).all() and (mk[words:] == 0x5A5A5A5A).all()
    return (yy[:n].reshape(N, G), mk[:words], pk[:nb], s32.cpu().numpy(), m32.cpu().numpy(),
            sbf.cpu().numpy().view(np.uint16), mbf.cpu().numpy().view(np.uint16))


def _same(got, want):
    for name, g_, w_ in zip(("y", "mask", "packed", "scale", "min", "scale_bf16", "min_bf16"), got, want):
        assert np.ascontiguousarray(g_).tobytes() == np.ascontiguousarray(w_).tobytes(), name


SHAPES = [(1, 8), (37, 40), (64, 256), (203, 256), (33, 1024), (129, 104), (19, 520), (20011, 256)]


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", SHAPES)
@pytest.mark.parametrize("supplied", [True, False])
def test_relu_dropout_pack_equals_the_oracle_chain(N, G, bits, supplied):
    print(f"case fused N={N} G={G} bits={bits} supplied={supplied}", flush=True)
    rng = np.random.default_rng(N * 1000 + G + bits)
    x = (rng.standard_normal((N, G)) * 2).astype(F32)
    if N > 3:
        x[2] = -np.abs(x[2])                      # a row that ReLU zeroes entirely -> constant row
    if supplied:
        act_noise, noise = rng.random((N, G), dtype=F32), rng.random((N, G), dtype=F32)
    else:
        act_noise = o.philox_noise_flat(11, 3, N * G).reshape(N, G)
        noise = o.philox_noise_rows(12, 4, N, G)
    got = _launch(x, 0.5, bits, act_noise if supplied else None, noise if supplied else None, (11, 3, 12, 4))
    _same(got, _chain(x, 0.5, bits, act_noise, noise))


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", SHAPES)
@pytest.mark.parametrize("supplied", [True, False])
def test_bn_relu_dropout_pack_equals_the_oracle_chain_on_the_normalised_input(N, G, bits, supplied):
    print(f"case bn-fused N={N} G={G} bits={bits} supplied={supplied}", flush=True)
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
    got = _launch(x, 0.25, bits, act_noise if supplied else None, noise if supplied else None, (21, 8, 22, 12),
                  norm=(mean, mult, shift))
    normalised = ((x - mean[None, :]) * mult[None, :] + shift[None, :]).astype(F32)   # three fp32 roundings
    _same(got, _chain(normalised, 0.25, bits, act_noise, noise))


@pytest.mark.parametrize("folded", [False, True])
def test_fused_epilogues_at_config_2_size(folded):
    """Every output of the fused pass on a [169343, 256] activation (INT2, internal Philox
    streams), with and without the batch norm, bit for bit against the oracle chain."""
    N, G, bits = 169343, 256, 2
    print(f"case fused full size folded={folded}", flush=True)
    rng = np.random.default_rng(2 + folded)
    x = (rng.standard_normal((N, G), dtype=F32) * F32(2) + F32(0.5)).astype(F32)
    act_noise = o.philox_noise_flat(31, 16, N * G).reshape(N, G)
    noise = o.philox_noise_rows(32, 20, N, G)
    if folded:
        mean = rng.standard_normal(G).astype(F32)
        mult = (rng.random(G, dtype=F32) + F32(0.5)).astype(F32)
        shift = rng.standard_normal(G).astype(F32)
        got = _launch(x, 0.5, bits, None, None, (31, 16, 32, 20), norm=(mean, mult, shift))
        x = ((x - mean[None, :]) * mult[None, :] + shift[None, :]).astype(F32)
    else:
        got = _launch(x, 0.5, bits, None, None, (31, 16, 32, 20))
    _same(got, _chain(x, 0.5, bits, act_noise, noise))
