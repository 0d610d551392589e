"""CPU restatement of the reference's fp16 (at::Half) instantiation of the path:
what its kernels compute when the activations are fp16, i.e. under autocast
(ops.py:130, 260, 313 cast the Functions' inputs to torch.float16).  TEST
INFRASTRUCTURE ONLY (see the header of exact_oracle.py).

at::Half's binary operators evaluate in fp32 and round the result to fp16
(c10/util/Half-inl.h), and a Half combined with a float yields a float.  So

  scale  = h(h(1 / h(mx - mn)) * B)            torch: (2**bits - 1) / (mx - mn) on fp16 tensors, ops.py:39
  q      = rn(fmax(h(h(x - mn) * scale) + u - 0.5, 0))      quantization_cuda_kernel.cu:88-89 (u is a float)
  x_hat  = h(h(q / scale) + mn)                              quantization_cuda_kernel.cu:182
  y      = h(x * keep * pinv), dx = h(dy / p1m)              :490, :566
  y      = h(x * slope)                                      :356

with h() = round to nearest even fp16.  Pinned in tests/test_oracle_half.py
against torch's CPU fp16 tensor arithmetic (which rounds the same way).
PARITY UNPINNED against the reference itself: its fp16 kernels cannot be run
here and its tests hold no fp16 vectors."""
import numpy as np

import exact_oracle as o

F32, F16 = np.float32, np.float16


def h(x):
    """fp32 array -> the fp32 values of its fp16 rounding."""
    with np.errstate(over="ignore", invalid="ignore"):
        return np.asarray(x, dtype=F32).astype(F16).astype(F32)


def compute_scale(mn, mx, bits):
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        return h(h(F32(1.0) / h(np.asarray(mx, F32) - np.asarray(mn, F32))) * F32(2 ** bits - 1))


def quantize_activation(x, bits, noise):
    """x fp16 [N, G] -> (packed uint8, scale fp16, min fp16)."""
    x = np.asarray(x)
    assert x.dtype == F16
    xf = x.astype(F32)
    mn, mx = xf.min(1), xf.max(1)
    scale = compute_scale(mn, mx, bits)
    with np.errstate(invalid="ignore", over="ignore"):
        t = h(h(xf - mn[:, None]) * scale[:, None])
        t = (t + np.asarray(noise, F32)).astype(F32)
        t = (t - F32(0.5)).astype(F32)
        t = np.fmax(t, F32(0.0))
        # cvt.rni.s32.f32 clamps to the int32 range: +inf (a scale that overflowed fp16) gives INT_MAX
        big = t >= F32(2147483648.0)
        q = np.where(big, np.int64(2147483647), np.rint(np.where(big, F32(0.0), t)).astype(np.int64))
    N, G = x.shape
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    qpad = np.zeros((n_round, G), np.int64)
    qpad[:N] = q
    qpad = qpad.reshape(n_round // wpt, wpt, G)
    acc = np.zeros((n_round // wpt, G), np.int64)
    for i in range(wpt):
        acc |= qpad[:, i, :] << (i * bits)
    out = np.zeros(o.packed_nbytes(N, G, bits), np.uint8)
    out[:acc.size] = (acc & 0xFF).astype(np.uint8).reshape(-1)
    return out, scale.astype(F16), mn.astype(F16)


def unpack(packed, bits, scale, mn, N, G):
    """-> fp16 [N, G]."""
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    p = np.asarray(packed).view(np.uint8)[:(n_round // wpt) * G].reshape(n_round // wpt, 1, G).astype(np.int32)
    shifts = (np.arange(wpt, dtype=np.int32) * bits).reshape(1, wpt, 1)
    q = ((p >> shifts) & (2 ** bits - 1)).reshape(n_round, G)[:N].astype(F32)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        v = h(q / np.asarray(scale, F16).astype(F32)[:, None])
        return (v + np.asarray(mn, F16).astype(F32)[:, None]).astype(F32).astype(F16)


def relu_fwd(x):
    x = np.asarray(x)
    assert x.dtype == F16
    bit = x > 0
    return np.where(bit, x, F16(0)), o._pack_bits(bit)


def relu_bwd(dy, mask_words):
    dy = np.asarray(dy)
    bit = o._unpack_bits(mask_words, dy.size).reshape(dy.shape)
    return np.where(bit, dy, F16(0))


def leaky_relu_fwd(x, slope):
    x = np.asarray(x)
    bit = x > 0
    with np.errstate(over="ignore"):
        return np.where(bit, x, (x.astype(F32) * F32(slope)).astype(F16)), o._pack_bits(bit)


def leaky_relu_bwd(dy, mask_words, slope):
    dy = np.asarray(dy)
    bit = o._unpack_bits(mask_words, dy.size).reshape(dy.shape)
    with np.errstate(over="ignore"):
        return np.where(bit, dy, (dy.astype(F32) * F32(slope)).astype(F16))


def dropout_fwd(x, p, noise, relu=False):
    x = np.asarray(x)
    pf = F32(p)
    pinv = F32(1.0 / (1.0 - float(pf)))
    keep = np.asarray(noise, F32) > pf
    xf = x.astype(F32)
    bit = keep
    if relu:
        pos = xf > 0
        xf = np.where(pos, xf, F32(0))
        bit = keep & pos
    with np.errstate(over="ignore", invalid="ignore"):
        y = ((xf * keep.astype(F32)).astype(F32) * pinv).astype(F32).astype(F16)
    return y, o._pack_bits(bit)


def dropout_bwd(dy, mask_words, p):
    dy = np.asarray(dy)
    p1m = F32(1.0 - float(F32(p)))
    bit = o._unpack_bits(mask_words, dy.size).reshape(dy.shape)
    with np.errstate(over="ignore"):
        return np.where(bit, (dy.astype(F32) / p1m).astype(F32).astype(F16), F16(0))
