"""Load the SIMT-emulated build of the kernels (tests/emu) and call its C ABI
with NumPy arrays.  The emulated library is compiled from the very same .hip
sources as libexact_hip.so; it exists so that the kernels' indexing and
arithmetic are checked on machines without a GPU."""
import ctypes
import importlib.util
import os

import numpy as np

from exact_amd import _lib

HERE = os.path.dirname(os.path.abspath(__file__))
_spec = importlib.util.spec_from_file_location("build_emu", os.path.join(HERE, "emu", "build_emu.py"))
build_emu = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(build_emu)

_emu = None


def _newest_source_mtime():
    files = [os.path.join(build_emu.CSRC, f) for f in os.listdir(build_emu.CSRC) if f.endswith((".hip", ".hpp"))]
    files.append(os.path.join(HERE, "emu", "include", "hip", "hip_runtime.h"))
    return max(os.path.getmtime(f) for f in files)


def emu():
    global _emu
    if _emu is None:
        if not os.path.exists(build_emu.LIB) or os.path.getmtime(build_emu.LIB) < _newest_source_mtime():
            build_emu.build_lib()
        handle = ctypes.CDLL(build_emu.LIB)
        for name, (res, args) in _lib.SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _emu = handle
    return _emu


def p(a):
    return None if a is None else a.ctypes.data


def f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def minmax_pack(x, bits, noise=None, seed=0, offset=0, guard=64):
    """-> (packed u8, scale f32, min f32, scale bf16 bits, min bf16 bits); the
    packed buffer has `guard` sentinel bytes behind it that must stay intact."""
    x = f32(x)
    N, G = x.shape
    nb = int(emu().exact_packed_nbytes(N, G, bits))
    packed = np.full(nb + guard, 0xA5, np.uint8)
    s32, m32 = np.zeros(N, np.float32), np.zeros(N, np.float32)
    sbf, mbf = np.zeros(N, np.uint16), np.zeros(N, np.uint16)
    noise = None if noise is None else f32(noise)
    rc = emu().exact_minmax_pack_f32(p(x), p(noise), seed, offset, N, G, bits, p(packed), p(s32), p(m32), p(sbf),
                                     p(mbf), None)
    assert rc == 0, rc
    assert (packed[nb:] == 0xA5).all(), "pack wrote past the packed stream"
    return packed[:nb], s32, m32, sbf, mbf


def pack(x, mn, scale, bits, noise=None, seed=0, offset=0, guard=64):
    x = f32(x)
    N, G = x.shape
    nb = int(emu().exact_packed_nbytes(N, G, bits))
    packed = np.full(nb + guard, 0xA5, np.uint8)
    noise = None if noise is None else f32(noise)
    rc = emu().exact_pack_f32(p(x), p(f32(mn)), p(f32(scale)), p(noise), seed, offset, N, G, bits, p(packed), None)
    assert rc == 0, rc
    assert (packed[nb:] == 0xA5).all()
    return packed[:nb]


def unpack(packed, bits, scale, mn, N, G, bf16=False, guard=64):
    out = np.full(N * G + guard, np.float32(-12345.0), np.float32)
    packed = np.ascontiguousarray(packed)
    if bf16:
        rc = emu().exact_unpack_bf16param_f32(p(packed), bits, p(np.ascontiguousarray(scale, np.uint16)),
                                              p(np.ascontiguousarray(mn, np.uint16)), N, G, p(out), None)
    else:
        rc = emu().exact_unpack_f32(p(packed), bits, p(f32(scale)), p(f32(mn)), N, G, p(out), None)
    assert rc == 0, rc
    assert (out[N * G:] == np.float32(-12345.0)).all(), "unpack wrote past the output"
    return out[:N * G].reshape(N, G)


def row_minmax(x):
    x = f32(x)
    N, G = x.shape
    mn, mx = np.zeros(N, np.float32), np.zeros(N, np.float32)
    assert emu().exact_row_minmax_f32(p(x), N, G, p(mn), p(mx), None) == 0
    return mn, mx


def relu_fwd(x, guard=8):
    x = f32(x).reshape(-1)
    n = x.size
    y = np.full(n + guard, np.float32(7.0), np.float32)
    words = (n + 31) // 32
    mask = np.full(words + guard, 0x5A5A5A5A, np.uint32)
    assert emu().exact_relu_fwd_f32(p(x), n, p(y), p(mask), None) == 0
    assert (y[n:] == 7.0).all() and (mask[words:] == 0x5A5A5A5A).all()
    return y[:n], mask[:words]


def relu_bwd(dy, mask):
    dy = f32(dy).reshape(-1)
    dx = np.zeros_like(dy)
    assert emu().exact_relu_bwd_f32(p(dy), p(np.ascontiguousarray(mask, np.uint32)), dy.size, p(dx), None) == 0
    return dx


def dropout_fwd(x, prob, noise=None, seed=0, offset=0, guard=8):
    x = f32(x).reshape(-1)
    n = x.size
    y = np.full(n + guard, np.float32(7.0), np.float32)
    words = (n + 31) // 32
    mask = np.full(words + guard, 0x5A5A5A5A, np.uint32)
    noise = None if noise is None else f32(noise).reshape(-1)
    assert emu().exact_dropout_fwd_f32(p(x), p(noise), seed, offset, prob, n, p(y), p(mask), None) == 0
    assert (y[n:] == 7.0).all() and (mask[words:] == 0x5A5A5A5A).all()
    return y[:n], mask[:words]


def dropout_bwd(dy, mask, prob):
    dy = f32(dy).reshape(-1)
    dx = np.zeros_like(dy)
    assert emu().exact_dropout_bwd_f32(p(dy), p(np.ascontiguousarray(mask, np.uint32)), prob, dy.size, p(dx), None) == 0
    return dx


def spmm(rowptr, col, val, X, reduce, idx=np.int64, guard=16):
    rowptr = np.ascontiguousarray(rowptr, dtype=idx)
    col = np.ascontiguousarray(col, dtype=idx)
    X = f32(X)
    val = None if val is None else f32(val)
    M, K = rowptr.size - 1, X.shape[1]
    out = np.full(M * K + guard, np.float32(-777.0), np.float32)
    rc = emu().exact_spmm_csr_f32(p(rowptr), p(col), p(val), rowptr.itemsize, p(X), M, X.shape[0], K, col.size,
                                  1 if reduce == "mean" else 0, p(out), None)
    assert rc == 0, rc
    assert (out[M * K:] == np.float32(-777.0)).all()
    return out[:M * K].reshape(M, K)


RP_MODES = {"fp32": 0, "bf16_split": 1, "bf16_signs": 2}


def rp_table(R, mode, guard=64):
    """The operand-fragment table of R for the bf16 entry points (exactly sized, with a guard behind it)."""
    R = f32(R)
    if mode == "bf16_signs":
        assert (np.abs(R) == np.abs(R).max()).all() and np.abs(R).max() > 0, "the signs mode needs a +-c matrix"
    D, k = R.shape
    nb = int(emu().exact_rp_table_nbytes(D, k, RP_MODES[mode]))
    assert nb > 0 and nb % 16 == 0
    raw = np.full(nb + guard + 16, 0xC3, np.uint8)
    off = (-raw.ctypes.data) % 16
    table = raw[off:off + nb + guard]
    rc = emu().exact_rp_prepare_bf16(p(R), D, k, RP_MODES[mode], p(table), None)
    assert rc == 0, rc
    assert (table[nb:] == 0xC3).all()
    return table


def rp_fwd(X, R, guard=16, mode="fp32"):
    X, R = f32(X), f32(R)
    N, D = X.shape
    k = R.shape[1]
    out = np.full(N * k + guard, np.float32(-777.0), np.float32)
    if mode == "fp32":
        rc = emu().exact_rp_fwd_f32(p(X), p(R), N, D, k, p(out), None)
    else:
        table = rp_table(R, mode)          # held until the call has returned
        rc = emu().exact_rp_fwd_bf16_f32(p(X), p(table), N, D, k, RP_MODES[mode], p(out), None)
    assert rc == 0, rc
    assert (out[N * k:] == np.float32(-777.0)).all()
    return out[:N * k].reshape(N, k)


def rp_minmax_pack(X, R, bits, noise=None, seed=0, offset=0, guard=64, expect_rc=0, mode="fp32"):
    """-> (packed, scale f32, min f32, scale bf16 bits, min bf16 bits) of the projected X."""
    X, R = f32(X), f32(R)
    N, D = X.shape
    k = R.shape[1]
    nb = int(emu().exact_packed_nbytes(N, k, bits)) if bits in (1, 2, 4, 8) else 1
    packed = np.full(nb + guard, 0xA5, np.uint8)
    s32, m32 = np.full(N + 1, np.float32(-3.0), np.float32), np.full(N + 1, np.float32(-3.0), np.float32)
    sbf, mbf = np.full(N + 1, 0x1234, np.uint16), np.full(N + 1, 0x1234, np.uint16)
    noise = None if noise is None else f32(noise)
    if mode == "fp32":
        rc = emu().exact_rp_minmax_pack_f32(p(X), p(R), p(noise), seed, offset, N, D, k, bits, p(packed), p(s32), p(m32),
                                            p(sbf), p(mbf), None)
    else:
        table = rp_table(R, mode)
        rc = emu().exact_rp_minmax_pack_bf16_f32(p(X), p(table), RP_MODES[mode], p(noise), seed, offset,
                                                 N, D, k, bits, p(packed), p(s32), p(m32), p(sbf), p(mbf), None)
    assert rc == expect_rc, rc
    if rc != 0:
        return None
    assert (packed[nb:] == 0xA5).all() and s32[N] == -3.0 and m32[N] == -3.0 and sbf[N] == 0x1234 and mbf[N] == 0x1234
    return packed[:nb], s32[:N], m32[:N], sbf[:N], mbf[:N]


def rp_bwd(Xr, R, guard=16, mode="fp32"):
    Xr, R = f32(Xr), f32(R)
    N, k = Xr.shape
    D = R.shape[0]
    out = np.full(N * D + guard, np.float32(-777.0), np.float32)
    if mode == "fp32":
        rc = emu().exact_rp_bwd_f32(p(Xr), p(R), N, D, k, p(out), None)
    else:
        table = rp_table(R, mode)
        rc = emu().exact_rp_bwd_bf16_f32(p(Xr), p(table), N, D, k, RP_MODES[mode], p(out), None)
    assert rc == 0, rc
    assert (out[N * D:] == np.float32(-777.0)).all()
    return out[:N * D].reshape(N, D)


def leaky_relu_fwd(x, slope, guard=8):
    x = f32(x).reshape(-1)
    n = x.size
    y = np.full(n + guard, np.float32(7.0), np.float32)
    words = (n + 31) // 32
    mask = np.full(words + guard, 0x5A5A5A5A, np.uint32)
    assert emu().exact_leaky_relu_fwd_f32(p(x), n, slope, p(y), p(mask), None) == 0
    assert (y[n:] == 7.0).all() and (mask[words:] == 0x5A5A5A5A).all()
    return y[:n], mask[:words]


def leaky_relu_bwd(dy, mask, slope):
    dy = f32(dy).reshape(-1)
    dx = np.zeros_like(dy)
    assert emu().exact_leaky_relu_bwd_f32(p(dy), p(np.ascontiguousarray(mask, np.uint32)), dy.size, slope, p(dx), None) == 0
    return dx


def spmm_minmax(rowptr, col, val, X, is_max, idx=np.int64, guard=16):
    rowptr = np.ascontiguousarray(rowptr, dtype=idx)
    col = np.ascontiguousarray(col, dtype=idx)
    X = f32(X)
    val = None if val is None else f32(val)
    M, K = rowptr.size - 1, X.shape[1]
    out = np.full(M * K + guard, np.float32(-777.0), np.float32)
    arg = np.full(M * K + guard, -5, idx)
    rc = emu().exact_spmm_csr_minmax_f32(p(rowptr), p(col), p(val), rowptr.itemsize, p(X), M, X.shape[0], K, col.size,
                                         1 if is_max else 0, p(out), p(arg), None)
    assert rc == 0, rc
    assert (out[M * K:] == np.float32(-777.0)).all() and (arg[M * K:] == -5).all()
    return out[:M * K].reshape(M, K), arg[:M * K].reshape(M, K)


def sddmm(row, rowptr, col, mat, grad, reduce, idx=np.int64, guard=8):
    row, rowptr, col = (np.ascontiguousarray(a, dtype=idx) for a in (row, rowptr, col))
    mat, grad = f32(mat), f32(grad)
    out = np.full(row.size + guard, np.float32(-777.0), np.float32)
    rc = emu().exact_sddmm_f32(p(row), p(rowptr), p(col), row.itemsize, p(mat), p(grad), row.size, mat.shape[1],
                               1 if reduce == "mean" else 0, p(out), None)
    assert rc == 0, rc
    assert (out[row.size:] == np.float32(-777.0)).all()
    return out[:row.size]


def relu_dropout_fwd(x, prob, noise=None, seed=0, offset=0, guard=8):
    x = f32(x).reshape(-1)
    n = x.size
    y = np.full(n + guard, np.float32(7.0), np.float32)
    words = (n + 31) // 32
    mask = np.full(words + guard, 0x5A5A5A5A, np.uint32)
    noise = None if noise is None else f32(noise).reshape(-1)
    assert emu().exact_relu_dropout_fwd_f32(p(x), p(noise), seed, offset, prob, n, p(y), p(mask), None) == 0
    assert (y[n:] == 7.0).all() and (mask[words:] == 0x5A5A5A5A).all()
    return y[:n], mask[:words]


def relu_dropout_minmax_pack(x, prob, bits, act_noise=None, noise=None, act_seed=0, act_offset=0, seed=0, offset=0,
                             guard=64, expect_rc=0, norm=None):
    """-> (y, mask words, packed, scale f32, min f32, scale bf16 bits, min bf16 bits).
    norm = (mean, mult, shift) selects the entry point with batch norm ahead of the ReLU."""
    x = f32(x)
    N, G = x.shape
    n = N * G
    nb = int(emu().exact_packed_nbytes(N, G, bits))
    packed = np.full(nb + guard, 0xA5, np.uint8)
    y = np.full(n + guard, np.float32(7.0), np.float32)
    words = (n + 31) // 32
    mask = np.full(words + guard, 0x5A5A5A5A, np.uint32)
    s32, m32 = np.zeros(N, np.float32), np.zeros(N, np.float32)
    sbf, mbf = np.zeros(N, np.uint16), np.zeros(N, np.uint16)
    act_noise = None if act_noise is None else f32(act_noise)
    noise = None if noise is None else f32(noise)
    if norm is None:
        rc = emu().exact_relu_dropout_minmax_pack_f32(p(x), prob, p(act_noise), act_seed, act_offset, p(noise), seed,
                                                      offset, N, G, bits, p(y), p(mask), p(packed), p(s32), p(m32),
                                                      p(sbf), p(mbf), None)
    else:
        mean, mult, shift = (None if v is None else f32(v) for v in norm)
        rc = emu().exact_bn_relu_dropout_minmax_pack_f32(p(x), p(mean), p(mult), p(shift), prob, p(act_noise), act_seed,
                                                         act_offset, p(noise), seed, offset, N, G, bits, p(y), p(mask),
                                                         p(packed), p(s32), p(m32), p(sbf), p(mbf), None)
    assert rc == expect_rc, rc
    if rc != 0:
        return None
    assert (packed[nb:] == 0xA5).all() and (y[n:] == 7.0).all() and (mask[words:] == 0x5A5A5A5A).all()
    return y[:n].reshape(N, G), mask[:words], packed[:nb], s32, m32, sbf, mbf


# ---- fp16 entry points -------------------------------------------------------
def f16(a):
    return np.ascontiguousarray(a, dtype=np.float16)


def minmax_pack_f16(x, bits, noise=None, seed=0, offset=0, guard=64, expect_rc=0):
    x = f16(x)
    N, G = x.shape
    nb = int(emu().exact_packed_nbytes(N, G, bits))
    packed = np.full(nb + guard, 0xA5, np.uint8)
    sc, mn = np.zeros(N, np.float16), np.zeros(N, np.float16)
    noise = None if noise is None else f32(noise)
    rc = emu().exact_minmax_pack_f16(p(x), p(noise), seed, offset, N, G, bits, p(packed), p(sc), p(mn), None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (packed[nb:] == 0xA5).all()
    return packed[:nb], sc, mn


def unpack_f16(packed, bits, scale, mn, N, G, guard=64):
    out = np.full(N * G + guard, np.float16(-123.0), np.float16)
    rc = emu().exact_unpack_f16(p(np.ascontiguousarray(packed)), bits, p(f16(scale)), p(f16(mn)), N, G, p(out), None)
    assert rc == 0, rc
    assert (out[N * G:] == np.float16(-123.0)).all()
    return out[:N * G].reshape(N, G)


def _mask_fwd_f16(fn, x, *args, guard=8):
    x = f16(x).reshape(-1)
    n = x.size
    y = np.full(n + guard, np.float16(7.0), np.float16)
    words = (n + 31) // 32
    mask = np.full(words + guard, 0x5A5A5A5A, np.uint32)
    assert fn(x, n, y, mask, *args) == 0
    assert (y[n:] == 7.0).all() and (mask[words:] == 0x5A5A5A5A).all()
    return y[:n], mask[:words]


def relu_fwd_f16(x):
    return _mask_fwd_f16(lambda x, n, y, m: emu().exact_relu_fwd_f16(p(x), n, p(y), p(m), None), x)


def leaky_relu_fwd_f16(x, slope):
    return _mask_fwd_f16(lambda x, n, y, m: emu().exact_leaky_relu_fwd_f16(p(x), n, slope, p(y), p(m), None), x)


def dropout_fwd_f16(x, prob, noise=None, seed=0, offset=0, relu=False):
    noise = None if noise is None else f32(noise).reshape(-1)
    fn = emu().exact_relu_dropout_fwd_f16 if relu else emu().exact_dropout_fwd_f16
    return _mask_fwd_f16(lambda x, n, y, m: fn(p(x), p(noise), seed, offset, prob, n, p(y), p(m), None), x)


def mask_bwd_f16(kind, dy, mask, arg=None):
    dy = f16(dy).reshape(-1)
    dx = np.zeros_like(dy)
    mask = np.ascontiguousarray(mask, np.uint32)
    if kind == "relu":
        rc = emu().exact_relu_bwd_f16(p(dy), p(mask), dy.size, p(dx), None)
    elif kind == "leaky":
        rc = emu().exact_leaky_relu_bwd_f16(p(dy), p(mask), dy.size, arg, p(dx), None)
    else:
        rc = emu().exact_dropout_bwd_f16(p(dy), p(mask), arg, dy.size, p(dx), None)
    assert rc == 0, rc
    return dx


def minmax_pack_geom(x, bits, octs_per_lane, noise=None, seed=0, offset=0, guard=64, expect_rc=0):
    """exact_minmax_pack_geom_f32 -> (packed, scale bf16 bits, min bf16 bits)."""
    x = f32(x)
    N, G = x.shape
    nb = int(emu().exact_packed_nbytes(N, G, bits))
    packed = np.full(nb + guard, 0xA5, np.uint8)
    sbf, mbf = np.zeros(N, np.uint16), np.zeros(N, np.uint16)
    noise = None if noise is None else f32(noise)
    rc = emu().exact_minmax_pack_geom_f32(p(x), p(noise), seed, offset, N, G, bits, p(packed), None, None, p(sbf),
                                          p(mbf), octs_per_lane, None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (packed[nb:] == 0xA5).all()
    return packed[:nb], sbf, mbf


def spmm_rowwise(rowptr, col, val, X, reduce, idx=np.int64, guard=16):
    rowptr = np.ascontiguousarray(rowptr, dtype=idx)
    col = np.ascontiguousarray(col, dtype=idx)
    X = f32(X)
    val = None if val is None else f32(val)
    M, K = rowptr.size - 1, X.shape[1]
    out = np.full(M * K + guard, np.float32(-777.0), np.float32)
    rc = emu().exact_spmm_csr_rowwise_f32(p(rowptr), p(col), p(val), rowptr.itemsize, p(X), M, X.shape[0], K, col.size,
                                          1 if reduce == "mean" else 0, p(out), None)
    assert rc == 0, rc
    assert (out[M * K:] == np.float32(-777.0)).all()
    return out[:M * K].reshape(M, K)


def colsum(x, guard=8, expect_rc=0):
    """exact_colsum_f32 -> fp32 [K]."""
    x = f32(x)
    N, K = x.shape
    out = np.full(K + guard, np.float32(-777.0), np.float32)
    rc = emu().exact_colsum_f32(p(x), N, K, p(out), None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (out[K:] == np.float32(-777.0)).all()
    return out[:K]


def bn_backward_reduce(dy, x, mean, guard=8, expect_rc=0):
    """exact_bn_backward_reduce_f32 -> (sum_dy, sum_dy_xmu), fp32 [K] each."""
    dy, x, mean = f32(dy), f32(x), f32(mean)
    N, K = dy.shape
    a = np.full(K + guard, np.float32(-777.0), np.float32)
    b = np.full(K + guard, np.float32(-777.0), np.float32)
    rc = emu().exact_bn_backward_reduce_f32(p(dy), p(x), p(mean), N, K, p(a), p(b), None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (a[K:] == np.float32(-777.0)).all() and (b[K:] == np.float32(-777.0)).all()
    return a[:K], b[:K]


def col_moments(x, center, guard=8, expect_rc=0):
    """exact_col_moments_f32 -> (sum of (x - center), sum of (x - center)^2), fp32 [K] each."""
    x, center = f32(x), f32(center)
    N, K = x.shape
    a = np.full(K + guard, np.float32(-777.0), np.float32)
    b = np.full(K + guard, np.float32(-777.0), np.float32)
    rc = emu().exact_col_moments_f32(p(x), p(center), N, K, p(a), p(b), None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (a[K:] == np.float32(-777.0)).all() and (b[K:] == np.float32(-777.0)).all()
    return a[:K], b[:K]


def linear_dw(dy, x, ldy=None, ldx=None, guard=8, expect_rc=0, bf16=False):
    """exact_linear_dw_f32 / exact_linear_dw_bf16_f32 -> fp32 [Kout, D]; dy / x may be given wider than used (row strides)."""
    dy, x = f32(dy), f32(x)
    N, K = dy.shape
    D = x.shape[1]
    if ldy:
        wide = np.full((N, ldy), np.float32(np.nan), np.float32); wide[:, :K] = dy; dy = wide
    if ldx:
        wide = np.full((N, ldx), np.float32(np.nan), np.float32); wide[:, :D] = x; x = wide
    out = np.full(K * D + guard, np.float32(-777.0), np.float32)
    fn = emu().exact_linear_dw_bf16_f32 if bf16 else emu().exact_linear_dw_f32
    rc = fn(p(dy), dy.shape[1], p(x), x.shape[1], N, K, D, p(out), None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (out[K * D:] == np.float32(-777.0)).all()
    return out[:K * D].reshape(K, D)


def tall_gemm(X, M, bias=None, addend=None, transposed=False, ld=None, in_place=False, guard=16, expect_rc=0):
    """exact_tall_gemm_prepare_bf16 + exact_tall_gemm_bf16_f32: X [N, D] . M [D, K] (+ bias) (+ addend) -> fp32 [N, K].
    `M` is given as the [D, K] matrix; transposed=True hands it over as its [K, D] transpose, `ld` as a wider row
    stride with NaN in the padding; in_place=True passes the output (pre-filled with addend) as the addend."""
    X, M = f32(X), f32(M)
    N, D = X.shape
    K = M.shape[1]
    src = np.ascontiguousarray(M.T) if transposed else M
    if ld:
        wide = np.full((src.shape[0], ld), np.float32(np.nan), np.float32); wide[:, :src.shape[1]] = src; src = wide
    nb = int(emu().exact_tall_gemm_table_nbytes(D, K))
    assert nb > 0 and nb % 16 == 0
    raw = np.full(nb + 64 + 16, 0xC3, np.uint8)
    off = (-raw.ctypes.data) % 16
    table = raw[off:off + nb + 64]
    rc = emu().exact_tall_gemm_prepare_bf16(p(src), src.shape[1], int(transposed), D, K, p(table), None)
    assert rc == 0, rc
    assert (table[nb:] == 0xC3).all()
    out = np.full(N * K + guard, np.float32(-777.0), np.float32)
    b = None if bias is None else f32(bias)
    a = None if addend is None else f32(addend)
    if in_place and a is not None:
        out[:N * K] = a.reshape(-1)
        rc = emu().exact_tall_gemm_bf16_f32(p(X), p(table), N, D, K, p(b) if b is not None else None, p(out), K, p(out), K, None)
    else:
        rc = emu().exact_tall_gemm_bf16_f32(p(X), p(table), N, D, K, p(b) if b is not None else None,
                                            p(a) if a is not None else None, K, p(out), K, None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (out[N * K:] == np.float32(-777.0)).all()
    return out[:N * K].reshape(N, K)


def stream_probe(x, out_bytes, guard=32, expect_rc=0):
    """exact_stream_probe_f32 on a flat fp32 array -> the bytes it wrote."""
    x = f32(x).reshape(-1)
    nb = max(16, (x.size // 16) * out_bytes)
    out = np.full(nb + guard, 0xA5, np.uint8)
    rc = emu().exact_stream_probe_f32(p(x), x.size, out_bytes, p(out), None)
    assert rc == expect_rc, rc
    if rc:
        return None
    assert (out[nb:] == 0xA5).all()
    return out[:nb]

