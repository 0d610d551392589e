"""ctypes loader of the C restatement (oracle/exact_oracle.c).
TEST INFRASTRUCTURE ONLY -- see the header of exact_oracle.py."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "_build", "libexact_oracle.so")
_lib = None


def build():
    subprocess.run(["make", "-C", _HERE, "-B"], check=True, capture_output=True)
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = ctypes.CDLL(LIB_PATH)
        _lib.oracle_packed_nbytes.restype = ctypes.c_int64
        _lib.oracle_packed_nbytes.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]
        _lib.oracle_count_fast_division_mismatches.restype = ctypes.c_int64
        _lib.oracle_count_fast_division_mismatches.argtypes = [ctypes.c_int]
        _lib.oracle_f32_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_f32_to_bf16.argtypes = [ctypes.c_float]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


I64, U64, INT, F = ctypes.c_int64, ctypes.c_uint64, ctypes.c_int, ctypes.c_float


def num_threads():
    return lib().oracle_num_threads()


def philox4x32_10(ctr, key):
    c = np.ascontiguousarray(ctr, dtype=np.uint32)
    k = np.ascontiguousarray(key, dtype=np.uint32)
    out = np.empty(4, dtype=np.uint32)
    lib().oracle_philox4x32_10(_p(c), _p(k), _p(out))
    return out


def row_minmax(x):
    x = _f32(x)
    N, G = x.shape
    mn, mx = np.empty(N, np.float32), np.empty(N, np.float32)
    lib().oracle_row_minmax(_p(x), I64(N), I64(G), _p(mn), _p(mx))
    return mn, mx


def scale(mn, mx, bits):
    mn, mx = _f32(mn), _f32(mx)
    out = np.empty_like(mn)
    lib().oracle_scale(_p(mn), _p(mx), I64(mn.size), INT(bits), _p(out))
    return out


def pack(x, mn, sc, bits, noise=None, seed=0, offset=0):
    x, mn, sc, noise = _f32(x), _f32(mn), _f32(sc), _f32(noise)
    N, G = x.shape
    out = np.zeros(lib().oracle_packed_nbytes(N, G, bits), dtype=np.uint8)
    lib().oracle_pack(_p(x), _p(mn), _p(sc), _p(noise), U64(seed), U64(offset), I64(N), I64(G), INT(bits), _p(out))
    return out


def unpack(packed, bits, sc, mn, N, G):
    packed = np.ascontiguousarray(packed).view(np.uint8)
    sc, mn = _f32(sc), _f32(mn)
    out = np.empty((N, G), np.float32)
    lib().oracle_unpack(_p(packed), INT(bits), _p(sc), _p(mn), I64(N), I64(G), _p(out))
    return out


def pack_unpack_roundtrip(x, bits, noise=None, seed=0, offset=0):
    """The whole quantize_activation -> dequantize_activation chain; used as
    the timed CPU baseline."""
    x, noise = _f32(x), _f32(noise)
    N, G = x.shape
    packed = np.zeros(lib().oracle_packed_nbytes(N, G, bits), dtype=np.uint8)
    mn, mx, sc = (np.empty(N, np.float32) for _ in range(3))
    out = np.empty((N, G), np.float32)
    lib().oracle_pack_unpack_roundtrip(_p(x), _p(noise), U64(seed), U64(offset), I64(N), I64(G), INT(bits),
                                       _p(packed), _p(mn), _p(mx), _p(sc), _p(out))
    return packed, out


def relu_fwd(x):
    x = _f32(x).reshape(-1)
    y = np.empty_like(x)
    mask = np.zeros((x.size + 31) // 32, np.uint32)
    lib().oracle_relu_fwd(_p(x), I64(x.size), _p(y), _p(mask))
    return y, mask


def relu_bwd(dy, mask):
    dy = _f32(dy).reshape(-1)
    dx = np.empty_like(dy)
    mask = np.ascontiguousarray(mask, dtype=np.uint32)
    lib().oracle_relu_bwd(_p(dy), _p(mask), I64(dy.size), _p(dx))
    return dx


def dropout_fwd(x, p, noise=None, seed=0, offset=0):
    x, noise = _f32(x).reshape(-1), (None if noise is None else _f32(noise).reshape(-1))
    y = np.empty_like(x)
    mask = np.zeros((x.size + 31) // 32, np.uint32)
    lib().oracle_dropout_fwd(_p(x), _p(noise), U64(seed), U64(offset), F(p), I64(x.size), _p(y), _p(mask))
    return y, mask


def dropout_bwd(dy, mask, p):
    dy = _f32(dy).reshape(-1)
    dx = np.empty_like(dy)
    mask = np.ascontiguousarray(mask, dtype=np.uint32)
    lib().oracle_dropout_bwd(_p(dy), _p(mask), F(p), I64(dy.size), _p(dx))
    return dx


def spmm_csr(rowptr, col, val, X, reduce="sum"):
    rowptr = np.ascontiguousarray(rowptr, dtype=np.int64)
    col = np.ascontiguousarray(col, dtype=np.int64)
    val, X = _f32(val), _f32(X)
    M, K = rowptr.size - 1, X.shape[1]
    out = np.empty((M, K), np.float32)
    lib().oracle_spmm_csr(_p(rowptr), _p(col), _p(val), _p(X), I64(M), I64(K), INT(reduce == "mean"), _p(out))
    return out


def rp_fwd(X, R):
    X, R = _f32(X), _f32(R)
    out = np.empty((X.shape[0], R.shape[1]), np.float32)
    lib().oracle_rp_fwd(_p(X), _p(R), I64(X.shape[0]), I64(X.shape[1]), I64(R.shape[1]), _p(out))
    return out


def rp_bwd(Xr, R):
    Xr, R = _f32(Xr), _f32(R)
    out = np.empty((Xr.shape[0], R.shape[0]), np.float32)
    lib().oracle_rp_bwd(_p(Xr), _p(R), I64(Xr.shape[0]), I64(R.shape[0]), I64(R.shape[1]), _p(out))
    return out
