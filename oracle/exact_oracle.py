"""CPU restatement of EXACT's activation-compression + sparse-aggregation path.

TEST INFRASTRUCTURE ONLY.  This module is the parity checker for the HIP
library: only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg
may import it.  Nothing in exact_amd/ imports it, and it is never the thing
that is measured as the product or shipped.

Every function restates one piece of the reference algorithm in NumPy fp32
arithmetic (one IEEE-754 rounding per written operation, no fused
multiply-add) and cites the reference file:line it follows.  Paths are
relative to the reference checkout (exact/exact/...).

Pinning status (what fixes each function besides re-reading its own formula):

  philox4x32            Random123 known-answer vectors (three of them).
  bf16_round            torch.Tensor.to(torch.bfloat16) on CPU (library routine).
  row_min_max           numpy min/max (library routine), brute-force loops.
  pack/unpack           hand-computed bytes (0xE4, 0x55/0xAA, ragged N=5),
                        packed-length formula, brute-force Python loops,
                        invariants (0<=q<=B, error bound, constant rows),
                        noise==0.5 => round-half-even, unbiasedness of E[q].
  relu/dropout masks    F.relu + autograd, closed form keep=u>p, np.packbits.
  spmm_csr              scipy.sparse CSR @ dense, dense brute force, A^T.
  rp                    numpy matmul with the matrix passed in; k-formula table.

  parity unpinned:      the reference's own cuRAND noise stream for a torch
                        seed, and nvcc's choice to contract (x-mn)*scale+noise
                        into one FMA.  Neither can be observed without CUDA
                        hardware; the noise is therefore an INPUT here and the
                        arithmetic is defined as unfused fp32.
"""
from __future__ import annotations

import numpy as np

F32 = np.float32
U32 = np.uint32
U64 = np.uint64

# --------------------------------------------------------------------------
# Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
# SC'11).  The reference draws its noise from cuRAND's Philox4_32_10
# (cpp_extension/quantization_cuda_kernel.cu:77-79,88 and :452-453,463); the
# exact cuRAND stream is not reproducible here, so the build defines its own
# counter layout on top of the same published block function.
# --------------------------------------------------------------------------
PHILOX_M0 = 0xD2511F53
PHILOX_M1 = 0xCD9E8D57
PHILOX_W0 = 0x9E3779B9
PHILOX_W1 = 0xBB67AE85


def philox4x32(ctr: np.ndarray, key, rounds: int = 10) -> np.ndarray:
    """ctr: uint32[..., 4], key: (k0, k1) -> uint32[..., 4]."""
    c = np.asarray(ctr, dtype=U64) & U64(0xFFFFFFFF)
    c0, c1, c2, c3 = c[..., 0], c[..., 1], c[..., 2], c[..., 3]
    k0 = int(key[0]) & 0xFFFFFFFF
    k1 = int(key[1]) & 0xFFFFFFFF
    mask = U64(0xFFFFFFFF)
    for _ in range(rounds):
        p0 = U64(PHILOX_M0) * c0
        p1 = U64(PHILOX_M1) * c2
        hi0, lo0 = p0 >> U64(32), p0 & mask
        hi1, lo1 = p1 >> U64(32), p1 & mask
        c0, c1, c2, c3 = (hi1 ^ c1 ^ U64(k0)), lo1, (hi0 ^ c3 ^ U64(k1)), lo0
        k0 = (k0 + PHILOX_W0) & 0xFFFFFFFF
        k1 = (k1 + PHILOX_W1) & 0xFFFFFFFF
    return np.stack([c0, c1, c2, c3], axis=-1).astype(U32)


def _u16_to_uniform(h: np.ndarray) -> np.ndarray:
    """16 random bits -> fp32 uniform on the open interval (0,1):
    u = (h + 0.5) * 2^-16, exact in fp32."""
    return ((h.astype(F32) + F32(0.5)) * F32(2.0 ** -16)).astype(F32)


def philox_noise_rows(seed: int, offset: int, N: int, G: int) -> np.ndarray:
    """Noise the library's internal generator gives element (n, d) of an
    [N, G] activation: one Philox4x32-10 block per 8 consecutive columns,
    counter = (d // 8, n, offset_lo, offset_hi), key = (seed_lo, seed_hi);
    column d uses 16-bit half (d % 2) of output word ((d % 8) // 2),
    low half first."""
    octs = (G + 7) // 8
    n_idx, j_idx = np.meshgrid(np.arange(N, dtype=U64), np.arange(octs, dtype=U64), indexing="ij")
    ctr = np.empty((N, octs, 4), dtype=U64)
    ctr[..., 0] = j_idx
    ctr[..., 1] = n_idx
    ctr[..., 2] = U64(offset & 0xFFFFFFFF)
    ctr[..., 3] = U64((offset >> 32) & 0xFFFFFFFF)
    out = philox4x32(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    halves = np.empty((N, octs, 8), dtype=U32)
    halves[..., 0::2] = out & U32(0xFFFF)
    halves[..., 1::2] = out >> U32(16)
    return _u16_to_uniform(halves.reshape(N, octs * 8)[:, :G])


def philox_noise_flat(seed: int, offset: int, n: int) -> np.ndarray:
    """Noise for flat element i of an n-element tensor (dropout):
    counter = ((i // 8) lo32, (i // 8) hi32, offset_lo, offset_hi)."""
    octs = (n + 7) // 8
    j = np.arange(octs, dtype=U64)
    ctr = np.empty((octs, 4), dtype=U64)
    ctr[:, 0] = j & U64(0xFFFFFFFF)
    ctr[:, 1] = j >> U64(32)
    ctr[:, 2] = U64(offset & 0xFFFFFFFF)
    ctr[:, 3] = U64((offset >> 32) & 0xFFFFFFFF)
    out = philox4x32(ctr, (seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF))
    halves = np.empty((octs, 8), dtype=U32)
    halves[:, 0::2] = out & U32(0xFFFF)
    halves[:, 1::2] = out >> U32(16)
    return _u16_to_uniform(halves.reshape(-1)[:n])


# --------------------------------------------------------------------------
# bf16 detour of scale / min   (ops.py:80-81 cast, ops.py:94-96 cast back)
# --------------------------------------------------------------------------
def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 (round to nearest even) -> fp32, as uint16 bit patterns
    widened back.  Returns (bits_u16, value_f32)."""
    x = np.ascontiguousarray(x, dtype=F32)
    bits = x.view(U32).astype(U64)
    lsb = (bits >> U64(16)) & U64(1)
    rounded = ((bits + U64(0x7FFF) + lsb) >> U64(16)).astype(np.uint16)
    nan = np.isnan(x)
    if nan.any():
        rounded = np.where(nan, np.uint16(0x7FC0) | ((bits >> U64(16)).astype(np.uint16) & np.uint16(0x8000)), rounded)
    value = (rounded.astype(U32) << U32(16)).view(F32)
    return rounded, value


# --------------------------------------------------------------------------
# a1: per-row min / max     (qsheme.py:41-48, ops.py:61-66)
# --------------------------------------------------------------------------
def row_min_max(x: np.ndarray):
    x2 = np.ascontiguousarray(x, dtype=F32).reshape(x.shape[0], -1)
    return x2.min(axis=1), x2.max(axis=1)


# a2: scale = (2 ** bits - 1) / (mx - mn)      (ops.py:39)
def compute_scale(mn: np.ndarray, mx: np.ndarray, bits: int) -> np.ndarray:
    """`python_int / tensor` is Tensor.__rtruediv__, which torch defines as
    `tensor.reciprocal() * python_int`: TWO fp32 roundings (1/range, then * B),
    not one division.  Pinned by test_oracle.py against torch on the CPU."""
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        recip = (F32(1.0) / (mx.astype(F32) - mn.astype(F32))).astype(F32)
        return (recip * F32(2 ** bits - 1)).astype(F32)


def packed_nbytes(N: int, G: int, bits: int) -> int:
    """Length of the int8 stream (quantization_cuda_kernel.cu:107-113): the
    reference allocates (total_bits + 8) / 8 bytes; the last byte is padding
    that no kernel writes.  This build writes it as 0."""
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    return (bits * n_round * G + 8) // 8


# --------------------------------------------------------------------------
# a3: quantise + bit-pack   (quantization_cuda_kernel.cu:63-94)
# --------------------------------------------------------------------------
def quantize_values(x, mn, scale, noise) -> np.ndarray:
    """int32 q[n,d] = rn(fmax((x - mn[n]) * scale[n] + noise - 0.5, 0))
    (quantization_cuda_kernel.cu:89), each operation rounded to fp32, no FMA.
    The double literal 0.5 of the source changes nothing: the sum is exact in
    double and the later float conversion performs the one fp32 rounding."""
    x = np.asarray(x, dtype=F32)
    with np.errstate(invalid="ignore", over="ignore"):
        t = (x - mn.astype(F32)[:, None]).astype(F32)
        t = (t * scale.astype(F32)[:, None]).astype(F32)
        t = (t + np.asarray(noise, dtype=F32)).astype(F32)
        t = (t - F32(0.5)).astype(F32)
        t = np.fmax(t, F32(0.0))          # IEEE fmax: NaN -> 0
        # round half to even, like cvt.rni.s32.f32, which clamps to the int32 range: +inf (a row whose
        # spread is so small that its reciprocal overflows) gives INT_MAX
        big = t >= F32(2147483648.0)
        return np.where(big, np.int32(2147483647), np.rint(np.where(big, F32(0.0), t)).astype(np.int32)).astype(np.int32)


def pack_single_precision(x, mn, scale, bits: int, noise) -> np.ndarray:
    """uint8 stream of length packed_nbytes(N, G, bits).  Byte (n // wpt) * G + d
    holds rows n..n+wpt-1 of column d, row i of the group at bit offset i*bits
    (quantization_cuda_kernel.cu:70-93).  No upper clamp: a value of B+1
    produced by fp32 rounding ORs into the next field / is truncated by the
    uint8 accumulator exactly as `local_packed |= (val << (ni * bits))` does."""
    assert 8 % bits == 0
    x = np.ascontiguousarray(x, dtype=F32)
    N, G = x.shape
    wpt = 8 // bits
    q = quantize_values(x, mn, scale, noise)
    n_round = N + (wpt - N % wpt) % wpt
    qpad = np.zeros((n_round, G), dtype=np.int64)
    qpad[:N] = q
    qpad = qpad.reshape(n_round // wpt, wpt, G)
    acc = np.zeros((n_round // wpt, G), dtype=np.int64)
    for i in range(wpt):
        acc |= (qpad[:, i, :] << (i * bits))
    out = np.zeros(packed_nbytes(N, G, bits), dtype=np.uint8)
    out[: acc.size] = (acc & 0xFF).astype(np.uint8).reshape(-1)
    return out


# --------------------------------------------------------------------------
# a5: unpack + dequantise    (quantization_cuda_kernel.cu:158-185)
# --------------------------------------------------------------------------
def unpack_single_precision(packed, bits: int, scale, mn, N: int, G: int) -> np.ndarray:
    """x_hat[n,d] = float(field) / scale[n] + mn[n]  (true division, then add)."""
    wpt = 8 // bits
    n_round = N + (wpt - N % wpt) % wpt
    p = np.asarray(packed).view(np.uint8)[: (n_round // wpt) * G].reshape(n_round // wpt, 1, G).astype(np.int32)
    shifts = (np.arange(wpt, dtype=np.int32) * bits).reshape(1, wpt, 1)
    q = ((p >> shifts) & (2 ** bits - 1)).reshape(n_round, G)[:N]
    with np.errstate(divide="ignore", invalid="ignore"):
        v = (q.astype(F32) / scale.astype(F32)[:, None]).astype(F32)
        return (v + mn.astype(F32)[:, None]).astype(F32)


# --------------------------------------------------------------------------
# a4 / a6: the Python-level API     (ops.py:69-98)
# --------------------------------------------------------------------------
def quantize_activation(x, bits: int, noise):
    """-> (packed uint8, bits, scale bf16 bits, min bf16 bits); also returns the
    fp32 scale/min the quantiser itself used (ops.py:39 keeps fp32 for K1 and
    only the RETURNED copies are bf16, ops.py:80-81)."""
    x2 = np.ascontiguousarray(x, dtype=F32).reshape(x.shape[0], -1)
    mn, mx = row_min_max(x2)
    scale = compute_scale(mn, mx, bits)
    packed = pack_single_precision(x2, mn, scale, bits, noise)
    scale_bf, _ = bf16_round(scale)
    mn_bf, _ = bf16_round(mn)
    return packed, bits, scale_bf, mn_bf, scale, mn


def dequantize_activation(packed, bits, scale_bf16_bits, min_bf16_bits, shape) -> np.ndarray:
    """bf16 -> fp32 widening of scale/min, then K2 (ops.py:92-98)."""
    N = shape[0]
    G = int(np.prod(shape[1:]))
    scale = (np.asarray(scale_bf16_bits, dtype=np.uint16).astype(U32) << U32(16)).view(F32)
    mn = (np.asarray(min_bf16_bits, dtype=np.uint16).astype(U32) << U32(16)).view(F32)
    return unpack_single_precision(packed, bits, scale, mn, N, G).reshape(shape)


# --------------------------------------------------------------------------
# a7: random projection     (ops.py:107-125; k at ops.py:143)
# --------------------------------------------------------------------------
def kept_acts(kept_frac: float, D: int) -> int:
    return int(kept_frac * D + 0.999)


def rademacher_matrix(D: int, k: int, rng: np.random.Generator) -> np.ndarray:
    """(2*Bernoulli(1/2) - 1) / sqrt(k)   (ops.py:112-114)."""
    bern = rng.integers(0, 2, size=(D, k)).astype(F32)
    return ((F32(2.0) * bern - F32(1.0)) / F32(k ** 0.5)).astype(F32)


def gaussian_matrix(D: int, k: int, rng: np.random.Generator) -> np.ndarray:
    """N(0, 1/k) entries: the distribution the target metric names."""
    return (rng.standard_normal((D, k)) / np.sqrt(k)).astype(F32)


def input2rp(x, R) -> np.ndarray:
    """X[N,D] @ R[D,k], accumulated in float64 then rounded once: the
    tolerance-free centre that fp32 GEMMs are compared against (1e-5 rel)."""
    return (np.asarray(x, dtype=np.float64) @ np.asarray(R, dtype=np.float64)).astype(F32)


def rp2input(xr, R) -> np.ndarray:
    return (np.asarray(xr, dtype=np.float64) @ np.asarray(R, dtype=np.float64).T).astype(F32)


# --------------------------------------------------------------------------
# a13: ReLU with a 1-bit mask   (quantization_cuda_kernel.cu:237-331)
# The reference's mask word/bit order is private to its two kernels; this
# build uses the linear order: bit (i % 32) of int32 word (i // 32) <-> element i.
# --------------------------------------------------------------------------
def mask_nwords(n: int) -> int:
    return (n + 31) // 32       # quantization_cuda_kernel.cu:277


def _pack_bits(bits_bool: np.ndarray) -> np.ndarray:
    n = bits_bool.size
    padded = np.zeros(mask_nwords(n) * 32, dtype=np.uint8)
    padded[:n] = bits_bool.reshape(-1)
    return np.packbits(padded, bitorder="little").view(np.uint32).copy()


def _unpack_bits(mask_words: np.ndarray, n: int) -> np.ndarray:
    return np.unpackbits(np.asarray(mask_words).view(np.uint8), bitorder="little")[:n].astype(bool)


def relu_fwd(x):
    """bit = x > 0; y = bit ? x : 0   (quantization_cuda_kernel.cu:252-258)."""
    x = np.asarray(x, dtype=F32)
    bit = x > 0
    return np.where(bit, x, F32(0.0)).astype(F32), _pack_bits(bit)


def relu_bwd(dy, mask_words):
    dy = np.asarray(dy, dtype=F32)
    bit = _unpack_bits(mask_words, dy.size).reshape(dy.shape)
    return np.where(bit, dy, F32(0.0)).astype(F32)


# --------------------------------------------------------------------------
# a14: dropout with a 1-bit keep mask   (quantization_cuda_kernel.cu:442-594,
# quantization.cc:111-134)
# --------------------------------------------------------------------------
def dropout_fwd(x, p: float, noise):
    """keep = u > p (:465-468); y = x * keep * pinv with
    pinv = float(1.0 / (1.0 - double(float(p)))) (:456, :490)."""
    x = np.asarray(x, dtype=F32)
    pf = F32(p)
    pinv = F32(1.0 / (1.0 - float(pf)))
    keep = np.asarray(noise, dtype=F32) > pf
    with np.errstate(invalid="ignore"):
        y = ((x * keep.astype(F32)).astype(F32) * pinv).astype(F32)
    return y, _pack_bits(keep)


def dropout_bwd(dy, mask_words, p: float):
    """dx = bit ? dy / p1m : 0, p1m = float(1.0 - double(float(p)))
    (quantization.cc:121,127; quantization_cuda_kernel.cu:565-569)."""
    dy = np.asarray(dy, dtype=F32)
    p1m = F32(1.0 - float(F32(p)))
    bit = _unpack_bits(mask_words, dy.size).reshape(dy.shape)
    return np.where(bit, (dy / p1m).astype(F32), F32(0.0)).astype(F32)


# --------------------------------------------------------------------------
# a10 / a11: CSR SpMM, sum and mean; transpose for backward
# (spmm_cuda.cu:27-104, reducer.cuh:43-85, spmm.cc:57-79,115-139)
# --------------------------------------------------------------------------
def spmm_csr(rowptr, col, val, X, reduce: str = "sum") -> np.ndarray:
    """out[r,:] = sum_{e in row r} val[e] * X[col[e],:], accumulated in CSR
    order in fp32 (one multiply and one add per term, spmm_cuda.cu:85-90 with
    Reducer::update reducer.cuh:56-57); mean divides by max(deg,1)
    (reducer.cuh:75-76).  Rows without entries give 0."""
    rowptr = np.asarray(rowptr, dtype=np.int64)
    col = np.asarray(col, dtype=np.int64)
    X = np.ascontiguousarray(X, dtype=F32)
    M = rowptr.size - 1
    K = X.shape[1]
    out = np.zeros((M, K), dtype=F32)
    deg = np.diff(rowptr)
    # vectorised over rows, sequential over the position inside each row
    for j in range(int(deg.max()) if M else 0):
        rows = np.nonzero(deg > j)[0]
        e = rowptr[rows] + j
        term = X[col[e]]
        if val is not None:
            term = (np.asarray(val, dtype=F32)[e][:, None] * term).astype(F32)
        out[rows] = (out[rows] + term).astype(F32)
    if reduce == "mean":
        out = (out / np.maximum(deg, 1).astype(F32)[:, None]).astype(F32)
    elif reduce != "sum":
        raise ValueError(reduce)
    return out


def csr_transpose(rowptr, col, n_cols: int):
    """-> (row, colptr, csr2csc): what torch_sparse caches and the reference
    reads through spmm.py:21-31.  csr2csc is the stable sort of entries by
    column; colptr its row-pointer array."""
    rowptr = np.asarray(rowptr, dtype=np.int64)
    col = np.asarray(col, dtype=np.int64)
    M = rowptr.size - 1
    row = np.repeat(np.arange(M, dtype=np.int64), np.diff(rowptr))
    csr2csc = np.argsort(col, kind="stable").astype(np.int64)
    colptr = np.zeros(n_cols + 1, dtype=np.int64)
    np.cumsum(np.bincount(col, minlength=n_cols), out=colptr[1:])
    return row, colptr, csr2csc


def spmm_sum_bw(row, colptr, csr2csc, val, dY) -> np.ndarray:
    """grad_mat = A^T dY via the CSC arrays (spmm.cc:70-77)."""
    v = None if val is None else np.asarray(val, dtype=F32)[csr2csc]
    return spmm_csr(colptr, row[csr2csc], v, dY, "sum")


def spmm_mean_bw(row, rowcount, colptr, csr2csc, val, dY) -> np.ndarray:
    """Per-entry weight [val] / max(rowcount[row],1) in CSC order, then a sum
    SpMM on the CSC arrays (spmm.cc:128-137)."""
    r = row[csr2csc]
    cnt = np.maximum(np.asarray(rowcount)[r].astype(F32), F32(1.0))
    if val is not None:
        w = (np.asarray(val, dtype=F32)[csr2csc] / cnt).astype(F32)
    else:
        w = (F32(1.0) / cnt).astype(F32)          # rowcount.pow_(-1)
    return spmm_csr(colptr, r, w, dY, "sum")
