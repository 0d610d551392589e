"""CPU restatement of the remaining operators of the reference's extension
modules: LeakyReLU mask, ELU backward, max / min aggregation with arg output
and its backward, and the edge-value gradient.  TEST INFRASTRUCTURE ONLY (see
the header of exact_oracle.py).  Pinned in tests/test_oracle_extra.py against
torch (F.leaky_relu / F.elu autograd), dense brute force and scipy."""
import numpy as np

import exact_oracle as o

F32 = np.float32


def leaky_relu_fwd(x, slope):
    """bit = x > 0; y = bit ? x : x * slope  (quantization_cuda_kernel.cu:352-358)."""
    x = np.asarray(x, dtype=F32)
    bit = x > 0
    with np.errstate(invalid="ignore"):
        return np.where(bit, x, (x * F32(slope)).astype(F32)).astype(F32), o._pack_bits(bit)


def leaky_relu_bwd(dy, mask_words, slope):
    """dx = bit ? dy : dy * slope  (quantization_cuda_kernel.cu:405-411)."""
    dy = np.asarray(dy, dtype=F32)
    bit = o._unpack_bits(mask_words, dy.size).reshape(dy.shape)
    return np.where(bit, dy, (dy * F32(slope)).astype(F32)).astype(F32)


def spmm_minmax(rowptr, col, val, X, is_max):
    """-> (out [M, K], arg [M, K]): extreme of val[e] * X[col[e], k] over the
    entries of each row, the FIRST extreme entry in CSR order as arg (strict
    comparison, reducer.cuh:62-66); empty rows give 0 and arg = nnz
    (reducer.cuh:77-84, spmm_cuda.cu:151-153)."""
    rowptr, col = np.asarray(rowptr, np.int64), np.asarray(col, np.int64)
    X = np.ascontiguousarray(X, dtype=F32)
    M, K, nnz = rowptr.size - 1, X.shape[1], col.size
    out = np.zeros((M, K), F32)
    arg = np.full((M, K), nnz, np.int64)
    for r in range(M):
        best = np.full(K, np.finfo(F32).min if is_max else np.finfo(F32).max, F32)
        barg = np.full(K, nnz, np.int64)
        for e in range(rowptr[r], rowptr[r + 1]):
            t = X[col[e]] if val is None else (F32(val[e]) * X[col[e]]).astype(F32)
            better = (t > best) if is_max else (t < best)
            best = np.where(better, t, best)
            barg = np.where(better, e, barg)
        if rowptr[r + 1] > rowptr[r]:
            out[r], arg[r] = best, barg
    return out, arg


def spmm_minmax_bw(col, val, X, arg, dY, nnz):
    """(grad_value or None, grad_mat): the scatter of spmm_max_bw / spmm_min_bw
    (spmm.cc:159-193)."""
    col = np.asarray(col, np.int64)
    invalid = arg == nnz
    a = np.where(invalid, 0, arg)
    src = col[a]                                         # [M, K] source row of X per output element
    contrib = dY if val is None else (np.asarray(val, F32)[a] * dY).astype(F32)
    contrib = np.where(invalid, F32(0), contrib).astype(F32)
    grad_mat = np.zeros_like(X, dtype=np.float64)
    K = X.shape[1]
    np.add.at(grad_mat, (src.reshape(-1), np.tile(np.arange(K), src.shape[0])), contrib.reshape(-1))
    grad_val = None
    if val is not None:
        picked = np.take_along_axis(X[src.reshape(-1)].reshape(src.shape + (K,)),
                                    np.arange(K).reshape(1, K, 1).repeat(src.shape[0], 0), axis=2)[..., 0]
        gv = np.where(invalid, F32(0), (picked * dY).astype(F32))
        grad_val = np.zeros(nnz, np.float64)
        np.add.at(grad_val, a.reshape(-1), gv.reshape(-1))
        grad_val = grad_val.astype(F32)
    return grad_val, grad_mat.astype(F32)


def sddmm(row, rowptr, col, mat, grad, reduce):
    """out[e] = sum_k mat[col[e], k] * grad[row[e], k], / max(deg(row[e]), 1)
    for mean  (spmm_cuda.cu:172-209).  float64 centre for a 1e-5 comparison."""
    row, col, rowptr = np.asarray(row, np.int64), np.asarray(col, np.int64), np.asarray(rowptr, np.int64)
    out = np.einsum("ek,ek->e", np.asarray(mat, np.float64)[col], np.asarray(grad, np.float64)[row])
    if reduce == "mean":
        out = out / np.maximum(np.diff(rowptr), 1)[row]
    return out.astype(F32)
