"""Sparse-dense product dispatch, as exact/exact/spmm.py:7-90 of the
reference: QMatmul module and qmatmul function over a SparseTensor-like
operand (anything exposing .csr() and .storage with the cached vectors)."""
import torch

from .conf import config
from .ops import qspmm_max, qspmm_mean, qspmm_min, qspmm_sum
from .qsheme import QScheme


def _dispatch(src, other, reduce, quantized, randmat, scheme):
    rowptr, col, value = src.csr()
    has_value = value is not None
    st = src.storage
    row, csr2csc, colptr = st._row, st._csr2csc, st._colptr
    if has_value and value.requires_grad:
        row = st.row()
    if reduce == "sum":
        if other.requires_grad:
            row, csr2csc, colptr = st.row(), st.csr2csc(), st.colptr()
        return qspmm_sum.apply(row, rowptr, col, value, colptr, csr2csc, has_value, other,
                               quantized, randmat, scheme)
    if reduce == "mean":
        rowcount = st._rowcount
        if other.requires_grad:
            row, rowcount, csr2csc, colptr = st.row(), st.rowcount(), st.csr2csc(), st.colptr()
        return qspmm_mean.apply(row, rowptr, col, value, rowcount, colptr, csr2csc, has_value, other,
                                quantized, randmat, scheme)
    if reduce == "max":
        return qspmm_max.apply(rowptr, col, value, has_value, other, quantized, randmat, scheme)
    if reduce == "min":
        return qspmm_min.apply(rowptr, col, value, has_value, other, quantized, randmat, scheme)
    raise ValueError(reduce)


class QMatmul(torch.nn.Module):
    def __init__(self, reduce):
        super().__init__()
        if reduce in ["sum", "add"]:
            reduce = "sum"
        self.reduce = reduce
        self.scheme = QScheme("matmul") if config.single_precision else None

    def forward(self, src, other, quantized=None, randmat=None):
        return _dispatch(src, other, self.reduce, quantized, randmat, self.scheme)


def qmatmul(src, other, reduce="sum", quantized=None, randmat=None, scheme=None):
    if reduce in ["sum", "add"]:
        reduce = "sum"
    return _dispatch(src, other, reduce, quantized, randmat, scheme)
