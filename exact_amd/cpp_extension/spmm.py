"""Stand-in for the reference's `exact.cpp_extension.spmm` module
(spmm.cc:243-252): spmm_sum_fw/bw and spmm_mean_fw/bw with the reference's
argument lists.  max/min reductions and gradients with respect to the edge
values are outside this library's scope and raise.
"""
from __future__ import annotations

from collections import OrderedDict

import torch

from .. import _lib
from . import _checks
from ._checks import ptr

REDUCE = {"sum": 0, "mean": 1}


def _check_index(t, name):
    if not _checks.on_device(t):
        raise RuntimeError(f"{name} must be CUDA tensor")       # CHECK_CUDA, spmm_cuda.cu:111-116
    if t.dim() != 1:
        raise RuntimeError("Input mismatch")                     # CHECK_INPUT, spmm_cuda.cu:118-119
    if t.dtype not in (torch.int32, torch.int64):
        raise RuntimeError(f"{name} must be int32 or int64")


def spmm_csr(rowptr, col, value, mat, reduce):
    """spmm_cuda(rowptr, col, optional_value, mat, reduce) for reduce in
    {sum, mean} (spmm_cuda.cu:106-170)."""
    if reduce not in REDUCE:
        raise NotImplementedError(f"reduce='{reduce}' is not implemented by this library (sum, mean only)")
    _check_index(rowptr, "rowptr")
    _check_index(col, "col")
    if not _checks.on_device(mat):
        raise RuntimeError("mat must be CUDA tensor")
    if mat.dim() != 2:
        raise RuntimeError("Input mismatch: mat must be 2-D [N, K]")
    if mat.dtype != torch.float32:
        raise RuntimeError("The type of mat is not correct!")
    if value is not None:
        if not _checks.on_device(value):
            raise RuntimeError("value must be CUDA tensor")
        if value.dim() != 1 or value.size(0) != col.size(0):
            raise RuntimeError("Input mismatch")                 # spmm_cuda.cu:121-122
        if value.dtype != torch.float32:
            value = value.float()
        value = value.contiguous()
    if rowptr.dtype != col.dtype:
        wide = torch.int64 if torch.int64 in (rowptr.dtype, col.dtype) else torch.int32
        rowptr, col = rowptr.to(wide), col.to(wide)
    rowptr, col, mat = rowptr.contiguous(), col.contiguous(), mat.contiguous()
    M = rowptr.numel() - 1
    n_cols, K = mat.shape
    out = torch.empty((M, K), dtype=mat.dtype, device=mat.device)
    rc = _lib.lib().exact_spmm_csr_f32(ptr(rowptr), ptr(col), ptr(value), rowptr.element_size(), ptr(mat),
                                       M, n_cols, K, col.numel(), REDUCE[reduce], ptr(out), _checks.stream_ptr(mat))
    _lib.check(rc, f"spmm_{reduce}")
    return out


def _missing(name):
    raise RuntimeError(f"Argument `{name}` is missing")          # AT_ASSERTM, spmm.cc:39-46


def spmm_sum_fw(row, rowptr, col, value, colptr, csr2csc, mat):
    """spmm.cc:31-55."""
    if value is not None and value.requires_grad and row is None:
        _missing("row")
    if mat.requires_grad:
        if row is None:
            _missing("row")
        if colptr is None:
            _missing("colptr")
        if csr2csc is None:
            _missing("csr2csc")
    return spmm_csr(rowptr, col, value, mat, "sum")


def spmm_mean_fw(row, rowptr, col, value, rowcount, colptr, csr2csc, mat):
    """spmm.cc:84-113."""
    if value is not None and value.requires_grad and row is None:
        _missing("row")
    if mat.requires_grad:
        if row is None:
            _missing("row")
        if rowcount is None:
            _missing("rowcount")
        if colptr is None:
            _missing("colptr")
        if csr2csc is None:
            _missing("csr2csc")
    return spmm_csr(rowptr, col, value, mat, "mean")


# The reference re-gathers row[csr2csc], value[csr2csc] (and the mean weights)
# with index_select on EVERY backward (spmm.cc:73-75, 129-133).  They depend
# only on the graph, so they are built once per (graph, values) and kept.
_CSC_CACHE: "OrderedDict[tuple, tuple]" = OrderedDict()
_CSC_CACHE_MAX = 16


def _csc_operands(kind, row, value, rowcount, csr2csc, has_value, dtype):
    key = (kind, row.data_ptr(), csr2csc.data_ptr(), row.numel(),
           value.data_ptr() if has_value else 0, value._version if has_value else 0,
           rowcount.data_ptr() if rowcount is not None else 0)
    hit = _CSC_CACHE.get(key)
    if hit is not None:
        _CSC_CACHE.move_to_end(key)
        return hit[0], hit[1]
    row_csc = row.index_select(0, csr2csc)
    if kind == "sum":
        w = value.detach().index_select(0, csr2csc) if has_value else None
    else:
        cnt = rowcount.to(dtype).index_select(0, row_csc).clamp_(min=1)
        w = value.detach().index_select(0, csr2csc).div(cnt) if has_value else cnt.pow_(-1)
    # the inputs are kept alive with the entry so their addresses cannot be reused
    _CSC_CACHE[key] = (row_csc, w, (row, value, rowcount, csr2csc))
    while len(_CSC_CACHE) > _CSC_CACHE_MAX:
        _CSC_CACHE.popitem(last=False)
    return row_csc, w


def clear_csc_cache():
    _CSC_CACHE.clear()


def _no_value_grad(has_value, value_requires_grad):
    if has_value and value_requires_grad:
        raise NotImplementedError(
            "gradients with respect to the edge values (spmm_value_bw) are not implemented by this library")


def spmm_sum_bw(row, rowptr, col, value, colptr, csr2csc, mat, grad_out,
                has_value, value_requires_grad, mat_requires_grad):
    """spmm.cc:57-79 -> (grad_value, grad_mat)."""
    _no_value_grad(has_value, value_requires_grad)
    grad_mat = None
    if mat_requires_grad:
        row_csc, val_csc = _csc_operands("sum", row, value, None, csr2csc, has_value, grad_out.dtype)
        grad_mat = spmm_csr(colptr, row_csc, val_csc, grad_out, "sum")
    return None, grad_mat


def spmm_mean_bw(row, rowptr, col, value, rowcount, colptr, csr2csc, mat, grad_out,
                 has_value, value_requires_grad, mat_requires_grad):
    """spmm.cc:115-139 -> (grad_value, grad_mat)."""
    _no_value_grad(has_value, value_requires_grad)
    grad_mat = None
    if mat_requires_grad:
        row_csc, w_csc = _csc_operands("mean", row, value, rowcount, csr2csc, has_value, grad_out.dtype)
        grad_mat = spmm_csr(colptr, row_csc, w_csc, grad_out, "sum")
    return None, grad_mat


def _unsupported(*_a, **_k):
    raise NotImplementedError("max/min aggregation is not implemented by this library (sum, mean only)")


spmm_max_fw = spmm_max_bw = spmm_min_fw = spmm_min_bw = _unsupported
