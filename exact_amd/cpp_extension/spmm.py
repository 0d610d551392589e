"""Stand-in for the reference's `exact.cpp_extension.spmm` module
(spmm.cc:243-252): spmm_{sum,mean,max,min}_{fw,bw} with the reference's
argument lists, plus spmm_value_bw (the edge-value gradient).
"""
from __future__ import annotations


import torch
from torch.utils.weak import WeakIdKeyDictionary

from .. import _lib
from ..conf import config
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
        raise NotImplementedError(f"reduce='{reduce}': use spmm_max_fw / spmm_min_fw for max and min")
    if isinstance(mat, torch.Tensor) and mat.dtype == torch.float16:
        # fp16 activations (autocast): gather and accumulate in fp32, round the result once
        return spmm_csr(rowptr, col, value, mat.float(), reduce).to(torch.float16)
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
    rowptr, col = rowptr.contiguous(), col.contiguous()
    M = rowptr.numel() - 1
    n_cols, K = mat.shape
    out = torch.empty((M, K), dtype=mat.dtype, device=mat.device)
    reproducible = config.deterministic_spmm or torch.are_deterministic_algorithms_enabled()
    if reproducible:
        mat = mat.contiguous()
        rc = _lib.lib().exact_spmm_csr_rowwise_f32(ptr(rowptr), ptr(col), ptr(value), rowptr.element_size(), ptr(mat),
                                                   M, n_cols, K, col.numel(), REDUCE[reduce], ptr(out),
                                                   _checks.stream_ptr(mat))
    else:
        mat = _aligned_rows(mat, col.numel())
        rc = _lib.lib().exact_spmm_csr_strided_f32(ptr(rowptr), ptr(col), ptr(value), rowptr.element_size(), ptr(mat),
                                                   mat.stride(0), M, n_cols, K, col.numel(), REDUCE[reduce], ptr(out), K,
                                                   _checks.stream_ptr(mat))
    _lib.check(rc, f"spmm_{reduce}")
    return out


def _aligned_rows(mat, nnz):
    """The dense operand as the kernel wants it: unit column stride, any row
    stride.  Wide rows whose length is not a multiple of 128 bytes are copied
    into rows padded to one when the graph is dense enough to pay for the copy:
    a wavefront gathers 512-byte pieces of a row, and an unaligned piece
    straddles five 128-byte lines instead of four (602 columns, average degree
    100: 8.9 ms -> 7.2 ms per product for a 0.2 ms copy)."""
    if mat.stride(1) != 1 or mat.stride(0) < mat.shape[1]:
        mat = mat.contiguous()
    n_cols, K = mat.shape
    if K > 128 and K % 32 != 0 and mat.stride(0) == K and n_cols > 0 and nnz >= 16 * n_cols:
        padded = torch.empty((n_cols, (K + 31) // 32 * 32), dtype=mat.dtype, device=mat.device)
        padded[:, :K].copy_(mat)
        return padded[:, :K]
    return mat


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
# only on the graph, so they are built once and kept -- attached to the graph's
# own `csr2csc` tensor (the object a SparseTensor's storage caches), weakly: the
# entry dies with the graph, and a graph rebuilt every step (gcn_norm without
# caching, learned or attention edge values) leaves nothing behind.  Per graph
# there is ONE slot per reduction for the value-dependent part, replaced when
# the values change; values that require grad change every step and are never
# kept.  A slot holds the value tensor it was built from: an address alone does
# not identify a tensor (the allocator hands a freed block to the next tensor
# of the same size), but while the slot keeps the tensor alive its block cannot
# be handed out again, so "same address, same length, same version" then does
# mean "same values" (another Python wrapper of the same storage shares its
# version counter).
_CSC_CACHE = WeakIdKeyDictionary()          # csr2csc tensor -> {"row_csc": .., "sum": (value, version, w), "mean": ..}


def _slot_hit(entry, value, has_value):
    held, version, _ = entry
    if not has_value:
        return held is None
    if held is not value and (held.data_ptr() != value.data_ptr() or held.numel() != value.numel()
                              or held.stride() != value.stride()):
        return False
    return version == value._version and held._version == value._version


def _csc_operands(kind, row, value, rowcount, csr2csc, has_value, dtype):
    # fp16 values are per-call copies made by autocast, values that require grad are new every step
    cacheable = not (has_value and (value.dtype != torch.float32 or value.requires_grad))
    slot = _CSC_CACHE.get(csr2csc) if cacheable else None
    if slot is not None and slot["row"] != (row.data_ptr(), row.numel()):
        slot = None                                         # the same permutation handed in with other rows
    if slot is not None and kind in slot and _slot_hit(slot[kind], value, has_value):
        return slot["row_csc"], slot[kind][2]
    row_csc = slot["row_csc"] if slot is not None else row.index_select(0, csr2csc)
    if kind == "sum":
        w = value.detach().index_select(0, csr2csc) if has_value else None
    else:
        cnt = rowcount.to(torch.float32).index_select(0, row_csc).clamp_(min=1)   # fp32 whatever `dtype` is
        w = value.detach().index_select(0, csr2csc).div(cnt) if has_value else cnt.pow_(-1)
    if cacheable:
        if slot is None:
            slot = _CSC_CACHE[csr2csc] = {"row": (row.data_ptr(), row.numel()), "row_csc": row_csc, "keep": row}
        slot[kind] = (value, value._version, w) if has_value else (None, 0, w)
    return row_csc, w


def clear_csc_cache():
    _CSC_CACHE.clear()


def _same_index_dtype(*ts):
    wide = torch.int64 if any(t.dtype == torch.int64 for t in ts) else torch.int32
    return [t.to(wide).contiguous() for t in ts]


def spmm_value_bw(row, rowptr, col, mat, grad, reduce):
    """spmm_value_bw_cuda (spmm_cuda.cu:211-252): gradient with respect to the
    edge values, out[e] = mat[col[e]] . grad[row[e]] (/ row length for mean)."""
    if reduce not in REDUCE:
        raise NotImplementedError(f"reduce='{reduce}'")
    if torch.float16 in (mat.dtype, grad.dtype):
        return spmm_value_bw(row, rowptr, col, mat.float(), grad.float(), reduce).to(torch.float16)
    for t, name in ((row, "row"), (rowptr, "rowptr"), (col, "col")):
        _check_index(t, name)
    for t, name in ((mat, "mat"), (grad, "grad")):
        if not _checks.on_device(t):
            raise RuntimeError(f"{name} must be CUDA tensor")
        if t.dim() != 2 or t.dtype != torch.float32:
            raise RuntimeError(f"The type of {name} is not correct!")
    row, rowptr, col = _same_index_dtype(row, rowptr, col)
    mat, grad = mat.contiguous(), grad.contiguous()
    if mat.shape[1] != grad.shape[1]:
        raise RuntimeError("Input mismatch")
    out = torch.zeros(row.numel(), dtype=grad.dtype, device=grad.device)
    rc = _lib.lib().exact_sddmm_f32(ptr(row), ptr(rowptr), ptr(col), row.element_size(), ptr(mat), ptr(grad),
                                    row.numel(), mat.shape[1], REDUCE[reduce], ptr(out), _checks.stream_ptr(grad))
    _lib.check(rc, "spmm_value_bw")
    return out


def spmm_sum_bw(row, rowptr, col, value, colptr, csr2csc, mat, grad_out,
                has_value, value_requires_grad, mat_requires_grad):
    """spmm.cc:57-79 -> (grad_value, grad_mat)."""
    grad_value = None
    if has_value and value_requires_grad:
        grad_value = spmm_value_bw(row, rowptr, col, mat, grad_out, "sum")
    grad_mat = None
    if mat_requires_grad:
        row_csc, val_csc = _csc_operands("sum", row, value, None, csr2csc, has_value, grad_out.dtype)
        grad_mat = spmm_csr(colptr, row_csc, val_csc, grad_out, "sum")
    return grad_value, grad_mat


def spmm_mean_bw(row, rowptr, col, value, rowcount, colptr, csr2csc, mat, grad_out,
                 has_value, value_requires_grad, mat_requires_grad):
    """spmm.cc:115-139 -> (grad_value, grad_mat)."""
    grad_value = None
    if has_value and value_requires_grad:
        grad_value = spmm_value_bw(row, rowptr, col, mat, grad_out, "mean")
    grad_mat = None
    if mat_requires_grad:
        row_csc, w_csc = _csc_operands("mean", row, value, rowcount, csr2csc, has_value, grad_out.dtype)
        grad_mat = spmm_csr(colptr, row_csc, w_csc, grad_out, "sum")
    return grad_value, grad_mat


# ---- max / min aggregation ----------------------------------------------------
def _spmm_extreme_fw(rowptr, col, value, mat, is_max):
    """spmm_max_fw / spmm_min_fw (spmm.cc:145-157, 199-212) -> (out, arg_out)."""
    if isinstance(mat, torch.Tensor) and mat.dtype == torch.float16:
        out, arg = _spmm_extreme_fw(rowptr, col, value, mat.float(), is_max)
        return out.to(torch.float16), arg
    _check_index(rowptr, "rowptr")
    _check_index(col, "col")
    if not _checks.on_device(mat):
        raise RuntimeError("mat must be CUDA tensor")
    if mat.dim() != 2 or mat.dtype != torch.float32:
        raise RuntimeError("The type of mat is not correct!")
    if value is not None:
        if value.dim() != 1 or value.size(0) != col.size(0):
            raise RuntimeError("Input mismatch")
        value = value.detach().float().contiguous()
    rowptr, col = _same_index_dtype(rowptr, col)
    mat = mat.contiguous()
    M, K = rowptr.numel() - 1, mat.shape[1]
    out = torch.empty((M, K), dtype=mat.dtype, device=mat.device)
    arg_out = torch.empty((M, K), dtype=rowptr.dtype, device=mat.device)
    rc = _lib.lib().exact_spmm_csr_minmax_f32(ptr(rowptr), ptr(col), ptr(value), rowptr.element_size(), ptr(mat), M,
                                              mat.shape[0], K, col.numel(), 1 if is_max else 0, ptr(out), ptr(arg_out),
                                              _checks.stream_ptr(mat))
    _lib.check(rc, "spmm_max_fw" if is_max else "spmm_min_fw")
    return out, arg_out


def spmm_max_fw(rowptr, col, value, mat):
    return _spmm_extreme_fw(rowptr, col, value, mat, True)


def spmm_min_fw(rowptr, col, value, mat):
    return _spmm_extreme_fw(rowptr, col, value, mat, False)


def spmm_max_bw(col, value, mat, arg_out, grad_out, has_value, value_requires_grad, mat_requires_grad):
    """spmm.cc:159-193: route each output gradient back to the entry that won
    (torch gathers / scatters, as in the reference)."""
    arg_out = arg_out.long()
    invalid = arg_out == col.size(0)
    arg = arg_out.masked_fill(invalid, 0)
    src = col.long().index_select(0, arg.flatten()).view_as(arg)
    grad_value = None
    if has_value and value_requires_grad:
        picked = mat.gather(-2, src) * grad_out
        picked.masked_fill_(invalid, 0)
        grad_value = torch.zeros_like(value).scatter_add_(0, arg.flatten(), picked.flatten())
    grad_mat = None
    if mat_requires_grad:
        contrib = value.detach().index_select(0, arg.flatten()).view_as(arg) * grad_out if has_value else grad_out.clone()
        contrib.masked_fill_(invalid, 0)
        grad_mat = torch.zeros_like(mat).scatter_add_(-2, src, contrib)
    return grad_value, grad_mat


spmm_min_bw = spmm_max_bw      # identical routing (spmm.cc:214-241)
