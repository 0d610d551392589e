"""A minimal CSR container with the attribute surface of
torch_sparse.SparseTensor that the path touches (reference spmm.py:19-44):
.csr(), .storage._row/_rowcount/_colptr/_csr2csc and the lazy
row()/rowcount()/colptr()/csr2csc(), fill_cache_(), sparse_sizes().
torch_sparse itself is not a dependency; a real SparseTensor can be passed to
the ops instead of this class (duck typing).

Building and transposing the graph is a one-off format step done with torch
ops on whatever device the vectors live on.
"""
from __future__ import annotations

import torch


class SparseStorage:
    def __init__(self, rowptr, col, value, sparse_sizes):
        self._rowptr = rowptr
        self._col = col
        self._value = value
        self._sparse_sizes = tuple(sparse_sizes)
        self._row = None
        self._rowcount = None
        self._colptr = None
        self._csr2csc = None

    # -- lazily cached vectors (same names as torch_sparse's storage) --------
    def rowptr(self):
        return self._rowptr

    def col(self):
        return self._col

    def value(self):
        return self._value

    def rowcount(self):
        if self._rowcount is None:
            self._rowcount = self._rowptr[1:] - self._rowptr[:-1]
        return self._rowcount

    def row(self):
        if self._row is None:
            M = self._sparse_sizes[0]
            self._row = torch.repeat_interleave(
                torch.arange(M, device=self._col.device, dtype=self._col.dtype), self.rowcount().long())
        return self._row

    def csr2csc(self):
        if self._csr2csc is None:
            # entries ordered by (col, row): a stable sort of col keeps CSR's row order
            self._csr2csc = torch.sort(self._col.long(), stable=True).indices.to(self._col.dtype)
        return self._csr2csc

    def colptr(self):
        if self._colptr is None:
            n_cols = self._sparse_sizes[1]
            counts = torch.bincount(self._col.long(), minlength=n_cols)
            colptr = torch.zeros(n_cols + 1, dtype=self._rowptr.dtype, device=self._col.device)
            torch.cumsum(counts, 0, out=colptr[1:])
            self._colptr = colptr
        return self._colptr


class SparseTensor:
    def __init__(self, rowptr, col, value=None, sparse_sizes=None):
        M = rowptr.numel() - 1
        if sparse_sizes is None:
            sparse_sizes = (M, M)
        self.storage = SparseStorage(rowptr.contiguous(), col.contiguous(),
                                     None if value is None else value.contiguous(), sparse_sizes)

    # -- construction ---------------------------------------------------------
    @classmethod
    def from_edge_index(cls, row, col, value=None, sparse_sizes=None):
        """COO (row, col[, value]) -> CSR, entries sorted by (row, col)."""
        row, col = row.long(), col.long()
        if sparse_sizes is None:
            n = int(max(row.max(), col.max())) + 1 if row.numel() else 0
            sparse_sizes = (n, n)
        M, Ncol = sparse_sizes
        perm = torch.argsort(row * Ncol + col)
        row, col = row[perm], col[perm]
        if value is not None:
            value = value[perm]
        rowptr = torch.zeros(M + 1, dtype=torch.long, device=row.device)
        torch.cumsum(torch.bincount(row, minlength=M), 0, out=rowptr[1:])
        out = cls(rowptr, col, value, sparse_sizes)
        out.storage._row = row
        return out

    @classmethod
    def from_scipy(cls, mat, device="cpu"):
        mat = mat.tocsr()
        mat.sort_indices()
        value = torch.from_numpy(mat.data.astype("float32")).to(device)
        return cls(torch.from_numpy(mat.indptr.astype("int64")).to(device),
                   torch.from_numpy(mat.indices.astype("int64")).to(device), value, mat.shape)

    # -- accessors --------------------------------------------------------------
    def csr(self):
        st = self.storage
        return st._rowptr, st._col, st._value

    def coo(self):
        st = self.storage
        return st.row(), st._col, st._value

    def sparse_sizes(self):
        return self.storage._sparse_sizes

    def sparse_size(self, dim):
        return self.storage._sparse_sizes[dim]

    def size(self, dim):
        return self.storage._sparse_sizes[dim]

    def nnz(self):
        return self.storage._col.numel()

    def has_value(self):
        return self.storage._value is not None

    def device(self):
        return self.storage._col.device

    def set_value(self, value, layout=None):
        st = self.storage
        out = SparseTensor(st._rowptr, st._col, value, st._sparse_sizes)
        for name in ("_row", "_rowcount", "_colptr", "_csr2csc"):
            setattr(out.storage, name, getattr(st, name))
        return out

    def fill_cache_(self):
        st = self.storage
        st.row(), st.rowcount(), st.colptr(), st.csr2csc()
        return self

    def to(self, device):
        st = self.storage
        mv = lambda t: None if t is None else t.to(device)  # noqa: E731
        out = SparseTensor(mv(st._rowptr), mv(st._col), mv(st._value), st._sparse_sizes)
        for name in ("_row", "_rowcount", "_colptr", "_csr2csc"):
            setattr(out.storage, name, mv(getattr(st, name)))
        return out

    def cuda(self):
        return self.to("cuda")

    def to_int32_(self):
        """Narrow every index vector to int32 (the reference's cast_adj)."""
        st = self.storage
        for name in ("_rowptr", "_col", "_row", "_rowcount", "_colptr", "_csr2csc"):
            t = getattr(st, name)
            if t is not None:
                setattr(st, name, t.to(torch.int32))
        return self

    def to_dense(self):
        row, col, value = self.coo()
        M, N = self.sparse_sizes()
        dense = torch.zeros(M, N, dtype=torch.float32, device=col.device)
        v = value if value is not None else torch.ones(col.numel(), device=col.device)
        dense.index_put_((row.long(), col.long()), v, accumulate=True)
        return dense

    # -- graph normalisations used by the models ------------------------------
    def fill_diag(self, fill_value=1.0):
        """Add (or overwrite) the diagonal: A + I for graphs without self loops."""
        row, col, value = self.coo()
        M, N = self.sparse_sizes()
        keep = row != col
        diag = torch.arange(min(M, N), device=col.device, dtype=col.dtype)
        v = value if value is not None else torch.ones(col.numel(), device=col.device)
        new_row = torch.cat([row[keep], diag])
        new_col = torch.cat([col[keep], diag])
        new_val = torch.cat([v[keep], torch.full((diag.numel(),), fill_value, dtype=v.dtype, device=v.device)])
        return SparseTensor.from_edge_index(new_row, new_col, new_val, (M, N))


def gcn_norm(adj_t: SparseTensor, add_self_loops: bool = True) -> SparseTensor:
    """D^-1/2 (A [+ I]) D^-1/2 with D the row sums: the symmetric
    normalisation the reference applies once before training
    (mem_speed_bench/arxiv/train_full_batch.py:186-196)."""
    if not adj_t.has_value():
        adj_t = adj_t.set_value(torch.ones(adj_t.nnz(), device=adj_t.device()))
    if add_self_loops:
        adj_t = adj_t.fill_diag(1.0)
    row, col, value = adj_t.coo()
    M = adj_t.sparse_size(0)
    deg = torch.zeros(M, dtype=value.dtype, device=value.device).index_add_(0, row.long(), value)
    dinv = deg.pow(-0.5)
    dinv[torch.isinf(dinv)] = 0.0
    value = dinv[row.long()] * value * dinv[col.long()]
    return adj_t.set_value(value)
