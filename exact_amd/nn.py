"""Plain (uncompressed) GCNConv / SAGEConv with the constructor arguments and
parameter names of torch_geometric 1.7.2, the classes the reference's
QGCNConv / QSAGEConv subclass (layers.py:123, 215).  torch_geometric is not a
dependency: only the SparseTensor code path (message_and_aggregate) that the
full-batch trainers use is provided.  These are the layers QModule swaps."""
import math

import torch
import torch.nn.functional as F
from torch.nn import Linear, Parameter

from .cpp_extension import spmm as _spmm
from .sparse import gcn_norm


def glorot(tensor):
    if tensor is not None:
        stdv = math.sqrt(6.0 / (tensor.size(-2) + tensor.size(-1)))
        tensor.data.uniform_(-stdv, stdv)


class _SpMM(torch.autograd.Function):
    """Uncompressed A @ X with the transpose product as backward."""

    @staticmethod
    def forward(ctx, adj_t, x, reduce):
        rowptr, col, value = adj_t.csr()
        ctx.adj_t, ctx.reduce = adj_t, reduce
        return _spmm.spmm_csr(rowptr, col, value, x, reduce)

    @staticmethod
    def backward(ctx, grad_out):
        adj_t, reduce = ctx.adj_t, ctx.reduce
        rowptr, col, value = adj_t.csr()
        st = adj_t.storage
        has_value = value is not None
        grad_out = grad_out.contiguous()
        if reduce == "sum":
            _, g = _spmm.spmm_sum_bw(st.row(), rowptr, col, value, st.colptr(), st.csr2csc(), None, grad_out,
                                     has_value, False, True)
        else:
            _, g = _spmm.spmm_mean_bw(st.row(), rowptr, col, value, st.rowcount(), st.colptr(), st.csr2csc(),
                                      None, grad_out, has_value, False, True)
        return None, g, None


def matmul(adj_t, x, reduce="sum"):
    if reduce in ("add", "sum"):
        reduce = "sum"
    return _SpMM.apply(adj_t, x, reduce)


class GCNConv(torch.nn.Module):
    def __init__(self, in_channels, out_channels, improved=False, cached=False, add_self_loops=True,
                 normalize=True, bias=True, aggr="add"):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.improved, self.cached = improved, cached
        self.add_self_loops, self.normalize = add_self_loops, normalize
        self.aggr = aggr
        self._cached_adj_t = None
        self.weight = Parameter(torch.Tensor(in_channels, out_channels))
        if bias:
            self.bias = Parameter(torch.Tensor(out_channels))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight)
        if self.bias is not None:
            self.bias.data.zero_()
        self._cached_adj_t = None

    def _normalized(self, adj_t):
        if not self.normalize:
            return adj_t
        if self._cached_adj_t is not None:
            return self._cached_adj_t
        if self.improved:
            raise NotImplementedError("improved=True (A + 2I) is not provided")
        out = gcn_norm(adj_t, self.add_self_loops)
        if self.cached:
            self._cached_adj_t = out
        return out

    def message_and_aggregate(self, adj_t, x):
        return matmul(adj_t, x, reduce=self.aggr)

    def forward(self, x, edge_index, edge_weight=None):
        adj_t = self._normalized(edge_index)
        x = x @ self.weight
        out = self.message_and_aggregate(adj_t, x)
        if self.bias is not None:
            out = out + self.bias
        return out


class SAGEConv(torch.nn.Module):
    def __init__(self, in_channels, out_channels, normalize=False, root_weight=True, bias=True):
        super().__init__()
        self.in_channels, self.out_channels = in_channels, out_channels
        self.normalize, self.root_weight = normalize, root_weight
        self.aggr = "mean"
        if isinstance(in_channels, int):
            in_channels = (in_channels, in_channels)
        self.lin_l = Linear(in_channels[0], out_channels, bias=bias)
        if self.root_weight:
            self.lin_r = Linear(in_channels[1], out_channels, bias=False)
        self.reset_parameters()

    def reset_parameters(self):
        self.lin_l.reset_parameters()
        if self.root_weight:
            self.lin_r.reset_parameters()

    def message_and_aggregate(self, adj_t, x):
        return matmul(adj_t, x[0], reduce=self.aggr)

    def forward(self, x, edge_index, size=None):
        if isinstance(x, torch.Tensor):
            x = (x, x)
        out = self.message_and_aggregate(edge_index, x)
        out = self.lin_l(out)
        x_r = x[1]
        if self.root_weight and x_r is not None:
            out = out + self.lin_r(x_r)
        if self.normalize:
            out = F.normalize(out, p=2.0, dim=-1)
        return out


class ReLUDropout(torch.nn.Module):
    """ReLU followed by dropout as ONE module, so that QModule can swap the
    pair for a single fused pass (QReLUDropout)."""

    def __init__(self, p=0.5):
        super().__init__()
        self.p = p

    def forward(self, input):  # noqa: A002
        return F.dropout(F.relu(input), self.p, self.training)

    def extra_repr(self):
        return f"p={self.p}"
