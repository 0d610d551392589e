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

    def forward(self, input, norm=None):  # noqa: A002
        """`norm`: a normalisation layer to apply first (the quantised counterpart
        folds a batch norm into its pass)."""
        if norm is not None:
            input = norm(input)  # noqa: A001
        return F.dropout(F.relu(input), self.p, self.training)

    def extra_repr(self):
        return f"p={self.p}"


class GraphConv(torch.nn.Module):
    """out = lin_l(aggr_j w_ij x_j) + lin_r(x_i), the operator the reference's
    QGraphConv subclasses (layers.py:181-212; torch_geometric 1.7 parameter
    names lin_l / lin_r).  Edge weights are the values of the SparseTensor."""

    def __init__(self, in_channels, out_channels, aggr="add", bias=True):
        super().__init__()
        self.in_channels, self.out_channels, self.aggr = in_channels, out_channels, aggr
        if isinstance(in_channels, int):
            in_channels = (in_channels, in_channels)
        self.lin_l = Linear(in_channels[0], out_channels, bias=bias)
        self.lin_r = Linear(in_channels[1], out_channels, bias=False)
        self.reset_parameters()

    def reset_parameters(self):
        self.lin_l.reset_parameters()
        self.lin_r.reset_parameters()

    def message_and_aggregate(self, adj_t, x):
        return matmul(adj_t, x[0], reduce=self.aggr)

    def forward(self, x, edge_index, edge_weight=None, size=None):
        if isinstance(x, torch.Tensor):
            x = (x, x)
        out = self.lin_l(self.message_and_aggregate(edge_index, x))
        if x[1] is not None:
            out = out + self.lin_r(x[1])
        return out


class GCN2Conv(torch.nn.Module):
    """GCNII layer: out = (1 - beta) h + beta h W1 with h = (1 - alpha) A x +
    alpha x_0 (shared weights), or the two-weight form; beta = log(theta /
    layer + 1).  The operator the reference's QGCN2Conv subclasses
    (layers.py:66-120)."""

    def __init__(self, channels, alpha, theta=None, layer=None, shared_weights=True, cached=False,
                 add_self_loops=True, normalize=True, aggr="add"):
        super().__init__()
        self.channels, self.alpha, self.aggr = channels, alpha, aggr
        self.beta = 1.0 if theta is None or layer is None else math.log(theta / layer + 1)
        self.cached, self.normalize, self.add_self_loops = cached, normalize, add_self_loops
        self._cached_adj_t = None
        self.weight1 = Parameter(torch.Tensor(channels, channels))
        if shared_weights:
            self.register_parameter("weight2", None)
        else:
            self.weight2 = Parameter(torch.Tensor(channels, channels))
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight1)
        glorot(self.weight2)
        self._cached_adj_t = None

    def _normalized(self, adj_t):
        if not self.normalize:
            return adj_t
        if self._cached_adj_t is not None:
            return self._cached_adj_t
        out = gcn_norm(adj_t, self.add_self_loops)
        if self.cached:
            self._cached_adj_t = out
        return out

    def message_and_aggregate(self, adj_t, x):
        return matmul(adj_t, x, reduce=self.aggr)

    def _addmm(self, inp, mat, weight):
        return (1.0 - self.beta) * inp + self.beta * (mat @ weight)

    def forward(self, x, x_0, edge_index, edge_weight=None):
        x = self.message_and_aggregate(self._normalized(edge_index), x) * (1 - self.alpha)
        x_0 = self.alpha * x_0[:x.size(0)]
        if self.weight2 is None:
            out = x + x_0
            return self._addmm(out, out, self.weight1)
        return self._addmm(x, x, self.weight1) + self._addmm(x_0, x_0, self.weight2)


def edge_softmax(score, row, num_rows, eps=1e-16):
    """Softmax of score[E, H] over the entries that share a row (PyG's
    utils.softmax: shift by the group maximum, + 1e-16 in the denominator;
    torch_scatter's scatter_softmax is the same with eps = 0)."""
    idx = row.view(-1, 1).expand_as(score)
    top = torch.full((num_rows, score.size(1)), float("-inf"), dtype=score.dtype, device=score.device)
    top = top.scatter_reduce(0, idx, score.detach(), "amax", include_self=True)
    e = (score - top.index_select(0, row)).exp()
    denom = torch.zeros((num_rows, score.size(1)), dtype=score.dtype, device=score.device).index_add_(0, row, e)
    return e / (denom.index_select(0, row) + eps)


class CustomGATConv(torch.nn.Module):
    """Multi-head graph attention with an optional residual projection and an
    optional separate destination attention vector -- the reference's
    CustomGATConv (gatconv.py:18-144), on the SparseTensor path: entry (i, j)
    of adj_t carries the message from j to i."""

    def __init__(self, in_channels, out_channels, heads=1, concat=True, negative_slope=0.2, dropout=0.0,
                 add_self_loops=True, bias=True, residual=True, use_attn_dst=True):
        super().__init__()
        self.in_channels, self.out_channels, self.heads, self.concat = in_channels, out_channels, heads, concat
        self.negative_slope, self.dropout, self.add_self_loops = negative_slope, dropout, add_self_loops
        self.residual, self.use_attn_dst = residual, use_attn_dst
        self._build_linears(Linear)
        self.att_l = Parameter(torch.Tensor(1, heads, out_channels))
        self.att_r = Parameter(torch.Tensor(1, heads, out_channels)) if use_attn_dst else self.att_l
        if bias:
            self.bias = Parameter(torch.Tensor(heads * out_channels if concat else out_channels))
        else:
            self.register_parameter("bias", None)
        self.reset_parameters()

    def _build_linears(self, linear_cls):
        width = self.heads * self.out_channels
        if isinstance(self.in_channels, int):
            self.lin_l = linear_cls(self.in_channels, width, bias=False)
            self.lin_r = self.lin_l
        else:
            self.lin_l = linear_cls(self.in_channels[0], width, bias=False)
            self.lin_r = linear_cls(self.in_channels[1], width, bias=False)
        if self.residual:
            self.res_fc = Linear(self.in_channels, width, bias=False)
        else:
            self.res_fc = None

    def reset_parameters(self):
        gain = torch.nn.init.calculate_gain("relu")
        torch.nn.init.xavier_normal_(self.lin_l.weight, gain=gain)
        torch.nn.init.xavier_normal_(self.lin_r.weight, gain=gain)
        if self.res_fc is not None:
            torch.nn.init.xavier_normal_(self.res_fc.weight, gain=gain)
        torch.nn.init.xavier_normal_(self.att_l, gain=gain)
        if self.use_attn_dst:
            torch.nn.init.xavier_normal_(self.att_r, gain=gain)
        if self.bias is not None:
            self.bias.data.zero_()

    def _edges(self, adj_t):
        """(row, col, number of rows) of the graph with self loops set; kept for
        the graph object last seen, since building it sorts the entries."""
        cached = getattr(self, "_edge_cache", None)
        if cached is None or cached[0] is not adj_t:
            g = adj_t.fill_diag(1.0) if self.add_self_loops else adj_t
            row, col, _ = g.coo()
            cached = (adj_t, row.long(), col.long(), g.sparse_size(0))
            self._edge_cache = cached
        return cached[1], cached[2], cached[3]

    # the two hooks the quantised subclass replaces
    def _leaky_relu(self, score):
        return F.leaky_relu(score, self.negative_slope)

    def _attention_dropout(self, alpha):
        return F.dropout(alpha, p=self.dropout, training=self.training)

    def forward(self, x, edge_index, size=None):
        H, C = self.heads, self.out_channels
        if isinstance(x, torch.Tensor):
            x_l = x_r = self.lin_l(x).view(-1, H, C)
            alpha_l = (x_l * self.att_l).sum(dim=-1)
            alpha_r = (x_r * self.att_r).sum(dim=-1) if self.use_attn_dst else alpha_l
            x_res = x
        else:
            x_l = self.lin_l(x[0]).view(-1, H, C)
            alpha_l = (x_l * self.att_l).sum(dim=-1)
            alpha_r = None
            if x[1] is not None:
                alpha_r = (self.lin_r(x[1]).view(-1, H, C) * self.att_r).sum(dim=-1)
            x_res = x[1]
        row, col, num_rows = self._edges(edge_index)
        score = alpha_l.index_select(0, col)
        if alpha_r is not None:
            score = score + alpha_r.index_select(0, row)
        alpha = edge_softmax(self._leaky_relu(score), row, num_rows)
        alpha = self._attention_dropout(alpha)
        msg = x_l.index_select(0, col) * alpha.unsqueeze(-1)
        out = torch.zeros((num_rows, H, C), dtype=msg.dtype, device=msg.device).index_add_(0, row, msg)
        out = out.view(-1, H * C) if self.concat else out.mean(dim=1)
        if self.res_fc is not None:
            out = out + self.res_fc(x_res)
        if self.bias is not None:
            out = out + self.bias
        return out


class MLP(torch.nn.Sequential):
    """Linear (-> norm) -> ReLU -> Dropout blocks, the MLP of PyG's GENConv."""

    def __init__(self, channels, norm=None, bias=True, dropout=0.0):
        blocks = []
        for i in range(1, len(channels)):
            blocks.append(Linear(channels[i - 1], channels[i], bias))
            if i < len(channels) - 1:
                if norm == "batch":
                    blocks.append(torch.nn.BatchNorm1d(channels[i], affine=True))
                elif norm == "layer":
                    blocks.append(torch.nn.LayerNorm(channels[i], elementwise_affine=True))
                elif norm == "instance":
                    blocks.append(torch.nn.InstanceNorm1d(channels[i], affine=False))
                elif norm:
                    raise NotImplementedError(f'Normalization layer "{norm}" not supported.')
                blocks.append(torch.nn.ReLU())
                blocks.append(torch.nn.Dropout(dropout))
        super().__init__(*blocks)


class MessageNorm(torch.nn.Module):
    """msg / |msg| * |x| * scale (PyG's MessageNorm)."""

    def __init__(self, learn_scale=False):
        super().__init__()
        self.scale = Parameter(torch.Tensor([1.0]), requires_grad=learn_scale)

    def reset_parameters(self):
        self.scale.data.fill_(1.0)

    def forward(self, x, msg, p=2):
        return F.normalize(msg, p=p, dim=-1) * x.norm(p=p, dim=-1, keepdim=True) * self.scale


class GENConv(torch.nn.Module):
    """The generalised aggregation layer of DeeperGCN that the reference's
    QGENConv subclasses (layers.py:50-63; PyG 1.7 GENConv): per edge the
    message relu(x_j) + eps, aggregated per target node with a softmax (optionally
    stop-gradient) or a power mean, added to x_i and passed through an MLP.
    Entry (i, j) of adj_t carries the message from j to i; edge features are
    not supported on this path."""

    def __init__(self, in_channels, out_channels, aggr="softmax", t=1.0, learn_t=False, p=1.0, learn_p=False,
                 msg_norm=False, learn_msg_scale=False, norm="batch", num_layers=2, eps=1e-7):
        super().__init__()
        assert aggr in ("softmax", "softmax_sg", "power")
        self.in_channels, self.out_channels, self.aggr, self.eps = in_channels, out_channels, aggr, eps
        channels = [in_channels] + [in_channels * 2] * (num_layers - 1) + [out_channels]
        self.mlp = self._make_mlp(channels, norm)
        self.msg_norm = MessageNorm(learn_msg_scale) if msg_norm else None
        self.initial_t, self.initial_p = t, p
        self.t = Parameter(torch.Tensor([t]), requires_grad=True) if (learn_t and aggr == "softmax") else t
        self.p = Parameter(torch.Tensor([p]), requires_grad=True) if learn_p else p

    def _make_mlp(self, channels, norm):
        return MLP(channels, norm=norm)

    def reset_parameters(self):
        for m in self.mlp:
            if hasattr(m, "reset_parameters"):
                m.reset_parameters()
        if self.msg_norm is not None:
            self.msg_norm.reset_parameters()
        if isinstance(self.t, Parameter):
            self.t.data.fill_(self.initial_t)
        if isinstance(self.p, Parameter):
            self.p.data.fill_(self.initial_p)

    def message(self, x_j, edge_attr=None):
        msg = x_j if edge_attr is None else x_j + edge_attr
        return F.relu(msg) + self.eps

    def aggregate(self, inputs, row, num_rows):
        if self.aggr in ("softmax", "softmax_sg"):
            alpha = edge_softmax(inputs * self.t, row, num_rows, eps=0.0)
            if self.aggr == "softmax_sg":
                alpha = alpha.detach()
            out = torch.zeros((num_rows, inputs.size(1)), dtype=inputs.dtype, device=inputs.device)
            return out.index_add_(0, row, inputs * alpha)
        lo, hi = 1e-7, 1e1
        powered = torch.pow(inputs.clamp(lo, hi), self.p)
        total = torch.zeros((num_rows, inputs.size(1)), dtype=inputs.dtype, device=inputs.device).index_add_(0, row, powered)
        count = torch.zeros(num_rows, dtype=inputs.dtype, device=inputs.device).index_add_(
            0, row, torch.ones_like(row, dtype=inputs.dtype)).clamp_(min=1)
        return torch.pow((total / count.unsqueeze(-1)).clamp(lo, hi), 1 / self.p)

    def forward(self, x, edge_index, edge_attr=None, size=None):
        if edge_attr is not None:
            raise NotImplementedError("edge features are not supported on the SparseTensor path")
        if isinstance(x, torch.Tensor):
            x = (x, x)
        row, col, _ = edge_index.coo()
        row, col = row.long(), col.long()
        out = self.aggregate(self.message(x[0].index_select(0, col)), row, edge_index.sparse_size(0))
        if self.msg_norm is not None:
            out = self.msg_norm(x[0], out)
        if x[1] is not None:
            out = out + x[1]
        return self.mlp(out)
