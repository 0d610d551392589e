"""Drop-in quantised layers with the names, constructor arguments and
forward signatures of exact/exact/layers.py in the reference (QLinear :268,
QGCNConv :215, QSAGEConv :123, QGraphConv :181, QGCN2Conv :66, QGENConv :50,
QMLP :32, QBatchNorm1d :340, QReLU :284, QLeakyReLU :295, QELU :304,
QDropout :316, QDropout2 :328).  In eval mode a layer runs the stock op
wherever the reference's does.

Organisation (this library's own): the element-wise layers share one small
base class that picks the training or the evaluation op; the convolutions get
their QLinear / QMatmul parts from two helpers."""
import torch
import torch.nn.functional as F
from torch.nn import Parameter

from .conf import config
from .cpp_extension import quantization as ext_quantization
from .nn import GCN2Conv, GCNConv, GENConv, GraphConv, SAGEConv, glorot
from .ops import (CompressedActivation, bn_relu_dropout, consumer_bits, project_and_quantize, qbatch_norm, qelu,
                  qgcn, qlinear, qsage, quantize_activation, relu_dropout, take_compressed)
from .qsheme import QScheme
from .spmm import QMatmul, qmatmul


def _scheme(name):
    """Per-layer bookkeeping object of the reference (qsheme.py), attached only
    when config.single_precision is set at construction time."""
    return QScheme(name) if config.single_precision else None


def _channel_pair(in_channels):
    return (in_channels, in_channels) if isinstance(in_channels, int) else tuple(in_channels)


# ---------------------------------------------------------------------------
# linear
# ---------------------------------------------------------------------------
class QLinear(torch.nn.Linear):
    def __init__(self, input_features, output_features, bias=True, rp=True):
        super().__init__(input_features, output_features, bias)
        self.scheme = _scheme("linear")
        self.rp = rp

    def forward(self, input, quantized=None, randmat=None):  # noqa: A002
        if not self.training:
            return super().forward(input)
        if quantized is None:
            quantized = take_compressed(input, project=self.rp)   # a copy a fused producer made, if any
        return qlinear.apply(input, self.weight, self.bias, quantized, randmat, self.scheme, self.rp)


def qaddmm(input, mat1, mat2, beta=1.0, alpha=1):  # noqa: A002
    """layers.py:27-28.  As there, the product is qlinear(mat1, mat2) = mat1 @
    mat2^T (not torch.addmm's mat1 @ mat2): QGCN2Conv multiplies by the
    transposed weight in the reference, and so does this."""
    return beta * input + alpha * qlinear.apply(mat1, mat2, None)


class QMLP(torch.nn.Sequential):
    """layers.py:32-47: QLinear (-> QBatchNorm1d) -> QReLU -> QDropout blocks."""

    def __init__(self, channels, norm, bias=True, dropout=0.0):
        if norm and norm != "batch":
            raise NotImplementedError(f'Normalization layer "{norm}" not supported.')
        widths = list(zip(channels[:-1], channels[1:]))
        blocks = []
        for index, (fan_in, fan_out) in enumerate(widths):
            blocks.append(QLinear(fan_in, fan_out, bias))
            if index + 1 < len(widths):                 # every layer but the last
                if norm:
                    blocks.append(QBatchNorm1d(fan_out, affine=True))
                blocks += [QReLU(), QDropout(dropout)]
        super().__init__(*blocks)


# ---------------------------------------------------------------------------
# convolutions
# ---------------------------------------------------------------------------
class QGCNConv(GCNConv):
    """layers.py:215-265: the weight is stored [out, in] and the linear map is
    a qlinear; propagation is a quantised SpMM."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.weight = Parameter(torch.Tensor(self.out_channels, self.in_channels))
        self.msg_and_aggr_func = QMatmul(self.aggr)
        self.lin_scheme = _scheme("linear")
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight)
        if self.bias is not None:
            self.bias.data.zero_()
        self._cached_adj_t = None

    def _transform(self, x):
        if not self.training:
            return F.linear(x, self.weight, None)
        # layers.py:252 passes lin_scheme in the `randmat` slot; with
        # kept_frac == 1 that slot is unused, so the numbers are those of a
        # qlinear without a scheme.  Here the scheme is passed as scheme.
        return qlinear.apply(x, self.weight, None, take_compressed(x), None, self.lin_scheme)

    def _as_one_node(self, x, adj_t):
        """The whole layer through ops.qgcn where that node applies (fp32 2-D
        input, sum or mean aggregation, edge values without a gradient), else
        None."""
        reduce = self.msg_and_aggr_func.reduce
        if not (config.gcn_single_node and self.training and x.dim() == 2 and x.dtype == torch.float32
                and not torch.is_autocast_enabled(x.device.type) and reduce in ("sum", "mean")):
            return None
        rowptr, col, value = adj_t.csr()
        if value is not None and (value.requires_grad or value.dtype != torch.float32):
            return None
        st = adj_t.storage
        # the transpose operands: backward multiplies by A^T (the reference builds them whenever the dense operand
        # of its qspmm needs a gradient, spmm.py:34-44, which x W^T always does)
        graph = (st.row(), rowptr, col, value, st.rowcount(), st.colptr(), st.csr2csc())
        quantized = take_compressed(x)               # a copy a fused producer made, if any
        if quantized is not None:
            kept = CompressedActivation.adopt(x, quantized, None)
        else:
            kept = CompressedActivation.compress(x, self.lin_scheme)
        return qgcn.apply(x, self.weight, self.bias, graph, reduce, kept)

    def forward(self, x, edge_index, edge_weight=None):
        adj_t = self._normalized(edge_index)
        out = self._as_one_node(x, adj_t)
        if out is not None:
            return out
        out = self.message_and_aggregate(adj_t, self._transform(x))
        return out if self.bias is None else out + self.bias

    def message_and_aggregate(self, adj_t, x):
        return self.msg_and_aggr_func(adj_t, x)


def _quantise_two_linears(conv, root_optional):
    """lin_l / lin_r of a SAGE- or GraphConv-style layer as QLinear, plus the
    quantised aggregation (layers.py:124-139, 182-191)."""
    fan_l, fan_r = _channel_pair(conv.in_channels)
    conv.lin_l = QLinear(fan_l, conv.out_channels, bias=conv.lin_l.bias is not None, rp=True)
    if not root_optional or conv.root_weight:
        conv.lin_r = QLinear(fan_r, conv.out_channels, bias=False, rp=True)
    conv.msg_and_aggr_func = QMatmul(conv.aggr)


class QSAGEConv(SAGEConv):
    """layers.py:123-178: the input is projected + quantised ONCE and the same
    compressed copy serves the mean aggregation and lin_r."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        _quantise_two_linears(self, root_optional=True)
        self.scheme = _scheme("sage")
        self.reset_parameters()

    def _shared_copy(self, x):
        """-> (quantized, randmat) of x for both consumers (layers.py:153-159)."""
        handed_over = take_compressed(x)
        if handed_over is not None:
            return handed_over, None
        if config.kept_frac < 1.0:
            quantized, randmat, _ = project_and_quantize(x, self.scheme)
            return quantized, randmat
        return quantize_activation(x, self.scheme), None

    def _as_one_node(self, x, adj_t):
        """The whole layer through ops.qsage where that node applies (one fp32
        2-D input for both sides, root weight, sum or mean aggregation, edge
        values without a gradient), else None."""
        if not (config.sage_single_node and self.training and self.root_weight and x.dim() == 2
                and x.dtype == torch.float32 and not torch.is_autocast_enabled(x.device.type)
                and self.msg_and_aggr_func.reduce in ("sum", "mean")):
            return None
        rowptr, col, value = adj_t.csr()
        if value is not None and (value.requires_grad or value.dtype != torch.float32):
            return None
        st = adj_t.storage
        if x.requires_grad:
            graph = (st.row(), rowptr, col, value, st.rowcount(), st.colptr(), st.csr2csc())
        else:
            graph = (st._row, rowptr, col, value, st._rowcount, st._colptr, st._csr2csc)
        quantized, randmat = self._shared_copy(x)
        shared = CompressedActivation.adopt(x, quantized, randmat)
        return qsage.apply(x, self.lin_l.weight, self.lin_l.bias, self.lin_r.weight, graph,
                           self.msg_and_aggr_func.reduce, shared, self.lin_l.scheme)

    def forward(self, x, edge_index, size=None):
        same_both_sides = isinstance(x, torch.Tensor)
        if same_both_sides:
            out = self._as_one_node(x, edge_index)
            if out is not None:
                return F.normalize(out, p=2.0, dim=-1) if self.normalize else out
        x_l, x_r = (x, x) if same_both_sides else x
        quantized, randmat = self._shared_copy(x_l) if (same_both_sides and self.training) else (None, None)
        out = self.lin_l(self.message_and_aggregate(edge_index, (x_l, x_r), quantized=quantized, randmat=randmat))
        if self.root_weight and x_r is not None:
            out = out + self.lin_r(x_r, quantized, randmat)
        return F.normalize(out, p=2.0, dim=-1) if self.normalize else out

    def message_and_aggregate(self, adj_t, x, quantized=None, randmat=None):
        return self.msg_and_aggr_func(adj_t, x[0], quantized=quantized, randmat=randmat)


class QGraphConv(GraphConv):
    """layers.py:181-212: both linear maps are QLinear, the aggregation a
    quantised SpMM."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        _quantise_two_linears(self, root_optional=False)
        self.reset_parameters()

    def message_and_aggregate(self, adj_t, x):
        return self.msg_and_aggr_func(adj_t, x[0])


class QGCN2Conv(GCN2Conv):
    """layers.py:66-120."""

    def message_and_aggregate(self, adj_t, x):
        return qmatmul(adj_t, x, reduce=self.aggr)

    def _addmm(self, inp, mat, weight):
        return qaddmm(inp, mat, weight, beta=1.0 - self.beta, alpha=self.beta)


class QGENConv(GENConv):
    """layers.py:50-63: the MLP is a QMLP and the message ReLU keeps a 1-bit mask."""

    def _make_mlp(self, channels, norm):
        return QMLP(channels, norm)

    def message(self, x_j, edge_attr=None):
        msg = x_j if edge_attr is None else x_j + edge_attr
        return ext_quantization.act_quantized_relu(msg) + self.eps


# ---------------------------------------------------------------------------
# element-wise layers: a compressed op in training, the stock op in evaluation
# ---------------------------------------------------------------------------
class _TrainEval(torch.nn.Module):
    always_compressed = False        # QLeakyReLU keeps its mask in eval mode as well (layers.py:300-301)

    def _train(self, t):
        raise NotImplementedError

    def _eval(self, t):
        raise NotImplementedError

    def forward(self, input):  # noqa: A002
        return self._train(input) if (self.training or self.always_compressed) else self._eval(input)


class QReLU(_TrainEval):
    def __init__(self, inplace=False):
        super().__init__()

    def _train(self, t):
        return ext_quantization.act_quantized_relu(t)

    def _eval(self, t):
        return F.relu(t)


class QLeakyReLU(_TrainEval):
    always_compressed = True

    def __init__(self, negative_slope, inplace=False):
        super().__init__()
        self.negative_slope = negative_slope

    def _train(self, t):
        return ext_quantization.act_quantized_leaky_relu(t, self.negative_slope)


class QELU(_TrainEval):
    def __init__(self, alpha, inplace=False):
        super().__init__()
        self.alpha = alpha

    def _train(self, t):
        return qelu.apply(t, self.alpha)

    def _eval(self, t):
        return F.elu(t, self.alpha)


class QDropout(_TrainEval):
    def __init__(self, p):
        super().__init__()
        self.p = p

    def _train(self, t):
        return ext_quantization.act_quantized_dropout(t, self.p, True)

    def _eval(self, t):
        return t                      # F.dropout(t, p, training=False)


class QDropout2(QDropout):
    """layers.py:328-337: dropout whose survivors keep their magnitude (the
    1 / (1 - p) of dropout is undone); evaluation scales by (1 - p)."""

    def _train(self, t):
        return super()._train(t) * (1 - self.p)

    def _eval(self, t):
        return t * (1 - self.p)


class QReLUDropout(_TrainEval):
    """QReLU followed by QDropout (layers.py:284-325) as one pass that keeps one
    joint mask; with `for_consumer`, the compressed copy the following
    QLinear / QGCNConv / QSAGEConv would make of the result is produced in the
    same pass and handed to it.  Bit-identical to the separate layers."""

    def __init__(self, p, for_consumer=True):
        super().__init__()
        self.p = p
        self.for_consumer = for_consumer

    def forward(self, input, norm=None):  # noqa: A002
        """`norm`: a batch norm layer to apply ahead of the ReLU; a QBatchNorm1d in
        training mode is folded into the same pass where the kernel applies."""
        if norm is not None:
            fused = self._with_norm(input, norm) if self.training else None
            if fused is not None:
                return fused
            input = norm(input)  # noqa: A001
        return super().forward(input)

    def _with_norm(self, t, norm):
        if not (isinstance(norm, QBatchNorm1d) and norm.training and config.fuse_epilogue and config.fold_batch_norm
                and t.dim() == 2):
            return None
        bits = consumer_bits(t, self.for_consumer)
        if bits is None or t.shape[0] < 2:
            return None                      # not this kernel's case
        norm._check_input_dim(t)
        return bn_relu_dropout(t, norm, norm._averaging_factor(), self.p, bits)

    def _train(self, t):
        return relu_dropout(t, self.p, self.for_consumer)

    def _eval(self, t):
        return F.relu(t)

    def extra_repr(self):
        return f"p={self.p}, for_consumer={self.for_consumer}"


class QBatchNorm1d(torch.nn.BatchNorm1d):
    def __init__(self, num_features, eps=1e-05, momentum=0.1, affine=True, track_running_stats=True):
        super().__init__(num_features, eps, momentum, affine, track_running_stats)
        self.scheme = _scheme("batchnorm")

    def _averaging_factor(self):
        """Weight of this batch in the running statistics; counts the batch
        (torch.nn.BatchNorm1d's bookkeeping, layers.py:352-369)."""
        if not (self.track_running_stats and self.num_batches_tracked is not None):
            return 0.0 if self.momentum is None else self.momentum
        self.num_batches_tracked = self.num_batches_tracked + 1
        if self.momentum is None:                       # cumulative moving average
            return 1.0 / float(self.num_batches_tracked)
        return self.momentum

    def forward(self, input):  # noqa: A002
        if not self.training:
            return super().forward(input)
        self._check_input_dim(input)
        factor = self._averaging_factor()
        running = (self.running_mean, self.running_var) if self.track_running_stats else (None, None)
        return qbatch_norm.apply(input, *running, self.weight, self.bias, True, factor, self.eps, self.scheme)
