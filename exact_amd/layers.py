"""Drop-in quantised layers with the names, constructor arguments and
forward signatures of exact/exact/layers.py in the reference (QLinear :268,
QGCNConv :215, QSAGEConv :123, QBatchNorm1d :340, QReLU :284, QDropout :316,
QDropout2 :328).  In eval mode every layer runs the stock op, as there."""
import torch
import torch.nn.functional as F
from torch.nn import Parameter

from .conf import config
from .cpp_extension import quantization as ext_quantization
from .nn import GCN2Conv, GCNConv, GENConv, GraphConv, SAGEConv, glorot
from .ops import input2rp, qbatch_norm, qelu, qlinear, quantize_activation, relu_dropout, take_compressed
from .qsheme import QScheme
from .spmm import QMatmul, qmatmul


class QLinear(torch.nn.Linear):
    def __init__(self, input_features, output_features, bias=True, rp=True):
        super().__init__(input_features, output_features, bias)
        self.scheme = QScheme("linear") if config.single_precision else None
        self.rp = rp

    def forward(self, input, quantized=None, randmat=None):  # noqa: A002
        if self.training:
            if quantized is None:
                quantized = take_compressed(input, project=self.rp)
            return qlinear.apply(input, self.weight, self.bias, quantized, randmat, self.scheme, self.rp)
        return super().forward(input)


class QGCNConv(GCNConv):
    """layers.py:215-265: the weight is stored [out, in] and the linear map is
    a qlinear; propagation is a quantised SpMM."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self.weight = Parameter(torch.Tensor(self.out_channels, self.in_channels))
        self.msg_and_aggr_func = QMatmul(self.aggr)
        self.lin_scheme = QScheme("linear") if config.single_precision else None
        self.reset_parameters()

    def reset_parameters(self):
        glorot(self.weight)
        if self.bias is not None:
            self.bias.data.zero_()
        self._cached_adj_t = None

    def forward(self, x, edge_index, edge_weight=None):
        adj_t = self._normalized(edge_index)
        if self.training:
            # layers.py:252 passes lin_scheme in the `randmat` slot; with
            # kept_frac == 1 that slot is unused, so the numbers are those of
            # a qlinear without a scheme.  Here the scheme is passed as scheme.
            x = qlinear.apply(x, self.weight, None, take_compressed(x), None, self.lin_scheme)
        else:
            x = F.linear(x, self.weight, None)
        out = self.message_and_aggregate(adj_t, x)
        if self.bias is not None:
            out = out + self.bias
        return out

    def message_and_aggregate(self, adj_t, x):
        return self.msg_and_aggr_func(adj_t, x)


class QSAGEConv(SAGEConv):
    """layers.py:123-178: the input is projected + quantised ONCE and the same
    compressed copy serves the mean aggregation and lin_r."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        in_channels = self.in_channels
        if isinstance(in_channels, int):
            in_channels = (in_channels, in_channels)
        bias = self.lin_l.bias is not None
        self.lin_l = QLinear(in_channels[0], self.out_channels, bias=bias, rp=True)
        if self.root_weight:
            self.lin_r = QLinear(in_channels[1], self.out_channels, bias=False, rp=True)
        self.msg_and_aggr_func = QMatmul(self.aggr)
        self.scheme = QScheme("sage") if config.single_precision else None
        self.reset_parameters()

    def forward(self, x, edge_index, size=None):
        if isinstance(x, torch.Tensor):
            x = (x, x)
            l_eq_r = True
        else:
            l_eq_r = False
        if l_eq_r and self.training:
            if config.kept_frac < 1.0:
                kept_acts = int(config.kept_frac * x[0].shape[1] + 0.999)
                dim_reduced_input, randmat = input2rp(x[0], kept_acts)
            else:
                dim_reduced_input, randmat = x[0], None
            quantized = take_compressed(x[0]) or quantize_activation(dim_reduced_input, self.scheme)
        else:
            quantized, randmat = None, None
        out = self.message_and_aggregate(edge_index, x, quantized=quantized, randmat=randmat)
        out = self.lin_l(out)
        x_r = x[1]
        if self.root_weight and x_r is not None:
            out = out + self.lin_r(x_r, quantized, randmat)
        if self.normalize:
            out = F.normalize(out, p=2.0, dim=-1)
        return out

    def message_and_aggregate(self, adj_t, x, quantized=None, randmat=None):
        return self.msg_and_aggr_func(adj_t, x[0], quantized=quantized, randmat=randmat)


class QGraphConv(GraphConv):
    """layers.py:181-212: both linear maps are QLinear, the aggregation a
    quantised SpMM."""

    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        in_channels = self.in_channels
        if isinstance(in_channels, int):
            in_channels = (in_channels, in_channels)
        bias = self.lin_l.bias is not None
        self.lin_l = QLinear(in_channels[0], self.out_channels, bias=bias, rp=True)
        self.lin_r = QLinear(in_channels[1], self.out_channels, bias=False, rp=True)
        self.msg_and_aggr_func = QMatmul(self.aggr)
        self.reset_parameters()

    def message_and_aggregate(self, adj_t, x):
        return self.msg_and_aggr_func(adj_t, x[0])


def qaddmm(input, mat1, mat2, beta=1.0, alpha=1):  # noqa: A002
    """layers.py:27-28.  As there, the product is qlinear(mat1, mat2) = mat1 @
    mat2^T (not torch.addmm's mat1 @ mat2): QGCN2Conv multiplies by the
    transposed weight in the reference, and so does this."""
    return beta * input + alpha * qlinear.apply(mat1, mat2, None)


class QGCN2Conv(GCN2Conv):
    """layers.py:66-120."""

    def message_and_aggregate(self, adj_t, x):
        return qmatmul(adj_t, x, reduce=self.aggr)

    def _addmm(self, inp, mat, weight):
        return qaddmm(inp, mat, weight, beta=1.0 - self.beta, alpha=self.beta)


class QMLP(torch.nn.Sequential):
    """layers.py:32-47: QLinear (-> QBatchNorm1d) -> QReLU -> QDropout blocks."""

    def __init__(self, channels, norm, bias=True, dropout=0.0):
        blocks = []
        for i in range(1, len(channels)):
            blocks.append(QLinear(channels[i - 1], channels[i], bias))
            if i < len(channels) - 1:
                if norm == "batch":
                    blocks.append(QBatchNorm1d(channels[i], affine=True))
                elif norm:
                    raise NotImplementedError(f'Normalization layer "{norm}" not supported.')
                blocks.append(QReLU())
                blocks.append(QDropout(dropout))
        super().__init__(*blocks)


class QGENConv(GENConv):
    """layers.py:50-63: the MLP is a QMLP and the message ReLU keeps a 1-bit mask."""

    def _make_mlp(self, channels, norm):
        return QMLP(channels, norm)

    def message(self, x_j, edge_attr=None):
        msg = x_j if edge_attr is None else x_j + edge_attr
        return ext_quantization.act_quantized_relu(msg) + self.eps


class QReLU(torch.nn.Module):
    def __init__(self, inplace=False):
        super().__init__()

    def forward(self, input):  # noqa: A002
        if self.training:
            return ext_quantization.act_quantized_relu(input)
        return F.relu(input)


class QLeakyReLU(torch.nn.Module):
    """layers.py:295-301 of the reference (compressed in train and eval alike)."""

    def __init__(self, negative_slope, inplace=False):
        super().__init__()
        self.negative_slope = negative_slope

    def forward(self, input):  # noqa: A002
        return ext_quantization.act_quantized_leaky_relu(input, self.negative_slope)


class QELU(torch.nn.Module):
    """layers.py:304-313 of the reference."""

    def __init__(self, alpha, inplace=False):
        super().__init__()
        self.alpha = alpha

    def forward(self, input):  # noqa: A002
        if self.training:
            return qelu.apply(input, self.alpha)
        return F.elu(input, self.alpha)


class QDropout(torch.nn.Module):
    def __init__(self, p):
        super().__init__()
        self.p = p

    def forward(self, input):  # noqa: A002
        if self.training:
            return ext_quantization.act_quantized_dropout(input, self.p, self.training)
        return F.dropout(input, self.p, self.training)


class QDropout2(torch.nn.Module):
    def __init__(self, p):
        super().__init__()
        self.p = p

    def forward(self, input):  # noqa: A002
        if self.training:
            return ext_quantization.act_quantized_dropout(input, self.p, self.training) * (1 - self.p)
        return F.dropout(input, self.p, self.training) * (1 - self.p)


class QReLUDropout(torch.nn.Module):
    """QReLU followed by QDropout (layers.py:284-325) as one pass that keeps one
    joint mask; with `for_consumer`, the compressed copy the following
    QLinear / QGCNConv / QSAGEConv would make of the result is produced in the
    same pass and handed to it.  Bit-identical to the separate layers."""

    def __init__(self, p, for_consumer=True):
        super().__init__()
        self.p = p
        self.for_consumer = for_consumer

    def forward(self, input):  # noqa: A002
        if self.training:
            return relu_dropout(input, self.p, self.for_consumer)
        return F.relu(input)

    def extra_repr(self):
        return f"p={self.p}, for_consumer={self.for_consumer}"


class QBatchNorm1d(torch.nn.BatchNorm1d):
    def __init__(self, num_features, eps=1e-05, momentum=0.1, affine=True, track_running_stats=True):
        super().__init__(num_features, eps, momentum, affine, track_running_stats)
        self.scheme = QScheme("batchnorm") if config.single_precision else None

    def forward(self, input):  # noqa: A002
        if not self.training:
            return super().forward(input)
        self._check_input_dim(input)
        exponential_average_factor = 0.0 if self.momentum is None else self.momentum
        if self.track_running_stats and self.num_batches_tracked is not None:
            self.num_batches_tracked = self.num_batches_tracked + 1
            if self.momentum is None:
                exponential_average_factor = 1.0 / float(self.num_batches_tracked)
        return qbatch_norm.apply(
            input,
            self.running_mean if self.track_running_stats else None,
            self.running_var if self.track_running_stats else None,
            self.weight, self.bias, True, exponential_average_factor, self.eps, self.scheme)
