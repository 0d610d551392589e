"""QModule: wrap a model and swap its stock layers for the quantised ones, as
exact/exact/module.py:18-112 of the reference does (Linear, BatchNorm1d, ReLU,
Dropout, GCNConv, SAGEConv, GCN2Conv, GraphConv, CustomGATConv, GENConv).

The conversion is table driven: `_RULES` pairs a predicate on the stock layer
with a builder of its quantised counterpart; the first match wins, layers
without a rule are searched recursively."""
from collections import OrderedDict

import torch
import torch.nn as nn

from .conf import config
from .gatconv import QCustomGATConv
from .layers import (QBatchNorm1d, QDropout, QDropout2, QGCN2Conv, QGCNConv, QGENConv, QGraphConv, QLinear,
                     QReLU, QReLUDropout, QSAGEConv)
from .nn import CustomGATConv, GCN2Conv, GCNConv, GENConv, GraphConv, ReLUDropout, SAGEConv

_ALREADY_QUANTISED = (QBatchNorm1d, QLinear, QReLU, QGCNConv, QDropout, QDropout2, QSAGEConv, QReLUDropout,
                      QGCN2Conv, QGraphConv, QCustomGATConv, QGENConv)


def _kind(cls, pyg_name=None):
    """Predicate: an instance of `cls`, or torch_geometric's class of that name
    (whose attributes the library's stock layers mirror)."""
    def matches(layer):
        if isinstance(layer, cls):
            return True
        return pyg_name is not None and type(layer).__name__ == pyg_name \
            and type(layer).__module__.startswith("torch_geometric")
    return matches


def _dropout(p):
    return QDropout2(p) if config.dropout2 else QDropout(p)        # module.py:38-42


class _ReLUThenDropout(nn.Sequential):
    """The two quantised layers one after the other, callable like ReLUDropout."""

    def forward(self, input, norm=None):  # noqa: A002
        return super().forward(input if norm is None else norm(input))


def _relu_dropout(src):
    if config.fuse_epilogue and not config.dropout2:
        return QReLUDropout(src.p)
    return _ReLUThenDropout(QReLU(), _dropout(src.p))


def _gcn2(src):                                                      # module.py:47-53
    layer = QGCN2Conv(src.channels, alpha=src.alpha, theta=None, layer=None, shared_weights=src.weight2 is None,
                      cached=src.cached, add_self_loops=src.add_self_loops, normalize=src.normalize)
    layer.beta = src.beta
    return layer


def _gen(src):                                                       # module.py:63-85
    kinds = {nn.LayerNorm: "layer", nn.InstanceNorm1d: "instance"}
    norm = next((kinds[type(m)] for m in src.mlp if type(m) in kinds), "batch")
    has_norm = src.msg_norm is not None
    return QGENConv(src.in_channels, src.out_channels, src.aggr,
                    t=src.initial_t, learn_t=src.aggr == "softmax" and isinstance(src.t, nn.Parameter),
                    p=src.initial_p, learn_p=isinstance(src.p, nn.Parameter),
                    msg_norm=has_norm, learn_msg_scale=has_norm and src.msg_norm.scale.requires_grad,
                    norm=norm, num_layers=sum(isinstance(m, nn.Linear) for m in src.mlp), eps=src.eps)


_RULES = (
    (lambda m: isinstance(m, nn.BatchNorm1d) and config.enable_quantized_bn,
     lambda m: QBatchNorm1d(m.num_features, m.eps, m.momentum, m.affine, m.track_running_stats)),
    (_kind(nn.Linear), lambda m: QLinear(m.in_features, m.out_features, m.bias is not None)),
    (_kind(nn.ReLU), lambda m: QReLU()),
    (_kind(nn.Dropout), lambda m: _dropout(m.p)),
    (_kind(ReLUDropout), _relu_dropout),
    (_kind(GCNConv, "GCNConv"),
     lambda m: QGCNConv(m.in_channels, m.out_channels, m.improved, m.cached, m.add_self_loops, m.normalize,
                        m.bias is not None, aggr=m.aggr)),
    (_kind(SAGEConv, "SAGEConv"),
     lambda m: QSAGEConv(m.in_channels, m.out_channels, m.normalize, m.root_weight, m.lin_l.bias is not None)),
    (_kind(GCN2Conv), _gcn2),
    (_kind(GraphConv), lambda m: QGraphConv(m.in_channels, m.out_channels, m.aggr, m.lin_l.bias is not None)),
    (_kind(CustomGATConv),
     lambda m: QCustomGATConv(m.in_channels, m.out_channels, m.heads, m.concat, m.negative_slope, m.dropout,
                              m.add_self_loops, m.bias is not None, m.residual, m.use_attn_dst)),
    (_kind(GENConv), _gen),
)


def _quantised_counterpart(layer):
    for applies, build in _RULES:
        if applies(layer):
            return build(layer)
    return None


class QModule(nn.Module):
    def __init__(self, model):
        super().__init__()
        self.model = model
        QModule.convert_layers(model)

    @staticmethod
    def convert_layers(module):
        for name, child in module.named_children():
            if isinstance(child, _ALREADY_QUANTISED):
                continue
            replacement = _quantised_counterpart(child)
            if replacement is None:
                QModule.convert_layers(child)
            else:
                setattr(module, name, replacement)

    def forward(self, *args, **kwargs):
        return self.model(*args, **kwargs)

    # The wrapper's weights interchange with the unwrapped model's: the "model."
    # prefix this wrapper adds is hidden in both directions (module.py:93-107).
    def load_state_dict(self, state_dict, strict=True):
        return super().load_state_dict(OrderedDict(("model." + k, v) for k, v in state_dict.items()), strict)

    def state_dict(self, destination=None, prefix="", keep_vars=False):
        wrapped = super().state_dict(destination=destination, prefix=prefix, keep_vars=keep_vars)
        return OrderedDict((k[len("model."):], v) for k, v in wrapped.items())

    def reset_parameters(self):
        self.model.reset_parameters()

    @torch.no_grad()
    def mini_inference(self, x_all, loader):
        return self.model.mini_inference(x_all, loader)
