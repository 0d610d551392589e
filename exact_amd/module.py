"""QModule: wrap a model and swap its stock layers for the quantised ones, as
exact/exact/module.py:18-112 of the reference does for the layer types on this
library's path (Linear, BatchNorm1d, ReLU, Dropout, GCNConv, SAGEConv, GCN2Conv,
GraphConv, CustomGATConv, GENConv)."""
from collections import OrderedDict

import torch
import torch.nn as nn

from .conf import config
from .gatconv import QCustomGATConv
from .layers import (QBatchNorm1d, QDropout, QDropout2, QGCN2Conv, QGCNConv, QGENConv, QGraphConv, QLinear,
                     QReLU, QReLUDropout, QSAGEConv)
from .nn import CustomGATConv, GCN2Conv, GCNConv, GENConv, GraphConv, ReLUDropout, SAGEConv

_QUANTIZED = (QBatchNorm1d, QLinear, QReLU, QGCNConv, QDropout, QDropout2, QSAGEConv, QReLUDropout, QGCN2Conv,
              QGraphConv, QCustomGATConv, QGENConv)


def _is_pyg(child, name):
    return type(child).__name__ == name and type(child).__module__.startswith("torch_geometric")


class QModule(nn.Module):
    def __init__(self, model):
        super().__init__()
        self.model = model
        QModule.convert_layers(model)

    @staticmethod
    def convert_layers(module):
        for name, child in module.named_children():
            if isinstance(child, _QUANTIZED):
                continue
            if isinstance(child, nn.BatchNorm1d) and config.enable_quantized_bn:
                new = QBatchNorm1d(child.num_features, child.eps, child.momentum, child.affine,
                                   child.track_running_stats)
            elif isinstance(child, nn.Linear):
                new = QLinear(child.in_features, child.out_features, child.bias is not None)
            elif isinstance(child, nn.ReLU):
                new = QReLU()
            elif isinstance(child, nn.Dropout):
                new = QDropout2(child.p) if config.dropout2 else QDropout(child.p)
            elif isinstance(child, ReLUDropout):
                if config.fuse_epilogue and not config.dropout2:
                    new = QReLUDropout(child.p)
                else:
                    new = nn.Sequential(QReLU(), QDropout2(child.p) if config.dropout2 else QDropout(child.p))
            elif isinstance(child, GCNConv) or _is_pyg(child, "GCNConv"):
                new = QGCNConv(child.in_channels, child.out_channels, child.improved, child.cached,
                               child.add_self_loops, child.normalize, child.bias is not None, aggr=child.aggr)
            elif isinstance(child, SAGEConv) or _is_pyg(child, "SAGEConv"):
                new = QSAGEConv(child.in_channels, child.out_channels, child.normalize, child.root_weight,
                                child.lin_l.bias is not None)
            elif isinstance(child, GCN2Conv):
                new = QGCN2Conv(child.channels, alpha=child.alpha, theta=None, layer=None,
                                shared_weights=child.weight2 is None, cached=child.cached,
                                add_self_loops=child.add_self_loops, normalize=child.normalize)
                new.beta = child.beta
            elif isinstance(child, GraphConv):
                new = QGraphConv(child.in_channels, child.out_channels, child.aggr, child.lin_l.bias is not None)
            elif isinstance(child, CustomGATConv):
                new = QCustomGATConv(child.in_channels, child.out_channels, child.heads, child.concat,
                                     child.negative_slope, child.dropout, child.add_self_loops,
                                     child.bias is not None, child.residual, child.use_attn_dst)
            elif isinstance(child, GENConv):
                norm = "batch"
                for m in child.mlp:
                    if isinstance(m, nn.LayerNorm):
                        norm = "layer"
                    elif isinstance(m, nn.InstanceNorm1d):
                        norm = "instance"
                new = QGENConv(child.in_channels, child.out_channels, child.aggr, child.initial_t,
                               child.aggr == "softmax" and isinstance(child.t, nn.Parameter), child.initial_p,
                               isinstance(child.p, nn.Parameter), child.msg_norm is not None,
                               child.msg_norm is not None and child.msg_norm.scale.requires_grad, norm,
                               sum(isinstance(m, nn.Linear) for m in child.mlp), child.eps)
            else:
                QModule.convert_layers(child)
                continue
            setattr(module, name, new)

    def forward(self, *args, **kwargs):
        return self.model(*args, **kwargs)

    def load_state_dict(self, state_dict, strict=True):
        # weights interchange with the unwrapped model: add the "model." prefix
        return super().load_state_dict(OrderedDict(("model." + k, v) for k, v in state_dict.items()), strict)

    def state_dict(self, destination=None, prefix="", keep_vars=False):
        ret = super().state_dict(destination=destination, prefix=prefix, keep_vars=keep_vars)
        return OrderedDict((k[len("model."):], v) for k, v in ret.items())

    def reset_parameters(self):
        self.model.reset_parameters()

    @torch.no_grad()
    def mini_inference(self, x_all, loader):
        return self.model.mini_inference(x_all, loader)
