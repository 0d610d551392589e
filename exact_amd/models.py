"""The two model shapes of the full-batch benchmarks: GCN and GraphSAGE with
optional BatchNorm -> ReLU -> Dropout between convolutions, as
mem_speed_bench/models/gcn.py:10-61 and sage.py:13-78 of the reference build
them from stock layers (QModule then swaps the layers)."""
import torch
from torch.nn import BatchNorm1d, ModuleList

from .nn import GCNConv, ReLUDropout, SAGEConv


class _Stack(torch.nn.Module):
    def __init__(self, conv_cls, conv_kwargs, in_channels, hidden_channels, out_channels, num_layers,
                 dropout=0.0, batch_norm=False, residual=False, drop_input=False):
        super().__init__()
        self.in_channels, self.out_channels, self.num_layers = in_channels, out_channels, num_layers
        self.act_drop = ReLUDropout(p=dropout)  # one module for the pair: QModule fuses it
        self.drop_input = drop_input
        if drop_input:
            self.input_dropout = torch.nn.Dropout(p=dropout)
        self.batch_norm, self.residual = batch_norm, residual
        self.convs = ModuleList()
        for i in range(num_layers):
            in_dim = in_channels if i == 0 else hidden_channels
            out_dim = out_channels if i == num_layers - 1 else hidden_channels
            self.convs.append(conv_cls(in_dim, out_dim, **conv_kwargs))
        if batch_norm:
            self.bns = ModuleList(BatchNorm1d(hidden_channels) for _ in range(num_layers - 1))

    def reset_parameters(self):
        for conv in self.convs:
            conv.reset_parameters()
        if self.batch_norm:
            for bn in self.bns:
                bn.reset_parameters()

    def forward(self, x, adj_t, *args):
        if self.drop_input:
            x = self.input_dropout(x)
        for idx, conv in enumerate(self.convs[:-1]):
            h = conv(x, adj_t)
            norm = self.bns[idx] if self.batch_norm else None
            if self.residual and h.size(-1) == x.size(-1):
                if norm is not None:
                    h = norm(h)
                x = self.act_drop(h + x[:h.size(0)])
            else:
                x = self.act_drop(h, norm=norm)    # norm -> ReLU -> dropout as one unit (one pass when quantised)
        return self.convs[-1](x, adj_t)


class GCN(_Stack):
    def __init__(self, in_channels, hidden_channels, out_channels, num_layers, dropout=0.0,
                 drop_input=False, batch_norm=False, residual=False):
        super().__init__(GCNConv, {"normalize": False}, in_channels, hidden_channels, out_channels, num_layers,
                         dropout, batch_norm, residual, drop_input)


class SAGE(_Stack):
    def __init__(self, in_channels, hidden_channels, out_channels, num_layers, dropout=0.0,
                 batch_norm=False, residual=False):
        super().__init__(SAGEConv, {}, in_channels, hidden_channels, out_channels, num_layers,
                         dropout, batch_norm, residual, False)
