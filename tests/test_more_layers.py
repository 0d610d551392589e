"""The other convolution layers the reference quantises -- GraphConv, GCN2Conv,
CustomGATConv, the QMLP block -- on both back ends: stock layers against dense
restatements, quantised layers against the stock ones (compression off: same
numbers; INT8: close gradients), and QModule's conversion of them."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

import exact_amd as exact
from exact_amd import nn as xnn
from exact_amd.conf import config
from exact_amd.sparse import SparseTensor, gcn_norm


def graph(n, m, seed, backend, valued=False):
    rng = np.random.default_rng(seed)
    A = sp.coo_matrix((rng.random(m).astype(np.float32) + 0.5, (rng.integers(0, n, m), rng.integers(0, n, m))),
                      shape=(n, n)).tocsr()
    A.sum_duplicates()
    A.setdiag(0)
    A.eliminate_zeros()
    A.sort_indices()
    if not valued:
        A.data[:] = 1.0
    adj = SparseTensor.from_scipy(A, backend)
    return A, (adj if valued else adj.set_value(None))


def copy_params(dst, src):
    sd = src.state_dict()
    missing = dst.load_state_dict(sd, strict=True)
    assert not missing.missing_keys and not missing.unexpected_keys


def grads_of(layer, out):
    out.square().sum().backward()
    return {k: p.grad.detach().clone() for k, p in layer.named_parameters() if p.grad is not None}


def close(a, b, backend, loose=False):
    tol = dict(rtol=1e-5, atol=1e-5) if backend.type == "cpu" else dict(rtol=2e-4, atol=2e-4)
    if loose:
        tol = dict(rtol=0.1, atol=0.1 * float(b.abs().max()))
    assert torch.allclose(a, b, **tol), float((a - b).abs().max())


def test_graph_conv(backend):
    A, adj = graph(80, 500, 1, backend, valued=True)
    torch.manual_seed(0)
    stock = xnn.GraphConv(24, 16).to(backend)
    x = torch.randn(80, 24, device=backend)
    want = (torch.from_numpy(A.toarray()).to(backend) @ x) @ stock.lin_l.weight.t() + stock.lin_l.bias + x @ stock.lin_r.weight.t()
    close(stock(x, adj), want, backend)
    g_stock = grads_of(stock, stock(x, adj))
    q = exact.QGraphConv(24, 16).to(backend).train()
    copy_params(q, stock)
    config.compress_activation = False
    close(q(x, adj), want, backend)
    g_q = grads_of(q, q(x, adj))
    for k in g_stock:
        close(g_q[k], g_stock[k], backend)
    config.compress_activation = True
    config.activation_compression_bits = [8]
    q.zero_grad()
    g_q8 = grads_of(q, q(x, adj))
    for k in g_stock:
        close(g_q8[k], g_stock[k], backend, loose=True)
        assert not torch.equal(g_q8[k], g_stock[k]) or k.endswith("bias")


@pytest.mark.parametrize("shared", [True, False])
def test_gcn2_conv(backend, shared):
    A, adj = graph(70, 420, 2, backend)
    torch.manual_seed(1)
    stock = xnn.GCN2Conv(20, alpha=0.1, theta=0.5, layer=2, shared_weights=shared).to(backend)
    assert abs(stock.beta - np.log(0.5 / 2 + 1)) < 1e-12
    x, x0 = torch.randn(70, 20, device=backend), torch.randn(70, 20, device=backend)
    An = gcn_norm(SparseTensor.from_scipy(A).set_value(None)).to_dense().to(backend)
    h, h0, b = 0.9 * (An @ x), 0.1 * x0, stock.beta
    if shared:
        want = (1 - b) * (h + h0) + b * ((h + h0) @ stock.weight1)
    else:
        want = (1 - b) * h + b * (h @ stock.weight1) + (1 - b) * h0 + b * (h0 @ stock.weight2)
    close(stock(x, x0, adj), want, backend)
    q = exact.QModule(torch.nn.ModuleList([stock])).model[0].to(backend).train()
    assert type(q).__name__ == "QGCN2Conv" and q.beta == stock.beta and (q.weight2 is None) == shared
    copy_params(q, stock)
    config.compress_activation = False
    # the reference multiplies by the TRANSPOSED weight in the quantised layer (qaddmm -> qlinear)
    if shared:
        want_q = (1 - b) * (h + h0) + b * ((h + h0) @ stock.weight1.t())
    else:
        want_q = (1 - b) * h + b * (h @ stock.weight1.t()) + (1 - b) * h0 + b * (h0 @ stock.weight2.t())
    close(q(x, x0, adj), want_q, backend)
    config.compress_activation = True
    out = q(x, x0, adj)
    out.sum().backward()
    assert torch.isfinite(q.weight1.grad).all() and q.weight1.grad.abs().sum() > 0


def dense_gat(layer, A, x):
    """Dense restatement: masked softmax over the neighbours (with self loops)."""
    n = A.shape[0]
    H, C = layer.heads, layer.out_channels
    M = torch.from_numpy(((A + sp.eye(n)).toarray() != 0)).to(x.device)
    xl = (x @ layer.lin_l.weight.t()).view(n, H, C)
    al = (xl * layer.att_l).sum(-1)
    ar = (xl * layer.att_r).sum(-1)
    score = F.leaky_relu(ar.unsqueeze(1) + al.unsqueeze(0), layer.negative_slope)      # [i, j, H]
    score = score.masked_fill(~M.unsqueeze(-1), float("-inf"))
    alpha = torch.softmax(score, dim=1)
    out = torch.einsum("ijh,jhc->ihc", alpha, xl)
    out = out.reshape(n, H * C) if layer.concat else out.mean(1)
    if layer.res_fc is not None:
        out = out + x @ layer.res_fc.weight.t()
    return out + layer.bias


@pytest.mark.parametrize("heads,concat,dst", [(3, True, True), (2, False, True), (1, True, False)])
def test_gat_conv(backend, heads, concat, dst):
    A, adj = graph(60, 300, 3, backend)
    torch.manual_seed(2)
    # the residual projection is heads * out_channels wide, so (as in the reference) it needs concat
    stock = xnn.CustomGATConv(12, 8, heads=heads, concat=concat, dropout=0.0, use_attn_dst=dst,
                              residual=concat).to(backend)
    stock.bias.data.normal_()
    x = torch.randn(60, 12, device=backend)
    close(stock(x, adj), dense_gat(stock, A, x), backend)
    g_stock = grads_of(stock, stock(x, adj))
    q = exact.QModule(torch.nn.ModuleList([stock])).model[0].to(backend).train()
    assert type(q).__name__ == "QCustomGATConv" and type(q.lin_l).__name__ == "QLinear" and q.lin_r is q.lin_l
    assert (type(q.res_fc).__name__ == "Linear") == concat and q.use_attn_dst == dst
    copy_params(q, stock)
    config.compress_activation = False
    close(q(x, adj), dense_gat(stock, A, x), backend)
    g_q = grads_of(q, q(x, adj))
    for k in g_stock:
        close(g_q[k], g_stock[k], backend)
    config.compress_activation = True
    config.activation_compression_bits = [8]
    q.zero_grad()
    g_q8 = grads_of(q, q(x, adj))
    for k in g_stock:
        close(g_q8[k], g_stock[k], backend, loose=True)
    # attention dropout goes through the 1-bit-mask kernel and still trains
    q.dropout_module.p = 0.5
    q.zero_grad()
    q(x, adj).sum().backward()
    assert all(torch.isfinite(p.grad).all() for p in q.parameters())
    close(q.eval()(x, adj), dense_gat(stock, A, x), backend)   # eval: no dropout, the stock arithmetic


def test_qmlp_block(backend):
    torch.manual_seed(3)
    mlp = exact.QMLP([16, 32, 8], "batch", dropout=0.0).to(backend).train()
    kinds = [type(m).__name__ for m in mlp]
    assert kinds == ["QLinear", "QBatchNorm1d", "QReLU", "QDropout", "QLinear"]
    x = torch.randn(40, 16, device=backend)
    config.compress_activation = False
    want = mlp[4](F.relu(F.batch_norm(mlp[0](x), None, None, mlp[1].weight, mlp[1].bias, True)))
    close(mlp(x), want, backend)
    with pytest.raises(NotImplementedError):
        exact.QMLP([4, 4, 4], "layer")


def dense_gen(layer, A, x):
    """Dense restatement of GENConv's aggregation."""
    M = torch.from_numpy(A.toarray() != 0).to(x.device)                  # [i, j]
    msg = F.relu(x) + layer.eps                                           # [j, C]
    if layer.aggr in ("softmax", "softmax_sg"):
        score = (msg * layer.t).unsqueeze(0).expand(M.shape[0], -1, -1).masked_fill(~M.unsqueeze(-1), float("-inf"))
        alpha = torch.softmax(score, dim=1)
        alpha = torch.nan_to_num(alpha, nan=0.0)                          # rows without neighbours
        agg = (alpha * msg.unsqueeze(0)).sum(1)
    else:
        powered = msg.clamp(1e-7, 1e1).pow(layer.p)
        cnt = M.sum(1, keepdim=True).clamp(min=1)
        agg = ((M.unsqueeze(-1) * powered.unsqueeze(0)).sum(1) / cnt).clamp(1e-7, 1e1).pow(1 / layer.p)
    if layer.msg_norm is not None:
        agg = F.normalize(agg, p=2, dim=-1) * x.norm(p=2, dim=-1, keepdim=True) * layer.msg_norm.scale
    return layer.mlp(agg + x)


@pytest.mark.parametrize("aggr,msg_norm,learn", [("softmax", False, True), ("softmax_sg", True, False), ("power", False, True)])
def test_gen_conv(backend, aggr, msg_norm, learn):
    A, adj = graph(50, 260, 4, backend)
    torch.manual_seed(5)
    stock = xnn.GENConv(12, 8, aggr=aggr, t=0.7, learn_t=learn, p=2.0, learn_p=learn, msg_norm=msg_norm,
                        learn_msg_scale=msg_norm, num_layers=2).to(backend).train()
    x = torch.randn(50, 12, device=backend)
    close(stock(x, adj), dense_gen(stock, A, x), backend)
    g_stock = grads_of(stock, stock(x, adj))
    q = exact.QModule(torch.nn.ModuleList([stock])).model[0].to(backend).train()
    assert type(q).__name__ == "QGENConv" and type(q.mlp).__name__ == "QMLP"
    assert [type(m).__name__ for m in q.mlp] == ["QLinear", "QBatchNorm1d", "QReLU", "QDropout", "QLinear"]
    assert isinstance(q.t, torch.nn.Parameter) == (learn and aggr == "softmax") and isinstance(q.p, torch.nn.Parameter) == learn
    assert (q.msg_norm is not None) == msg_norm and q.eps == stock.eps
    copy_params(q, stock)
    config.compress_activation = False
    close(q(x, adj), dense_gen(stock, A, x), backend)
    g_q = grads_of(q, q(x, adj))
    for k in g_stock:
        close(g_q[k], g_stock[k], backend)
    config.compress_activation = True
    config.activation_compression_bits = [8]
    q.zero_grad()
    g_q8 = grads_of(q, q(x, adj))
    for k in g_stock:
        if g_stock[k].abs().max() > 1e-4:       # a bias in front of a batch norm has an exactly vanishing gradient
            close(g_q8[k], g_stock[k], backend, loose=True)
    with pytest.raises(NotImplementedError):
        exact.QGENConv(4, 4, norm="layer")
