"""The reference's own test strategy turned into assertions (its test/test_op.py
and test/test_conv.py only PRINT these figures):

* statistical: the mean of repeated quantised gradients approaches the exact
  gradient -- for qelu, the edge-value gradient of the quantised SpMM, QGCNConv
  and QSAGEConv (test_op.py:245-269, 533-562; test_conv.py:26-54, 97-134);
* memory: what a layer keeps for backward, in bytes, against the fp32
  activation it replaces (test_op.py:44-67, 333-371; test_conv.py:57-93).

Both back ends: emulated kernels always, the GPU with -m gpu."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch
import torch.nn.functional as F

import exact_amd as exact
from exact_amd import nn as xnn
from exact_amd import ops
from exact_amd.conf import config
from exact_amd.sparse import SparseTensor, gcn_norm
from exact_amd.spmm import qmatmul
from exact_amd.utils import compute_tensor_bytes


def graph(n, nnz, seed, backend, valued):
    rng = np.random.default_rng(seed)
    A = sp.coo_matrix((rng.random(nnz).astype(np.float32) + 0.5, (rng.integers(0, n, nnz), rng.integers(0, n, nnz))),
                      shape=(n, n)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    adj = SparseTensor.from_scipy(A, backend)
    return adj if valued else adj.set_value(None)


def bias_and_spread(run, ref, reps):
    """-> (relative error of one draw, relative error of the mean of `reps` draws)."""
    draws = torch.stack([run() for _ in range(reps)])
    scale = ref.norm()
    return ((draws[0] - ref).norm() / scale).item(), ((draws.mean(0) - ref).norm() / scale).item()


def test_qelu_gradient_error_shrinks_with_bits_and_repeats(backend):
    """ELU's gradient is not linear in the saved input (exp and the sign test
    act on the dequantised values), so it keeps a bias floor at low precision;
    averaging still helps, and at 8 bits the error is small."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1500, 32, generator=g).to(backend)
    dy = torch.randn(1500, 32, generator=g).to(backend)
    xr = x.clone().requires_grad_()
    F.elu(xr, 1.0).backward(dy)

    def run():
        xq = x.clone().requires_grad_()
        ops.qelu.apply(xq, 1.0, None).backward(dy)
        return xq.grad

    single, mean = bias_and_spread(run, xr.grad, 16)
    assert single > 0.01 and mean < 0.7 * single
    config.activation_compression_bits = [8]
    single8, _ = bias_and_spread(run, xr.grad, 1)
    assert single8 < 0.01


@pytest.mark.parametrize("reduce", ["sum", "mean"])
def test_edge_value_gradient_of_quantised_spmm_is_unbiased(backend, reduce):
    adj = graph(400, 3000, 1, backend, valued=True)
    g = torch.Generator().manual_seed(1)
    x = torch.randn(400, 32, generator=g).to(backend)
    dy = torch.randn(400, 32, generator=g).to(backend)

    def grad_of_values(compress):
        config.compress_activation = compress
        value = adj.storage._value.detach().clone().requires_grad_()
        qmatmul(adj.set_value(value), x.clone().requires_grad_(), reduce).backward(dy)
        config.compress_activation = True
        return value.grad

    ref = grad_of_values(False)
    single, mean = bias_and_spread(lambda: grad_of_values(True), ref, 16)
    assert single > 0.01 and mean < single / 2.5


@pytest.mark.parametrize("layer", ["gcn", "sage"])
def test_conv_layer_weight_gradients_are_unbiased(backend, layer):
    """test_conv.py:26-54, 97-134 with an assertion: INT2 activations, same
    weights, repeated backward passes against the uncompressed layer."""
    adj = graph(600, 4000, 2, backend, valued=False)
    if layer == "gcn":
        adj = gcn_norm(adj, add_self_loops=True)
    torch.manual_seed(3)
    stock = (xnn.GCNConv(32, 16, normalize=False) if layer == "gcn" else xnn.SAGEConv(32, 16)).to(backend)
    q = exact.QModule(torch.nn.ModuleList([stock])).model[0].to(backend).train()
    g = torch.Generator().manual_seed(4)
    x = torch.randn(600, 32, generator=g).to(backend)
    dy = torch.randn(600, 16, generator=g).to(backend)
    first = "weight" if layer == "gcn" else "lin_l.weight"

    def grad(compress):
        config.compress_activation = compress
        q.zero_grad()
        q(x, adj).backward(dy)
        config.compress_activation = True
        return dict(q.named_parameters())[first].grad.clone()

    ref = grad(False)
    single, mean = bias_and_spread(lambda: grad(True), ref, 16)
    assert single > 0.01 and mean < single / 2.5


def kept_bytes(fn_output):
    """Bytes of everything the autograd node of `fn_output` keeps for backward."""
    node = fn_output.grad_fn
    held = []
    kept = getattr(node, "kept", None)
    if kept is not None:
        held += [t for t in kept.quantized if isinstance(t, torch.Tensor)]
        if kept.randmat is not None:
            held.append(kept.randmat)
    held += [t for t in getattr(node, "saved_tensors", ()) if isinstance(t, torch.Tensor)]
    return compute_tensor_bytes(held)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_bytes_kept_for_backward(backend, bits):
    """What replaces the [N, G] fp32 activation: bits/8 bytes per element plus a
    bf16 scale and min per row (+ 1 pad byte); the 1-bit masks of ReLU /
    dropout; with a projection, the reduced width."""
    N, G = 1024, 128
    config.activation_compression_bits = [bits]
    x = torch.randn(N, G, device=backend, requires_grad=True)
    w = torch.randn(16, G, device=backend, requires_grad=True)
    full = 4 * N * G
    y = ops.qlinear.apply(x, w, None, None, None, None, True)
    assert kept_bytes(y) == bits * N * G // 8 + 1 + 2 * 2 * N
    assert full / kept_bytes(y) > 0.95 * 32 / (bits + 32 / G)
    relu_out = exact.QReLU().train()(x)
    assert kept_bytes(relu_out) == N * G // 8                      # vs 4 N G for the stock ReLU
    drop_out = exact.QDropout(0.5).train()(x)
    assert kept_bytes(drop_out) == N * G // 8
    fused = exact.QReLUDropout(0.5, for_consumer=False).train()(x)
    assert kept_bytes(fused) == N * G // 8                          # one joint mask for the pair
    config.kept_frac = 0.125
    k = int(0.125 * G + 0.999)
    y = ops.qlinear.apply(x, w, None, None, None, None, True)
    assert kept_bytes(y) == bits * N * k // 8 + 1 + 2 * 2 * N + 4 * G * k


def test_unused_spmm_operand_is_not_kept(backend):
    """The reference keeps a compressed copy of the dense SpMM operand in every
    case (ops.py:272-280); it is read only for the edge-value gradient."""
    adj = gcn_norm(graph(300, 2000, 5, backend, valued=False), add_self_loops=True)
    x = torch.randn(300, 64, device=backend, requires_grad=True)
    y = qmatmul(adj, x, "sum")
    assert getattr(y.grad_fn, "kept", None) is None
    config.keep_unused_spmm_operand = True
    y = qmatmul(adj, x, "sum")
    assert kept_bytes(y) == 2 * 300 * 64 // 8 + 1 + 4 * 300
