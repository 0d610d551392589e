"""CPU restatement of the reference's quantised layers and of the two
full-batch models built from them (TEST INFRASTRUCTURE ONLY, see the header of
exact_oracle.py).  torch-CPU autograd Functions whose saved state goes through
the NumPy oracle, in the reference's order of operations:

  qlinear        exact/exact/ops.py:128-178        (+ backward_func.cc:83-93)
  qbatch_norm    exact/exact/ops.py:206-254
  qspmm sum/mean exact/exact/ops.py:257-371, spmm.cc:57-79,115-139
  ReLU / dropout quantization.cc:66-84, 111-134
  QGCNConv / QSAGEConv / GCN / SAGE   layers.py:123-178,215-265;
                                      mem_speed_bench/models/gcn.py:54-61, sage.py:56-78

Noise and projection matrices are drawn from the `noise` / `rp_matrix`
callables handed in, in the same call order as the product (one draw per
quantize_activation, per dropout and per input2rp)."""
import numpy as np
import torch
import torch.nn.functional as F

import exact_oracle as o


class _Native:
    """The element-wise and sparse pieces through the C restatement
    (exact_oracle.c), which tests/test_oracle.py holds bit for bit to the NumPy
    functions of the same name: the only way to run a model of benchmark size
    on the CPU in seconds.  Same signatures as the NumPy module."""

    def __init__(self):
        import c_oracle
        self.c = c_oracle

    def quantize_activation(self, x, bits, noise):
        x2 = np.ascontiguousarray(x, dtype=np.float32).reshape(x.shape[0], -1)
        mn, mx = self.c.row_minmax(x2)
        scale = self.c.scale(mn, mx, bits)
        packed = self.c.pack(x2, mn, scale, bits, noise)
        return packed, bits, o.bf16_round(scale)[0], o.bf16_round(mn)[0], scale, mn

    def dequantize_activation(self, packed, bits, scale_bf16_bits, min_bf16_bits, shape):
        scale = (np.asarray(scale_bf16_bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
        mn = (np.asarray(min_bf16_bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
        return self.c.unpack(packed, bits, scale, mn, shape[0], int(np.prod(shape[1:]))).reshape(shape)

    def relu_fwd(self, x):
        y, mask = self.c.relu_fwd(x)
        return y.reshape(np.shape(x)), mask

    def relu_bwd(self, dy, mask):
        return self.c.relu_bwd(dy, mask).reshape(np.shape(dy))

    def dropout_fwd(self, x, p, noise):
        y, mask = self.c.dropout_fwd(x, p, noise)
        return y.reshape(np.shape(x)), mask

    def dropout_bwd(self, dy, mask, p):
        return self.c.dropout_bwd(dy, mask, p).reshape(np.shape(dy))

    def spmm_csr(self, rowptr, col, val, X, reduce="sum"):
        return self.c.spmm_csr(rowptr, col, val, X, reduce)

    def spmm_sum_bw(self, row, colptr, csr2csc, val, dY):
        v = None if val is None else np.asarray(val, dtype=np.float32)[csr2csc]
        return self.c.spmm_csr(colptr, row[csr2csc], v, dY, "sum")

    def spmm_mean_bw(self, row, rowcount, colptr, csr2csc, val, dY):
        r = row[csr2csc]
        cnt = np.maximum(np.asarray(rowcount)[r].astype(np.float32), np.float32(1.0))
        w = (np.float32(1.0) / cnt).astype(np.float32) if val is None else \
            (np.asarray(val, dtype=np.float32)[csr2csc] / cnt).astype(np.float32)
        return self.c.spmm_csr(colptr, r, w, dY, "sum")


_impl = o          # the module whose functions the classes below call: the NumPy oracle, or _Native()


def use_native(on=True):
    """Route quantise / dequantise / masks / SpMM through the C restatement."""
    global _impl
    _impl = _Native() if on else o


class Ctx:
    """What the reference keeps in exact.config plus the random sources."""

    def __init__(self, bits=2, kept_frac=1.0, noise=None, rp_matrix=None):
        self.bits, self.kept_frac, self.noise, self.rp_matrix = bits, kept_frac, noise, rp_matrix

    def quantize(self, x):                                   # ops.py:69-83
        x2 = x.detach().numpy().reshape(x.shape[0], -1)
        u = self.noise(x2.shape).numpy()
        packed, bits, sbf, mbf, _, _ = _impl.quantize_activation(x2, self.bits, u)
        return packed, bits, sbf, mbf

    def dequantize(self, q, shape):                          # ops.py:86-98
        return torch.from_numpy(_impl.dequantize_activation(q[0], q[1], q[2], q[3], tuple(shape)))

    def compress(self, x):                                   # ops.py:141-149
        if self.kept_frac < 1.0:
            k = o.kept_acts(self.kept_frac, x.shape[1])
            R = self.rp_matrix(x.shape[1], k)
            xr = torch.from_numpy(o.input2rp(x.detach().numpy(), R.numpy()))
            return self.quantize(xr), R, xr.shape
        return self.quantize(x), None, x.shape

    def decompress(self, q, R, proj_shape, ori_shape):       # ops.py:163-165
        x = self.dequantize(q, proj_shape)
        if R is not None:
            x = torch.from_numpy(o.rp2input(x.numpy(), R.numpy())).view(ori_shape)
        return x


class QLinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, c, x, weight, bias, quantized, R, proj_shape):
        if quantized is None:
            quantized, R, proj_shape = c.compress(x)
        ctx.c, ctx.saved = c, (quantized, R, proj_shape, x.shape, weight, bias)
        return F.linear(x, weight, bias)

    @staticmethod
    def backward(ctx, g):
        quantized, R, proj_shape, ori_shape, weight, bias = ctx.saved
        x = ctx.c.decompress(quantized, R, proj_shape, ori_shape)
        return None, g.mm(weight), g.t().mm(x), (g.sum(0) if bias is not None else None), None, None, None


class QBatchNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, c, x, running_mean, running_var, weight, bias, momentum, eps):
        quantized = c.quantize(x)
        out, save_mean, save_invstd = torch.ops.aten.native_batch_norm(x, weight, bias, running_mean, running_var,
                                                                       True, momentum, eps)
        ctx.c, ctx.saved = c, (quantized, x.shape, weight, running_mean, running_var, save_mean, save_invstd, eps)
        return out

    @staticmethod
    def backward(ctx, g):
        quantized, shape, weight, rm, rv, save_mean, save_invstd, eps = ctx.saved
        x = ctx.c.dequantize(quantized, shape)
        gi, gw, gb = torch.ops.aten.native_batch_norm_backward(g.contiguous(), x, weight, rm, rv, save_mean,
                                                               save_invstd, True, eps, [True, True, True])
        return None, gi, None, None, gw, gb, None, None


class ReLUFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        y, mask = _impl.relu_fwd(x.detach().numpy())
        ctx.mask = mask
        return torch.from_numpy(y)

    @staticmethod
    def backward(ctx, g):
        return torch.from_numpy(_impl.relu_bwd(g.contiguous().numpy(), ctx.mask))


class DropoutFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, c, x, p):
        u = c.noise(tuple(x.shape)).numpy()
        y, mask = _impl.dropout_fwd(x.detach().numpy(), p, u)
        ctx.mask, ctx.p = mask, p
        return torch.from_numpy(y)

    @staticmethod
    def backward(ctx, g):
        return None, torch.from_numpy(_impl.dropout_bwd(g.contiguous().numpy(), ctx.mask, ctx.p)), None


class Graph:
    """CSR arrays + the cached transpose, as NumPy."""

    def __init__(self, rowptr, col, value):
        self.rowptr, self.col = np.asarray(rowptr, np.int64), np.asarray(col, np.int64)
        self.value = None if value is None else np.asarray(value, np.float32)
        self.n = self.rowptr.size - 1
        self.row, self.colptr, self.csr2csc = o.csr_transpose(self.rowptr, self.col, self.n)
        self.rowcount = np.diff(self.rowptr)


class SpMMFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, x, reduce):
        ctx.g, ctx.reduce = g, reduce
        return torch.from_numpy(_impl.spmm_csr(g.rowptr, g.col, g.value, x.detach().numpy(), reduce))

    @staticmethod
    def backward(ctx, grad):
        g, dY = ctx.g, grad.contiguous().numpy()
        if ctx.reduce == "sum":
            out = _impl.spmm_sum_bw(g.row, g.colptr, g.csr2csc, g.value, dY)
        else:
            out = _impl.spmm_mean_bw(g.row, g.rowcount, g.colptr, g.csr2csc, g.value, dY)
        return None, torch.from_numpy(out), None


def gcn_forward(c, params, graph, x, dropout_p, batch_norm=True, bn_state=None):
    """mem_speed_bench/models/gcn.py:54-61 over QGCNConv (layers.py:226-262):
    qlinear (no bias) -> sum SpMM -> + bias, then BN -> ReLU -> dropout."""
    n_layers = len(params["conv_w"])
    for i in range(n_layers):
        h = QLinearFn.apply(c, x, params["conv_w"][i], None, None, None, None)
        h = SpMMFn.apply(graph, h, "sum")
        if params["conv_b"][i] is not None:
            h = h + params["conv_b"][i]
        if i == n_layers - 1:
            return h
        if batch_norm:
            rm, rv = bn_state[i] if bn_state is not None else (None, None)
            h = QBatchNormFn.apply(c, h, rm, rv, params["bn_w"][i], params["bn_b"][i], 0.1, 1e-5)
        x = ReLUFn.apply(h)
        x = DropoutFn.apply(c, x, dropout_p)


def sage_forward(c, params, graph, x, dropout_p, batch_norm=False, bn_state=None):
    """mem_speed_bench/models/sage.py:56-78 over QSAGEConv (layers.py:142-178):
    the input is compressed once and shared by the mean SpMM and lin_r; lin_l
    compresses the aggregated tensor itself."""
    n_layers = len(params["lin_l_w"])
    for i in range(n_layers):
        quantized, R, proj_shape = c.compress(x)
        agg = SpMMFn.apply(graph, x, "mean")
        h = QLinearFn.apply(c, agg, params["lin_l_w"][i], params["lin_l_b"][i], None, None, None)
        h = h + QLinearFn.apply(c, x, params["lin_r_w"][i], None, quantized, R, proj_shape)
        if i == n_layers - 1:
            return h
        if batch_norm:
            rm, rv = bn_state[i] if bn_state is not None else (None, None)
            h = QBatchNormFn.apply(c, h, rm, rv, params["bn_w"][i], params["bn_b"][i], 0.1, 1e-5)
        x = ReLUFn.apply(h)
        x = DropoutFn.apply(c, x, dropout_p)
