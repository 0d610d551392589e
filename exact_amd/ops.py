"""Compress / decompress API and the quantised autograd Functions.

Public names, signatures and return conventions follow the reference's
exact/exact/ops.py (quantize_activation :69, dequantize_activation :86,
input2rp :108, rp2input :122, qlinear :128, qbatch_norm :206, qspmm_sum :257,
qspmm_mean :310).  Every tensor-sized operation of the path runs in
libexact_hip.so; the GEMMs of the linear layers and the batch-norm statistics
stay with torch's ROCm libraries, as they stay with ATen in the reference.

Internally each Function keeps one `CompressedActivation` (packed codes,
bf16 scale/min, optional projection matrix and the two shapes) instead of the
reference's loose tuples, and restores the activation from it in backward.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch.amp import custom_bwd, custom_fwd
from torch.autograd.function import Function
from torch.utils.weak import WeakIdKeyDictionary

from . import _lib
from .conf import config
from .cpp_extension import _checks
from .cpp_extension import backward_func as ext_backward_func
from .cpp_extension import quantization as ext_quantization
from .cpp_extension import spmm
from .cpp_extension._checks import FLOAT_OR_HALF, check_device_tensor, ptr
from .utils import empty_cache, swap_to_cpu


def _simulated_quantize(data, bits, mn, mx):
    """config.simulate (reference ops.py:18-31): the reference's debugging
    stand-in for the kernels, plain tensor ops that keep the codes UNPACKED as
    int32 [N, G] -- min / max widened by 1e-6, uniform(-0.5, 0.5) noise from
    the torch generator, relu, round.  -> (codes, scale)."""
    levels = 2 ** bits - 1
    mn = mn - 1e-6
    mx = mx + 1e-6
    scale = levels / (mx - mn)
    out = (data - mn.view(-1, 1)) * scale.view(-1, 1)
    if config.stochastic:
        out = out + torch.empty_like(out).uniform_(-0.5, 0.5)
    return F.relu(out).round_().int(), scale


def _rows_by_features(t):
    rows = t.shape[0]
    return t.reshape(rows, math.prod(t.shape[1:]))


# ---------------------------------------------------------------------------
# quantise / dequantise
# ---------------------------------------------------------------------------
def no_scheme_compute_quantization_bits(input):  # noqa: A002
    """Reference ops.py:61-66 -> (input viewed [N, -1], bits, row min, row max)."""
    flat = _rows_by_features(input)
    lo, hi = ext_quantization.row_minmax(flat)
    return flat, config.activation_compression_bits[0], lo, hi


def quantize_and_pack(data, bits, mn, mx):
    """Two-step form with the row extrema given (reference ops.py:20-43):
    -> (packed int8 stream, fp32 scale)."""
    if config.simulate:
        return _simulated_quantize(data, bits, mn, mx)
    if type(bits) is not int:
        raise TypeError("bits must be an int")
    scale = (2 ** bits - 1) / (mx - mn)      # reciprocal() * int, as torch evaluates it
    packed = ext_quantization.pack_single_precision(data, mn, mx, scale.to(data.dtype), bits, config.stochastic)
    if config.swap:
        packed = swap_to_cpu(packed)         # reference ops.py:41-42
    return packed, scale


def dequantize_and_unpack(data, shape, bits, scale, mn):
    """Reference ops.py:46-58; scale / min may be fp32 or the bf16 tensors that
    quantize_activation returned."""
    if config.simulate:
        scale, mn = scale.to(torch.float32), mn.to(torch.float32)
        return data / scale.view(-1, 1) + mn.view(-1, 1)        # reference ops.py:47-48
    rows, feats = shape[0], math.prod(shape[1:])
    if data.device != scale.device:          # offloaded by config.swap (reference ops.py:50-51)
        data = data.to(scale.device, non_blocking=True)
    unpack = ext_quantization.unpack_bf16param if scale.dtype == torch.bfloat16 else ext_quantization.unpack_single_precision
    return unpack(data, bits, scale, mn, rows, feats)


def quantize_activation(input, scheme):  # noqa: A002
    """Reference ops.py:69-83 -> (q_input, q_bits, q_scale, q_min) with bf16
    scale / min.  Row min/max, scale, stochastic quantiser, bit packer and the
    bf16 casts are ONE kernel launch here."""
    if not config.compress_activation:
        return input, None, None, None
    if scheme:
        scheme.note_use()
    check_device_tensor(input, "input", None, FLOAT_OR_HALF)
    bits = config.activation_compression_bits[0]
    if config.simulate:
        flat = _rows_by_features(input)
        lo, hi = ext_quantization.row_minmax(flat.float())
        codes, scale = _simulated_quantize(flat, bits, lo.to(flat.dtype), hi.to(flat.dtype))
        if input.dtype == torch.float32:
            return codes, bits, scale.to(torch.bfloat16), lo.to(torch.bfloat16)
        return codes, bits, scale, lo.to(flat.dtype)
    packed, scale_bf16, min_bf16 = ext_quantization.minmax_pack(_rows_by_features(input), bits)
    if config.swap:
        packed = swap_to_cpu(packed)
    return packed, bits, scale_bf16, min_bf16


def dequantize_activation(quantized, q_input_shape):
    """Reference ops.py:86-98."""
    if not config.compress_activation:
        return quantized[0]
    packed, bits, scale, mn = quantized
    return dequantize_and_unpack(packed, q_input_shape, bits, scale, mn).view(q_input_shape)


# ---------------------------------------------------------------------------
# random projection
# ---------------------------------------------------------------------------
def _projection_matrix(D, k, device, dtype):
    if config.rp_matrix_source is not None:
        R = config.rp_matrix_source(D, k, device)
        check_device_tensor(R, "rand_matrix", 2)
        return R.to(dtype)
    if config.rp_distribution == "gaussian":
        return torch.randn((D, k), device=device, dtype=dtype) / k ** 0.5
    # reference ops.py:112-114: Rademacher entries +-1/sqrt(k)
    signs = torch.randint(2, size=(D, k), device=device, dtype=dtype)
    matrix = (2.0 * signs - 1) / k ** 0.5
    matrix._exact_sign_matrix = True     # every entry is +-c with one c: the projection kernels may work on the signs alone
    return matrix


RP_KERNEL_MAX_COLUMNS = 128      # k of exact_rp_fwd_f32 / exact_rp_bwd_f32 / exact_rp_minmax_pack_f32


def kept_columns(width):
    """k of the projection D -> k (reference ops.py:143)."""
    return int(config.kept_frac * width + 0.999)


@torch.no_grad()
def input2rp(input, kept_acts):  # noqa: A002
    """Reference ops.py:107-118 -> (dim_reduced_input [N, k], rand_matrix [D, k])."""
    assert input.dim() == 2
    check_device_tensor(input, "input", 2, FLOAT_OR_HALF)
    N, D = input.shape
    rand_matrix = _projection_matrix(D, kept_acts, input.device, input.dtype).contiguous()
    if input.dtype != torch.float32 or kept_acts > RP_KERNEL_MAX_COLUMNS:
        # fp16 activations (autocast), or more projected columns than the kernel's
        # accumulators hold: a plain library GEMM, as torch.matmul is in the reference
        return torch.matmul(input, rand_matrix), rand_matrix
    reduced = torch.empty((N, kept_acts), dtype=input.dtype, device=input.device)
    mode = ext_quantization.rp_mode(rand_matrix)
    if mode == ext_quantization.RP_FP32:
        rc = _lib.lib().exact_rp_fwd_f32(ptr(input), ptr(rand_matrix), N, D, kept_acts, ptr(reduced),
                                         _checks.stream_ptr(input))
    else:
        rc = _lib.lib().exact_rp_fwd_bf16_f32(ptr(input), ptr(ext_quantization.rp_table(rand_matrix, mode)), N, D, kept_acts, mode,
                                              ptr(reduced),
                                              _checks.stream_ptr(input))
    _lib.check(rc, "input2rp")
    return reduced, rand_matrix


@torch.no_grad()
def rp2input(dim_reduced_input, input_shape, rand_matrix):
    """Reference ops.py:121-125."""
    assert dim_reduced_input.dim() == 2
    check_device_tensor(dim_reduced_input, "dim_reduced_input", 2, FLOAT_OR_HALF)
    check_device_tensor(rand_matrix, "rand_matrix", 2, (dim_reduced_input.dtype,))
    if dim_reduced_input.dtype != torch.float32 or dim_reduced_input.shape[1] > RP_KERNEL_MAX_COLUMNS:
        return torch.matmul(dim_reduced_input, rand_matrix.t()).view(input_shape)
    N, k = dim_reduced_input.shape
    D = rand_matrix.shape[0]
    if rand_matrix.shape[1] != k:
        raise RuntimeError("rand_matrix does not match the reduced input")
    full = torch.empty((N, D), dtype=dim_reduced_input.dtype, device=dim_reduced_input.device)
    mode = ext_quantization.rp_mode(rand_matrix)
    if mode == ext_quantization.RP_FP32:
        rc = _lib.lib().exact_rp_bwd_f32(ptr(dim_reduced_input), ptr(rand_matrix), N, D, k, ptr(full),
                                         _checks.stream_ptr(dim_reduced_input))
    else:
        rc = _lib.lib().exact_rp_bwd_bf16_f32(ptr(dim_reduced_input), ptr(ext_quantization.rp_table(rand_matrix, mode)), N, D, k, mode,
                                              ptr(full),
                                              _checks.stream_ptr(dim_reduced_input))
    _lib.check(rc, "rp2input")
    return full.view(input_shape)


def project_and_quantize(input, scheme):  # noqa: A002
    """input2rp followed by quantize_activation of the result (reference
    ops.py:141-149, layers.py:153-159) -> (quantized, rand_matrix, reduced shape).
    One launch that never writes the [N, k] product where the kernel applies
    (fp32, k <= 128, compression on), bit-identical to the two calls, which
    run otherwise."""
    k = kept_columns(input.shape[1])
    fused = (config.fuse_epilogue and config.compress_activation and not config.simulate
             and input.dim() == 2 and input.dtype == torch.float32 and not torch.is_autocast_enabled()
             and 0 < k <= ext_quantization.RP_PACK_MAX_COLUMNS)
    if not fused:
        reduced, rand_matrix = input2rp(input, k)
        return quantize_activation(reduced, scheme), rand_matrix, reduced.shape
    check_device_tensor(input, "input", 2)
    rand_matrix = _projection_matrix(input.shape[1], k, input.device, input.dtype).contiguous()
    if scheme:
        scheme.note_use()
    bits = config.activation_compression_bits[0]
    packed, scale_bf16, min_bf16 = ext_quantization.rp_minmax_pack(input, rand_matrix, bits)
    if config.swap:
        packed = swap_to_cpu(packed)
    return (packed, bits, scale_bf16, min_bf16), rand_matrix, torch.Size((input.shape[0], k))


class CompressedActivation:
    """The only trace of an activation a quantised node keeps for backward:
    the packed codes with their bf16 scale/min, the projection matrix when the
    activation was projected first, and the shapes before / after projection."""

    __slots__ = ("quantized", "randmat", "full_shape", "stored_shape")

    def __init__(self, quantized, randmat, full_shape, stored_shape):
        self.quantized, self.randmat = quantized, randmat
        self.full_shape, self.stored_shape = full_shape, stored_shape

    @classmethod
    def compress(cls, x, scheme, project=True):
        """Project (when kept_frac < 1 and allowed) and quantise x
        (reference ops.py:141-149, 272-280, 326-334)."""
        if project and config.kept_frac < 1.0:
            quantized, randmat, stored_shape = project_and_quantize(x, scheme)
            return cls(quantized, randmat, x.shape, stored_shape)
        return cls(quantize_activation(x, scheme), None, x.shape, x.shape)

    @classmethod
    def adopt(cls, x, quantized, randmat, project=True):
        """Wrap a compressed copy the caller made earlier (QSAGEConv shares one
        between its aggregation and lin_r; reference ops.py:133-140)."""
        if randmat is None:
            assert (not project) or config.kept_frac == 1.0
            return cls(quantized, None, x.shape, x.shape)
        assert project and config.kept_frac < 1.0 and x.shape[1] == randmat.shape[0]
        return cls(quantized, randmat, x.shape, torch.Size([x.shape[0], randmat.shape[1]]))

    def restore(self):
        x = dequantize_activation(self.quantized, self.stored_shape)
        if self.randmat is not None:
            x = rp2input(x, self.full_shape, self.randmat)
        return x


# ---------------------------------------------------------------------------
# autograd Functions
# ---------------------------------------------------------------------------
# Inside an autocast region the reference's Functions receive fp16 copies of
# their floating-point inputs and run with autocast off (custom_fwd(cast_inputs=
# torch.float16), reference ops.py:130, 260, 313, 377, 408); so do these.
_amp_fwd = custom_fwd(device_type="cuda", cast_inputs=torch.float16)
_amp_bwd = custom_bwd(device_type="cuda")

class qlinear(Function):
    """y = x W^T + b, keeping x only in compressed form (reference ops.py:128-178)."""

    @staticmethod
    @_amp_fwd
    def forward(ctx, input, weight, bias=None, quantized=None, randmat=None, scheme=None, rp=True):  # noqa: A002
        if quantized is None:
            kept = CompressedActivation.compress(input, scheme, project=rp)
        else:
            kept = CompressedActivation.adopt(input, quantized, randmat, project=rp)
        empty_cache(config.empty_cache_threshold)
        ctx.kept, ctx.weight, ctx.bias = kept, weight, bias
        if input.dim() == 2:
            return ext_backward_func.tall_matmul(input, weight, transposed=True, bias=bias)
        return F.linear(input, weight, bias)

    @staticmethod
    @_amp_bwd
    def backward(ctx, grad_output):
        kept, ctx.kept = ctx.kept, None
        if kept.randmat is None:
            grads = ext_backward_func.linear_backward(grad_output, kept.restore(), ctx.weight, ctx.bias,
                                                      ctx.needs_input_grad[0])
        else:
            # dW = dY^T (X_r R^T) = (dY^T X_r) R^T: the [N, D] decompressed input of
            # the reference (ops.py:163-165) is never formed; only the order in
            # which fp32 sums are taken differs.
            x_r = dequantize_activation(kept.quantized, kept.stored_shape)
            grad_input = ext_backward_func.tall_matmul(grad_output, ctx.weight) if ctx.needs_input_grad[0] else None
            grad_weight = ext_backward_func.weight_gradient(grad_output, x_r).mm(kept.randmat.t())
            grads = (grad_input, grad_weight,
                     ext_backward_func.column_sums(grad_output) if ctx.bias is not None else None)
        empty_cache(config.empty_cache_threshold)
        return (*grads, None, None, None, None)


class qbatch_norm(Function):
    """Training-mode batch norm that keeps its input compressed (reference ops.py:206-254)."""

    @staticmethod
    def forward(ctx, input, running_mean, running_var, weight, bias,  # noqa: A002
                training, exponential_average_factor, eps, scheme):
        kept = CompressedActivation.compress(input, scheme, project=False)
        output, save_mean, save_invstd = ext_backward_func.native_batch_norm(
            input, weight, bias, running_mean, running_var, training, exponential_average_factor, eps)
        ctx.kept = kept
        ctx.stats = (weight, running_mean, running_var, save_mean, save_invstd, training, eps)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        weight, running_mean, running_var, save_mean, save_invstd, training, eps = ctx.stats
        x_hat = ctx.kept.restore()
        ctx.kept = None
        empty_cache(config.empty_cache_threshold)
        wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[3], ctx.needs_input_grad[4]]
        g_in, g_w, g_b = ext_backward_func.native_batch_norm_backward(
            grad_output.contiguous(), x_hat, weight, running_mean, running_var, save_mean, save_invstd, training, eps,
            wanted)
        # the device routine returns tensors for masked-out outputs too (e.g. without affine parameters)
        g_in, g_w, g_b = (g if w else None for g, w in zip((g_in, g_w, g_b), wanted))
        return g_in, None, None, g_w, g_b, None, None, None, None


def _keep_for_spmm(other, value, has_value, quantized, randmat, scheme):
    """The dense operand of A @ X is read again in backward only for the
    gradient with respect to the edge values (reference spmm.cc:65-67,
    123-125).  The reference compresses and keeps it regardless
    (ops.py:272-280, 326-334); here it is kept when that gradient is wanted
    or when the caller hands in a compressed copy.  -> (kept or None, flag)."""
    value_requires_grad = bool(has_value and value.requires_grad)
    if quantized is not None:
        return CompressedActivation.adopt(other, quantized, randmat), value_requires_grad
    if value_requires_grad or config.keep_unused_spmm_operand:
        return CompressedActivation.compress(other, scheme), value_requires_grad
    return None, value_requires_grad


class qspmm_sum(Function):
    """out = A @ X with sum aggregation (reference ops.py:257-307)."""

    @staticmethod
    @_amp_fwd
    def forward(ctx, row, rowptr, col, value, colptr, csr2csc, has_value, other,
                quantized=None, randmat=None, scheme=None):
        result = spmm.spmm_sum_fw(row, rowptr, col, value, colptr, csr2csc, other)
        ctx.kept, value_requires_grad = _keep_for_spmm(other, value, has_value, quantized, randmat, scheme)
        empty_cache(config.empty_cache_threshold)
        ctx.graph = (row, rowptr, col, value, colptr, csr2csc)
        ctx.flags = (has_value, value_requires_grad, other.requires_grad)
        return result

    @staticmethod
    @_amp_bwd
    def backward(ctx, grad_outputs):
        row, rowptr, col, value, colptr, csr2csc = ctx.graph
        has_value, value_requires_grad, mat_requires_grad = ctx.flags
        other = ctx.kept.restore() if value_requires_grad else None
        ctx.kept = None
        empty_cache(config.empty_cache_threshold)
        grad_value, grad_mat = spmm.spmm_sum_bw(row, rowptr, col, value, colptr, csr2csc, other,
                                                grad_outputs.contiguous(), has_value, value_requires_grad,
                                                mat_requires_grad)
        return None, None, None, grad_value, None, None, None, grad_mat, None, None, None


class qspmm_mean(Function):
    """out = D^-1 A @ X, mean aggregation (reference ops.py:310-371)."""

    @staticmethod
    @_amp_fwd
    def forward(ctx, row, rowptr, col, value, rowcount, colptr, csr2csc, has_value, other,
                quantized=None, randmat=None, scheme=None):
        result = spmm.spmm_mean_fw(row, rowptr, col, value, rowcount, colptr, csr2csc, other)
        ctx.kept, value_requires_grad = _keep_for_spmm(other, value, has_value, quantized, randmat, scheme)
        empty_cache(config.empty_cache_threshold)
        ctx.graph = (row, rowptr, col, value, rowcount, colptr, csr2csc)
        ctx.flags = (has_value, value_requires_grad, other.requires_grad)
        return result

    @staticmethod
    @_amp_bwd
    def backward(ctx, grad_outputs):
        row, rowptr, col, value, rowcount, colptr, csr2csc = ctx.graph
        has_value, value_requires_grad, mat_requires_grad = ctx.flags
        other = ctx.kept.restore() if value_requires_grad else None
        ctx.kept = None
        empty_cache(config.empty_cache_threshold)
        grad_value, grad_mat = spmm.spmm_mean_bw(row, rowptr, col, value, rowcount, colptr, csr2csc, other,
                                                 grad_outputs.contiguous(), has_value, value_requires_grad,
                                                 mat_requires_grad)
        return None, None, None, grad_value, None, None, None, None, grad_mat, None, None, None


def _restored_weight_gradient(grad_output, kept):
    """dW = dY^T X_hat for a compressed X (reference ops.py:163-169).  With a
    projection, dY^T (X_r R^T) = (dY^T X_r) R^T: the [N, D] decompressed input
    is never formed; only the order of the fp32 sums differs."""
    if kept.randmat is None:
        return ext_backward_func.weight_gradient(grad_output, kept.restore())
    x_r = dequantize_activation(kept.quantized, kept.stored_shape)
    return ext_backward_func.weight_gradient(grad_output, x_r).mm(kept.randmat.t())


class qsage(Function):
    """`lin_l(aggregate(x)) + lin_r(x)` of a GraphSAGE layer as ONE autograd node:
    the chain qspmm_mean -> qlinear -> qlinear -> add of the reference's
    QSAGEConv.forward (layers.py:142-149), keeping exactly what that chain keeps
    for backward (the shared compressed copy of x for lin_r, a compressed copy
    of the aggregate for lin_l) and returning the same gradients.  Being one
    node, it may place the linear maps on whichever side of the aggregation
    moves fewer bytes through the sparse product -- aggregation and the linear
    maps commute, A (X W) = (A X) W:

      backward   dX = A^T (dY W_l) + dY W_r  is computed as  (A^T dY) W_l + dY W_r
                 when out < in (config.sage_reassociate_backward): the sparse
                 product runs at width `out` instead of `in`; same numbers up to
                 the order of fp32 sums.
      forward    with a projection (kept_frac < 1) the layer needs aggregate(x)
                 only as aggregate(x) W_l^T (the output) and aggregate(x) R (the
                 copy lin_l keeps).  When k + out < in
                 (config.sage_aggregate_projected) it aggregates x [R | W_l^T] at
                 that width instead; the kept copy is then the quantised
                 aggregate of x R, equal to the reference's up to fp32 rounding
                 ahead of the quantiser.

    The second GEMM of each pair accumulates into the first one's result, so no
    separate full-tensor addition runs.  `graph` = (row, rowptr, col, value,
    rowcount, colptr, csr2csc) without a gradient for `value`; `shared` = the
    CompressedActivation of x that serves lin_r."""

    @staticmethod
    def forward(ctx, x, weight_l, bias_l, weight_r, graph, reduce, shared, scheme_l):
        row, rowptr, col, value, rowcount, colptr, csr2csc = graph
        n, cin = x.shape
        cout = weight_l.shape[0]
        k = kept_columns(cin)
        narrow = (config.sage_aggregate_projected and config.compress_activation and config.kept_frac < 1.0
                  and not config.simulate and 0 < k and k + cout < cin)
        if narrow:
            if scheme_l:
                scheme_l.note_use()
            rand_matrix = _projection_matrix(cin, k, x.device, x.dtype).contiguous()
            width = k + cout
            # The sparse product gathers rows of x [R | W_l^T]: rows padded to whole 128-byte lines, and an
            # even number of columns (a zero column if need be) so that it can gather 8 bytes per lane.
            both = x.new_zeros((cin, (width + 31) // 32 * 32))
            both[:, :k] = rand_matrix
            both[:, k:width] = weight_l.detach().t()
            aggregated = spmm.spmm_csr(rowptr, col, value, ext_backward_func.tall_matmul(x, both)[:, :width + (width & 1)], reduce)
            quantized = quantize_activation(aggregated[:, :k].contiguous(), None)
            kept_l = CompressedActivation(quantized, rand_matrix, x.shape, torch.Size((n, k)))
            out = ext_backward_func.tall_matmul(x, weight_r, transposed=True, bias=bias_l, addend=aggregated[:, k:width])
        else:
            aggregated = spmm.spmm_csr(rowptr, col, value, x, reduce)
            kept_l = CompressedActivation.compress(aggregated, scheme_l)
            out = ext_backward_func.tall_matmul(aggregated, weight_l, transposed=True, bias=bias_l)
            ext_backward_func.tall_matmul(x, weight_r, transposed=True, addend=out, into=out)
        del aggregated
        empty_cache(config.empty_cache_threshold)
        ctx.kept = (kept_l, shared)
        ctx.weights = (weight_l, weight_r, bias_l is not None)
        ctx.graph, ctx.reduce = graph, reduce
        return out

    @staticmethod
    def backward(ctx, grad_output):
        row, rowptr, col, value, rowcount, colptr, csr2csc = ctx.graph
        weight_l, weight_r, has_bias = ctx.weights
        (kept_l, shared), ctx.kept = ctx.kept, None
        grad_output = grad_output.contiguous()
        has_value = value is not None

        def transpose_product(t):
            if ctx.reduce == "sum":
                return spmm.spmm_sum_bw(row, rowptr, col, value, colptr, csr2csc, None, t, has_value, False, True)[1]
            return spmm.spmm_mean_bw(row, rowptr, col, value, rowcount, colptr, csr2csc, None, t, has_value, False,
                                     True)[1]

        grad_x = None
        if ctx.needs_input_grad[0]:
            cout, cin = weight_l.shape
            if config.sage_reassociate_backward and cout < cin:
                grad_x = ext_backward_func.tall_matmul(transpose_product(grad_output), weight_l)
            else:
                grad_x = transpose_product(ext_backward_func.tall_matmul(grad_output, weight_l))
            ext_backward_func.tall_matmul(grad_output, weight_r, addend=grad_x, into=grad_x)
        grad_wl = _restored_weight_gradient(grad_output, kept_l) if ctx.needs_input_grad[1] else None
        del kept_l
        grad_wr = _restored_weight_gradient(grad_output, shared) if ctx.needs_input_grad[3] else None
        del shared
        grad_b = ext_backward_func.column_sums(grad_output) if (has_bias and ctx.needs_input_grad[2]) else None
        empty_cache(config.empty_cache_threshold)
        return grad_x, grad_wl, grad_b, grad_wr, None, None, None, None


class qgcn(Function):
    """`aggregate(x W^T) + b` of a GCN layer as ONE autograd node: the chain
    qlinear -> qspmm_sum -> bias add of the reference's QGCNConv.forward
    (layers.py:244-262), keeping exactly what that chain keeps for backward
    (the compressed copy of x that serves the weight gradient) and returning
    the same gradients.  Aggregation and the linear map commute,
    A (X W^T) = (A X) W^T, so the node runs the sparse product on the narrower
    side (config.gcn_aggregate_narrow):

      forward   in < out: (A X) W^T + b, the bias folded into the GEMM;
                otherwise A (X W^T) + b as in the reference.
      backward  G = A^T dY serves both dX = G W and dW = G^T X_hat.  Where dX is
                not wanted (the first layer) and the kept copy is narrower
                than `out`, dW = dY^T (A X_hat) instead: the sparse product
                runs on the restored (still projected) copy.

    Same numbers up to the order of fp32 sums.  `graph` = (row, rowptr, col,
    value, rowcount, colptr, csr2csc) without a gradient for `value`; `kept` =
    the CompressedActivation of x."""

    @staticmethod
    def forward(ctx, x, weight, bias, graph, reduce, kept):
        row, rowptr, col, value, rowcount, colptr, csr2csc = graph
        cout, cin = weight.shape
        if config.gcn_aggregate_narrow and cin < cout:
            aggregated = spmm.spmm_csr(rowptr, col, value, x, reduce)
            out = ext_backward_func.tall_matmul(aggregated, weight, transposed=True, bias=bias)
            del aggregated
        else:
            out = spmm.spmm_csr(rowptr, col, value, ext_backward_func.tall_matmul(x, weight, transposed=True), reduce)
            if bias is not None:
                out += bias
        empty_cache(config.empty_cache_threshold)
        ctx.kept, ctx.weight, ctx.has_bias = kept, weight, bias is not None
        ctx.graph, ctx.reduce = graph, reduce
        return out

    @staticmethod
    def backward(ctx, grad_output):
        row, rowptr, col, value, rowcount, colptr, csr2csc = ctx.graph
        weight = ctx.weight
        kept, ctx.kept = ctx.kept, None
        grad_output = grad_output.contiguous()
        has_value = value is not None
        cout = weight.shape[0]
        grad_x = grad_w = None
        stored_width = kept.stored_shape[1]
        if not ctx.needs_input_grad[0] and ctx.needs_input_grad[1] and config.gcn_aggregate_narrow and stored_width < cout:
            # dW = dY^T (A X_hat); with a projection X_hat = X_r R^T and the sparse product runs on X_r
            x_r = dequantize_activation(kept.quantized, kept.stored_shape)
            grad_w = ext_backward_func.weight_gradient(grad_output, spmm.spmm_csr(rowptr, col, value, x_r, ctx.reduce))
            if kept.randmat is not None:
                grad_w = grad_w.mm(kept.randmat.t())
        else:
            if ctx.reduce == "sum":
                g = spmm.spmm_sum_bw(row, rowptr, col, value, colptr, csr2csc, None, grad_output, has_value, False, True)[1]
            else:
                g = spmm.spmm_mean_bw(row, rowptr, col, value, rowcount, colptr, csr2csc, None, grad_output, has_value,
                                      False, True)[1]
            if ctx.needs_input_grad[0]:
                grad_x = ext_backward_func.tall_matmul(g, weight)
            if ctx.needs_input_grad[1]:
                grad_w = _restored_weight_gradient(g, kept)
        del kept
        grad_b = ext_backward_func.column_sums(grad_output) if (ctx.has_bias and ctx.needs_input_grad[2]) else None
        empty_cache(config.empty_cache_threshold)
        return grad_x, grad_w, grad_b, None, None, None


class qelu(Function):
    """ELU that keeps its input compressed (reference ops.py:182-204)."""

    @staticmethod
    def forward(ctx, input, alpha, scheme=None):  # noqa: A002
        ctx.kept = CompressedActivation.compress(input, scheme, project=False)
        ctx.alpha = alpha
        empty_cache(config.empty_cache_threshold)
        return F.elu(input, alpha)

    @staticmethod
    def backward(ctx, grad_output):
        x_hat = ctx.kept.restore()
        ctx.kept = None
        empty_cache(config.empty_cache_threshold)
        return ext_backward_func._elu_backward_cuda(grad_output, x_hat, ctx.alpha), None, None


def _extreme_forward(ctx, is_max, rowptr, col, value, has_value, other, quantized, scheme):
    """Shared forward of qspmm_max / qspmm_min (reference ops.py:374-436).  The
    dense operand is read again in backward only for the edge-value gradient,
    so it is compressed and kept only then (or when the caller supplies it)."""
    fw = spmm.spmm_max_fw if is_max else spmm.spmm_min_fw
    output, arg_out = fw(rowptr, col, value, other)
    value_requires_grad = bool(has_value and value.requires_grad)
    if quantized is not None:
        assert isinstance(quantized, tuple)
        kept = CompressedActivation(quantized, None, other.shape, other.shape)
    elif value_requires_grad or config.keep_unused_spmm_operand:
        kept = CompressedActivation.compress(other, scheme, project=False)
    else:
        kept = None
    empty_cache(config.empty_cache_threshold)
    ctx.kept, ctx.graph, ctx.operand_shape = kept, (col, value, arg_out), other.shape
    ctx.flags = (has_value, value_requires_grad, other.requires_grad)
    ctx.mark_non_differentiable(arg_out)
    return output


def _extreme_backward(ctx, grad_outputs):
    col, value, arg_out = ctx.graph
    has_value, value_requires_grad, mat_requires_grad = ctx.flags
    if value_requires_grad:
        other = ctx.kept.restore()
    else:  # only the operand's shape is needed to size grad_mat
        other = grad_outputs.new_empty(ctx.operand_shape)
    ctx.kept = None
    empty_cache(config.empty_cache_threshold)
    grad_value, grad_mat = spmm.spmm_max_bw(col, value, other, arg_out, grad_outputs.contiguous(), has_value,
                                            value_requires_grad, mat_requires_grad)
    return None, None, grad_value, None, grad_mat, None, None, None


class qspmm_max(Function):
    """out = max over the entries of each row of val * X[col]  (reference ops.py:374-403)."""

    @staticmethod
    @_amp_fwd
    def forward(ctx, rowptr, col, value, has_value, other, quantized=None, randmat=None, scheme=None):
        return _extreme_forward(ctx, True, rowptr, col, value, has_value, other, quantized, scheme)

    @staticmethod
    @_amp_bwd
    def backward(ctx, grad_outputs):
        return _extreme_backward(ctx, grad_outputs)


class qspmm_min(Function):
    """Reference ops.py:406-436; gradients are routed as for max (spmm.cc:214-241)."""

    @staticmethod
    @_amp_fwd
    def forward(ctx, rowptr, col, value, has_value, other, quantized=None, randmat=None, scheme=None):
        return _extreme_forward(ctx, False, rowptr, col, value, has_value, other, quantized, scheme)

    @staticmethod
    @_amp_bwd
    def backward(ctx, grad_outputs):
        return _extreme_backward(ctx, grad_outputs)


# ---------------------------------------------------------------------------
# fused epilogue: ReLU -> dropout -> compressed copy for the consumer
# ---------------------------------------------------------------------------
class qrelu_dropout(Function):
    """dropout(relu(input)) in one pass with one joint 1-bit mask kept for
    backward -- the pair QReLU -> QDropout of the reference (layers.py:284-325).
    With `bits`, the same pass also quantises the result the way the next
    layer's quantize_activation would (ops.py:69-83) and returns that copy:
    -> (output, packed | None, scale bf16 | None, min bf16 | None)."""

    @staticmethod
    def forward(ctx, input, p, bits=None):  # noqa: A002
        flat = _rows_by_features(input) if input.dim() >= 2 else input
        if bits is None:
            out, mask = ext_quantization.relu_dropout_fwd(flat, p)
            packed = scale = mn = None
        else:
            out, mask, packed, scale, mn = ext_quantization.relu_dropout_minmax_pack(flat, p, bits)
            ctx.mark_non_differentiable(packed, scale, mn)
        ctx.save_for_backward(mask)
        ctx.p = float(p)
        return out.view(input.shape), packed, scale, mn

    @staticmethod
    def backward(ctx, grad_output, *unused):
        (mask,) = ctx.saved_tensors
        return ext_quantization.dropout_bwd(grad_output, mask, ctx.p), None, None


class qbn_relu_dropout(Function):
    """Training-mode batch norm -> ReLU -> dropout, the chain QBatchNorm1d ->
    QReLU -> QDropout of the reference (layers.py:340-369, 284-325; ops.py:206-254),
    in two passes over the input instead of six: the batch norm's compressed
    copy of its input (ops.py:213), the batch statistics, and then ONE pass that
    normalises, applies ReLU and dropout with one joint mask and quantises the
    result for the following layer.  Backward: the joint mask, then
    native_batch_norm_backward on the dequantised input as in ops.py:228-254.
    -> (output, packed, scale bf16, min bf16)."""

    @staticmethod
    def forward(ctx, input, running_mean, running_var, weight, bias,  # noqa: A002
                exponential_average_factor, eps, p, bits, scheme):
        kept = CompressedActivation.compress(input, scheme, project=False)
        rows = input.shape[0]
        var, mean = ext_backward_func.batch_statistics(input)
        invstd = torch.rsqrt(var + eps)
        if running_mean is not None:                       # the bookkeeping of native_batch_norm
            running_mean.mul_(1 - exponential_average_factor).add_(mean, alpha=exponential_average_factor)
            running_var.mul_(1 - exponential_average_factor).add_(var * (rows / max(rows - 1, 1)),
                                                                   alpha=exponential_average_factor)
        mult = invstd if weight is None else weight * invstd
        shift = torch.zeros_like(mean) if bias is None else bias.detach()
        out, mask, packed, scale, mn = ext_quantization.bn_relu_dropout_minmax_pack(
            input, mean, mult.contiguous(), shift.contiguous(), p, bits)
        ctx.mark_non_differentiable(packed, scale, mn)
        ctx.save_for_backward(mask)
        ctx.kept = kept
        ctx.stats = (weight, running_mean, running_var, mean, invstd, eps)
        ctx.p = float(p)
        return out, packed, scale, mn

    @staticmethod
    def backward(ctx, grad_output, *unused):
        (mask,) = ctx.saved_tensors
        weight, running_mean, running_var, save_mean, save_invstd, eps = ctx.stats
        grad_normalised = ext_quantization.dropout_bwd(grad_output, mask, ctx.p)
        x_hat = ctx.kept.restore()
        ctx.kept = None
        empty_cache(config.empty_cache_threshold)
        wanted = [ctx.needs_input_grad[0], ctx.needs_input_grad[3], ctx.needs_input_grad[4]]
        g_in, g_w, g_b = ext_backward_func.native_batch_norm_backward(
            grad_normalised, x_hat, weight, running_mean, running_var, save_mean, save_invstd, True, eps, wanted)
        g_in, g_w, g_b = (g if w else None for g, w in zip((g_in, g_w, g_b), wanted))
        return g_in, None, None, g_w, g_b, None, None, None, None, None


# Compressed copies made ahead of their consumer, keyed by the tensor they
# describe.  The entry dies with the tensor; `_version` guards against an
# in-place change between producer and consumer.
_HANDED_OVER = WeakIdKeyDictionary()  # keyed by identity: Tensor.__eq__ is elementwise


def hand_over_compressed(tensor, quantized):
    _HANDED_OVER[tensor] = (tensor._version, quantized)


def take_compressed(tensor, project=True):
    """The compressed copy a fused producer made of exactly this tensor for a
    consumer that would call quantize_activation(tensor) itself, or None."""
    entry = _HANDED_OVER.pop(tensor, None) if isinstance(tensor, torch.Tensor) else None
    if entry is None:
        return None
    version, quantized = entry
    usable = (config.compress_activation and version == tensor._version and not torch.is_autocast_enabled()
              and quantized[1] == config.activation_compression_bits[0]
              and not (project and config.kept_frac < 1.0))
    return quantized if usable else None


def consumer_bits(input, for_consumer):  # noqa: A002
    """Bit width of the compressed copy the fused pass can make of its result for
    the next layer, or None where it cannot (needs 2-D fp32 rows of a multiple
    of 8 <= 1024 columns, compression on, no projection, no autocast)."""
    if (for_consumer and config.compress_activation and config.kept_frac == 1.0 and input.dim() == 2
            and input.dtype == torch.float32 and not torch.is_autocast_enabled()
            and not config.simulate and ext_quantization.fusable_width(input.shape[1])):
        return config.activation_compression_bits[0]
    return None


def bn_relu_dropout(input, norm, exponential_average_factor, p, bits):  # noqa: A002
    """dropout(relu(batch_norm(input))) in training mode through qbn_relu_dropout;
    `bits` from consumer_bits(input, True) (not None), at least two rows.
    `norm` supplies running statistics, affine parameters, eps and scheme of a
    QBatchNorm1d; the compressed copy of the result is handed over to the layer
    that receives it."""
    check_device_tensor(input, "input", 2)
    running = (norm.running_mean, norm.running_var) if norm.track_running_stats else (None, None)
    out, packed, scale, mn = qbn_relu_dropout.apply(input, *running, norm.weight, norm.bias,
                                                    exponential_average_factor, norm.eps, p, bits, norm.scheme)
    hand_over_compressed(out, (swap_to_cpu(packed) if config.swap else packed, bits, scale, mn))
    return out


def relu_dropout(input, p, for_consumer=False):  # noqa: A002
    """dropout(relu(input)); with `for_consumer`, the compressed copy of the
    result is made in the same pass where the kernel can (2-D rows of a
    multiple of 8 <= 1024 columns, compression on, no projection) and handed
    over to the layer that receives the result."""
    check_device_tensor(input, "input", None, FLOAT_OR_HALF)
    bits = consumer_bits(input, for_consumer)
    out, packed, scale, mn = qrelu_dropout.apply(input, p, bits)
    if bits is not None:
        hand_over_compressed(out, (swap_to_cpu(packed) if config.swap else packed, bits, scale, mn))
    return out
