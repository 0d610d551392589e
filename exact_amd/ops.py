"""Compress / decompress API and the quantised autograd Functions.

Same names, signatures and return conventions as the reference's
exact/exact/ops.py (quantize_activation :69, dequantize_activation :86,
input2rp :108, rp2input :122, qlinear :128, qbatch_norm :206, qspmm_sum :257,
qspmm_mean :310).  Every tensor-sized operation of the path runs in
libexact_hip.so; GEMMs of the linear layers and batch-norm statistics stay
with torch's ROCm libraries, as they stay with ATen in the reference.
"""
from __future__ import annotations

import numpy as np
import torch
import torch.nn.functional as F
from torch.autograd.function import Function

from . import _lib
from .conf import config
from .cpp_extension import backward_func as ext_backward_func
from .cpp_extension import quantization as ext_quantization
from .cpp_extension import spmm
from .cpp_extension import _checks
from .cpp_extension._checks import check_device_tensor, ptr
from .utils import empty_cache, swap_to_cpu


# ---------------------------------------------------------------------------
# quantise / dequantise
# ---------------------------------------------------------------------------
def quantize_and_pack(data, bits, mn, mx):
    """ops.py:20-43 of the reference (two-step form: min / max given)."""
    if config.simulate:
        B = 2 ** bits - 1
        mn = mn - 1e-6
        mx = mx + 1e-6
        scale = B / (mx - mn)
        output = (data - mn.view(-1, 1)) * scale.view(-1, 1)
        if config.stochastic:
            noise = output.new(output.shape).uniform_(-0.5, 0.5)
            output.add_(noise)
        output = F.relu(output)
        output = output.round_().int()
    else:
        assert type(bits) == int
        scale = (2 ** bits - 1) / (mx - mn)
        output = ext_quantization.pack_single_precision(data, mn, mx, scale.to(data.dtype), bits, config.stochastic)
        if config.swap:
            output = swap_to_cpu(output)
    return output, scale


def dequantize_and_unpack(data, shape, bits, scale, mn):
    """ops.py:46-58."""
    if config.simulate:
        data = data / scale.view(-1, 1) + mn.view(-1, 1)
    else:
        if config.swap:
            data = data.cuda()
        N = shape[0]
        num_features = int(np.prod(shape[1:]))
        assert type(bits) == int
        if scale.dtype == torch.bfloat16:
            data = ext_quantization.unpack_bf16param(data, bits, scale, mn, N, num_features)
        else:
            data = ext_quantization.unpack_single_precision(data, bits, scale, mn, N, num_features)
    return data


def no_scheme_compute_quantization_bits(input):  # noqa: A002
    """ops.py:61-66."""
    N = input.shape[0]
    input_flatten = input.view(N, -1)
    mn, mx = ext_quantization.row_minmax(input_flatten)
    b = config.activation_compression_bits[0]
    return input_flatten, b, mn, mx


def quantize_activation(input, scheme):  # noqa: A002
    """ops.py:69-83 -> (q_input, q_bits, q_scale, q_min); bf16 scale / min for
    fp32 inputs.  The min/max reductions, the scale, the quantiser, the packer
    and the bf16 casts are one kernel launch here."""
    if not config.compress_activation:
        if config.swap:
            input = swap_to_cpu(input)  # noqa: A001
        return input, None, None, None
    if config.simulate:
        if scheme:
            input_groups, q_bits, q_min, mx = scheme.compute_quantization_bits(input)
        else:
            input_groups, q_bits, q_min, mx = no_scheme_compute_quantization_bits(input)
        q_input, q_scale = quantize_and_pack(input_groups, q_bits, q_min, mx)
        return q_input, q_bits, q_scale.to(torch.bfloat16), q_min.to(torch.bfloat16)
    if scheme:
        scheme.note_use()
    check_device_tensor(input, "input")
    N = input.shape[0]
    q_bits = config.activation_compression_bits[0]
    q_input, q_scale, q_min = ext_quantization.minmax_pack(input.reshape(N, input[0].numel() if N else int(np.prod(input.shape[1:]))), q_bits)
    if config.swap:
        q_input = swap_to_cpu(q_input)
    return q_input, q_bits, q_scale, q_min


def dequantize_activation(quantized, q_input_shape):
    """ops.py:86-98."""
    if not config.compress_activation:
        ret = quantized[0]
        if config.swap:
            ret = ret.cuda(non_blocking=True)
        return ret
    q_input, q_bits, q_scale, q_min = quantized
    if config.simulate and q_scale.dtype == torch.bfloat16:
        q_scale = q_scale.to(torch.float32)
        q_min = q_min.to(torch.float32)
    input = dequantize_and_unpack(q_input, q_input_shape, q_bits, q_scale, q_min)  # noqa: A001
    return input.view(q_input_shape).contiguous()


# ---------------------------------------------------------------------------
# random projection
# ---------------------------------------------------------------------------
def _gen_rand_matrix(D, k, device, dtype):
    if config.rp_matrix_source is not None:
        R = config.rp_matrix_source(D, k, device)
        check_device_tensor(R, "rand_matrix", 2)
        return R
    if config.rp_distribution == "gaussian":
        return torch.randn((D, k), device=device, dtype=dtype) / k ** 0.5
    # ops.py:112-114: Rademacher entries +-1/sqrt(k)
    bern = torch.randint(2, size=(D, k), device=device, requires_grad=False, dtype=dtype)
    return (2.0 * bern - 1) / k ** 0.5


@torch.no_grad()
def input2rp(input, kept_acts):  # noqa: A002
    """ops.py:107-118 -> (dim_reduced_input [N, k], rand_matrix [D, k])."""
    assert len(input.size()) == 2
    check_device_tensor(input, "input", 2)
    N, D = input.shape
    rand_matrix = _gen_rand_matrix(D, kept_acts, input.device, input.dtype).contiguous()
    out = torch.empty((N, kept_acts), dtype=input.dtype, device=input.device)
    rc = _lib.lib().exact_rp_fwd_f32(ptr(input), ptr(rand_matrix), N, D, kept_acts, ptr(out), _checks.stream_ptr(input))
    _lib.check(rc, "input2rp")
    return out, rand_matrix


@torch.no_grad()
def rp2input(dim_reduced_input, input_shape, rand_matrix):
    """ops.py:121-125."""
    assert len(dim_reduced_input.size()) == 2
    check_device_tensor(dim_reduced_input, "dim_reduced_input", 2)
    check_device_tensor(rand_matrix, "rand_matrix", 2)
    N, k = dim_reduced_input.shape
    D = rand_matrix.shape[0]
    if rand_matrix.shape[1] != k:
        raise RuntimeError("rand_matrix does not match the reduced input")
    out = torch.empty((N, D), dtype=dim_reduced_input.dtype, device=dim_reduced_input.device)
    rc = _lib.lib().exact_rp_bwd_f32(ptr(dim_reduced_input), ptr(rand_matrix), N, D, k, ptr(out),
                                     _checks.stream_ptr(dim_reduced_input))
    _lib.check(rc, "rp2input")
    return out.view(input_shape)


def _compress(x, scheme):
    """Shared front half of the Functions below (ops.py:141-149, 272-280,
    326-334): optional projection, then quantise."""
    if config.kept_frac < 1.0:
        kept_acts = int(config.kept_frac * x.shape[1] + 0.999)
        reduced, randmat = input2rp(x, kept_acts)
        proj_shape = reduced.shape
    else:
        reduced, randmat = x, None
        proj_shape = x.shape
    return quantize_activation(reduced, scheme), randmat, x.shape, proj_shape


# ---------------------------------------------------------------------------
# autograd Functions
# ---------------------------------------------------------------------------
class qlinear(Function):
    """ops.py:128-178."""

    @staticmethod
    def forward(ctx, input, weight, bias=None, quantized=None, randmat=None, scheme=None, rp=True):  # noqa: A002
        if quantized is not None:
            if randmat is None:
                assert rp is False or config.kept_frac == 1.0
                ori_input_shape, proj_input_shape = input.shape, input.shape
            else:
                assert (rp is True and config.kept_frac < 1.0) and (input.shape[1] == randmat.shape[0])
                ori_input_shape, proj_input_shape = input.shape, torch.Size([input.shape[0], randmat.shape[1]])
        else:
            if config.kept_frac < 1.0 and rp:
                quantized, randmat, ori_input_shape, proj_input_shape = _compress(input, scheme)
            else:
                randmat = None
                ori_input_shape, proj_input_shape = input.shape, input.shape
                quantized = quantize_activation(input, scheme)

        empty_cache(config.empty_cache_threshold)
        ctx.scheme = scheme
        ctx.saved = quantized, weight, bias, randmat
        ctx.other_args = ori_input_shape, proj_input_shape, rp
        return F.linear(input, weight, bias)

    @staticmethod
    def backward(ctx, grad_output):
        quantized, weight, bias, randmat = ctx.saved
        ori_input_shape, q_input_shape, rp = ctx.other_args
        input = dequantize_activation(quantized, q_input_shape)  # noqa: A001
        if config.kept_frac < 1.0 and rp:
            input = rp2input(input, ori_input_shape, randmat)  # noqa: A001
        del quantized, ctx.saved
        empty_cache(config.empty_cache_threshold)
        grad_input, grad_weight, grad_bias = ext_backward_func.linear_backward(grad_output, input, weight, bias)
        del input, grad_output
        empty_cache(config.empty_cache_threshold)
        return grad_input, grad_weight, grad_bias, None, None, None, None


class qbatch_norm(Function):
    """ops.py:206-254."""

    @staticmethod
    def forward(ctx, input, running_mean, running_var, weight, bias,  # noqa: A002
                training, exponential_average_factor, eps, scheme):
        quantized = quantize_activation(input, scheme)
        output, save_mean, save_var = ext_backward_func.native_batch_norm(
            input, weight, bias, running_mean, running_var, training, exponential_average_factor, eps)
        ctx.scheme = scheme
        ctx.other_args = input.shape
        ctx.saved = (quantized, weight, running_mean, running_var, save_mean, save_var, training, eps)
        return output

    @staticmethod
    def backward(ctx, grad_output):
        quantized, weight, running_mean, running_var, save_mean, save_var, training, eps = ctx.saved
        q_input_shape = ctx.other_args
        input = dequantize_activation(quantized, q_input_shape)  # noqa: A001
        del quantized, ctx.saved
        empty_cache(config.empty_cache_threshold)
        grad_input, grad_weight, grad_bias = ext_backward_func.native_batch_norm_backward(
            grad_output.contiguous(), input, weight, running_mean, running_var, save_mean, save_var, training, eps,
            [ctx.needs_input_grad[0], ctx.needs_input_grad[3], ctx.needs_input_grad[4]])
        return grad_input, None, None, grad_weight, grad_bias, None, None, None, None


def _spmm_saved_shapes(other, quantized, randmat, scheme):
    """Compression bookkeeping shared by qspmm_sum / qspmm_mean
    (ops.py:263-280, 317-334)."""
    if quantized is not None:
        if randmat is None:
            assert config.kept_frac == 1.0
            return quantized, randmat, other.shape, other.shape
        assert config.kept_frac < 1.0 and (other.shape[1] == randmat.shape[0])
        return quantized, randmat, other.shape, torch.Size([other.shape[0], randmat.shape[1]])
    return _compress(other, scheme)


class qspmm_sum(Function):
    """ops.py:257-307."""

    @staticmethod
    def forward(ctx, row, rowptr, col, value, colptr, csr2csc, has_value, other,
                quantized=None, randmat=None, scheme=None):
        result = spmm.spmm_sum_fw(row, rowptr, col, value, colptr, csr2csc, other)
        value_requires_grad = value.requires_grad if has_value else False
        if value_requires_grad or quantized is not None:
            # `other` is read in backward only for the edge-value gradient
            # (spmm.cc:65-67); a caller-supplied `quantized` is kept as given.
            quantized, randmat, ori_input_shape, proj_input_shape = _spmm_saved_shapes(other, quantized, randmat, scheme)
        else:
            quantized, randmat = None, None
            ori_input_shape = proj_input_shape = other.shape
        empty_cache(config.empty_cache_threshold)
        ctx.saved = row, rowptr, col, value, colptr, csr2csc, quantized, randmat
        ctx.other_args = has_value, ori_input_shape, proj_input_shape, value_requires_grad, other.requires_grad
        ctx.scheme = scheme
        return result

    @staticmethod
    def backward(ctx, grad_outputs):
        row, rowptr, col, value, colptr, csr2csc, quantized, randmat = ctx.saved
        has_value, ori_input_shape, q_input_shape, value_requires_grad, mat_requires_grad = ctx.other_args
        other = None
        if value_requires_grad:
            other = dequantize_activation(quantized, q_input_shape)
            if config.kept_frac < 1.0:
                other = rp2input(other, ori_input_shape, randmat)
        del quantized, ctx.saved
        empty_cache(config.empty_cache_threshold)
        grad_value, grad_mat = spmm.spmm_sum_bw(row, rowptr, col, value, colptr, csr2csc, other,
                                                grad_outputs.contiguous(), has_value, value_requires_grad,
                                                mat_requires_grad)
        del other
        empty_cache(config.empty_cache_threshold)
        return None, None, None, grad_value, None, None, None, grad_mat, None, None, None


class qspmm_mean(Function):
    """ops.py:310-371."""

    @staticmethod
    def forward(ctx, row, rowptr, col, value, rowcount, colptr, csr2csc, has_value, other,
                quantized=None, randmat=None, scheme=None):
        result = spmm.spmm_mean_fw(row, rowptr, col, value, rowcount, colptr, csr2csc, other)
        value_requires_grad = value.requires_grad if has_value else False
        if value_requires_grad or quantized is not None:
            quantized, randmat, ori_input_shape, proj_input_shape = _spmm_saved_shapes(other, quantized, randmat, scheme)
        else:
            quantized, randmat = None, None
            ori_input_shape = proj_input_shape = other.shape
        empty_cache(config.empty_cache_threshold)
        ctx.saved = row, rowptr, col, value, rowcount, colptr, csr2csc, quantized, randmat
        ctx.other_args = has_value, ori_input_shape, proj_input_shape, value_requires_grad, other.requires_grad
        ctx.scheme = scheme
        return result

    @staticmethod
    def backward(ctx, grad_outputs):
        row, rowptr, col, value, rowcount, colptr, csr2csc, quantized, randmat = ctx.saved
        has_value, ori_input_shape, q_input_shape, value_requires_grad, mat_requires_grad = ctx.other_args
        # ops.py:351-364: `other` is needed only for the edge-value gradient
        other = None
        if value_requires_grad:
            other = dequantize_activation(quantized, q_input_shape)
            if config.kept_frac < 1.0:
                other = rp2input(other, ori_input_shape, randmat)
        del quantized, ctx.saved
        empty_cache(config.empty_cache_threshold)
        grad_value, grad_mat = spmm.spmm_mean_bw(row, rowptr, col, value, rowcount, colptr, csr2csc, other,
                                                 grad_outputs.contiguous(), has_value, value_requires_grad,
                                                 mat_requires_grad)
        del other
        empty_cache(config.empty_cache_threshold)
        return None, None, None, grad_value, None, None, None, None, grad_mat, None, None, None
