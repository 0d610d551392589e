"""Stand-in for the reference's `exact.cpp_extension.backward_func` module
(backward_func.cc:83-107).  The reference only re-exports ATen routines plus
the two-GEMM linear backward; the same ATen routines are reachable from
Python, so no native code is needed here."""
import torch


def linear_backward(grad_output, input, weight, bias):  # noqa: A002
    """backward_func.cc:83-93."""
    grad_input = grad_output.mm(weight)
    grad_weight = grad_output.t().mm(input)
    grad_bias = grad_output.sum(0) if bias is not None else None
    return grad_input, grad_weight, grad_bias


def native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps):  # noqa: A002
    return torch.ops.aten.native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps)


def native_batch_norm_backward(grad_out, input, weight, running_mean, running_var, save_mean, save_invstd,  # noqa: A002
                               train, eps, output_mask):
    return torch.ops.aten.native_batch_norm_backward(grad_out, input, weight, running_mean, running_var,
                                                     save_mean, save_invstd, train, eps, list(output_mask))


def _elu_backward_cuda(grad_output, data, alpha):
    """backward_func_cuda_kernel.cu:6-36: x >= 0 ? grad : alpha * grad * exp(x)."""
    return torch.where(data >= 0, grad_output, alpha * grad_output * torch.exp(data))
