"""Stand-in for the reference's `exact.cpp_extension.backward_func` module
(backward_func.cc:83-107).  The reference only re-exports ATen routines plus
the two-GEMM linear backward, which are reachable from Python as they are;
its one kernel of its own, the ELU derivative, is a kernel of the library."""
import torch

from .. import _lib
from . import _checks


def column_sums(matrix):
    """`matrix.sum(0)` of a 2-D tensor.  fp32 device matrices go through the
    library's streaming kernel (the framework's reduction runs far off the
    memory roofline for narrow matrices: 19 ms for [2.4M, 47]); its atomics
    fix no summation order, so deterministic mode and everything else keep the
    framework's reduction."""
    usable = (matrix.dim() == 2 and matrix.dtype == torch.float32 and _checks.on_device(matrix)
              and matrix.is_contiguous() and 0 < matrix.shape[1] <= 8192 and matrix.shape[0] >= 4096
              and matrix.data_ptr() % 16 == 0 and not torch.are_deterministic_algorithms_enabled())
    if not usable:
        return matrix.sum(0)
    out = torch.empty(matrix.shape[1], dtype=torch.float32, device=matrix.device)
    rc = _lib.lib().exact_colsum_f32(_checks.ptr(matrix), matrix.shape[0], matrix.shape[1], _checks.ptr(out),
                                     _checks.stream_ptr(matrix))
    _lib.check(rc, "column_sums")
    return out


def linear_backward(grad_output, input, weight, bias, need_input_grad=True):  # noqa: A002
    """backward_func.cc:83-93.  `need_input_grad=False` leaves out the product
    the caller would discard (the reference forms all three regardless)."""
    grad_input = grad_output.mm(weight) if need_input_grad else None
    grad_weight = grad_output.t().mm(input)
    grad_bias = column_sums(grad_output) if bias is not None else None
    return grad_input, grad_weight, grad_bias


def native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps):  # noqa: A002
    return torch.ops.aten.native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps)


def native_batch_norm_backward(grad_out, input, weight, running_mean, running_var, save_mean, save_invstd,  # noqa: A002
                               train, eps, output_mask):
    return torch.ops.aten.native_batch_norm_backward(grad_out, input, weight, running_mean, running_var,
                                                     save_mean, save_invstd, train, eps, list(output_mask))


def _elu_backward_cuda(grad_output, data, alpha):
    """backward_func_cuda_kernel.cu:6-36: x >= 0 ? grad : alpha * grad * exp(x)."""
    grad_output, data = grad_output.contiguous(), data.contiguous()
    _checks.check_device_tensor(grad_output, "grad_output", None, _checks.FLOAT_OR_HALF)
    _checks.check_device_tensor(data, "data", None, (grad_output.dtype,))
    if data.numel() != grad_output.numel():
        raise RuntimeError("grad_output and data must have the same number of elements")
    grad_input = torch.empty_like(grad_output)
    fn = getattr(_lib.lib(), "exact_elu_bwd_" + _checks.suffix(grad_output))
    rc = fn(_checks.ptr(grad_output), _checks.ptr(data), float(alpha), grad_output.numel(), _checks.ptr(grad_input),
            _checks.stream_ptr(grad_output))
    _lib.check(rc, "_elu_backward_cuda")
    return grad_input
