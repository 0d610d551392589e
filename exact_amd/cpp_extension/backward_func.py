"""Stand-in for the reference's `exact.cpp_extension.backward_func` module
(backward_func.cc:83-107).  The reference only re-exports ATen routines plus
the two-GEMM linear backward, which are reachable from Python as they are;
its one kernel of its own, the ELU derivative, is a kernel of the library."""
import torch

from .. import _lib
from ..conf import config
from . import _checks


def _atomics_allowed():
    """The library's reductions meet in memory through atomics; both the
    framework's deterministic mode and config.deterministic_reductions ask for
    reproducible sums instead."""
    return not (torch.are_deterministic_algorithms_enabled() or config.deterministic_reductions)


def column_sums(matrix):
    """`matrix.sum(0)` of a 2-D tensor.  fp32 device matrices go through the
    library's streaming kernel (the framework's reduction runs far off the
    memory roofline for narrow matrices: 19 ms for [2.4M, 47]); its atomics
    fix no summation order, so deterministic mode
    (config.deterministic_reductions or the framework's own switch) and
    everything else keep the framework's reduction."""
    usable = (matrix.dim() == 2 and matrix.dtype == torch.float32 and _checks.on_device(matrix)
              and matrix.is_contiguous() and 0 < matrix.shape[1] <= 256 and matrix.shape[0] >= 4096
              and _atomics_allowed())
    if not usable:
        return matrix.sum(0)
    out = torch.empty(matrix.shape[1], dtype=torch.float32, device=matrix.device)
    rc = _lib.lib().exact_colsum_f32(_checks.ptr(matrix), matrix.shape[0], matrix.shape[1], _checks.ptr(out),
                                     _checks.stream_ptr(matrix))
    _lib.check(rc, "column_sums")
    return out


def batch_statistics(matrix):
    """(biased variance, mean) of every column of a 2-D tensor, what
    torch.var_mean(matrix, dim=0, unbiased=False) returns.  Tall fp32 device
    matrices of at most 256 columns take the library's one-pass kernel (moments
    centred on the mean of 256 rows spread evenly over the matrix -- also for
    sorted or clustered rows a centre within a fraction of a standard deviation
    of the column mean, so that the difference of the two moments loses no
    digits); everything else the framework's reduction."""
    usable = (matrix.dim() == 2 and matrix.dtype == torch.float32 and _checks.on_device(matrix) and matrix.is_contiguous()
              and 0 < matrix.shape[1] <= 256 and matrix.shape[0] >= 4096
              and _atomics_allowed())
    if not usable:
        return torch.var_mean(matrix, dim=0, unbiased=False)
    N, K = matrix.shape
    center = matrix[::N // 256][:256].mean(0)
    sums = torch.empty((2, K), dtype=torch.float32, device=matrix.device)
    rc = _lib.lib().exact_col_moments_f32(_checks.ptr(matrix), _checks.ptr(center), N, K, _checks.ptr(sums[0]),
                                          _checks.ptr(sums[1]), _checks.stream_ptr(matrix))
    _lib.check(rc, "batch_statistics")
    shift = sums[0] / N
    return (sums[1] / N - shift * shift).clamp_(min=0.0), center + shift


def weight_gradient(grad_output, input):  # noqa: A002
    """`grad_output.t().mm(input)` (backward_func.cc:88-89): [N, out]^T . [N, in].
    Tall fp32 device operands take the library's matrix-core kernel for this
    shape -- on the bf16 instruction with operands split in three, or on the
    fp32 instruction (config.matrix_cores) -- whose slabs meet through atomics,
    so deterministic mode and everything else keep the framework's GEMM."""
    usable = (grad_output.dim() == 2 and input.dim() == 2 and grad_output.dtype == torch.float32
              and input.dtype == torch.float32 and _checks.on_device(grad_output) and _checks.on_device(input)
              and grad_output.shape[0] == input.shape[0] and grad_output.shape[0] >= 16384
              and 0 < grad_output.shape[1] <= 1024 and 0 < input.shape[1] <= 1024
              and grad_output.stride(1) == 1 and input.stride(1) == 1
              and grad_output.stride(0) >= grad_output.shape[1] and input.stride(0) >= input.shape[1]
              and _atomics_allowed())
    if not usable:
        return grad_output.t().mm(input)
    N, K = grad_output.shape
    D = input.shape[1]
    out = torch.empty((K, D), dtype=torch.float32, device=grad_output.device)
    if config.matrix_cores not in ("bf16", "fp32"):
        raise ValueError("config.matrix_cores must be 'bf16' or 'fp32'")
    kernel = _lib.lib().exact_linear_dw_bf16_f32 if config.matrix_cores == "bf16" else _lib.lib().exact_linear_dw_f32
    rc = kernel(_checks.ptr(grad_output), grad_output.stride(0), _checks.ptr(input), input.stride(0),
                N, K, D, _checks.ptr(out), _checks.stream_ptr(grad_output))
    _lib.check(rc, "weight_gradient")
    return out


# ---- the dense products of a layer on the bf16 matrix cores ---------------------
def _gemm_table(matrix, transposed, D, K):
    """Operand fragments of `matrix` for exact_tall_gemm_bf16_f32, remembered on the
    tensor until it changes (a weight is prepared once per optimiser step)."""
    key = (bool(transposed), matrix._version, matrix.data_ptr(), tuple(matrix.shape), matrix.stride(0))
    cached = getattr(matrix, "_exact_gemm_table", None)
    if cached is not None and cached[0] == key:
        return cached[1]
    L = _lib.lib()
    table = torch.empty(int(L.exact_tall_gemm_table_nbytes(D, K)), dtype=torch.uint8, device=matrix.device)
    rc = L.exact_tall_gemm_prepare_bf16(_checks.ptr(matrix), matrix.stride(0), int(bool(transposed)), D, K, _checks.ptr(table),
                                        _checks.stream_ptr(matrix))
    _lib.check(rc, "tall_matmul (prepare)")
    try:
        matrix._exact_gemm_table = (key, table)
    except AttributeError:
        pass
    return table


def tall_matmul(x, matrix, transposed=False, bias=None, addend=None, into=None):
    """x[N, D] . M (+ bias[K]) (+ addend[N, K]) -> [N, K], where M = `matrix`
    ([D, K]) or, with transposed=True, the transpose of `matrix` ([K, D]: a weight
    as F.linear holds it).  `into` names the result tensor; it may be `addend`
    itself (accumulate in place).  Tall fp32 device operands with a narrow result
    (config.tall_gemm_min_rows; a result of at most 64 columns or a reduction over
    at least config.tall_gemm_min_depth features of at most
    config.tall_gemm_max_rows_wide rows) take the library's
    kernel (six bf16 matrix-core products per fp32 product, fp32 accuracy,
    reproducible; config.matrix_cores == "bf16"); everything else the
    framework's GEMM."""
    M = matrix.t() if transposed else matrix
    usable = (config.matrix_cores == "bf16" and x.dim() == 2 and matrix.dim() == 2 and x.dtype == torch.float32
              and matrix.dtype == torch.float32 and _checks.on_device(x) and _checks.on_device(matrix)
              and x.shape[1] == M.shape[0] and x.shape[0] >= config.tall_gemm_min_rows and x.shape[1] % 2 == 0
              and 0 < x.shape[1] <= 4096 and 0 < M.shape[1] <= 4096
              and (M.shape[1] <= 64 or (x.shape[1] >= config.tall_gemm_min_depth and x.shape[0] <= config.tall_gemm_max_rows_wide))
              and x.is_contiguous() and x.data_ptr() % 8 == 0
              and matrix.stride(1) == 1 and matrix.stride(0) >= matrix.shape[1]
              and (bias is None or (bias.dtype == torch.float32 and bias.is_contiguous() and bias.numel() == M.shape[1]
                                    and _checks.on_device(bias)))
              and (addend is None or (addend.dtype == torch.float32 and addend.dim() == 2 and addend.stride(1) == 1
                                      and addend.shape == (x.shape[0], M.shape[1]) and _checks.on_device(addend)))
              and (into is None or (into.dtype == torch.float32 and into.dim() == 2 and into.stride(1) == 1
                                    and into.shape == (x.shape[0], M.shape[1]) and _checks.on_device(into)))
              and not (torch.is_grad_enabled() and (x.requires_grad or matrix.requires_grad
                                                    or (bias is not None and bias.requires_grad)
                                                    or (addend is not None and addend.requires_grad))))
    if not usable:
        if addend is not None:
            out = torch.addmm(addend, x, M) if into is None or into is not addend else addend.addmm_(x, M)
            if bias is not None:
                out += bias
        else:
            out = x.mm(M) if bias is None else torch.addmm(bias, x, M)
        if into is not None and into is not out:
            into.copy_(out)
            out = into
        return out
    N, D = x.shape
    K = M.shape[1]
    out = into if into is not None else torch.empty((N, K), dtype=torch.float32, device=x.device)
    table = _gemm_table(matrix, transposed, D, K)
    rc = _lib.lib().exact_tall_gemm_bf16_f32(_checks.ptr(x), _checks.ptr(table), N, D, K,
                                             _checks.ptr(bias) if bias is not None else None,
                                             _checks.ptr(addend) if addend is not None else None,
                                             addend.stride(0) if addend is not None else K, _checks.ptr(out), out.stride(0),
                                             _checks.stream_ptr(x))
    _lib.check(rc, "tall_matmul")
    return out


def linear_backward(grad_output, input, weight, bias, need_input_grad=True):  # noqa: A002
    """backward_func.cc:83-93.  `need_input_grad=False` leaves out the product
    the caller would discard (the reference forms all three regardless)."""
    grad_input = tall_matmul(grad_output, weight) if need_input_grad else None
    grad_weight = weight_gradient(grad_output, input)
    grad_bias = column_sums(grad_output) if bias is not None else None
    return grad_input, grad_weight, grad_bias


def native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps):  # noqa: A002
    return torch.ops.aten.native_batch_norm(input, weight, bias, running_mean, running_var, training, momentum, eps)


def native_batch_norm_backward(grad_out, input, weight, running_mean, running_var, save_mean, save_invstd,  # noqa: A002
                               train, eps, output_mask):
    """at::native_batch_norm_backward as re-exported by backward_func.cc:99-104.
    For a tall fp32 [N, K <= 256] training-mode batch on the device, its two
    column reductions (sum of dy, sum of dy * (x - mean)) run in the library's
    one-pass kernel -- the framework's reduction kernel reads the same two
    matrices at a tenth of the memory bandwidth -- and the element-wise half is
    the framework's batch_norm_backward_elemt, which computes
      dx = (dy - sum_dy / N - (x - mean) * invstd^2 * sum_dy_xmu / N) * invstd * weight
    exactly as the one-call routine does."""
    def stat_ok(t, optional=False):
        if t is None:
            return optional
        return t.dtype == torch.float32 and t.device == grad_out.device and t.numel() == grad_out.shape[1]

    fast = (train and grad_out.dim() == 2 and grad_out.is_cuda and grad_out.dtype == torch.float32
            and input.dtype == torch.float32 and input.device == grad_out.device
            and grad_out.is_contiguous() and input.is_contiguous()
            and 4096 <= grad_out.shape[0] < 2 ** 31 and 0 < grad_out.shape[1] <= 256 and grad_out.shape == input.shape
            and stat_ok(save_mean) and stat_ok(save_invstd) and stat_ok(weight, optional=True)
            and _atomics_allowed())
    if not fast:
        return torch.ops.aten.native_batch_norm_backward(grad_out, input, weight, running_mean, running_var,
                                                         save_mean, save_invstd, train, eps, list(output_mask))
    N, K = grad_out.shape
    mean = save_mean.contiguous()
    sums = torch.empty((2, K), dtype=torch.float32, device=grad_out.device)
    rc = _lib.lib().exact_bn_backward_reduce_f32(_checks.ptr(grad_out), _checks.ptr(input), _checks.ptr(mean), N, K,
                                                 _checks.ptr(sums[0]), _checks.ptr(sums[1]), _checks.stream_ptr(grad_out))
    _lib.check(rc, "native_batch_norm_backward")
    sum_dy, sum_dy_xmu = sums[0], sums[1]
    grad_input = grad_weight = grad_bias = None
    if output_mask[0]:
        count = torch.full((1,), N, dtype=torch.int32, device=grad_out.device)
        grad_input = torch.batch_norm_backward_elemt(grad_out, input, mean, save_invstd, weight, sum_dy, sum_dy_xmu, count)
    if output_mask[1]:
        grad_weight = sum_dy_xmu * save_invstd
    if output_mask[2]:
        grad_bias = sum_dy
    return grad_input, grad_weight, grad_bias


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
