"""Argument checks with the reference's error convention
(exact/exact/cpp_extension/ext_common.h:2-27): RuntimeError with the same
message for non-device, non-contiguous, wrong-rank or wrong-dtype tensors.
fp32 everywhere; fp16 where the library has fp16 kernels (pack / unpack and the
mask activations), as the reference's AT_DISPATCH_FLOATING_TYPES_AND_HALF admits."""
import torch


def _fail(msg):
    raise RuntimeError(msg)


def on_device(t):
    """True for tensors the kernels may touch (device memory)."""
    return t.is_cuda


def check_device_tensor(t, name, dim=None, dtypes=(torch.float32,)):
    if not isinstance(t, torch.Tensor):
        _fail(f"{name} must be a tensor!")
    if not on_device(t):
        _fail(f"{name} must be a CUDA tensor!")
    if not t.is_contiguous():
        _fail(f"{name} must be contiguous!")
    if dim is not None and t.dim() != dim:
        _fail(f"The dimension of {name} is not correct!")
    if t.dtype not in dtypes:
        _fail(f"The type of {name} is not correct!")


FLOAT_OR_HALF = (torch.float32, torch.float16)


def suffix(t):
    """Entry-point suffix for the element type of t."""
    return "f16" if t.dtype == torch.float16 else "f32"


def stream_ptr(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def ptr(t):
    return 0 if t is None else t.data_ptr()
