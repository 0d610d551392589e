"""Stand-in for the reference's `exact.cpp_extension.quantization` module
(quantization.cc:137-143): pack_single_precision, unpack_single_precision,
act_quantized_relu, act_quantized_dropout -- same names, argument order and
error behaviour -- plus the fused entry points this library adds.

Everything here is host glue: argument checks, output allocation with torch,
and one call into libexact_hip.so on the current stream.
"""
from __future__ import annotations

import torch

from .. import _lib
from ..conf import config
from ..rng import next_philox
from . import _checks
from ._checks import FLOAT_OR_HALF, check_device_tensor, ptr, suffix


def packed_nbytes(N: int, G: int, bits: int) -> int:
    return int(_lib.lib().exact_packed_nbytes(N, G, bits))


def _check_bits(bits):
    if not isinstance(bits, int) or bits <= 0 or 8 % bits != 0:
        # TORCH_CHECK(8 % bits == 0), quantization_cuda_kernel.cu:108,198
        raise RuntimeError("Expected 8 % bits == 0 to be true, but got false.")


def _noise_for(shape, device):
    """(noise tensor or None, seed, offset)."""
    if config.noise_source is not None:
        noise = config.noise_source(tuple(shape), device)
        check_device_tensor(noise, "noise")
        if noise.numel() != int(torch.Size(shape).numel()):
            raise RuntimeError("noise has the wrong number of elements")
        return noise, 0, 0
    seed, offset = next_philox(device)
    return None, seed, offset


def pack_single_precision(data, min, max, scale, bits, stochastic):  # noqa: A002
    """quantization.cc:37-48.  `max` is accepted and checked but, as in the
    reference kernel, not used by the arithmetic."""
    check_device_tensor(data, "data", 2)
    check_device_tensor(min, "min", 1)
    check_device_tensor(max, "max", 1)
    check_device_tensor(scale, "scale", 1)
    _check_bits(bits)
    if not stochastic:
        # TORCH_CHECK(stochastic), quantization_cuda_kernel.cu:123
        raise RuntimeError("Expected stochastic to be true, but got false.")
    N, G = data.shape
    if min.numel() != N or scale.numel() != N:
        raise RuntimeError("min / scale must have one entry per row of data")
    packed = torch.empty(packed_nbytes(N, G, bits), dtype=torch.int8, device=data.device)
    noise, seed, offset = _noise_for(data.shape, data.device)
    rc = _lib.lib().exact_pack_f32(ptr(data), ptr(min), ptr(scale), ptr(noise), seed, offset,
                                   N, G, bits, ptr(packed), _checks.stream_ptr(data))
    _lib.check(rc, "pack_single_precision")
    return packed


def unpack_single_precision(data, bits, scale, min, N, group_size):  # noqa: A002
    """quantization.cc:50-62."""
    check_device_tensor(data, "data", 1, (torch.int8,))
    check_device_tensor(scale, "scale", 1, FLOAT_OR_HALF)
    check_device_tensor(min, "min", 1, (scale.dtype,))
    _check_bits(bits)
    N, G = int(N), int(group_size)
    if data.numel() < packed_nbytes(N, G, bits) - 1 or scale.numel() < N or min.numel() < N:
        raise RuntimeError("packed data / scale / min are too short for N x group_size")
    out = torch.empty((N, G), dtype=scale.dtype, device=data.device)     # the dtype of scale decides, as at :209
    unpack = getattr(_lib.lib(), "exact_unpack_" + suffix(scale))
    rc = unpack(ptr(data), bits, ptr(scale), ptr(min), N, G, ptr(out), _checks.stream_ptr(data))
    _lib.check(rc, "unpack_single_precision")
    return out


# ---- work split of the fused pack kernel ---------------------------------------
# (G, bits) -> octs per lane found fastest by tune_pack_geometry; 0 or absent = the library's default
_PACK_GEOMETRY = {}
_TUNE_MIN_ELEMENTS = 1 << 20


def pack_geometry_candidates(G):
    """Octs (8-column groups) per lane the kernel accepts for rows of G columns."""
    octs = (G + 7) // 8
    return [c for c in (1, 2, 4) if (octs + c - 1) // c <= 32 and (c == 1 or octs >= c)]


def tune_pack_geometry(data, bits, reps=5):
    """Time exact_minmax_pack_geom_f32 on `data` (read only; outputs go to
    scratch buffers, no random numbers are consumed) with every candidate split,
    remember the fastest for (G, bits) and return {candidate: seconds}.  The
    launches rotate over up to four copies of the input, about 400 MB apart: in
    a training step the tensor to compress has just been written once and is
    not found in the 256 MB memory-side cache, and a candidate must not win on
    re-reading one cached input."""
    N, G = data.shape
    dev = data.device
    nbytes = data.numel() * data.element_size()
    extra = 0 if nbytes >= (400 << 20) else min(3, -(-(400 << 20) // max(nbytes, 1)))
    inputs = [data] + [data.clone() for _ in range(extra)]
    turn = [0]
    packed = torch.empty(packed_nbytes(N, G, bits), dtype=torch.int8, device=dev)
    scale_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    min_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    stream = _checks.stream_ptr(data)
    fn = _lib.lib().exact_minmax_pack_geom_f32
    timings = {}
    for cand in pack_geometry_candidates(G):
        def launch():
            turn[0] += 1
            rc = fn(ptr(inputs[turn[0] % len(inputs)]), None, 0x7E57, 4, N, G, bits, ptr(packed), None, None, ptr(scale_bf),
                    ptr(min_bf), cand, stream)
            _lib.check(rc, "tune_pack_geometry")
        launch()                                            # warm-up (first touch, code load)
        best = None
        for _ in range(3):                                  # the fastest of three runs: one run is now and then disturbed
            start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for _ in range(reps):
                launch()
            stop.record()
            stop.synchronize()
            t = start.elapsed_time(stop) * 1e-3 / reps
            best = t if best is None else min(best, t)
        timings[cand] = best
    _PACK_GEOMETRY[(G, bits)] = min(timings, key=timings.get)
    return timings


def _pack_geometry(data, bits):
    """The split to ask for: the remembered one, after tuning when that is due."""
    key = (data.shape[1], bits)
    if key not in _PACK_GEOMETRY:
        if not (config.autotune_pack and data.is_cuda and data.numel() >= _TUNE_MIN_ELEMENTS
                and len(pack_geometry_candidates(key[0])) > 1) or torch.cuda.is_current_stream_capturing():
            return 0
        tune_pack_geometry(data, bits)
    return _PACK_GEOMETRY[key]


# ---- fused forms (no counterpart module function in the reference) ----------
def minmax_pack(data, bits, want_fp32=False):
    """One pass over data[N, G]: per-row min and scale (ops.py:39, 61-66),
    quantise + pack, and the bf16 copies of scale / min (ops.py:80-81).
    -> (packed int8, scale bf16, min bf16[, scale fp32, min fp32])."""
    check_device_tensor(data, "data", 2, FLOAT_OR_HALF)
    _check_bits(bits)
    N, G = data.shape
    dev = data.device
    packed = torch.empty(packed_nbytes(N, G, bits), dtype=torch.int8, device=dev)
    if data.dtype == torch.float16:
        # fp16 activations: scale / min come back in fp16 (reference ops.py:82-83)
        if G > 1024:
            raise RuntimeError("fp16 activations: at most 1024 values per row")
        scale_h = torch.empty(N, dtype=torch.float16, device=dev)
        min_h = torch.empty(N, dtype=torch.float16, device=dev)
        noise, seed, offset = _noise_for(data.shape, dev)
        rc = _lib.lib().exact_minmax_pack_f16(ptr(data), ptr(noise), seed, offset, N, G, bits, ptr(packed),
                                              ptr(scale_h), ptr(min_h), _checks.stream_ptr(data))
        _lib.check(rc, "minmax_pack")
        if want_fp32:
            return packed, scale_h, min_h, scale_h.float(), min_h.float()
        return packed, scale_h, min_h
    scale_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    min_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    need32 = want_fp32 or G > 1024
    scale32 = torch.empty(N, dtype=torch.float32, device=dev) if need32 else None
    min32 = torch.empty(N, dtype=torch.float32, device=dev) if need32 else None
    noise, seed, offset = _noise_for(data.shape, dev)
    rc = _lib.lib().exact_minmax_pack_geom_f32(ptr(data), ptr(noise), seed, offset, N, G, bits, ptr(packed),
                                               ptr(scale32), ptr(min32), ptr(scale_bf), ptr(min_bf),
                                               _pack_geometry(data, bits), _checks.stream_ptr(data))
    _lib.check(rc, "minmax_pack")
    if want_fp32:
        return packed, scale_bf, min_bf, scale32, min32
    return packed, scale_bf, min_bf


RP_PACK_MAX_COLUMNS = 128


RP_FP32, RP_BF16_SPLIT, RP_BF16_SIGNS = 0, 1, 2      # EXACT_RP_* of the C header (0: the fp32 instruction)


def rp_mode(rand_matrix):
    """Which matrix-core path multiplies by this projection matrix.
    config.matrix_cores == "fp32": the fp32 instruction.  "bf16" (default):
    the bf16 instruction on operands split into three bf16 pieces each -- for a
    matrix that ops._projection_matrix drew as +-c (it marks the tensor) on its
    signs alone, scaled by c at the end; for any other matrix the general
    six-product form."""
    if config.matrix_cores == "fp32":
        return RP_FP32
    if config.matrix_cores != "bf16":
        raise ValueError("config.matrix_cores must be 'bf16' or 'fp32'")
    return RP_BF16_SIGNS if getattr(rand_matrix, "_exact_sign_matrix", False) else RP_BF16_SPLIT


def rp_table(rand_matrix, mode):
    """The matrix-core operand fragments of a projection matrix for the bf16 entry
    points (exact_rp_prepare_bf16), built on first use and kept on the tensor
    object for as long as the matrix is not written to: a layer's forward and
    backward share one."""
    kept = getattr(rand_matrix, "_exact_rp_table", None)
    if kept is not None and kept[0] == (mode, rand_matrix._version, rand_matrix.data_ptr()):
        return kept[1]
    D, k = rand_matrix.shape
    nbytes = int(_lib.lib().exact_rp_table_nbytes(D, k, mode))
    if nbytes <= 0:
        raise RuntimeError("the projection kernels take 1 to 128 projected columns")
    table = torch.empty(nbytes, dtype=torch.uint8, device=rand_matrix.device)
    rc = _lib.lib().exact_rp_prepare_bf16(ptr(rand_matrix), D, k, mode, ptr(table), _checks.stream_ptr(rand_matrix))
    _lib.check(rc, "rp_table")
    rand_matrix._exact_rp_table = ((mode, rand_matrix._version, rand_matrix.data_ptr()), table)
    return table


def rp_minmax_pack(data, rand_matrix, bits):
    """minmax_pack of the projection data[N, D] . rand_matrix[D, k] in one launch:
    the [N, k] product is quantised in the registers that accumulate it
    (input2rp then quantize_activation, ops.py:141-149; k <= 128)
    -> (packed int8, scale bf16, min bf16)."""
    check_device_tensor(data, "data", 2)
    check_device_tensor(rand_matrix, "rand_matrix", 2)
    _check_bits(bits)
    N, D = data.shape
    if rand_matrix.shape[0] != D:
        raise RuntimeError("rand_matrix does not match the input")
    k = rand_matrix.shape[1]
    if not 0 < k <= RP_PACK_MAX_COLUMNS:
        raise RuntimeError(f"rp_minmax_pack takes 1 to {RP_PACK_MAX_COLUMNS} projected columns")
    dev = data.device
    packed = torch.empty(packed_nbytes(N, k, bits), dtype=torch.int8, device=dev)
    scale_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    min_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    noise, seed, offset = _noise_for((N, k), dev)
    mode = rp_mode(rand_matrix)
    if mode == RP_FP32:
        rc = _lib.lib().exact_rp_minmax_pack_f32(ptr(data), ptr(rand_matrix), ptr(noise), seed, offset, N, D, k, bits,
                                                 ptr(packed), None, None, ptr(scale_bf), ptr(min_bf),
                                                 _checks.stream_ptr(data))
    else:
        rc = _lib.lib().exact_rp_minmax_pack_bf16_f32(ptr(data), ptr(rp_table(rand_matrix, mode)), mode, ptr(noise), seed,
                                                      offset, N, D, k, bits, ptr(packed), None, None, ptr(scale_bf),
                                                      ptr(min_bf), _checks.stream_ptr(data))
    _lib.check(rc, "rp_minmax_pack")
    return packed, scale_bf, min_bf


def unpack_bf16param(data, bits, scale_bf16, min_bf16, N, group_size):
    """unpack_single_precision with the bf16 -> fp32 widening of
    dequantize_activation (ops.py:92-96) folded into the kernel."""
    check_device_tensor(data, "data", 1, (torch.int8,))
    check_device_tensor(scale_bf16, "scale", 1, (torch.bfloat16,))
    check_device_tensor(min_bf16, "min", 1, (torch.bfloat16,))
    _check_bits(bits)
    N, G = int(N), int(group_size)
    if data.numel() < packed_nbytes(N, G, bits) - 1 or scale_bf16.numel() < N or min_bf16.numel() < N:
        raise RuntimeError("packed data / scale / min are too short for N x group_size")
    out = torch.empty((N, G), dtype=torch.float32, device=data.device)
    rc = _lib.lib().exact_unpack_bf16param_f32(ptr(data), bits, ptr(scale_bf16), ptr(min_bf16), N, G,
                                               ptr(out), _checks.stream_ptr(data))
    _lib.check(rc, "unpack_bf16param")
    return out


def row_minmax(data):
    check_device_tensor(data, "data", 2)
    N, G = data.shape
    mn = torch.empty(N, dtype=torch.float32, device=data.device)
    mx = torch.empty(N, dtype=torch.float32, device=data.device)
    rc = _lib.lib().exact_row_minmax_f32(ptr(data), N, G, ptr(mn), ptr(mx), _checks.stream_ptr(data))
    _lib.check(rc, "row_minmax")
    return mn, mx


# ---- 1-bit-mask activations --------------------------------------------------
def mask_nwords(n: int) -> int:
    return (n + 31) // 32


class ActQuantizedReLU(torch.autograd.Function):
    """quantization.cc:66-79: the only tensor kept for backward is the mask."""

    @staticmethod
    def forward(ctx, input):  # noqa: A002
        n = input.numel()
        out = torch.empty_like(input)
        mask = torch.empty(mask_nwords(n), dtype=torch.int32, device=input.device)
        rc = getattr(_lib.lib(), "exact_relu_fwd_" + suffix(input))(ptr(input), n, ptr(out), ptr(mask), _checks.stream_ptr(input))
        _lib.check(rc, "act_quantized_relu")
        ctx.save_for_backward(mask)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        (mask,) = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_input = torch.empty_like(grad_output)
        rc = getattr(_lib.lib(), "exact_relu_bwd_" + suffix(grad_output))(ptr(grad_output), ptr(mask), grad_output.numel(),
                                           ptr(grad_input), _checks.stream_ptr(grad_output))
        _lib.check(rc, "act_quantized_relu backward")
        return grad_input


def act_quantized_relu(input):  # noqa: A002
    """quantization.cc:81-84."""
    check_device_tensor(input, "input", None, FLOAT_OR_HALF)
    return ActQuantizedReLU.apply(input)


class ActQuantizedLeakyReLU(torch.autograd.Function):
    """quantization.cc:87-103."""

    @staticmethod
    def forward(ctx, input, slope):  # noqa: A002
        n = input.numel()
        out = torch.empty_like(input)
        mask = torch.empty(mask_nwords(n), dtype=torch.int32, device=input.device)
        rc = getattr(_lib.lib(), "exact_leaky_relu_fwd_" + suffix(input))(ptr(input), n, float(slope), ptr(out), ptr(mask),
                                                 _checks.stream_ptr(input))
        _lib.check(rc, "act_quantized_leaky_relu")
        ctx.save_for_backward(mask)
        ctx.slope = float(slope)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        (mask,) = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_input = torch.empty_like(grad_output)
        rc = getattr(_lib.lib(), "exact_leaky_relu_bwd_" + suffix(grad_output))(ptr(grad_output), ptr(mask), grad_output.numel(), ctx.slope,
                                                 ptr(grad_input), _checks.stream_ptr(grad_output))
        _lib.check(rc, "act_quantized_leaky_relu backward")
        return grad_input, None


def act_quantized_leaky_relu(input, slope):  # noqa: A002
    """quantization.cc:105-108."""
    check_device_tensor(input, "input", None, FLOAT_OR_HALF)
    return ActQuantizedLeakyReLU.apply(input, slope)


class ActQuantizedDropout(torch.autograd.Function):
    """quantization.cc:111-129."""

    @staticmethod
    def forward(ctx, input, p, train):  # noqa: A002
        if not train:
            return input
        n = input.numel()
        out = torch.empty_like(input)
        mask = torch.empty(mask_nwords(n), dtype=torch.int32, device=input.device)
        noise, seed, offset = _noise_for(input.shape, input.device)
        rc = getattr(_lib.lib(), "exact_dropout_fwd_" + suffix(input))(ptr(input), ptr(noise), seed, offset, float(p), n,
                                              ptr(out), ptr(mask), _checks.stream_ptr(input))
        _lib.check(rc, "act_quantized_dropout")
        ctx.save_for_backward(mask)
        ctx.p = float(p)
        ctx.train = True
        return out

    @staticmethod
    def backward(ctx, grad_output):
        if not getattr(ctx, "train", False):
            return grad_output, None, None
        (mask,) = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        grad_input = torch.empty_like(grad_output)
        rc = getattr(_lib.lib(), "exact_dropout_bwd_" + suffix(grad_output))(ptr(grad_output), ptr(mask), ctx.p, grad_output.numel(),
                                              ptr(grad_input), _checks.stream_ptr(grad_output))
        _lib.check(rc, "act_quantized_dropout backward")
        return grad_input, None, None


def act_quantized_dropout(input, p, train):  # noqa: A002
    """quantization.cc:131-134."""
    check_device_tensor(input, "input", None, FLOAT_OR_HALF)
    if not train:
        return input                      # quantization.cc:115-117
    return ActQuantizedDropout.apply(input, p, train)


# ---- fused epilogues (no counterpart module function in the reference) -------
def fusable_width(G: int) -> bool:
    """Row widths the one-pass ReLU + dropout + quantise kernel takes."""
    return G > 0 and G % 8 == 0 and G <= 1024


def relu_dropout_fwd(input, p):  # noqa: A002
    """dropout(relu(input)) in one pass -> (output, joint 1-bit mask); the
    gradient of the pair is dropout_bwd on that mask."""
    check_device_tensor(input, "input", None, FLOAT_OR_HALF)
    n = input.numel()
    out = torch.empty_like(input)
    mask = torch.empty(mask_nwords(n), dtype=torch.int32, device=input.device)
    noise, seed, offset = _noise_for(input.shape, input.device)
    rc = getattr(_lib.lib(), "exact_relu_dropout_fwd_" + suffix(input))(ptr(input), ptr(noise), seed, offset, float(p), n, ptr(out), ptr(mask),
                                               _checks.stream_ptr(input))
    _lib.check(rc, "relu_dropout")
    return out, mask


def _aligned16(t):
    """t itself, or a copy when its first element is not on a 16-byte boundary
    (a view into the middle of a buffer): the fused kernels use 16-byte accesses."""
    return t if t.data_ptr() % 16 == 0 else t.clone()


def relu_dropout_minmax_pack(input, p, bits):  # noqa: A002
    """dropout(relu(input)) and minmax_pack of the result in one pass over
    input[N, G] -> (output, mask, packed int8, scale bf16, min bf16).  Draws
    the dropout noise first, then the quantiser's, as the separate calls do."""
    check_device_tensor(input, "input", 2)
    _check_bits(bits)
    N, G = input.shape
    if not fusable_width(G):
        raise RuntimeError("relu_dropout_minmax_pack needs a row width that is a multiple of 8 and at most 1024")
    input = _aligned16(input)  # noqa: A001
    dev = input.device
    out = torch.empty_like(input)
    mask = torch.empty(mask_nwords(N * G), dtype=torch.int32, device=dev)
    packed = torch.empty(packed_nbytes(N, G, bits), dtype=torch.int8, device=dev)
    scale_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    min_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    act_noise, act_seed, act_offset = _noise_for(input.shape, dev)
    noise, seed, offset = _noise_for(input.shape, dev)
    rc = _lib.lib().exact_relu_dropout_minmax_pack_f32(
        ptr(input), float(p), ptr(act_noise), act_seed, act_offset, ptr(noise), seed, offset, N, G, bits,
        ptr(out), ptr(mask), ptr(packed), None, None, ptr(scale_bf), ptr(min_bf), _checks.stream_ptr(input))
    _lib.check(rc, "relu_dropout_minmax_pack")
    return out, mask, packed, scale_bf, min_bf


def bn_relu_dropout_minmax_pack(input, mean, mult, shift, p, bits):  # noqa: A002
    """relu_dropout_minmax_pack of the batch-normalised input, (input - mean) *
    mult + shift per column (three fp32 operations), in the same single pass
    -> (output, mask, packed int8, scale bf16, min bf16)."""
    check_device_tensor(input, "input", 2)
    _check_bits(bits)
    N, G = input.shape
    for name, vec in (("mean", mean), ("mult", mult), ("shift", shift)):
        check_device_tensor(vec, name, 1)
        if vec.shape[0] != G:
            raise RuntimeError(f"The dimension of {name} is not correct!")
    if not fusable_width(G):
        raise RuntimeError("bn_relu_dropout_minmax_pack needs a row width that is a multiple of 8 and at most 1024")
    input, mean, mult, shift = (_aligned16(t) for t in (input, mean, mult, shift))  # noqa: A001
    dev = input.device
    out = torch.empty_like(input)
    mask = torch.empty(mask_nwords(N * G), dtype=torch.int32, device=dev)
    packed = torch.empty(packed_nbytes(N, G, bits), dtype=torch.int8, device=dev)
    scale_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    min_bf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    act_noise, act_seed, act_offset = _noise_for(input.shape, dev)
    noise, seed, offset = _noise_for(input.shape, dev)
    rc = _lib.lib().exact_bn_relu_dropout_minmax_pack_f32(
        ptr(input), ptr(mean), ptr(mult), ptr(shift), float(p), ptr(act_noise), act_seed, act_offset, ptr(noise), seed,
        offset, N, G, bits, ptr(out), ptr(mask), ptr(packed), None, None, ptr(scale_bf), ptr(min_bf),
        _checks.stream_ptr(input))
    _lib.check(rc, "bn_relu_dropout_minmax_pack")
    return out, mask, packed, scale_bf, min_bf


def dropout_bwd(grad_output, mask, p):
    """dx = bit ? dy / (1 - p) : 0 (quantization_cuda_kernel.cu:565-569)."""
    grad_output = grad_output.contiguous()
    check_device_tensor(grad_output, "grad_output", None, FLOAT_OR_HALF)
    grad_input = torch.empty_like(grad_output)
    rc = getattr(_lib.lib(), "exact_dropout_bwd_" + suffix(grad_output))(ptr(grad_output), ptr(mask), float(p), grad_output.numel(),
                                          ptr(grad_input), _checks.stream_ptr(grad_output))
    _lib.check(rc, "dropout backward")
    return grad_input
