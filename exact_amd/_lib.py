"""ctypes binding of libexact_hip.so (the C ABI declared in include/exact_hip.h).

The library is the only compute back end of this package: if it cannot be
loaded, every op raises -- there is no eager/CPU fallback.
"""
from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
# EXACT_AMD_LIB overrides the path (e.g. to load a differently built library)
LIB_PATH = os.environ.get("EXACT_AMD_LIB") or os.path.join(_HERE, "libexact_hip.so")

_c_i64 = ctypes.c_int64
_c_u64 = ctypes.c_uint64
_c_int = ctypes.c_int
_c_ptr = ctypes.c_void_p
_c_f32 = ctypes.c_float

# name -> (restype, argtypes); mirrors include/exact_hip.h one to one
SIGNATURES = {
    "exact_abi_version": (_c_int, []),
    "exact_strerror": (ctypes.c_char_p, [_c_int]),
    "exact_packed_nbytes": (_c_i64, [_c_i64, _c_i64, _c_int]),
    "exact_row_minmax_f32": (_c_int, [_c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_pack_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_minmax_pack_f32": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "exact_minmax_pack_geom_f32": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]),
    "exact_unpack_f32": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_unpack_bf16param_f32": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_relu_fwd_f32": (_c_int, [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_relu_bwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr]),
    "exact_dropout_fwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_f32, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_dropout_bwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_f32, _c_i64, _c_ptr, _c_ptr]),
    "exact_spmm_csr_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_spmm_csr_strided_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_i64, _c_ptr]),
    "exact_spmm_csr_rowwise_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_spmm_csr_minmax_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr]),
    "exact_sddmm_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_leaky_relu_fwd_f32": (_c_int, [_c_ptr, _c_i64, _c_f32, _c_ptr, _c_ptr, _c_ptr]),
    "exact_leaky_relu_bwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_f32, _c_ptr, _c_ptr]),
    "exact_relu_dropout_fwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_f32, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_relu_dropout_minmax_pack_f32": (_c_int, [_c_ptr, _c_f32, _c_ptr, _c_u64, _c_u64, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_int,
                                                    _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "exact_bn_relu_dropout_minmax_pack_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_f32, _c_ptr, _c_u64, _c_u64, _c_ptr, _c_u64, _c_u64,
                                                       _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "exact_rp_minmax_pack_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr,
                                          _c_ptr, _c_ptr, _c_ptr]),
    "exact_minmax_pack_f16": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "exact_unpack_f16": (_c_int, [_c_ptr, _c_int, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_relu_fwd_f16": (_c_int, [_c_ptr, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_relu_bwd_f16": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_ptr, _c_ptr]),
    "exact_leaky_relu_fwd_f16": (_c_int, [_c_ptr, _c_i64, _c_f32, _c_ptr, _c_ptr, _c_ptr]),
    "exact_leaky_relu_bwd_f16": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_f32, _c_ptr, _c_ptr]),
    "exact_dropout_fwd_f16": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_f32, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_relu_dropout_fwd_f16": (_c_int, [_c_ptr, _c_ptr, _c_u64, _c_u64, _c_f32, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_dropout_bwd_f16": (_c_int, [_c_ptr, _c_ptr, _c_f32, _c_i64, _c_ptr, _c_ptr]),
    "exact_elu_bwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_f32, _c_i64, _c_ptr, _c_ptr]),
    "exact_linear_dw_f32": (_c_int, [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_linear_dw_bf16_f32": (_c_int, [_c_ptr, _c_i64, _c_ptr, _c_i64, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_colsum_f32": (_c_int, [_c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_stream_probe_f32": (_c_int, [_c_ptr, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_col_moments_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_bn_backward_reduce_f32": (_c_int, [_c_ptr, _c_ptr, _c_ptr, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_ptr]),
    "exact_elu_bwd_f16": (_c_int, [_c_ptr, _c_ptr, _c_f32, _c_i64, _c_ptr, _c_ptr]),
    "exact_rp_fwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_rp_bwd_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_rp_table_nbytes": (_c_i64, [_c_i64, _c_i64, _c_int]),
    "exact_rp_prepare_bf16": (_c_int, [_c_ptr, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_rp_fwd_bf16_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_rp_bwd_bf16_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_int, _c_ptr, _c_ptr]),
    "exact_rp_minmax_pack_bf16_f32": (_c_int, [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_u64, _c_u64, _c_i64, _c_i64, _c_i64,
                                               _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr]),
    "exact_tall_gemm_table_nbytes": (_c_i64, [_c_i64, _c_i64]),
    "exact_tall_gemm_prepare_bf16": (_c_int, [_c_ptr, _c_i64, _c_int, _c_i64, _c_i64, _c_ptr, _c_ptr]),
    "exact_tall_gemm_bf16_f32": (_c_int, [_c_ptr, _c_ptr, _c_i64, _c_i64, _c_i64, _c_ptr, _c_ptr, _c_i64, _c_ptr, _c_i64, _c_ptr]),
}

_lib = None
_lock = threading.Lock()


class ExactLibraryError(RuntimeError):
    pass


def lib() -> ctypes.CDLL:
    """The loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise ExactLibraryError(
                        f"{LIB_PATH} is missing: build it with `python -m exact_amd.build` "
                        "(hipcc, gfx950). exact_amd has no fallback path.")
                # torch must bring up its HIP runtime first: the library then binds
                # to that same runtime (one libamdhip64 per process), and a library
                # loaded ahead of torch's device initialisation has left torch
                # unable to see the GPU.
                import torch
                if torch.cuda.is_available():
                    torch.cuda.init()
                handle = ctypes.CDLL(LIB_PATH)
                for name, (res, args) in SIGNATURES.items():
                    fn = getattr(handle, name)  # AttributeError if the symbol is not exported
                    fn.restype = res
                    fn.argtypes = args
                _lib = handle
    return _lib


def check(rc: int, what: str) -> None:
    """Turn a non-zero return code into the RuntimeError the reference's
    TORCH_CHECK / AT_ASSERTM would have raised."""
    if rc != 0:
        msg = lib().exact_strerror(rc).decode()
        raise RuntimeError(f"{what}: {msg} (code {rc})")
