"""CPU-only checks of the C ABI: the library loads, exports every symbol that
include/exact_hip.h declares, and rejects bad arguments before touching a GPU."""
import ctypes
import os
import re

import pytest

from exact_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "exact_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(exact_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 15
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), n
    assert sorted(_lib.SIGNATURES) == names      # the ctypes table covers exactly the header


def test_version_and_strerror():
    L = _lib.lib()
    assert L.exact_abi_version() == 1
    assert b"bits" in L.exact_strerror(-2)
    assert L.exact_strerror(0) == b"ok"


@pytest.mark.parametrize("N,G,bits,want", [(169343, 256, 2, 10838017), (5, 3, 2, 7), (0, 256, 1, 1), (8, 1, 1, 2)])
def test_packed_nbytes(N, G, bits, want):
    assert _lib.lib().exact_packed_nbytes(N, G, bits) == want


def test_argument_errors_need_no_gpu():
    L = _lib.lib()
    assert L.exact_packed_nbytes(8, 8, 3) == -2
    # bits are checked before any pointer is used or any kernel is launched
    assert L.exact_pack_f32(None, None, None, None, 0, 0, 8, 8, 3, None, None) == -2
    assert L.exact_minmax_pack_f32(None, None, 0, 0, 8, 8, 5, None, None, None, None, None, None) == -2
    assert L.exact_unpack_f32(None, 16, None, None, 8, 8, None, None) == -2
    assert L.exact_pack_f32(None, None, None, None, 0, 0, -1, 8, 2, None, None) == -3
    assert L.exact_pack_f32(None, None, None, None, 0, 0, 8, 8, 2, None, None) == -1     # packed is NULL
    assert L.exact_unpack_f32(None, 2, None, None, 8, 8, None, None) == -1
    assert L.exact_relu_fwd_f32(None, 10, None, None, None) == -1
    assert L.exact_relu_fwd_f32(None, -1, None, None, None) == -3
    assert L.exact_dropout_fwd_f32(None, None, 0, 0, 1.0, 10, None, None, None) == -5    # p must be < 1
    assert L.exact_dropout_bwd_f32(None, None, -0.1, 10, None, None) == -5
    assert L.exact_spmm_csr_f32(None, None, None, 2, None, 4, 4, 4, 4, 0, None, None) == -5   # idx_bytes
    assert L.exact_spmm_csr_f32(None, None, None, 8, None, 4, 4, 4, 4, 7, None, None) == -5   # reduce
    assert L.exact_spmm_csr_f32(None, None, None, 8, None, 4, 4, 4, 4, 0, None, None) == -1
    assert L.exact_rp_fwd_f32(None, None, 4, 0, 4, None, None) == -3
    assert L.exact_rp_fwd_f32(None, None, 4, 8, 4, None, None) == -1
    assert L.exact_rp_bwd_f32(None, None, 4, 8, 0, None, None) == -3
    with pytest.raises(RuntimeError, match="EXACT_E_BITS"):
        _lib.check(-2, "x")
