"""Python-level stand-ins for the reference's four pybind extension modules
(exact/setup.py:6-22): same module and function names, implemented as thin
argument-checking shims over the C ABI of libexact_hip.so."""
from . import quantization, spmm, backward_func  # noqa: F401
