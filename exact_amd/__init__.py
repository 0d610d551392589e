"""exact_amd: EXACT's activation-compression and sparse-aggregation hot path
for MI355X (gfx950), behind EXACT's own Python API.

    import exact_amd as exact
    exact.config.activation_compression_bits = [2]
    model = exact.QModule(model)

`install_as_exact()` registers the package under the name `exact` so that code
written against the reference (`from exact import QModule, config`,
`import exact.cpp_extension.quantization as ext_quantization`) runs unchanged.
"""
import sys

from . import cpp_extension, ops, spmm  # noqa: F401
from .conf import config  # noqa: F401
from .gatconv import QCustomGATConv  # noqa: F401
from .layers import (QELU, QMLP, QBatchNorm1d, QDropout, QDropout2, QGCN2Conv, QGCNConv,  # noqa: F401
                     QGENConv, QGraphConv, QLeakyReLU, QLinear, QReLU, QReLUDropout, QSAGEConv)
from .module import QModule  # noqa: F401
from .sparse import SparseTensor, gcn_norm  # noqa: F401
from .utils import (cast_adj, cast_low_bit_int, compute_tensor_bytes,  # noqa: F401
                    exp_recorder, get_memory_usage)

__all__ = ["config", "QModule", "QLinear", "QGCNConv", "QSAGEConv", "QBatchNorm1d", "QReLU", "QDropout",
           "QDropout2", "QLeakyReLU", "QELU", "QReLUDropout", "QGCN2Conv", "QGENConv", "QGraphConv", "QMLP", "QCustomGATConv", "SparseTensor", "gcn_norm", "ops", "spmm", "cpp_extension", "install_as_exact"]


def install_as_exact():
    """Make `import exact`, `exact.ops`, `exact.spmm`, `exact.layers`,
    `exact.cpp_extension.quantization` ... resolve to this package."""
    pkg = sys.modules[__name__]
    sys.modules.setdefault("exact", pkg)
    for name, mod in list(sys.modules.items()):
        if name.startswith(__name__ + "."):
            sys.modules.setdefault("exact" + name[len(__name__):], mod)
    return pkg
