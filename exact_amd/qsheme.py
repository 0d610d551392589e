"""Per-layer quantisation scheme object, as exact/exact/qsheme.py:8-47 of the
reference: names layers, and computes the per-row min / max with which a row
is quantised (bits always config.activation_compression_bits[0])."""
from .conf import config
from .cpp_extension import quantization as ext_quantization


class QScheme(object):
    num_samples = 1
    num_matmul_layer = 0
    num_lin_layer = 0
    num_batchnorm_layer = 0
    num_sage_layer = 0
    batch = None
    update_scale = True
    layers = []
    prev_layer = None

    def __init__(self, name):
        self.initial_bits = config.initial_bits
        self.bits = config.activation_compression_bits[0]
        QScheme.layers.append(self)
        counters = {"linear": "num_lin_layer", "matmul": "num_matmul_layer",
                    "batchnorm": "num_batchnorm_layer", "sage": "num_sage_layer"}
        assert name in counters
        attr = counters[name]
        self.name = f"{name}_{getattr(QScheme, attr)}"
        setattr(QScheme, attr, getattr(QScheme, attr) + 1)

    def note_use(self):
        QScheme.prev_layer = self

    def compute_quantization_bits(self, input):  # noqa: A002
        """qsheme.py:41-48 -> (input_flatten, bits, min, max)."""
        self.note_use()
        N = input.shape[0]
        input_flatten = input.view(N, -1)
        mn, mx = ext_quantization.row_minmax(input_flatten)
        return input_flatten, config.activation_compression_bits[0], mn, mx
