"""Per-layer quantisation scheme objects (the reference's QScheme,
exact/exact/qsheme.py:8-47): every quantised layer owns one; it names the
layer and can report the per-row range its activation is quantised over.
The bit width is always config.activation_compression_bits[0]."""
from .conf import config
from .cpp_extension import quantization as ext_quantization

_KINDS = ("linear", "matmul", "batchnorm", "sage")


class QScheme(object):
    layers = []          # every scheme ever created, in creation order
    prev_layer = None    # the scheme of the most recent quantisation
    _created = dict.fromkeys(_KINDS, 0)

    def __init__(self, name):
        if name not in _KINDS:
            raise ValueError(f"unknown layer kind {name!r}")
        self.initial_bits = config.initial_bits
        self.bits = config.activation_compression_bits[0]
        self.name = f"{name}_{QScheme._created[name]}"
        QScheme._created[name] += 1
        QScheme.layers.append(self)

    def note_use(self):
        QScheme.prev_layer = self

    def compute_quantization_bits(self, input):  # noqa: A002
        """-> (input viewed [N, -1], bits, row min, row max)  (qsheme.py:41-48)."""
        self.note_use()
        flat = input.reshape(input.shape[0], -1)
        lo, hi = ext_quantization.row_minmax(flat)
        return flat, config.activation_compression_bits[0], lo, hi
