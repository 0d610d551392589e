"""QCustomGATConv: the attention layer of the reference's gatconv.py:147-172.
Only what the reference quantises is quantised: the linear maps (QLinear), the
LeakyReLU on the attention scores (1-bit mask) and the attention dropout
(1-bit mask); the residual projection stays a stock Linear, as there."""
from .cpp_extension import quantization as ext_quantization
from .layers import QDropout, QLinear
from .nn import CustomGATConv  # noqa: F401  (re-exported, as the reference module does)


class QCustomGATConv(CustomGATConv):
    def __init__(self, *args, **kwargs):
        super().__init__(*args, **kwargs)
        self._build_linears(QLinear)
        self.dropout_module = QDropout(p=self.dropout)
        self.reset_parameters()

    def _leaky_relu(self, score):
        return ext_quantization.act_quantized_leaky_relu(score, self.negative_slope)

    def _attention_dropout(self, alpha):
        return self.dropout_module(alpha)
