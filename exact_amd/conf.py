"""Global quantisation config: same singleton and field names as the
reference's exact/exact/conf.py:1-24, read at call time by the ops."""


class QuantizationConfig:
    def __init__(self):
        self.compress_activation = True
        self.activation_compression_bits = [2]
        self.initial_bits = 8
        self.stochastic = True
        self.use_gradient = False
        self.simulate = False
        self.enable_quantized_bn = True
        self.kept_frac = 1.0
        self.single_precision = True
        self.dropout2 = False
        # Memory management flags
        self.empty_cache_threshold = None
        self.swap = False
        self.amp = False
        # Debug flags
        self.debug_memory_op_forward = False
        self.debug_memory_op_backward = False
        self.debug_remove_bn = False
        self.debug_remove_relu = False
        self.debug_remove_dropout = False

        # ---- additions of this implementation (not in the reference) ----
        # Distribution of the random-projection matrix: "rademacher" is what
        # the reference draws (ops.py:112-114); "gaussian" is N(0, 1/k).
        self.rp_distribution = "rademacher"
        # None: the kernels draw their own Philox noise, keyed by torch's CUDA
        # generator.  A callable (shape, device) -> fp32 tensor of uniforms in
        # [0, 1) supplies the noise instead (stochastic rounding and dropout);
        # parity tests use this to feed the oracle and the kernels the same bits.
        self.noise_source = None
        # None: input2rp draws the projection matrix on the device.  A callable
        # (D, k, device) -> fp32 [D, k] tensor supplies it instead.
        self.rp_matrix_source = None


config = QuantizationConfig()
