"""The global quantisation config.  A mutable module-level singleton with the
field names of the reference's QuantizationConfig (exact/exact/conf.py:3-22),
read by the ops at call time; the trainers of the reference set these fields
from their command lines, so the names are part of the API."""
import copy

# field -> default.  First block: the reference's fields, same defaults.
_REFERENCE_FIELDS = {
    "compress_activation": True,          # False: every Q-layer keeps full-precision activations
    "activation_compression_bits": [2],   # bits per element; element 0 is the one used
    "initial_bits": 8,
    "stochastic": True,                   # the kernels implement stochastic rounding only
    "use_gradient": False,
    "simulate": False,                    # the reference's tensor-op stand-in for the kernels (unpacked int32 codes)
    "enable_quantized_bn": True,          # QModule swaps BatchNorm1d only when set
    "kept_frac": 1.0,                     # < 1: random projection D -> int(kept_frac * D + 0.999)
    "single_precision": True,             # read at layer construction: attach QScheme objects
    "dropout2": False,                    # QModule uses QDropout2 instead of QDropout
    "empty_cache_threshold": None,
    "swap": False,                        # keep the packed codes in pinned host memory between fwd and bwd
    "amp": False,
    "debug_memory_op_forward": False,
    "debug_memory_op_backward": False,
    "debug_remove_bn": False,
    "debug_remove_relu": False,
    "debug_remove_dropout": False,
}

# Second block: additions of this implementation.
_EXTRA_FIELDS = {
    # Distribution of the projection matrix: "rademacher" (+-1/sqrt(k), what the
    # reference draws, ops.py:112-114) or "gaussian" (N(0, 1/k)).
    "rp_distribution": "rademacher",
    # Matrix-core path of the projection and weight-gradient kernels: "bf16" --
    # the bf16 instruction on fp32 operands split without error into three bf16
    # pieces (for the +-c projection matrices drawn here, on the signs alone);
    # "fp32" -- the fp32 instruction.  Both are within fp32 rounding of the exact
    # product; they differ from each other in the last bits.
    "matrix_cores": "bf16",
    # None: the kernels draw Philox noise keyed by torch's CUDA generator.  A
    # callable (shape, device) -> fp32 uniforms in [0, 1) supplies the noise of
    # stochastic rounding and dropout instead (parity tests feed the oracle and
    # the kernels the same bits this way).
    "noise_source": None,
    # None: input2rp draws the projection matrix.  A callable (D, k, device) ->
    # fp32 [D, k] supplies it instead.
    "rp_matrix_source": None,
    # The reference compresses and keeps the dense operand of every quantised
    # SpMM although backward reads it only for edge-value gradients; set this to
    # reproduce that memory behaviour.  Results do not depend on it.
    "keep_unused_spmm_operand": False,
    # ReLU -> dropout -> (quantise for the next layer) as one pass where the
    # model offers the pair as one module (QReLUDropout).  Results are
    # bit-identical to the separate layers; False runs them separately.
    "fuse_epilogue": True,
    # A QBatchNorm1d ahead of that pair joins the same pass (normalise -> ReLU ->
    # dropout -> quantise).  The batch statistics then come from torch.var_mean
    # instead of native_batch_norm, so results agree with the separate layers to
    # rounding (about 1e-6 relative), not bit for bit.  Needs fuse_epilogue.
    "fold_batch_norm": True,
    # QGCNConv as one autograd node (aggregate(x W^T) + b) that keeps what the
    # reference's chain qlinear -> qspmm keeps.  False: the chain.
    "gcn_single_node": True,
    # In that node the sparse product runs on the narrower side of the linear
    # map: (A X) W^T when in < out, and, where no input gradient is wanted,
    # dW = dY^T (A X_hat) instead of (A^T dY)^T X_hat.  Same numbers up to the
    # order of fp32 sums; nothing kept changes.
    "gcn_aggregate_narrow": True,
    # QSAGEConv as one autograd node (lin_l(aggregate(x)) + lin_r(x)) that keeps
    # what the reference's chain of three nodes keeps.  False: the chain.
    "sage_single_node": True,
    # In that node's backward, A^T (dY W_l) is computed as (A^T dY) W_l when the
    # layer narrows (out < in): the sparse product runs at the smaller width.
    # Same numbers up to the order of fp32 sums; nothing kept changes.
    "sage_reassociate_backward": True,
    # In that node's forward, with a projection (kept_frac < 1) and k + out < in,
    # aggregate x [R | W_l^T] instead of x: the layer's output and the copy lin_l
    # keeps are both linear in the aggregate.  The kept codes are those of
    # aggregate(x R) instead of aggregate(x) R: equal up to fp32 rounding ahead
    # of the quantiser (a stochastic rounding can fall the other way for a value
    # within an ulp of a boundary), so results agree with the chain to rounding,
    # not bit for bit.
    "sage_aggregate_projected": True,
    # Time the alternative work splits of the pack kernel (1, 2 or 4 column
    # groups per lane) the first time a large activation of a new (width, bits)
    # is compressed on a GPU, and keep the fastest.  Results do not depend on it.
    "autotune_pack": True,
    # Sparse products with a reproducible (CSR-order, atomics-free) summation;
    # also switched on by torch.use_deterministic_algorithms(True).  The default
    # kernel balances hub rows across wavefronts and adds their parts atomically.
    "deterministic_spmm": False,
    # Column sums, weight gradients, batch statistics and the batch-norm
    # backward reductions combine partial results with fp32 atomics (no fixed
    # summation order: the last bits vary from run to run).  True sends all four
    # to the framework's own, reproducible routines, as
    # torch.use_deterministic_algorithms(True) does.
    "deterministic_reductions": False,
    # The dense products of a layer (x W^T, dY W) go to the library's bf16
    # matrix-core kernel (config.matrix_cores == "bf16") from this many rows on;
    # shorter operands keep the framework's GEMM, which is as fast there.
    "tall_gemm_min_rows": 16384,
    # ... when the result has at most 64 columns (20 - 35 % faster than the
    # framework's fp32 GEMM there) or the reduction runs over at least this many
    # features (10 - 20 % faster at 256 and 604; slower at 100 - 128).
    "tall_gemm_min_depth": 192,
    # ... and, for such wide results, at most this many rows: at 2.4 M rows the
    # framework's GEMM reaches 127 TFLOP/s and the two are equal.
    "tall_gemm_max_rows_wide": 1000000,
}


class QuantizationConfig:
    def __init__(self):
        for table in (_REFERENCE_FIELDS, _EXTRA_FIELDS):
            for name, default in table.items():
                setattr(self, name, copy.copy(default))

    def __repr__(self):
        return "QuantizationConfig(" + ", ".join(f"{k}={v!r}" for k, v in vars(self).items()) + ")"


config = QuantizationConfig()
