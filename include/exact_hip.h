/*
 * exact_hip.h -- C ABI of libexact_hip.so, the gfx950 (MI355X) implementation
 * of EXACT's activation-compression and sparse-aggregation hot path.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer unless
 *     stated otherwise; the caller allocates every output; the library never
 *     allocates, frees or keeps a pointer after the call returns;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); work
 *     is enqueued on it and the call returns without synchronising;
 *   - return value: 0 = ok, negative = argument error (EXACT_E_*), positive =
 *     the hipError_t of a failed launch;
 *   - re-entrant, no global state.
 *
 * Each declaration cites the interface of the reference extension it replaces
 * (paths relative to exact/exact/cpp_extension/ of the reference unless they
 * name another file).
 */
#ifndef EXACT_HIP_H_
#define EXACT_HIP_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define EXACT_ABI_VERSION 1

#define EXACT_OK 0
#define EXACT_E_NULL (-1)      /* a required pointer is NULL                    */
#define EXACT_E_BITS (-2)      /* bits not in {1,2,4,8} (8 % bits != 0)          */
#define EXACT_E_SHAPE (-3)     /* negative / overflowing / unsupported size      */
#define EXACT_E_ALIGN (-4)     /* pointer alignment the kernel needs is missing  */
#define EXACT_E_ARG (-5)       /* any other bad argument (reduce, idx_bytes, p)  */

#define EXACT_REDUCE_SUM 0
#define EXACT_REDUCE_MEAN 1

int exact_abi_version(void);
/* Static string for a return code (EXACT_E_* name or hipGetErrorString). */
const char *exact_strerror(int code);

/* Bytes of the packed stream for an [N, G] activation at `bits`:
 * (bits * N_round * G + 8) / 8 with N_round = N rounded up to 8/bits rows --
 * the allocation of pack_single_precision_cuda, quantization_cuda_kernel.cu:107-113
 * (the final byte is padding; this library writes it as 0). */
int64_t exact_packed_nbytes(int64_t N, int64_t G, int bits);

/* a1. Per-row minimum and maximum of x[N, G] (row-major fp32).
 * Replaces the two torch reductions of QScheme.compute_quantization_bits
 * (qsheme.py:41-48) / no_scheme_compute_quantization_bits (ops.py:61-66). */
int exact_row_minmax_f32(const float *x, int64_t N, int64_t G,
                         float *mn, float *mx, void *stream);

/* a3. Stochastic-rounding quantise + bit-pack with caller-supplied per-row
 * min and scale: replaces pack_single_precision(data, min, max, scale, bits,
 * stochastic) (quantization.cc:37-48 -> quantization_cuda_kernel.cu:63-155).
 *   q = rn(fmax((x - mn[n]) * scale[n] + u - 0.5, 0)), unfused fp32;
 *   byte[(n / wpt) * G + d] |= q << ((n % wpt) * bits), wpt = 8 / bits.
 * noise: fp32 [N, G] uniforms to use as u, or NULL to draw u from the
 * library's Philox4x32-10 stream keyed by (seed, offset) (16 random bits per
 * element, u = (h + 0.5) / 65536; counter = (d / 8, n, offset_lo, offset_hi)).
 * packed must hold exact_packed_nbytes(N, G, bits) bytes. */
int exact_pack_f32(const float *x, const float *mn, const float *scale,
                   const float *noise, uint64_t seed, uint64_t offset,
                   int64_t N, int64_t G, int bits, uint8_t *packed, void *stream);

/* a1+a2+a3(+a4) fused: one read of x produces per-row min, scale =
 * (2^bits - 1) / (max - min) (ops.py:39), the packed stream, and optionally
 * the bf16 copies that quantize_activation returns (ops.py:80-81).
 * Any of scale_f32 / min_f32 / scale_bf16 / min_bf16 may be NULL (skipped),
 * except that rows longer than 1024 columns need scale_f32 and min_f32.
 * Replaces quantize_activation's chain ops.py:69-83. */
int exact_minmax_pack_f32(const float *x, const float *noise, uint64_t seed,
                          uint64_t offset, int64_t N, int64_t G, int bits,
                          uint8_t *packed, float *scale_f32, float *min_f32,
                          uint16_t *scale_bf16, uint16_t *min_bf16, void *stream);

/* The same with the work split chosen by the caller: octs_per_lane = 1, 2 or 4
 * consecutive 8-column groups per lane (0 = the library's default; a value the
 * row length does not allow is ignored).  The result does not depend on it;
 * the host side times the alternatives once per (G, bits) and keeps the
 * fastest. */
int exact_minmax_pack_geom_f32(const float *x, const float *noise, uint64_t seed,
                               uint64_t offset, int64_t N, int64_t G, int bits,
                               uint8_t *packed, float *scale_f32, float *min_f32,
                               uint16_t *scale_bf16, uint16_t *min_bf16,
                               int octs_per_lane, void *stream);

/* a5. Unpack + dequantise: out[n, d] = float(field) / scale[n] + mn[n].
 * Replaces unpack_single_precision(data, bits, scale, min, N, group_size)
 * (quantization.cc:50-62 -> quantization_cuda_kernel.cu:158-229). */
int exact_unpack_f32(const uint8_t *packed, int bits, const float *scale,
                     const float *mn, int64_t N, int64_t G, float *out, void *stream);

/* a6. Same with scale / min given as bf16 bit patterns (what
 * quantize_activation returned): folds the bf16 -> fp32 widening of
 * dequantize_activation (ops.py:92-98) into the kernel. */
int exact_unpack_bf16param_f32(const uint8_t *packed, int bits,
                               const uint16_t *scale_bf16, const uint16_t *min_bf16,
                               int64_t N, int64_t G, float *out, void *stream);

/* a13. ReLU that keeps a 1-bit mask: y = x > 0 ? x : 0; bit (i % 32) of
 * mask[i / 32] = (x[i] > 0).  mask holds (n + 31) / 32 int32 words, all of
 * them fully written.  Replaces act_quantized_relu_forward_cuda /
 * act_quantized_relu_backward_cuda (quantization_cuda_kernel.cu:237-331). */
int exact_relu_fwd_f32(const float *x, int64_t n, float *y, uint32_t *mask, void *stream);
int exact_relu_bwd_f32(const float *dy, const uint32_t *mask, int64_t n, float *dx, void *stream);

/* a14. Dropout that keeps a 1-bit keep mask: keep = u > p,
 * y = x * keep * (1 / (1 - p)); backward dx = keep ? dy / (1 - p) : 0.
 * noise NULL -> Philox (counter = (i / 8, offset)).  0 <= p < 1.
 * Replaces act_quantized_dropout_forward_cuda / _backward_cuda
 * (quantization_cuda_kernel.cu:442-594; quantization.cc:111-134). */
int exact_dropout_fwd_f32(const float *x, const float *noise, uint64_t seed,
                          uint64_t offset, float p, int64_t n, float *y,
                          uint32_t *mask, void *stream);
int exact_dropout_bwd_f32(const float *dy, const uint32_t *mask, float p,
                          int64_t n, float *dx, void *stream);

/* a10 / a11. CSR SpMM out[M, K] = reduce_{e in row r} val[e] * X[col[e], :].
 * rowptr has M + 1 entries, col / val have nnz; idx_bytes is 4 (int32) or 8
 * (int64) for both index arrays; val may be NULL (implicit ones); X is
 * [n_cols, K] row-major fp32; nnz = rowptr[M] (passed in so the host never
 * reads device memory); reduce is EXACT_REDUCE_SUM or _MEAN (mean divides by
 * max(row length, 1)).  The entry stream is cut into equal chunks, one per
 * wavefront, so hub rows are split across wavefronts.  Replaces spmm_cuda (spmm_cuda.cu:106-170,
 * kernel :27-104, Reducer reducer.cuh:43-85); the backward products of
 * spmm_sum_bw / spmm_mean_bw (spmm.cc:57-79, 115-139) are the same call on
 * the CSC arrays. */
int exact_spmm_csr_f32(const void *rowptr, const void *col, const float *val,
                       int idx_bytes, const float *X, int64_t M, int64_t n_cols,
                       int64_t K, int64_t nnz, int reduce, float *out, void *stream);

/* The same with explicit row strides (in elements, >= K) of X and out, for
 * operands that are column slices of wider buffers -- e.g. rows padded to a
 * multiple of 128 bytes, which the 512-byte gathers of the kernel like. */
int exact_spmm_csr_strided_f32(const void *rowptr, const void *col, const float *val,
                               int idx_bytes, const float *X, int64_t ldx, int64_t M,
                               int64_t n_cols, int64_t K, int64_t nnz, int reduce,
                               float *out, int64_t ldo, void *stream);

/* The same product with a reproducible result: one wavefront per row, entries
 * added in CSR order with one multiply and one add each (the order of the
 * reference kernel, spmm_cuda.cu:85-90), no atomics.  Slower on hub rows. */
int exact_spmm_csr_rowwise_f32(const void *rowptr, const void *col, const float *val,
                               int idx_bytes, const float *X, int64_t M, int64_t n_cols,
                               int64_t K, int64_t nnz, int reduce, float *out, void *stream);

/* Max / min aggregation: out[r, k] = max (is_max != 0) or min over the entries
 * e of row r of val[e] * X[col[e], k]; arg_out[r, k] (same index type as
 * rowptr / col, [M, K]) = the first entry index attaining it; rows without
 * entries give out = 0 and arg_out = nnz.  Replaces spmm_cuda(..., "max" |
 * "min") as called by spmm_max_fw / spmm_min_fw (spmm.cc:145-157, 199-212;
 * kernel spmm_cuda.cu:27-104 with Reducer<MAX|MIN> reducer.cuh:43-85). */
int exact_spmm_csr_minmax_f32(const void *rowptr, const void *col, const float *val,
                              int idx_bytes, const float *X, int64_t M, int64_t n_cols,
                              int64_t K, int64_t nnz, int is_max, float *out,
                              void *arg_out, void *stream);

/* Gradient with respect to the edge values: out[e] = sum_k mat[col[e], k] *
 * grad[row[e], k], divided by max(length of row[e], 1) for EXACT_REDUCE_MEAN.
 * row is the COO row index of every entry.  Replaces spmm_value_bw_cuda
 * (spmm_cuda.cu:172-252) as called by spmm_sum_bw / spmm_mean_bw
 * (spmm.cc:65-67, 123-125). */
int exact_sddmm_f32(const void *row, const void *rowptr, const void *col, int idx_bytes,
                    const float *mat, const float *grad, int64_t nnz, int64_t K,
                    int reduce, float *out, void *stream);

/* LeakyReLU with the 1-bit mask of a13: y = x > 0 ? x : x * slope;
 * dx = bit ? dy : dy * slope.  Replaces act_quantized_leakyrelu_forward_cuda /
 * _backward_cuda (quantization_cuda_kernel.cu:339-435). */
int exact_leaky_relu_fwd_f32(const float *x, int64_t n, float slope, float *y,
                             uint32_t *mask, void *stream);
int exact_leaky_relu_bwd_f32(const float *dy, const uint32_t *mask, int64_t n,
                             float slope, float *dx, void *stream);

/* ELU backward on the decompressed input: dx = x >= 0 ? dy : alpha * dy * exp(x).
 * Replaces _elu_backward_cuda (backward_func_cuda_kernel.cu:6-36) as called by
 * qelu.backward (ops.py:195-203).  exact_elu_bwd_f16: the same on fp16 tensors. */
int exact_elu_bwd_f32(const float *dy, const float *x, float alpha, int64_t n,
                      float *dx, void *stream);
int exact_elu_bwd_f16(const uint16_t *dy, const uint16_t *x, float alpha, int64_t n,
                      uint16_t *dx, void *stream);

/* Column sums of a row-major [N, K] fp32 matrix, out[k] = sum_n x[n, k], K <= 8192.  Replaces `grad_output.sum(0)`, the bias gradient of
 * linear_backward (backward_func.cc:90-91), whose library reduction is far off
 * the memory roofline for narrow matrices.  fp32 atomics: the summation order
 * is not fixed. */
int exact_colsum_f32(const float *x, int64_t N, int64_t K, float *out, void *stream);

/* The two column reductions of a training-mode batch norm's backward over
 * row-major [N, K] fp32 matrices, K <= 256, in one pass:
 *   sum_dy[k] = sum_n dy[n, k],  sum_dy_xmu[k] = sum_n dy[n, k] * (x[n, k] - mean[k]).
 * Replaces the reduction inside at::native_batch_norm_backward as called by
 * qbatch_norm.backward (ops.py:228-254); the element-wise half of that routine
 * stays the framework's.  fp32 atomics: the summation order is not fixed. */
int exact_bn_backward_reduce_f32(const float *dy, const float *x, const float *mean, int64_t N, int64_t K,
                                 float *sum_dy, float *sum_dy_xmu, void *stream);

/* Centred column moments of a row-major [N, K] fp32 matrix, K <= 256, in one pass:
 *   sum_d[k] = sum_n (x[n, k] - center[k]),  sum_d2[k] = sum_n (x[n, k] - center[k])^2,
 * from which mean = center + sum_d / N and the biased variance = sum_d2 / N - (sum_d / N)^2
 * (free of cancellation when `center` is near the column means, e.g. the mean of a few rows).
 * Replaces the batch statistics inside at::native_batch_norm as called by
 * qbatch_norm.forward (ops.py:213) where the normalisation itself is folded
 * into the next pass.  fp32 atomics: the summation order is not fixed. */
int exact_col_moments_f32(const float *x, const float *center, int64_t N, int64_t K, float *sum_d, float *sum_d2,
                          void *stream);

/* FOR BENCHMARKS ONLY -- not part of the operator interface; no product code calls it and a binding of the
 * reference's operators has no use for it.  Measurement aid with no counterpart in the reference: the memory
 * traffic of the pack kernel without its arithmetic.  Every lane reads 64 bytes of x (n floats,
 * whole tiles of 4096 floats; the remainder is not touched) and writes
 * out_bytes (0, 2, 4, 8 or 16: what 1 / 2 / 4 / 8 bits per element make of 16
 * elements) to `out`, which holds (n / 16) * out_bytes bytes (at least 16).  x
 * and out 16-byte aligned.  bench.py times it beside the pack kernels: what it
 * reaches is what the device's memory system delivers for that read/write mix. */
int exact_stream_probe_f32(const float *x, int64_t n, int out_bytes, void *out, void *stream);

/* Weight gradient of a linear layer, dW[Kout, D] = dY[N, Kout]^T . X[N, D], row-major
 * fp32 with row strides ldy >= Kout and ldx >= D (in elements), N >> Kout, D.
 * Replaces `grad_output.t().mm(input)` of linear_backward (backward_func.cc:88-89)
 * with an fp32 matrix-core kernel shaped for the long reduction.  The row range
 * is cut into slabs combined by fp32 atomics: the summation order is not fixed. */
int exact_linear_dw_f32(const float *dY, int64_t ldy, const float *X, int64_t ldx, int64_t N,
                        int64_t Kout, int64_t D, float *out, void *stream);
/* The same product on the bf16 matrix cores at fp32 accuracy: both operands are split, without error, into three
 * bf16 pieces and six bf16 products replace each fp32 product (the neglected ones are below 2^-24 of it).  Same
 * arguments and limits; results agree with exact_linear_dw_f32 to fp32 rounding. */
int exact_linear_dw_bf16_f32(const float *dY, int64_t ldy, const float *X, int64_t ldx, int64_t N,
                             int64_t Kout, int64_t D, float *out, void *stream);

/* Fused epilogues (no single counterpart in the reference: each replaces a
 * chain of its calls with one pass over the data, bit-identical to the chain).
 *
 * ReLU then dropout: y = dropout(relu(x)) with ONE mask, bit = (x > 0) && keep;
 * replaces act_quantized_relu followed by act_quantized_dropout
 * (quantization.cc:66-84, 111-134).  The backward of the pair is
 * exact_dropout_bwd_f32 on that mask.  Noise as in exact_dropout_fwd_f32. */
int exact_relu_dropout_fwd_f32(const float *x, const float *noise, uint64_t seed,
                               uint64_t offset, float p, int64_t n, float *y,
                               uint32_t *mask, void *stream);

/* ReLU, dropout and the quantisation of the result (the next layer's saved
 * input) in one pass over x[N, G]: y and mask as exact_relu_dropout_fwd_f32
 * with (act_noise | act_seed, act_offset); packed / scale / min as
 * exact_minmax_pack_f32 applied to y with (noise | seed, offset).  Replaces
 * layers.py:288-292 + :321-325 + the quantize_activation of the following
 * qlinear (ops.py:149).  Needs G % 8 == 0, G <= 1024, 16-byte aligned x, y and
 * noise (else EXACT_E_SHAPE / EXACT_E_ALIGN: call the separate entry points);
 * act_noise and noise are both given or both NULL. */
int exact_relu_dropout_minmax_pack_f32(const float *x, float p, const float *act_noise,
                                       uint64_t act_seed, uint64_t act_offset,
                                       const float *noise, uint64_t seed, uint64_t offset,
                                       int64_t N, int64_t G, int bits, float *y,
                                       uint32_t *mask, uint8_t *packed, float *scale_f32,
                                       float *min_f32, uint16_t *scale_bf16,
                                       uint16_t *min_bf16, void *stream);

/* The same pass with training-mode batch norm ahead of the ReLU: every element
 * of column c first becomes (x - mean[c]) * mult[c] + shift[c] (three separate
 * fp32 operations), i.e. native_batch_norm's weight * (x - mean) * invstd + bias
 * (layers.py:340-369, ops.py:206-225) with mult = weight * invstd and the batch
 * statistics supplied by the caller; then ReLU, dropout, mask and the packed
 * copy of the result exactly as exact_relu_dropout_minmax_pack_f32.  mean,
 * mult and shift are fp32[G], 16-byte aligned.  Same shape conditions. */
int exact_bn_relu_dropout_minmax_pack_f32(const float *x, const float *mean, const float *mult,
                                          const float *shift, float p, const float *act_noise,
                                          uint64_t act_seed, uint64_t act_offset,
                                          const float *noise, uint64_t seed, uint64_t offset,
                                          int64_t N, int64_t G, int bits, float *y,
                                          uint32_t *mask, uint8_t *packed, float *scale_f32,
                                          float *min_f32, uint16_t *scale_bf16,
                                          uint16_t *min_bf16, void *stream);

/* fp16 activations (row f4: the reference instantiates its kernels for
 * at::Half as well -- AT_DISPATCH_FLOATING_TYPES_AND_HALF at
 * quantization_cuda_kernel.cu:132-150, 209-226, 284, 324, 387, 428, 535, 586 --
 * and its Functions cast their inputs to fp16 under autocast, ops.py:130, 260,
 * 313).  fp16 tensors are passed as uint16_t bit patterns.  The arithmetic
 * follows at::Half's operators (evaluate in fp32, round the result to fp16):
 *   scale = h(h(1 / h(max - min)) * (2^bits - 1));
 *   q = rn(fmax(h(h(x - min) * scale) + u - 0.5, 0));
 *   unpacked = h(h(q / scale) + min);
 * G <= 1024 (the reference's block-size limit). */
int exact_minmax_pack_f16(const uint16_t *x, const float *noise, uint64_t seed,
                          uint64_t offset, int64_t N, int64_t G, int bits,
                          uint8_t *packed, uint16_t *scale_f16, uint16_t *min_f16,
                          void *stream);
int exact_unpack_f16(const uint8_t *packed, int bits, const uint16_t *scale_f16,
                     const uint16_t *min_f16, int64_t N, int64_t G, uint16_t *out_f16,
                     void *stream);
/* The mask activations on fp16 tensors: same masks, values rounded to fp16 once
 * on store (y = h(x * keep * pinv), dx = h(dy / (1 - p)), y = h(x * slope)). */
int exact_relu_fwd_f16(const uint16_t *x, int64_t n, uint16_t *y, uint32_t *mask, void *stream);
int exact_relu_bwd_f16(const uint16_t *dy, const uint32_t *mask, int64_t n, uint16_t *dx, void *stream);
int exact_leaky_relu_fwd_f16(const uint16_t *x, int64_t n, float slope, uint16_t *y,
                             uint32_t *mask, void *stream);
int exact_leaky_relu_bwd_f16(const uint16_t *dy, const uint32_t *mask, int64_t n,
                             float slope, uint16_t *dx, void *stream);
int exact_dropout_fwd_f16(const uint16_t *x, const float *noise, uint64_t seed,
                          uint64_t offset, float p, int64_t n, uint16_t *y,
                          uint32_t *mask, void *stream);
int exact_relu_dropout_fwd_f16(const uint16_t *x, const float *noise, uint64_t seed,
                               uint64_t offset, float p, int64_t n, uint16_t *y,
                               uint32_t *mask, void *stream);
int exact_dropout_bwd_f16(const uint16_t *dy, const uint32_t *mask, float p,
                          int64_t n, uint16_t *dx, void *stream);

/* a7. Random projection: out[N, k] = X[N, D] . R[D, k]  (input2rp, ops.py:107-118)
 * and back: out[N, D] = Xr[N, k] . R[D, k]^T  (rp2input, ops.py:121-125).
 * fp32 in, fp32 accumulate on the matrix cores. */
int exact_rp_fwd_f32(const float *X, const float *R, int64_t N, int64_t D,
                     int64_t k, float *out, void *stream);
int exact_rp_bwd_f32(const float *Xr, const float *R, int64_t N, int64_t D,
                     int64_t k, float *out, void *stream);

/* Projection and quantisation in one launch: what exact_rp_fwd_f32 followed by
 * exact_minmax_pack_f32 (on the [N, k] product, G = k) computes, bit for bit,
 * without the [N, k] tensor reaching memory -- input2rp then
 * quantize_activation as qlinear.forward and QSAGEConv.forward chain them
 * (ops.py:141-149, layers.py:153-159).  k <= 128.  noise: NULL or [N, k]
 * uniforms; seed / offset, packed, scale and min outputs as in
 * exact_minmax_pack_f32 (packed holds exact_packed_nbytes(N, k, bits) bytes). */
int exact_rp_minmax_pack_f32(const float *X, const float *R, const float *noise, uint64_t seed,
                             uint64_t offset, int64_t N, int64_t D, int64_t k, int bits,
                             uint8_t *packed, float *scale_f32, float *min_f32,
                             uint16_t *scale_bf16, uint16_t *min_bf16, void *stream);

/* The same three products on the bf16 matrix cores (v_mfma_f32_32x32x16_bf16,
 * fp32 accumulate) at fp32 accuracy: every fp32 operand is split, without error,
 * into three bf16 pieces.  No counterpart in the reference beyond the two
 * torch.matmul calls of ops.py:117,124 (which ran on TF32 tensor cores there).
 *   mode EXACT_RP_BF16_SIGNS  R = +-c with one c > 0, the matrix the reference
 *        draws (ops.py:112-114: (2 * Bernoulli(1/2) - 1) / sqrt(k)); only the
 *        signs of R are used and the product is scaled once by c = |R[0][0]|.
 *        The caller vouches that |R| is the same everywhere and not 0.
 *   mode EXACT_RP_BF16_SPLIT  any R: six bf16 products per fp32 product, the
 *        neglected ones below 2^-24 of it.
 * The kernels read R as a TABLE of matrix-core operand fragments, which
 * exact_rp_prepare_bf16 writes from R[D, k] (row-major fp32) into a buffer of
 * exact_rp_table_nbytes(D, k, mode) bytes (16-byte aligned) that the caller
 * allocates and owns; one table serves all three products for as long as R,
 * D, k and mode stay the same.  exact_rp_table_nbytes returns 0 for shapes
 * the kernels do not take (k > 128).
 * exact_rp_minmax_pack_bf16_f32 equals exact_rp_fwd_bf16_f32 followed by
 * exact_minmax_pack_f32 bit for bit (same mode).  Results differ from the
 * fp32-matrix-core entry points above in the last bits (different order and
 * number of roundings); both are within fp32 rounding of the exact product.
 * Non-finite inputs: a row of X holding inf or NaN gives NaN in that row. */
#define EXACT_RP_BF16_SPLIT 1
#define EXACT_RP_BF16_SIGNS 2
int64_t exact_rp_table_nbytes(int64_t D, int64_t k, int mode);
int exact_rp_prepare_bf16(const float *R, int64_t D, int64_t k, int mode, void *table, void *stream);
int exact_rp_fwd_bf16_f32(const float *X, const void *table, int64_t N, int64_t D, int64_t k, int mode,
                          float *out, void *stream);
int exact_rp_bwd_bf16_f32(const float *Xr, const void *table, int64_t N, int64_t D, int64_t k, int mode,
                          float *out, void *stream);
int exact_rp_minmax_pack_bf16_f32(const float *X, const void *table, int mode, const float *noise,
                                  uint64_t seed, uint64_t offset, int64_t N, int64_t D, int64_t k,
                                  int bits, uint8_t *packed, float *scale_f32, float *min_f32,
                                  uint16_t *scale_bf16, uint16_t *min_bf16, void *stream);

/* The dense products of a layer around the compressed activation: out[N, K] =
 * X[N, D] . M[D, K] (+ bias[K]) (+ addend[N, K]), row-major fp32, N >> D, K.
 * Replaces `F.linear(input, weight, bias)` of qlinear.forward (ops.py:150) with
 * M = weight^T, and `grad_output.mm(weight)` of linear_backward
 * (backward_func.cc:85-86) with M = weight, by the forward projection kernel
 * above in its any-matrix form: M is split without error into three bf16
 * matrices and six bf16 matrix-core products stand for each fp32 product (the
 * neglected ones are below 2^-24 of it), accumulated in fp32.  No atomics: the
 * result is reproducible.
 * exact_tall_gemm_prepare_bf16 writes the operand fragments of M into `table`
 * (exact_tall_gemm_table_nbytes(D, K) bytes, 16-byte aligned, owned by the
 * caller, valid while M is unchanged); M has row stride `ld` elements and is
 * read as M[d * ld + c], or as M[c * ld + d] when `transposed` is 1 (a weight
 * [K, D] as F.linear holds it).
 * exact_tall_gemm_bf16_f32: X contiguous [N, D], D even, 8-byte aligned (16-byte
 * loads are used when D % 4 == 0 and X is 16-byte aligned, else 8-byte ones),
 * D and K at most 4096; `bias` and `addend` may be NULL; `addend` (row stride
 * ldc) may be `out` itself (row stride ldo >= K): out += X . M. */
int64_t exact_tall_gemm_table_nbytes(int64_t D, int64_t K);
int exact_tall_gemm_prepare_bf16(const float *M, int64_t ld, int transposed, int64_t D, int64_t K,
                                 void *table, void *stream);
int exact_tall_gemm_bf16_f32(const float *X, const void *table, int64_t N, int64_t D, int64_t K,
                             const float *bias, const float *addend, int64_t ldc, float *out,
                             int64_t ldo, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* EXACT_HIP_H_ */
