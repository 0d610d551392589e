// The remaining sparse kernels of the reference's spmm extension:
//   * max / min aggregation with the arg-entry output
//     (spmm_kernel<.., MAX|MIN, ..> spmm_cuda.cu:27-104, Reducer reducer.cuh:43-85);
//   * the gradient with respect to the edge values, a sampled dense-dense
//     product (spmm_value_bw_kernel spmm_cuda.cu:172-209).
// Neither is on the sum / mean path of the GCN / GraphSAGE benchmarks; they are
// plain one-wavefront-per-row (resp. per-entry) kernels, 64 lanes spanning
// 64 * VEC feature columns.

#include "exact_common.hpp"

namespace exact {

template <int VEC>
__device__ __forceinline__ void load_cols(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 4) { const float4 q = *reinterpret_cast<const float4*>(p); v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
  else if constexpr (VEC == 2) { const float2 q = *reinterpret_cast<const float2*>(p); v[0] = q.x; v[1] = q.y; }
  else { v[0] = *p; }
}

// out[r, k] = max / min over the entries e of row r of val[e] * X[col[e], k];
// arg_out[r, k] = the entry index that attained it (first one in CSR order),
// nnz for rows without entries, whose output is 0 (reducer.cuh:77-84).
template <typename I, int VEC, bool HAS_VAL, bool IS_MAX>
__global__ __launch_bounds__(kBlock) void spmm_minmax_kernel(const I* __restrict__ rowptr,
                                                             const I* __restrict__ col,
                                                             const float* __restrict__ val,
                                                             const float* __restrict__ X, int64_t M, int64_t K,
                                                             int64_t nnz, float* __restrict__ out,
                                                             I* __restrict__ arg_out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + (threadIdx.x >> 6);
  if (r >= M) return;
  const int64_t kcol = (static_cast<int64_t>(blockIdx.y) * kWave + lane) * VEC;
  if (kcol >= K) return;
  const int64_t rs = static_cast<int64_t>(rowptr[r]), re = static_cast<int64_t>(rowptr[r + 1]);
  float best[VEC];
  int64_t arg[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) {
    best[c] = IS_MAX ? -3.402823466e+38f : 3.402823466e+38f;  // numeric_limits lowest() / max(), reducer.cuh:47-50
    arg[c] = nnz;
  }
  for (int64_t e = rs; e < re; ++e) {
    const int64_t cidx = static_cast<int64_t>(col[e]);
    float xv[VEC];
    load_cols<VEC>(X + cidx * K + kcol, xv);
    const float w = HAS_VAL ? val[e] : 1.f;
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      const float t = HAS_VAL ? w * xv[c] : xv[c];
      if (IS_MAX ? (t > best[c]) : (t < best[c])) {  // strict: the first extreme entry wins
        best[c] = t;
        arg[c] = e;
      }
    }
  }
#pragma unroll
  for (int c = 0; c < VEC; ++c) {
    out[r * K + kcol + c] = (re > rs) ? best[c] : 0.f;
    arg_out[r * K + kcol + c] = static_cast<I>((re > rs) ? arg[c] : nnz);
  }
}

// Deterministic sum / mean: one wavefront per row (and per slab of 64 * VEC
// columns), the row's entries taken one after the other in CSR order with one
// multiply and one add each -- the summation order of the reference kernel
// (spmm_cuda.cu:85-90) and of the CPU oracle, so results are reproducible bit
// for bit.  No atomics, every output element is stored exactly once.  Hub rows
// serialise, which is why the default path is the chunked kernel in spmm.hip.
template <typename I, int VEC, bool HAS_VAL, bool MEAN>
__global__ __launch_bounds__(kBlock) void spmm_rowwise_kernel(const I* __restrict__ rowptr,
                                                              const I* __restrict__ col,
                                                              const float* __restrict__ val,
                                                              const float* __restrict__ X, int64_t M, int64_t K,
                                                              float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t r = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + (threadIdx.x >> 6);
  if (r >= M) return;
  const int64_t kcol = (static_cast<int64_t>(blockIdx.y) * kWave + lane) * VEC;
  if (kcol >= K) return;
  const int64_t rs = static_cast<int64_t>(rowptr[r]), re = static_cast<int64_t>(rowptr[r + 1]);
  float acc[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) acc[c] = 0.f;
  for (int64_t e = rs; e < re; ++e) {
    float xv[VEC];
    load_cols<VEC>(X + static_cast<int64_t>(col[e]) * K + kcol, xv);
    const float w = HAS_VAL ? val[e] : 1.f;
#pragma unroll
    for (int c = 0; c < VEC; ++c) {
      const float term = HAS_VAL ? w * xv[c] : xv[c];
      acc[c] = acc[c] + term;
    }
  }
  if (MEAN) {
    const float cnt = static_cast<float>(re > rs ? re - rs : 1);  // reducer.cuh:75-76
#pragma unroll
    for (int c = 0; c < VEC; ++c) acc[c] = acc[c] / cnt;
  }
#pragma unroll
  for (int c = 0; c < VEC; ++c) out[r * K + kcol + c] = acc[c];
}

// out[e] = sum_k mat[col[e], k] * grad[row[e], k]   (/ max(deg(row[e]), 1) for mean)
template <typename I, int VEC, bool MEAN>
__global__ __launch_bounds__(kBlock) void sddmm_kernel(const I* __restrict__ row, const I* __restrict__ rowptr,
                                                       const I* __restrict__ col, const float* __restrict__ mat,
                                                       const float* __restrict__ grad, int64_t E, int64_t K,
                                                       float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t e = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + (threadIdx.x >> 6);
  if (e >= E) return;  // whole wavefront
  const int64_t r = static_cast<int64_t>(row[e]), c = static_cast<int64_t>(col[e]);
  const float* mrow = mat + c * K;
  const float* grow = grad + r * K;
  float acc = 0.f;
  for (int64_t k = static_cast<int64_t>(lane) * VEC; k < K; k += kWave * VEC) {
    float a[VEC], b[VEC];
    load_cols<VEC>(mrow + k, a);
    load_cols<VEC>(grow + k, b);
#pragma unroll
    for (int i = 0; i < VEC; ++i) acc = __fmaf_rn(a[i], b[i], acc);
  }
  for (int m = kWave / 2; m > 0; m >>= 1) acc += __shfl_xor(acc, m);
  if (lane == 0) {
    if (MEAN) {
      const int64_t deg = static_cast<int64_t>(rowptr[r + 1]) - static_cast<int64_t>(rowptr[r]);
      acc /= static_cast<float>(deg > 0 ? deg : 1);
    }
    out[e] = acc;
  }
}

static bool aligned_to(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

template <typename I, int VEC>
static void minmax_dispatch(const I* rowptr, const I* col, const float* val, const float* X, int64_t M, int64_t K,
                            int64_t nnz, bool is_max, float* out, I* arg_out, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>((M + 3) / 4), static_cast<unsigned>((K + kWave * VEC - 1) / (kWave * VEC)));
  const dim3 block(kBlock);
  if (val) {
    if (is_max) hipLaunchKernelGGL((spmm_minmax_kernel<I, VEC, true, true>), grid, block, 0, s, rowptr, col, val, X, M, K, nnz, out, arg_out);
    else hipLaunchKernelGGL((spmm_minmax_kernel<I, VEC, true, false>), grid, block, 0, s, rowptr, col, val, X, M, K, nnz, out, arg_out);
  } else {
    if (is_max) hipLaunchKernelGGL((spmm_minmax_kernel<I, VEC, false, true>), grid, block, 0, s, rowptr, col, val, X, M, K, nnz, out, arg_out);
    else hipLaunchKernelGGL((spmm_minmax_kernel<I, VEC, false, false>), grid, block, 0, s, rowptr, col, val, X, M, K, nnz, out, arg_out);
  }
}

template <typename I, int VEC>
static void sddmm_dispatch(const I* row, const I* rowptr, const I* col, const float* mat, const float* grad, int64_t E,
                           int64_t K, bool mean, float* out, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>((E + 3) / 4));
  if (mean) hipLaunchKernelGGL((sddmm_kernel<I, VEC, true>), grid, dim3(kBlock), 0, s, row, rowptr, col, mat, grad, E, K, out);
  else hipLaunchKernelGGL((sddmm_kernel<I, VEC, false>), grid, dim3(kBlock), 0, s, row, rowptr, col, mat, grad, E, K, out);
}

template <typename I, int VEC>
static void rowwise_dispatch(const I* rowptr, const I* col, const float* val, const float* X, int64_t M, int64_t K,
                             bool mean, float* out, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>((M + 3) / 4), static_cast<unsigned>((K + kWave * VEC - 1) / (kWave * VEC)));
  const dim3 block(kBlock);
  if (val) {
    if (mean) hipLaunchKernelGGL((spmm_rowwise_kernel<I, VEC, true, true>), grid, block, 0, s, rowptr, col, val, X, M, K, out);
    else hipLaunchKernelGGL((spmm_rowwise_kernel<I, VEC, true, false>), grid, block, 0, s, rowptr, col, val, X, M, K, out);
  } else {
    if (mean) hipLaunchKernelGGL((spmm_rowwise_kernel<I, VEC, false, true>), grid, block, 0, s, rowptr, col, val, X, M, K, out);
    else hipLaunchKernelGGL((spmm_rowwise_kernel<I, VEC, false, false>), grid, block, 0, s, rowptr, col, val, X, M, K, out);
  }
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_spmm_csr_minmax_f32(const void* rowptr, const void* col, const float* val, int idx_bytes, const float* X,
                              int64_t M, int64_t n_cols, int64_t K, int64_t nnz, int is_max, float* out,
                              void* arg_out, void* stream) {
  if (idx_bytes != 4 && idx_bytes != 8) return EXACT_E_ARG;
  if (M < 0 || K < 0 || nnz < 0 || n_cols < 0 || n_cols > 0x7FFFFFFFll) return EXACT_E_SHAPE;
  if (idx_bytes == 4 && nnz > 0x7FFFFFFFll) return EXACT_E_SHAPE;
  if (M > (int64_t{1} << 32) || K > (int64_t{1} << 24)) return EXACT_E_SHAPE;  // launch-grid limits
  if (M == 0 || K == 0) return EXACT_OK;
  if (!rowptr || !out || !arg_out || (nnz > 0 && (!col || !X))) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int vec = (K % 4 == 0 && aligned_to(X, 16)) ? 4 : (K % 2 == 0 && aligned_to(X, 8)) ? 2 : 1;
#define EXACT_MM_GO(I, V) \
  minmax_dispatch<I, V>(static_cast<const I*>(rowptr), static_cast<const I*>(col), val, X, M, K, nnz, is_max != 0, out, static_cast<I*>(arg_out), s)
  if (idx_bytes == 4) {
    if (vec == 4) EXACT_MM_GO(int32_t, 4); else if (vec == 2) EXACT_MM_GO(int32_t, 2); else EXACT_MM_GO(int32_t, 1);
  } else {
    if (vec == 4) EXACT_MM_GO(int64_t, 4); else if (vec == 2) EXACT_MM_GO(int64_t, 2); else EXACT_MM_GO(int64_t, 1);
  }
#undef EXACT_MM_GO
  return launch_status();
}

int exact_sddmm_f32(const void* row, const void* rowptr, const void* col, int idx_bytes, const float* mat,
                    const float* grad, int64_t nnz, int64_t K, int reduce, float* out, void* stream) {
  if (idx_bytes != 4 && idx_bytes != 8) return EXACT_E_ARG;
  if (reduce != EXACT_REDUCE_SUM && reduce != EXACT_REDUCE_MEAN) return EXACT_E_ARG;
  if (nnz < 0 || K < 0 || nnz > (int64_t{1} << 32)) return EXACT_E_SHAPE;  // one wavefront per entry, 4 per workgroup
  if (nnz == 0) return EXACT_OK;
  if (!row || !rowptr || !col || !mat || !grad || !out) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int vec = (K % 4 == 0 && aligned_to(mat, 16) && aligned_to(grad, 16)) ? 4
                  : (K % 2 == 0 && aligned_to(mat, 8) && aligned_to(grad, 8)) ? 2 : 1;
  const bool mean = reduce == EXACT_REDUCE_MEAN;
#define EXACT_SD_GO(I, V) \
  sddmm_dispatch<I, V>(static_cast<const I*>(row), static_cast<const I*>(rowptr), static_cast<const I*>(col), mat, grad, nnz, K, mean, out, s)
  if (idx_bytes == 4) {
    if (vec == 4) EXACT_SD_GO(int32_t, 4); else if (vec == 2) EXACT_SD_GO(int32_t, 2); else EXACT_SD_GO(int32_t, 1);
  } else {
    if (vec == 4) EXACT_SD_GO(int64_t, 4); else if (vec == 2) EXACT_SD_GO(int64_t, 2); else EXACT_SD_GO(int64_t, 1);
  }
#undef EXACT_SD_GO
  return launch_status();
}

int exact_spmm_csr_rowwise_f32(const void* rowptr, const void* col, const float* val, int idx_bytes, const float* X,
                               int64_t M, int64_t n_cols, int64_t K, int64_t nnz, int reduce, float* out,
                               void* stream) {
  if (idx_bytes != 4 && idx_bytes != 8) return EXACT_E_ARG;
  if (reduce != EXACT_REDUCE_SUM && reduce != EXACT_REDUCE_MEAN) return EXACT_E_ARG;
  if (M < 0 || K < 0 || nnz < 0 || n_cols < 0 || n_cols > 0x7FFFFFFFll) return EXACT_E_SHAPE;
  if (idx_bytes == 4 && nnz > 0x7FFFFFFFll) return EXACT_E_SHAPE;
  if (M > (int64_t{1} << 32) || K > (int64_t{1} << 24)) return EXACT_E_SHAPE;  // launch-grid limits
  if (M == 0 || K == 0) return EXACT_OK;
  if (!rowptr || !out || (nnz > 0 && (!col || !X))) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const bool mean = reduce == EXACT_REDUCE_MEAN;
  const int vec = (K % 4 == 0 && aligned_to(X, 16)) ? 4 : (K % 2 == 0 && aligned_to(X, 8)) ? 2 : 1;
#define EXACT_RW_GO(I, V) \
  rowwise_dispatch<I, V>(static_cast<const I*>(rowptr), static_cast<const I*>(col), val, X, M, K, mean, out, s)
  if (idx_bytes == 4) {
    if (vec == 4) EXACT_RW_GO(int32_t, 4); else if (vec == 2) EXACT_RW_GO(int32_t, 2); else EXACT_RW_GO(int32_t, 1);
  } else {
    if (vec == 4) EXACT_RW_GO(int64_t, 4); else if (vec == 2) EXACT_RW_GO(int64_t, 2); else EXACT_RW_GO(int64_t, 1);
  }
#undef EXACT_RW_GO
  return launch_status();
}

}  // extern "C"
