// Column sums of a row-major [N, K] fp32 matrix: out[k] = sum_n x[n, k].
//
// The bias gradient of the reference's linear backward (`grad_output.sum(0)`,
// backward_func.cc:90-91).  The matrix is read as one flat stream, element e
// belonging to column e % K.  A workgroup takes a block of rows; thread t owns
// the stream positions t, t + P, t + 2P, .. of every "pass" of P elements, where
// P is a multiple of K (P = K * floor(256 / K) for K <= 256, else K rounded up
// to the threads), so the columns a thread meets never change and its partial
// sums stay in registers; consecutive threads read consecutive addresses.  The
// partial sums of the threads that share a column meet in LDS, and every
// workgroup then adds its K sums to the output with one global atomic each, so
// the order of the fp32 additions varies from run to run (callers that need a
// reproducible sum use a sequential reduction instead).

#include "exact_common.hpp"

namespace exact {

constexpr int kColsumMaxK = 8192;
constexpr int kColsumCols = kColsumMaxK / kBlock;  // columns per thread at most (K > 256)
constexpr int kColsumUnroll = 8;                   // loads in flight per thread

__global__ __launch_bounds__(kBlock) void colsum_zero_kernel(float* __restrict__ out, int64_t K) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i < K) out[i] = 0.f;
}

// Rows of at most 256 units (a unit is VEC = 1 or 4 consecutive columns, one
// load): a pass is `rpp` whole rows = rpp * K / VEC consecutive units, one per thread.
//
// PAIR: two sums in one pass over two matrices, out[k] = sum_n x[n, k] and
// out2[k] = sum_n x[n, k] * (y[n, k] - center[k]) -- the two column reductions
// of a batch norm's backward (sum of the incoming gradient, and of its product
// with the centred input).
//
// MOMENTS (with PAIR's extra outputs, one matrix): out[k] = sum_n (x[n, k] - center[k])
// and out2[k] = sum_n (x[n, k] - center[k])^2, from which the caller forms the
// column mean and variance; centring near the column mean (the caller passes
// the mean of the first rows) keeps the difference of the two moments free of
// cancellation.
template <int VEC, bool PAIR, bool MOMENTS = false>
__global__ __launch_bounds__(kBlock) void colsum_narrow_kernel(const float* __restrict__ x, const float* __restrict__ y,
                                                               const float* __restrict__ center, int64_t N, int K,
                                                               int rpp, int64_t rows_per_wg, float* __restrict__ out,
                                                               float* __restrict__ out2) {
  __shared__ float part[kBlock * VEC];
  __shared__ float part2[(PAIR || MOMENTS) ? kBlock * VEC : 1];
  const int t = threadIdx.x;
  const int upr = K / VEC;     // units per row
  const int span = rpp * upr;  // active threads == units per pass
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * rows_per_wg;
  const int64_t r1 = (r0 + rows_per_wg < N) ? r0 + rows_per_wg : N;
  constexpr int U = PAIR ? kColsumUnroll / 2 : kColsumUnroll;  // loads in flight per thread and matrix
  float acc[VEC], acc2[VEC], ctr[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) acc[c] = acc2[c] = ctr[c] = 0.f;
  auto load_unit = [&](const float* __restrict__ src, int64_t u, float (&v)[VEC]) {
    if constexpr (VEC == 4) {
      const f32x4 q = nt_load4(src + 4 * u);
      v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
    } else {
      v[0] = __builtin_nontemporal_load(src + u);
    }
  };
  if (t < span) {
    if constexpr (PAIR || MOMENTS) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) ctr[c] = center[(t % upr) * VEC + c];
    }
    const int64_t u1 = r1 * upr;
    int64_t u = r0 * upr + t;
    for (; u + static_cast<int64_t>(U - 1) * span < u1; u += static_cast<int64_t>(U) * span) {
      float v[U][VEC], w[PAIR ? U : 1][VEC];
#pragma unroll
      for (int i = 0; i < U; ++i) {
        load_unit(x, u + static_cast<int64_t>(i) * span, v[i]);
        if constexpr (PAIR) load_unit(y, u + static_cast<int64_t>(i) * span, w[i]);
      }
#pragma unroll
      for (int i = 0; i < U; ++i)
#pragma unroll
        for (int c = 0; c < VEC; ++c) {
          if constexpr (MOMENTS) {
            const float d = v[i][c] - ctr[c];
            acc[c] += d;
            acc2[c] = __fmaf_rn(d, d, acc2[c]);
          } else {
            acc[c] += v[i][c];
            if constexpr (PAIR) acc2[c] = __fmaf_rn(v[i][c], w[i][c] - ctr[c], acc2[c]);
          }
        }
    }
    for (; u < u1; u += span) {
      float v[VEC], w[VEC];
      load_unit(x, u, v);
      if constexpr (PAIR) load_unit(y, u, w);
#pragma unroll
      for (int c = 0; c < VEC; ++c) {
        if constexpr (MOMENTS) {
          const float d = v[c] - ctr[c];
          acc[c] += d;
          acc2[c] = __fmaf_rn(d, d, acc2[c]);
        } else {
          acc[c] += v[c];
          if constexpr (PAIR) acc2[c] = __fmaf_rn(v[c], w[c] - ctr[c], acc2[c]);
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < VEC; ++c) {
    part[t * VEC + c] = acc[c];  // thread t holds columns (t % upr) * VEC + c
    if constexpr (PAIR || MOMENTS) part2[t * VEC + c] = acc2[c];
  }
  __syncthreads();
  if (t < K) {
    // column t = unit t / VEC, component t % VEC, of every row of the pass
    float s = 0.f, s2 = 0.f;
    for (int i = t / VEC; i < span; i += upr) {
      s += part[i * VEC + t % VEC];
      if constexpr (PAIR || MOMENTS) s2 += part2[i * VEC + t % VEC];
    }
    if (s != 0.f) unsafeAtomicAdd(out + t, s);
    if constexpr (PAIR || MOMENTS) {
      if (s2 != 0.f) unsafeAtomicAdd(out2 + t, s2);
    }
  }
}

// K > 256: a pass is one row; thread t owns columns t, t + 256, ..
__global__ __launch_bounds__(kBlock) void colsum_wide_kernel(const float* __restrict__ x, int64_t N, int K,
                                                             int64_t rows_per_wg, float* __restrict__ out) {
  const int t = threadIdx.x;
  const int64_t r0 = static_cast<int64_t>(blockIdx.x) * rows_per_wg;
  const int64_t r1 = (r0 + rows_per_wg < N) ? r0 + rows_per_wg : N;
  float acc[kColsumCols];
#pragma unroll
  for (int c = 0; c < kColsumCols; ++c) acc[c] = 0.f;
  for (int64_t r = r0; r < r1; ++r) {
    const float* row = x + r * K;
#pragma unroll
    for (int c = 0; c < kColsumCols; ++c) {
      const int k = t + c * kBlock;
      if (k < K) acc[c] += __builtin_nontemporal_load(row + k);
    }
  }
#pragma unroll
  for (int c = 0; c < kColsumCols; ++c) {
    const int k = t + c * kBlock;
    if (k < K && acc[c] != 0.f) unsafeAtomicAdd(out + k, acc[c]);
  }
}

}  // namespace exact

using namespace exact;

// Every workgroup ends with one atomic add per column into the SAME K words,
// and atomics on one address are served one after the other: a few hundred
// long-lived workgroups (about 1024, at least 16 KiB of the stream each)
// instead of thousands of short ones.
static int64_t colsum_rows_per_wg(int64_t N, int64_t K) {
  int64_t rows = (N + 1023) / 1024;
  const int64_t least = (4096 + K - 1) / K;
  return rows < least ? least : rows;
}

extern "C" {

int exact_colsum_f32(const float* x, int64_t N, int64_t K, float* out, void* stream) {
  if (N < 0 || K < 0 || K > kColsumMaxK || N > (int64_t{1} << 40) / (K > 0 ? K : 1)) return EXACT_E_SHAPE;
  if (K == 0) return EXACT_OK;
  if (!out || (N > 0 && !x)) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(colsum_zero_kernel, dim3(static_cast<unsigned>((K + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, out, K);
  if (N > 0) {
    int64_t rows_per_wg = colsum_rows_per_wg(N, K);
    const dim3 grid(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg));
    if (K <= kBlock) {
      const bool vec4 = (K % 4 == 0) && (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
      const int rpp = static_cast<int>(kBlock / (vec4 ? K / 4 : K));
      rows_per_wg = (rows_per_wg + rpp - 1) / rpp * rpp;  // whole passes
      const dim3 g2(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg));
      const float* none = nullptr;
      float* none_out = nullptr;
      if (vec4) hipLaunchKernelGGL((colsum_narrow_kernel<4, false>), g2, dim3(kBlock), 0, s, x, none, none, N, static_cast<int>(K), rpp, rows_per_wg, out, none_out);
      else hipLaunchKernelGGL((colsum_narrow_kernel<1, false>), g2, dim3(kBlock), 0, s, x, none, none, N, static_cast<int>(K), rpp, rows_per_wg, out, none_out);
    } else {
      hipLaunchKernelGGL(colsum_wide_kernel, grid, dim3(kBlock), 0, s, x, N, static_cast<int>(K), rows_per_wg, out);
    }
  }
  return launch_status();
}

int exact_bn_backward_reduce_f32(const float* dy, const float* x, const float* mean, int64_t N, int64_t K,
                                 float* sum_dy, float* sum_dy_xmu, void* stream) {
  if (N < 0 || K < 0 || K > kBlock || N > (int64_t{1} << 40) / (K > 0 ? K : 1)) return EXACT_E_SHAPE;
  if (K == 0) return EXACT_OK;
  if (!sum_dy || !sum_dy_xmu || !mean || (N > 0 && (!dy || !x))) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 zgrid(static_cast<unsigned>((K + kBlock - 1) / kBlock));
  hipLaunchKernelGGL(colsum_zero_kernel, zgrid, dim3(kBlock), 0, s, sum_dy, K);
  hipLaunchKernelGGL(colsum_zero_kernel, zgrid, dim3(kBlock), 0, s, sum_dy_xmu, K);
  if (N > 0) {
    const bool vec4 = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(dy) | reinterpret_cast<uintptr_t>(x)) & 15u) == 0;
    const int rpp = static_cast<int>(kBlock / (vec4 ? K / 4 : K));
    int64_t rows_per_wg = colsum_rows_per_wg(N, K);
    rows_per_wg = (rows_per_wg + rpp - 1) / rpp * rpp;  // whole passes
    const dim3 grid(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg));
    if (vec4) hipLaunchKernelGGL((colsum_narrow_kernel<4, true>), grid, dim3(kBlock), 0, s, dy, x, mean, N, static_cast<int>(K), rpp, rows_per_wg, sum_dy, sum_dy_xmu);
    else hipLaunchKernelGGL((colsum_narrow_kernel<1, true>), grid, dim3(kBlock), 0, s, dy, x, mean, N, static_cast<int>(K), rpp, rows_per_wg, sum_dy, sum_dy_xmu);
  }
  return launch_status();
}

int exact_col_moments_f32(const float* x, const float* center, int64_t N, int64_t K, float* sum_d, float* sum_d2,
                          void* stream) {
  if (N < 0 || K < 0 || K > kBlock || N > (int64_t{1} << 40) / (K > 0 ? K : 1)) return EXACT_E_SHAPE;
  if (K == 0) return EXACT_OK;
  if (!sum_d || !sum_d2 || !center || (N > 0 && !x)) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 zgrid(static_cast<unsigned>((K + kBlock - 1) / kBlock));
  hipLaunchKernelGGL(colsum_zero_kernel, zgrid, dim3(kBlock), 0, s, sum_d, K);
  hipLaunchKernelGGL(colsum_zero_kernel, zgrid, dim3(kBlock), 0, s, sum_d2, K);
  if (N > 0) {
    const bool vec4 = (K % 4 == 0) && (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    const int rpp = static_cast<int>(kBlock / (vec4 ? K / 4 : K));
    int64_t rows_per_wg = colsum_rows_per_wg(N, K);
    rows_per_wg = (rows_per_wg + rpp - 1) / rpp * rpp;  // whole passes
    const dim3 grid(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg));
    const float* none = nullptr;
    if (vec4) hipLaunchKernelGGL((colsum_narrow_kernel<4, false, true>), grid, dim3(kBlock), 0, s, x, none, center, N, static_cast<int>(K), rpp, rows_per_wg, sum_d, sum_d2);
    else hipLaunchKernelGGL((colsum_narrow_kernel<1, false, true>), grid, dim3(kBlock), 0, s, x, none, center, N, static_cast<int>(K), rpp, rows_per_wg, sum_d, sum_d2);
  }
  return launch_status();
}

}  // extern "C"
