// Column sums of a row-major [N, K] fp32 matrix: out[k] = sum_n x[n, k].
//
// The bias gradient of the reference's linear backward (`grad_output.sum(0)`,
// backward_func.cc:90-91).  The matrix is read as one flat stream of 16-byte
// quads whatever K is (element e belongs to column e % K; a lane tracks its
// column incrementally, so there is no division in the loop); every workgroup
// sums its share of the stream into K bins in LDS with LDS atomics and then
// adds its bins to the output with one global atomic per non-zero bin.  The
// order of the fp32 additions therefore varies from run to run (callers that
// need a reproducible sum use a sequential reduction instead).

#include "exact_common.hpp"

namespace exact {

constexpr int kColsumMaxK = 8192;   // bins held in LDS (32 KB)
constexpr int kColsumUnroll = 4;    // quads in flight per lane

__global__ __launch_bounds__(kBlock) void colsum_zero_kernel(float* __restrict__ out, int64_t K) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i < K) out[i] = 0.f;
}

__global__ __launch_bounds__(kBlock) void colsum_kernel(const float* __restrict__ x, int64_t total, int K,
                                                        int64_t quads_per_wg, float* __restrict__ out) {
  HIP_DYNAMIC_SHARED(float, bins)  // [K]
  const int t = threadIdx.x;
  for (int i = t; i < K; i += kBlock) bins[i] = 0.f;
  __syncthreads();
  const int64_t nquads = total / 4;
  const int64_t q0 = static_cast<int64_t>(blockIdx.x) * quads_per_wg;
  const int64_t q1 = (q0 + quads_per_wg < nquads) ? q0 + quads_per_wg : nquads;
  // column of the first element of this lane's first quad, and the advance per step
  int64_t q = q0 + t;
  int col = static_cast<int>((4 * q) % K);
  const int step = static_cast<int>((4LL * kBlock) % K);
  auto add_quad = [&](const f32x4& v, int c) {
    unsafeAtomicAdd(&bins[c], v.x);
    c = (c + 1 == K) ? 0 : c + 1;
    unsafeAtomicAdd(&bins[c], v.y);
    c = (c + 1 == K) ? 0 : c + 1;
    unsafeAtomicAdd(&bins[c], v.z);
    c = (c + 1 == K) ? 0 : c + 1;
    unsafeAtomicAdd(&bins[c], v.w);
  };
  for (; q + (kColsumUnroll - 1) * kBlock < q1; q += kColsumUnroll * kBlock) {
    f32x4 v[kColsumUnroll];
#pragma unroll
    for (int u = 0; u < kColsumUnroll; ++u) v[u] = nt_load4(x + 4 * (q + u * kBlock));
#pragma unroll
    for (int u = 0; u < kColsumUnroll; ++u) {
      add_quad(v[u], col);
      col += step;
      col = col >= K ? col - K : col;
    }
  }
  for (; q < q1; q += kBlock) {
    add_quad(nt_load4(x + 4 * q), col);
    col += step;
    col = col >= K ? col - K : col;
  }
  if (blockIdx.x == 0 && t == 0) {  // the up to three elements after the last whole quad
    for (int64_t e = nquads * 4; e < total; ++e) unsafeAtomicAdd(&bins[e % K], x[e]);
  }
  __syncthreads();
  for (int i = t; i < K; i += kBlock) {
    const float s = bins[i];
    if (s != 0.f) unsafeAtomicAdd(out + i, s);
  }
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_colsum_f32(const float* x, int64_t N, int64_t K, float* out, void* stream) {
  if (N < 0 || K < 0 || K > kColsumMaxK || N > (int64_t{1} << 40) / (K > 0 ? K : 1)) return EXACT_E_SHAPE;
  if (K == 0) return EXACT_OK;
  if (!out || (N > 0 && !x)) return EXACT_E_NULL;
  if ((reinterpret_cast<uintptr_t>(x) & 15u) != 0) return EXACT_E_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipLaunchKernelGGL(colsum_zero_kernel, dim3(static_cast<unsigned>((K + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, out, K);
  const int64_t total = N * K;
  if (total > 0) {
    const int64_t nquads = total / 4;
    // enough workgroups to fill the chip several times over, each with at least 16 KiB of the stream
    int64_t wgs = (nquads + 1023) / 1024;
    if (wgs > 4096) wgs = 4096;
    if (wgs < 1) wgs = 1;
    const int64_t quads_per_wg = (nquads + wgs - 1) / wgs;
    hipLaunchKernelGGL(colsum_kernel, dim3(static_cast<unsigned>(wgs)), dim3(kBlock), static_cast<size_t>(K) * sizeof(float), s,
                       x, total, static_cast<int>(K), quads_per_wg, out);
  }
  return launch_status();
}

}  // extern "C"
