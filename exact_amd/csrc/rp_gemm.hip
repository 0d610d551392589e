// Random-projection compress / decompress as fp32 GEMMs on the gfx950 matrix
// cores (v_mfma_f32_32x32x2_f32, fp32 in, fp32 accumulate):
//   forward   out[N, k] = X[N, D]  . R[D, k]      (input2rp, ops.py:107-118)
//   backward  out[N, D] = Xr[N, k] . R[D, k]^T    (rp2input, ops.py:121-125)
// N is huge, D <= a few hundred, k = ceil-ish(kept_frac * D) is tens: both
// products are bound by streaming the [N, D] operand through HBM once.
//
// One wavefront owns 32 consecutive rows.  The streamed operand goes
// global -> registers directly: lane l reads VEC consecutive floats of row
// (l % 32) at column offset VEC * (l / 32), i.e. the two half-waves hold two
// different k-slices of the same 32 rows.  Because a dot product does not
// care in which order its terms are paired, MFMA step t multiplies element t
// of every lane's vector, with the small matrix R read from LDS at the k
// index that lane's element really has.  R is staged in LDS once per
// workgroup (zero-padded, so out-of-range k contributes 0).
//
// MFMA 32x32x2 f32 register layout (wave64): A-operand lane l = A[l % 32][l / 32],
// B-operand lane l = B[l / 32][l % 32]; accumulator register v of lane l is
// C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].

#include "exact_common.hpp"

namespace exact {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 32;       // MFMA M and N
constexpr int kFwdDChunk = 64;  // rows of R staged per LDS fill (forward)

template <int VEC>
__device__ __forceinline__ void load_k_slice(const float* __restrict__ p, int kk, int klimit, float (&a)[VEC]) {
#pragma unroll
  for (int t = 0; t < VEC; ++t) a[t] = 0.f;
  if constexpr (VEC == 4) {
    if (kk < klimit) { const float4 q = *reinterpret_cast<const float4*>(p + kk); a[0] = q.x; a[1] = q.y; a[2] = q.z; a[3] = q.w; }
  } else if constexpr (VEC == 2) {
    if (kk < klimit) { const float2 q = *reinterpret_cast<const float2*>(p + kk); a[0] = q.x; a[1] = q.y; }
  } else {
    if (kk < klimit) a[0] = p[kk];
  }
}

// out[N, k] = X[N, D] . R[D, k];  NT * 32 >= k columns per wavefront.
template <int VEC, int NT>
__global__ __launch_bounds__(kBlock) void rp_fwd_kernel(const float* __restrict__ X,
                                                        const float* __restrict__ R, int64_t N, int D,
                                                        int k, float* __restrict__ out) {
  HIP_DYNAMIC_SHARED(float, Rl)  // [kFwdDChunk][NT * 32]
  constexpr int KP = NT * kTile;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kTile;
  const int64_t my_row = (row0 + l32 < N) ? row0 + l32 : N - 1;
  const float* xrow = X + my_row * D;

  floatx16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

  for (int dc = 0; dc < D; dc += kFwdDChunk) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < kFwdDChunk * KP; idx += kBlock) {
      const int rr = idx / KP, cc = idx - rr * KP;
      Rl[idx] = (dc + rr < D && cc < k) ? R[static_cast<int64_t>(dc + rr) * k + cc] : 0.f;
    }
    __syncthreads();
    const int dlim = (D - dc < kFwdDChunk) ? D - dc : kFwdDChunk;
    for (int kb = 0; kb < dlim; kb += 2 * VEC) {
      const int ks = kb + VEC * half;  // this lane's k-slice inside the chunk
      float a[VEC];
      load_k_slice<VEC>(xrow, dc + ks, D, a);
#pragma unroll
      for (int t = 0; t < VEC; ++t) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          const float b = Rl[(ks + t) * KP + nt * kTile + l32];
          acc[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b, acc[nt], 0, 0, 0);
        }
      }
    }
  }

#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int cj = nt * kTile + l32;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int64_t rr = row0 + 8 * (v / 4) + 4 * half + (v % 4);
      if (rr < N && cj < k) out[rr * k + cj] = acc[nt][v];
    }
  }
}

// out[N, D] = Xr[N, k] . R[D, k]^T;  grid.y tiles D in slabs of NT * 32 columns.
template <int VEC, int NT>
__global__ __launch_bounds__(kBlock) void rp_bwd_kernel(const float* __restrict__ Xr,
                                                        const float* __restrict__ R, int64_t N, int D,
                                                        int k, int kpad, float* __restrict__ out) {
  HIP_DYNAMIC_SHARED(float, Rl)  // [NT * 32][kpad + 1], odd pitch: conflict-free column reads
  const int pitch = kpad + 1;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int dbase = blockIdx.y * (NT * kTile);
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kTile;
  const int64_t my_row = (row0 + l32 < N) ? row0 + l32 : N - 1;
  const float* xrow = Xr + my_row * k;

  for (int idx = threadIdx.x; idx < NT * kTile * kpad; idx += kBlock) {
    const int jj = idx / kpad, kk = idx - jj * kpad;
    Rl[jj * pitch + kk] = (dbase + jj < D && kk < k) ? R[static_cast<int64_t>(dbase + jj) * k + kk] : 0.f;
  }
  __syncthreads();

  floatx16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

  for (int kb = 0; kb < kpad; kb += 2 * VEC) {
    const int ks = kb + VEC * half;
    float a[VEC];
    load_k_slice<VEC>(xrow, ks, k, a);
#pragma unroll
    for (int t = 0; t < VEC; ++t) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const float b = Rl[(nt * kTile + l32) * pitch + ks + t];
        acc[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t], b, acc[nt], 0, 0, 0);
      }
    }
  }

#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int cj = dbase + nt * kTile + l32;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int64_t rr = row0 + 8 * (v / 4) + 4 * half + (v % 4);
      if (rr < N && cj < D) __builtin_nontemporal_store(acc[nt][v], out + rr * D + cj);
    }
  }
}

static bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static bool al8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

template <int VEC>
static int rp_fwd_launch(const float* X, const float* R, int64_t N, int D, int k, float* out, hipStream_t s) {
  const int nt = (k + kTile - 1) / kTile;
  const dim3 grid(static_cast<unsigned>((N + 127) / 128));
  const size_t lds = static_cast<size_t>(kFwdDChunk) * nt * kTile * sizeof(float);
  switch (nt) {
    case 1: hipLaunchKernelGGL((rp_fwd_kernel<VEC, 1>), grid, dim3(kBlock), lds, s, X, R, N, D, k, out); break;
    case 2: hipLaunchKernelGGL((rp_fwd_kernel<VEC, 2>), grid, dim3(kBlock), lds, s, X, R, N, D, k, out); break;
    case 3: hipLaunchKernelGGL((rp_fwd_kernel<VEC, 3>), grid, dim3(kBlock), lds, s, X, R, N, D, k, out); break;
    case 4: hipLaunchKernelGGL((rp_fwd_kernel<VEC, 4>), grid, dim3(kBlock), lds, s, X, R, N, D, k, out); break;
    default: return EXACT_E_SHAPE;
  }
  return launch_status();
}

template <int VEC>
static int rp_bwd_launch(const float* Xr, const float* R, int64_t N, int D, int k, float* out, hipStream_t s) {
  const int kpad = ((k + 2 * VEC - 1) / (2 * VEC)) * (2 * VEC);
  // output slab per workgroup: 128 columns, 64 when R's slab would not fit 64 KB of LDS
  const int nt = (kpad <= 96) ? 4 : 2;
  const dim3 grid(static_cast<unsigned>((N + 127) / 128), static_cast<unsigned>((D + nt * kTile - 1) / (nt * kTile)));
  const size_t lds = static_cast<size_t>(nt) * kTile * (kpad + 1) * sizeof(float);
  if (nt == 4) hipLaunchKernelGGL((rp_bwd_kernel<VEC, 4>), grid, dim3(kBlock), lds, s, Xr, R, N, D, k, kpad, out);
  else hipLaunchKernelGGL((rp_bwd_kernel<VEC, 2>), grid, dim3(kBlock), lds, s, Xr, R, N, D, k, kpad, out);
  return launch_status();
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_rp_fwd_f32(const float* X, const float* R, int64_t N, int64_t D, int64_t k, float* out,
                     void* stream) {
  if (N < 0 || D <= 0 || k <= 0 || D > (1 << 20) || k > 128) return EXACT_E_SHAPE;
  if (N == 0) return EXACT_OK;
  if (!X || !R || !out) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (D % 4 == 0 && al16(X)) return rp_fwd_launch<4>(X, R, N, static_cast<int>(D), static_cast<int>(k), out, s);
  if (D % 2 == 0 && al8(X)) return rp_fwd_launch<2>(X, R, N, static_cast<int>(D), static_cast<int>(k), out, s);
  return rp_fwd_launch<1>(X, R, N, static_cast<int>(D), static_cast<int>(k), out, s);
}

int exact_rp_bwd_f32(const float* Xr, const float* R, int64_t N, int64_t D, int64_t k, float* out,
                     void* stream) {
  if (N < 0 || D <= 0 || k <= 0 || D > (1 << 20) || k > 128) return EXACT_E_SHAPE;
  if (N == 0) return EXACT_OK;
  if (!Xr || !R || !out) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (k % 4 == 0 && al16(Xr)) return rp_bwd_launch<4>(Xr, R, N, static_cast<int>(D), static_cast<int>(k), out, s);
  if (k % 2 == 0 && al8(Xr)) return rp_bwd_launch<2>(Xr, R, N, static_cast<int>(D), static_cast<int>(k), out, s);
  return rp_bwd_launch<1>(Xr, R, N, static_cast<int>(D), static_cast<int>(k), out, s);
}

}  // extern "C"
