// ReLU and dropout that keep only a 1-bit-per-element mask for backward.
//
// Semantics restated from the reference kernels
//   act_quantized_relu_{forward,backward}_kernel     quantization_cuda_kernel.cu:237-331
//   act_quantized_dropout_{forward,backward}_kernel  quantization_cuda_kernel.cu:442-594
// (host glue quantization.cc:66-84, 111-134).  The reference's mask bit order
// is private to its kernels; here bit (i % 32) of word (i / 32) belongs to
// element i, every word of the (n + 31) / 32-word mask is written in full, and
// nothing is written past it.
//
// Each lane owns one oct (8 consecutive elements, 32 B): its 8 mask bits are
// one byte, and four neighbouring lanes merge their bytes into the 32-bit
// mask word with two cross-lane ORs.

#include "exact_common.hpp"

namespace exact {

template <bool VEC4>
__device__ __forceinline__ void load8(const float* __restrict__ p, int nv, float (&v)[8]) {
  if (VEC4 && nv == 8) {
    const f32x4 a = nt_load4(p);
    const f32x4 b = nt_load4(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (i < nv) ? p[i] : 0.f;
  }
}

template <bool VEC4>
__device__ __forceinline__ void store8(float* __restrict__ p, int nv, const float (&v)[8]) {
  if (VEC4 && nv == 8) {
    nt_store4(p, v[0], v[1], v[2], v[3]);
    nt_store4(p + 4, v[4], v[5], v[6], v[7]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < nv) p[i] = v[i];
  }
}

// Merge the mask bytes of lanes 4m..4m+3 into one word; lane 4m stores it.
__device__ __forceinline__ void store_mask_byte(uint32_t byte, int64_t oct, int64_t n,
                                                uint32_t* __restrict__ mask) {
  uint32_t w = byte << (8 * (threadIdx.x & 3));
  w |= __shfl_xor(w, 1);
  w |= __shfl_xor(w, 2);
  if ((threadIdx.x & 3) == 0 && oct * 8 < n) mask[oct >> 2] = w;
}

__device__ __forceinline__ uint32_t load_mask_byte(const uint32_t* __restrict__ mask, int64_t oct) {
  return (mask[oct >> 2] >> (8 * (oct & 3))) & 0xFFu;
}

template <bool VEC4>
__global__ __launch_bounds__(kBlock) void relu_fwd_kernel(const float* __restrict__ x, int64_t n,
                                                          float* __restrict__ y,
                                                          uint32_t* __restrict__ mask) {
  const int64_t oct = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t left = n - oct * 8;
  const int nv = left >= 8 ? 8 : (left > 0 ? static_cast<int>(left) : 0);
  float v[8];
  uint32_t byte = 0;
  if (nv > 0) {
    load8<VEC4>(x + oct * 8, nv, v);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bool bit = v[i] > 0.f;  // quantization_cuda_kernel.cu:252-257
      v[i] = bit ? v[i] : 0.f;
      byte |= static_cast<uint32_t>(bit && i < nv) << i;
    }
    store8<VEC4>(y + oct * 8, nv, v);
  }
  store_mask_byte(byte, oct, n, mask);
}

template <bool VEC4>
__global__ __launch_bounds__(kBlock) void relu_bwd_kernel(const float* __restrict__ dy,
                                                          const uint32_t* __restrict__ mask, int64_t n,
                                                          float* __restrict__ dx) {
  const int64_t oct = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t left = n - oct * 8;
  if (left <= 0) return;
  const int nv = left >= 8 ? 8 : static_cast<int>(left);
  float v[8];
  load8<VEC4>(dy + oct * 8, nv, v);
  const uint32_t byte = load_mask_byte(mask, oct);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = ((byte >> i) & 1u) ? v[i] : 0.f;  // :305-310
  store8<VEC4>(dx + oct * 8, nv, v);
}

template <bool VEC4, bool NOISE_IN>
__global__ __launch_bounds__(kBlock) void dropout_fwd_kernel(const float* __restrict__ x,
                                                             const float* __restrict__ noise,
                                                             uint32_t seed_lo, uint32_t seed_hi,
                                                             uint32_t off_lo, uint32_t off_hi, float p,
                                                             float pinv, int64_t n, float* __restrict__ y,
                                                             uint32_t* __restrict__ mask) {
  const int64_t oct = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t left = n - oct * 8;
  const int nv = left >= 8 ? 8 : (left > 0 ? static_cast<int>(left) : 0);
  uint32_t byte = 0;
  if (nv > 0) {
    float v[8], u[8];
    load8<VEC4>(x + oct * 8, nv, v);
    if constexpr (NOISE_IN) {
      load8<VEC4>(noise + oct * 8, nv, u);
    } else {
      const Philox4 r = philox4x32_10(static_cast<uint32_t>(oct), static_cast<uint32_t>(oct >> 32),
                                      off_lo, off_hi, seed_lo, seed_hi);
      philox_uniform8(r, u);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const bool keep = u[i] > p;  // quantization_cuda_kernel.cu:465-468
      const float kf = keep ? 1.f : 0.f;
      float r = v[i] * kf;  // :490, left to right
      r = r * pinv;
      v[i] = r;
      byte |= static_cast<uint32_t>(keep && i < nv) << i;
    }
    store8<VEC4>(y + oct * 8, nv, v);
  }
  store_mask_byte(byte, oct, n, mask);
}

template <bool VEC4>
__global__ __launch_bounds__(kBlock) void dropout_bwd_kernel(const float* __restrict__ dy,
                                                             const uint32_t* __restrict__ mask, float p1m,
                                                             int64_t n, float* __restrict__ dx) {
  const int64_t oct = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  const int64_t left = n - oct * 8;
  if (left <= 0) return;
  const int nv = left >= 8 ? 8 : static_cast<int>(left);
  float v[8];
  load8<VEC4>(dy + oct * 8, nv, v);
  const uint32_t byte = load_mask_byte(mask, oct);
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = ((byte >> i) & 1u) ? v[i] / p1m : 0.f;  // :565-569
  store8<VEC4>(dx + oct * 8, nv, v);
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Octs rounded up to whole mask words (4 octs), then to workgroups.
static dim3 oct_grid(int64_t n) {
  const int64_t octs = ((n + 31) / 32) * 4;
  return dim3(static_cast<unsigned>((octs + kBlock - 1) / kBlock));
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_relu_fwd_f32(const float* x, int64_t n, float* y, uint32_t* mask, void* stream) {
  if (n < 0 || n > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (n == 0) return EXACT_OK;
  if (!x || !y || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (aligned16(x) && aligned16(y))
    hipLaunchKernelGGL((relu_fwd_kernel<true>), oct_grid(n), dim3(kBlock), 0, s, x, n, y, mask);
  else
    hipLaunchKernelGGL((relu_fwd_kernel<false>), oct_grid(n), dim3(kBlock), 0, s, x, n, y, mask);
  return launch_status();
}

int exact_relu_bwd_f32(const float* dy, const uint32_t* mask, int64_t n, float* dx, void* stream) {
  if (n < 0 || n > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (n == 0) return EXACT_OK;
  if (!dy || !dx || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (aligned16(dy) && aligned16(dx))
    hipLaunchKernelGGL((relu_bwd_kernel<true>), oct_grid(n), dim3(kBlock), 0, s, dy, mask, n, dx);
  else
    hipLaunchKernelGGL((relu_bwd_kernel<false>), oct_grid(n), dim3(kBlock), 0, s, dy, mask, n, dx);
  return launch_status();
}

int exact_dropout_fwd_f32(const float* x, const float* noise, uint64_t seed, uint64_t offset, float p,
                          int64_t n, float* y, uint32_t* mask, void* stream) {
  if (n < 0 || n > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (!(p >= 0.f && p < 1.f)) return EXACT_E_ARG;
  if (n == 0) return EXACT_OK;
  if (!x || !y || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // quantization_cuda_kernel.cu:456: float pinv = 1. / (1. - p), evaluated in double
  const float pinv = static_cast<float>(1.0 / (1.0 - static_cast<double>(p)));
  const uint32_t sl = static_cast<uint32_t>(seed), sh = static_cast<uint32_t>(seed >> 32);
  const uint32_t ol = static_cast<uint32_t>(offset), oh = static_cast<uint32_t>(offset >> 32);
  const bool v4 = aligned16(x) && aligned16(y) && (!noise || aligned16(noise));
  const dim3 grid = oct_grid(n);
  if (noise) {
    if (v4) hipLaunchKernelGGL((dropout_fwd_kernel<true, true>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
    else hipLaunchKernelGGL((dropout_fwd_kernel<false, true>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
  } else {
    if (v4) hipLaunchKernelGGL((dropout_fwd_kernel<true, false>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
    else hipLaunchKernelGGL((dropout_fwd_kernel<false, false>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
  }
  return launch_status();
}

int exact_dropout_bwd_f32(const float* dy, const uint32_t* mask, float p, int64_t n, float* dx,
                          void* stream) {
  if (n < 0 || n > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (!(p >= 0.f && p < 1.f)) return EXACT_E_ARG;
  if (n == 0) return EXACT_OK;
  if (!dy || !dx || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // quantization.cc:121,127: p1m = 1. - p stored as double, read back into a float
  const float p1m = static_cast<float>(1.0 - static_cast<double>(p));
  if (aligned16(dy) && aligned16(dx))
    hipLaunchKernelGGL((dropout_bwd_kernel<true>), oct_grid(n), dim3(kBlock), 0, s, dy, mask, p1m, n, dx);
  else
    hipLaunchKernelGGL((dropout_bwd_kernel<false>), oct_grid(n), dim3(kBlock), 0, s, dy, mask, p1m, n, dx);
  return launch_status();
}

}  // extern "C"
