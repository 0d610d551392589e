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
// Each lane owns two quads (4 consecutive elements, one 16-byte access each):
// quad t and quad t + 256 of its workgroup's 512-quad tile, so every vector
// memory instruction of a wavefront covers 1 KiB of consecutive addresses.
// The 4 mask bits of a quad are a nibble; eight neighbouring lanes merge their
// nibbles into one 32-bit mask word with three DPP ORs.  Dropout noise comes
// from one Philox block per 8 consecutive elements: the even lane of a lane
// pair draws the block of the pair's first quad, the odd lane that of its
// second quad, and the two trade halves.

#include "exact_common.hpp"

namespace exact {

constexpr int kTileQuads = 2 * kBlock;  // quads per workgroup

// Element type T is float or half_t (fp16: the reference instantiates these
// kernels for at::Half as well; values are widened to fp32 on load and rounded
// to fp16 once on store, which is what at::Half arithmetic amounts to here).
typedef half_t half4_t __attribute__((ext_vector_type(4)));

template <bool VEC4>
__device__ __forceinline__ void load4(const float* __restrict__ p, int nv, float (&v)[4]) {
  if (VEC4 && nv == 4) {
    const f32x4 a = nt_load4(p);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (i < nv) ? p[i] : 0.f;
  }
}
template <bool VEC4>
__device__ __forceinline__ void load4(const half_t* __restrict__ p, int nv, float (&v)[4]) {
  if (VEC4 && nv == 4) {
    const half4_t a = __builtin_nontemporal_load(reinterpret_cast<const half4_t*>(p));
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = static_cast<float>(a[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (i < nv) ? static_cast<float>(p[i]) : 0.f;
  }
}

template <bool VEC4>
__device__ __forceinline__ void store4(float* __restrict__ p, int nv, const float (&v)[4]) {
  if (VEC4 && nv == 4) {
    nt_store4(p, v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nv) p[i] = v[i];
  }
}
template <bool VEC4>
__device__ __forceinline__ void store4(half_t* __restrict__ p, int nv, const float (&v)[4]) {
  if (VEC4 && nv == 4) {
    const half4_t a = {to_half(v[0]), to_half(v[1]), to_half(v[2]),
                       to_half(v[3])};
    __builtin_nontemporal_store(a, reinterpret_cast<half4_t*>(p));
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nv) p[i] = to_half(v[i]);
  }
}

__device__ __forceinline__ int valid_in_quad(int64_t quad, int64_t n) {
  const int64_t left = n - quad * 4;
  return left >= 4 ? 4 : (left > 0 ? static_cast<int>(left) : 0);
}

template <int CTRL>
__device__ __forceinline__ uint32_t dpp(uint32_t v) {
  return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), CTRL, 0xF, 0xF, true));
}

// OR the nibbles of lanes 8m..8m+7 into one mask word; lane 8m stores it.
// quad_perm [1,0,3,2] and [2,3,0,1] fold within groups of four lanes, the
// half-row mirror (lane i <-> 7 - i) then folds the two groups.
__device__ __forceinline__ void store_mask_nibble(uint32_t nibble, int64_t quad, int64_t n,
                                                  uint32_t* __restrict__ mask) {
  uint32_t w = nibble << (4 * (threadIdx.x & 7));
  w |= dpp<0xB1>(w);
  w |= dpp<0x4E>(w);
  w |= dpp<0x141>(w);
  if ((threadIdx.x & 7) == 0 && quad * 4 < n) mask[quad >> 3] = w;
}

__device__ __forceinline__ uint32_t load_mask_nibble(const uint32_t* __restrict__ mask, int64_t quad) {
  return (mask[quad >> 3] >> (4 * (quad & 7))) & 0xFu;
}

template <bool VEC4, typename T>
__global__ __launch_bounds__(kBlock) void relu_fwd_kernel(const T* __restrict__ x, int64_t n,
                                                          T* __restrict__ y,
                                                          uint32_t* __restrict__ mask) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * kTileQuads + h * kBlock + threadIdx.x;
    const int nv = valid_in_quad(quad, n);
    float v[4];
    uint32_t nibble = 0;
    if (nv > 0) {
      load4<VEC4>(x + quad * 4, nv, v);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool bit = v[i] > 0.f;  // quantization_cuda_kernel.cu:252-257
        v[i] = bit ? v[i] : 0.f;
        nibble |= static_cast<uint32_t>(bit && i < nv) << i;
      }
      store4<VEC4>(y + quad * 4, nv, v);
    }
    store_mask_nibble(nibble, quad, n, mask);
  }
}

template <bool VEC4, typename T>
__global__ __launch_bounds__(kBlock) void relu_bwd_kernel(const T* __restrict__ dy,
                                                          const uint32_t* __restrict__ mask, int64_t n,
                                                          T* __restrict__ dx) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * kTileQuads + h * kBlock + threadIdx.x;
    const int nv = valid_in_quad(quad, n);
    if (nv == 0) continue;
    float v[4];
    load4<VEC4>(dy + quad * 4, nv, v);
    const uint32_t nibble = load_mask_nibble(mask, quad);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ((nibble >> i) & 1u) ? v[i] : 0.f;  // :305-310
    store4<VEC4>(dx + quad * 4, nv, v);
  }
}

// LeakyReLU with the same 1-bit mask (quantization_cuda_kernel.cu:339-371, 395-412):
// y = x > 0 ? x : x * slope; dx = bit ? dy : dy * slope.
template <bool VEC4, typename T>
__global__ __launch_bounds__(kBlock) void leaky_relu_fwd_kernel(const T* __restrict__ x, int64_t n, float slope,
                                                                T* __restrict__ y,
                                                                uint32_t* __restrict__ mask) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * kTileQuads + h * kBlock + threadIdx.x;
    const int nv = valid_in_quad(quad, n);
    float v[4];
    uint32_t nibble = 0;
    if (nv > 0) {
      load4<VEC4>(x + quad * 4, nv, v);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool bit = v[i] > 0.f;
        v[i] = bit ? v[i] : v[i] * slope;
        nibble |= static_cast<uint32_t>(bit && i < nv) << i;
      }
      store4<VEC4>(y + quad * 4, nv, v);
    }
    store_mask_nibble(nibble, quad, n, mask);
  }
}

template <bool VEC4, typename T>
__global__ __launch_bounds__(kBlock) void leaky_relu_bwd_kernel(const T* __restrict__ dy,
                                                                const uint32_t* __restrict__ mask, int64_t n,
                                                                float slope, T* __restrict__ dx) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * kTileQuads + h * kBlock + threadIdx.x;
    const int nv = valid_in_quad(quad, n);
    if (nv == 0) continue;
    float v[4];
    load4<VEC4>(dy + quad * 4, nv, v);
    const uint32_t nibble = load_mask_nibble(mask, quad);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ((nibble >> i) & 1u) ? v[i] : v[i] * slope;
    store4<VEC4>(dx + quad * 4, nv, v);
  }
}

// RELU: the input first goes through ReLU and the mask bit is (x > 0) && keep --
// ReLU followed by dropout in one pass, with one mask for the pair (the
// backward of the pair is dx = bit ? dy / (1 - p) : 0, i.e. dropout_bwd_kernel).
template <bool VEC4, bool NOISE_IN, bool RELU, typename T>
__global__ __launch_bounds__(kBlock) void dropout_fwd_kernel(const T* __restrict__ x,
                                                             const float* __restrict__ noise,
                                                             uint32_t seed_lo, uint32_t seed_hi,
                                                             uint32_t off_lo, uint32_t off_hi, float p,
                                                             float pinv, int64_t n, T* __restrict__ y,
                                                             uint32_t* __restrict__ mask) {
  const int64_t qa = static_cast<int64_t>(blockIdx.x) * kTileQuads + threadIdx.x;
  const int64_t qb = qa + kBlock;
  float u[2][4];
  if constexpr (!NOISE_IN) {
    // flat element i draws from block i / 8 = quad / 2: counter (block lo, block hi, offset)
    const bool odd = (threadIdx.x & 1) != 0;
    const int64_t blk = (odd ? qb : qa) >> 1;
    const Philox4 r = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32), off_lo, off_hi,
                                    seed_lo, seed_hi);
    const uint32_t got0 = dpp<0xB1>(odd ? r.x : r.z);
    const uint32_t got1 = dpp<0xB1>(odd ? r.y : r.w);
    const uint32_t a0 = odd ? got0 : r.x, a1 = odd ? got1 : r.y;
    const uint32_t b0 = odd ? r.z : got0, b1 = odd ? r.w : got1;
    u[0][0] = u16_to_uniform(a0 & 0xFFFFu); u[0][1] = u16_to_uniform(a0 >> 16);
    u[0][2] = u16_to_uniform(a1 & 0xFFFFu); u[0][3] = u16_to_uniform(a1 >> 16);
    u[1][0] = u16_to_uniform(b0 & 0xFFFFu); u[1][1] = u16_to_uniform(b0 >> 16);
    u[1][2] = u16_to_uniform(b1 & 0xFFFFu); u[1][3] = u16_to_uniform(b1 >> 16);
  }
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = h ? qb : qa;
    const int nv = valid_in_quad(quad, n);
    uint32_t nibble = 0;
    if (nv > 0) {
      float v[4];
      load4<VEC4>(x + quad * 4, nv, v);
      if constexpr (NOISE_IN) load4<VEC4>(noise + quad * 4, nv, u[h]);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool pos = !RELU || v[i] > 0.f;  // :252-257
        const bool keep = u[h][i] > p;         // :465-468
        const float kf = keep ? 1.f : 0.f;
        float r = pos ? v[i] : 0.f;
        r = r * kf;  // :490, left to right
        r = r * pinv;
        v[i] = r;
        nibble |= static_cast<uint32_t>(pos && keep && i < nv) << i;
      }
      store4<VEC4>(y + quad * 4, nv, v);
    }
    store_mask_nibble(nibble, quad, n, mask);
  }
}

template <bool VEC4, typename T>
__global__ __launch_bounds__(kBlock) void dropout_bwd_kernel(const T* __restrict__ dy,
                                                             const uint32_t* __restrict__ mask, float p1m,
                                                             int64_t n, T* __restrict__ dx) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * kTileQuads + h * kBlock + threadIdx.x;
    const int nv = valid_in_quad(quad, n);
    if (nv == 0) continue;
    float v[4];
    load4<VEC4>(dy + quad * 4, nv, v);
    const uint32_t nibble = load_mask_nibble(mask, quad);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ((nibble >> i) & 1u) ? v[i] / p1m : 0.f;  // :565-569
    store4<VEC4>(dx + quad * 4, nv, v);
  }
}

// ELU backward on the (decompressed) input: dx = x >= 0 ? dy : alpha * dy * exp(x)
// (backward_func_cuda_kernel.cu:6-20; alpha * dy first, then the exponential).
template <bool VEC4, typename T>
__global__ __launch_bounds__(kBlock) void elu_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                         float alpha, int64_t n, T* __restrict__ dx) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int64_t quad = static_cast<int64_t>(blockIdx.x) * kTileQuads + h * kBlock + threadIdx.x;
    const int nv = valid_in_quad(quad, n);
    if (nv == 0) continue;
    float g[4], v[4];
    load4<VEC4>(dy + quad * 4, nv, g);
    load4<VEC4>(x + quad * 4, nv, v);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float scaled = alpha * g[i];
      scaled = scaled * expf(v[i]);
      g[i] = v[i] >= 0.f ? g[i] : scaled;
    }
    store4<VEC4>(dx + quad * 4, nv, g);
  }
}

// a quad of T is one aligned vector access
template <typename T>
static bool quad_aligned(const void* p) { return (reinterpret_cast<uintptr_t>(p) & (4 * sizeof(T) - 1)) == 0; }
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static dim3 tile_grid(int64_t n) {
  const int64_t quads = (n + 3) / 4;
  return dim3(static_cast<unsigned>((quads + kTileQuads - 1) / kTileQuads));
}

static int check_n(int64_t n) { return (n < 0 || n > (int64_t{1} << 40)) ? EXACT_E_SHAPE : EXACT_OK; }

template <typename T>
static int relu_forward(const T* x, int64_t n, T* y, uint32_t* mask, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (n == 0) return EXACT_OK;
  if (!x || !y || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (quad_aligned<T>(x) && quad_aligned<T>(y))
    hipLaunchKernelGGL((relu_fwd_kernel<true, T>), tile_grid(n), dim3(kBlock), 0, s, x, n, y, mask);
  else
    hipLaunchKernelGGL((relu_fwd_kernel<false, T>), tile_grid(n), dim3(kBlock), 0, s, x, n, y, mask);
  return launch_status();
}

template <typename T>
static int relu_backward(const T* dy, const uint32_t* mask, int64_t n, T* dx, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (n == 0) return EXACT_OK;
  if (!dy || !dx || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (quad_aligned<T>(dy) && quad_aligned<T>(dx))
    hipLaunchKernelGGL((relu_bwd_kernel<true, T>), tile_grid(n), dim3(kBlock), 0, s, dy, mask, n, dx);
  else
    hipLaunchKernelGGL((relu_bwd_kernel<false, T>), tile_grid(n), dim3(kBlock), 0, s, dy, mask, n, dx);
  return launch_status();
}

template <typename T>
static int leaky_forward(const T* x, int64_t n, float slope, T* y, uint32_t* mask, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (n == 0) return EXACT_OK;
  if (!x || !y || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (quad_aligned<T>(x) && quad_aligned<T>(y))
    hipLaunchKernelGGL((leaky_relu_fwd_kernel<true, T>), tile_grid(n), dim3(kBlock), 0, s, x, n, slope, y, mask);
  else
    hipLaunchKernelGGL((leaky_relu_fwd_kernel<false, T>), tile_grid(n), dim3(kBlock), 0, s, x, n, slope, y, mask);
  return launch_status();
}

template <typename T>
static int leaky_backward(const T* dy, const uint32_t* mask, int64_t n, float slope, T* dx, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (n == 0) return EXACT_OK;
  if (!dy || !dx || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (quad_aligned<T>(dy) && quad_aligned<T>(dx))
    hipLaunchKernelGGL((leaky_relu_bwd_kernel<true, T>), tile_grid(n), dim3(kBlock), 0, s, dy, mask, n, slope, dx);
  else
    hipLaunchKernelGGL((leaky_relu_bwd_kernel<false, T>), tile_grid(n), dim3(kBlock), 0, s, dy, mask, n, slope, dx);
  return launch_status();
}

template <bool RELU, typename T>
static int dropout_forward(const T* x, const float* noise, uint64_t seed, uint64_t offset, float p, int64_t n,
                           T* y, uint32_t* mask, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (!(p >= 0.f && p < 1.f)) return EXACT_E_ARG;
  if (n == 0) return EXACT_OK;
  if (!x || !y || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // quantization_cuda_kernel.cu:456: float pinv = 1. / (1. - p), evaluated in double
  const float pinv = static_cast<float>(1.0 / (1.0 - static_cast<double>(p)));
  const uint32_t sl = static_cast<uint32_t>(seed), sh = static_cast<uint32_t>(seed >> 32);
  const uint32_t ol = static_cast<uint32_t>(offset), oh = static_cast<uint32_t>(offset >> 32);
  const bool v4 = quad_aligned<T>(x) && quad_aligned<T>(y) && (!noise || aligned16(noise));
  const dim3 grid = tile_grid(n);
  if (noise) {
    if (v4) hipLaunchKernelGGL((dropout_fwd_kernel<true, true, RELU, T>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
    else hipLaunchKernelGGL((dropout_fwd_kernel<false, true, RELU, T>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
  } else {
    if (v4) hipLaunchKernelGGL((dropout_fwd_kernel<true, false, RELU, T>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
    else hipLaunchKernelGGL((dropout_fwd_kernel<false, false, RELU, T>), grid, dim3(kBlock), 0, s, x, noise, sl, sh, ol, oh, p, pinv, n, y, mask);
  }
  return launch_status();
}

template <typename T>
static int dropout_backward(const T* dy, const uint32_t* mask, float p, int64_t n, T* dx, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (!(p >= 0.f && p < 1.f)) return EXACT_E_ARG;
  if (n == 0) return EXACT_OK;
  if (!dy || !dx || !mask) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  // quantization.cc:121,127: p1m = 1. - p stored as double, read back into a float
  const float p1m = static_cast<float>(1.0 - static_cast<double>(p));
  if (quad_aligned<T>(dy) && quad_aligned<T>(dx))
    hipLaunchKernelGGL((dropout_bwd_kernel<true, T>), tile_grid(n), dim3(kBlock), 0, s, dy, mask, p1m, n, dx);
  else
    hipLaunchKernelGGL((dropout_bwd_kernel<false, T>), tile_grid(n), dim3(kBlock), 0, s, dy, mask, p1m, n, dx);
  return launch_status();
}

template <typename T>
static int elu_backward(const T* dy, const T* x, float alpha, int64_t n, T* dx, void* stream) {
  if (int rc = check_n(n)) return rc;
  if (n == 0) return EXACT_OK;
  if (!dy || !x || !dx) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (quad_aligned<T>(dy) && quad_aligned<T>(x) && quad_aligned<T>(dx))
    hipLaunchKernelGGL((elu_bwd_kernel<true, T>), tile_grid(n), dim3(kBlock), 0, s, dy, x, alpha, n, dx);
  else
    hipLaunchKernelGGL((elu_bwd_kernel<false, T>), tile_grid(n), dim3(kBlock), 0, s, dy, x, alpha, n, dx);
  return launch_status();
}

}  // namespace exact

using namespace exact;

static const half_t* hp(const uint16_t* p) { return reinterpret_cast<const half_t*>(p); }
static half_t* hp(uint16_t* p) { return reinterpret_cast<half_t*>(p); }

extern "C" {

int exact_relu_fwd_f32(const float* x, int64_t n, float* y, uint32_t* mask, void* stream) {
  return relu_forward<float>(x, n, y, mask, stream);
}
int exact_relu_bwd_f32(const float* dy, const uint32_t* mask, int64_t n, float* dx, void* stream) {
  return relu_backward<float>(dy, mask, n, dx, stream);
}
int exact_leaky_relu_fwd_f32(const float* x, int64_t n, float slope, float* y, uint32_t* mask, void* stream) {
  return leaky_forward<float>(x, n, slope, y, mask, stream);
}
int exact_leaky_relu_bwd_f32(const float* dy, const uint32_t* mask, int64_t n, float slope, float* dx,
                             void* stream) {
  return leaky_backward<float>(dy, mask, n, slope, dx, stream);
}
int exact_dropout_fwd_f32(const float* x, const float* noise, uint64_t seed, uint64_t offset, float p,
                          int64_t n, float* y, uint32_t* mask, void* stream) {
  return dropout_forward<false, float>(x, noise, seed, offset, p, n, y, mask, stream);
}
int exact_relu_dropout_fwd_f32(const float* x, const float* noise, uint64_t seed, uint64_t offset, float p,
                               int64_t n, float* y, uint32_t* mask, void* stream) {
  return dropout_forward<true, float>(x, noise, seed, offset, p, n, y, mask, stream);
}
int exact_dropout_bwd_f32(const float* dy, const uint32_t* mask, float p, int64_t n, float* dx,
                          void* stream) {
  return dropout_backward<float>(dy, mask, p, n, dx, stream);
}

int exact_elu_bwd_f32(const float* dy, const float* x, float alpha, int64_t n, float* dx, void* stream) {
  return elu_backward<float>(dy, x, alpha, n, dx, stream);
}
int exact_elu_bwd_f16(const uint16_t* dy, const uint16_t* x, float alpha, int64_t n, uint16_t* dx, void* stream) {
  return elu_backward<half_t>(hp(dy), hp(x), alpha, n, hp(dx), stream);
}

// fp16 activations: the same kernels instantiated for 16-bit elements
int exact_relu_fwd_f16(const uint16_t* x, int64_t n, uint16_t* y, uint32_t* mask, void* stream) {
  return relu_forward<half_t>(hp(x), n, hp(y), mask, stream);
}
int exact_relu_bwd_f16(const uint16_t* dy, const uint32_t* mask, int64_t n, uint16_t* dx, void* stream) {
  return relu_backward<half_t>(hp(dy), mask, n, hp(dx), stream);
}
int exact_leaky_relu_fwd_f16(const uint16_t* x, int64_t n, float slope, uint16_t* y, uint32_t* mask,
                             void* stream) {
  return leaky_forward<half_t>(hp(x), n, slope, hp(y), mask, stream);
}
int exact_leaky_relu_bwd_f16(const uint16_t* dy, const uint32_t* mask, int64_t n, float slope, uint16_t* dx,
                             void* stream) {
  return leaky_backward<half_t>(hp(dy), mask, n, slope, hp(dx), stream);
}
int exact_dropout_fwd_f16(const uint16_t* x, const float* noise, uint64_t seed, uint64_t offset, float p,
                          int64_t n, uint16_t* y, uint32_t* mask, void* stream) {
  return dropout_forward<false, half_t>(hp(x), noise, seed, offset, p, n, hp(y), mask, stream);
}
int exact_relu_dropout_fwd_f16(const uint16_t* x, const float* noise, uint64_t seed, uint64_t offset, float p,
                               int64_t n, uint16_t* y, uint32_t* mask, void* stream) {
  return dropout_forward<true, half_t>(hp(x), noise, seed, offset, p, n, hp(y), mask, stream);
}
int exact_dropout_bwd_f16(const uint16_t* dy, const uint32_t* mask, float p, int64_t n, uint16_t* dx,
                          void* stream) {
  return dropout_backward<half_t>(hp(dy), mask, p, n, hp(dx), stream);
}

}  // extern "C"
