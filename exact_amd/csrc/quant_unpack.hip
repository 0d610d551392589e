// Unpack + dequantise of the packed activation stream for [N, G] fp32
// activations on gfx950.
//
// Algorithm restated from the reference kernel
//   unpack_single_precision_kernel  quantization_cuda_kernel.cu:158-185
// and dequantize_activation (ops.py:86-98); the decomposition is this
// library's own.
//
// Work unit: a "quad" = 4 consecutive columns of one row: one 32-bit load of
// packed bytes (4 columns x 8/bits rows), one 16-byte store of fp32.  A row is
// owned by `lpr` adjacent lanes (a power of two in [2, 64]); lane i of the row
// handles quad i (and, for long rows, quad i + lpr), so every vector store of a wavefront covers
// whole contiguous runs of 16 * lpr bytes -- the kernel is bound by writing
// the [N, G] fp32 output once.

#include "exact_common.hpp"

namespace exact {

template <int VEC>
__device__ __forceinline__ void store_quad(float* __restrict__ p, int nv, const float (&v)[4]) {
  if constexpr (VEC == 4) {
    if (nv > 0) nt_store4(p, v[0], v[1], v[2], v[3]);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nv) __builtin_nontemporal_store(v[i], p + i);
  }
}

// ---------------------------------------------------------------------------
// unpack
// ---------------------------------------------------------------------------
struct UnpackArgs {
  const uint8_t* packed;
  const void* scale;  // float* or bf16 bits
  const void* mn;
  int64_t N;
  int G;
  int qpr;
  int lpr_log2;
  int in_vec;  // 4 or 1: widest aligned load of packed bytes
  float* out;
};

// RN(q / s) from r = RN(1 / s): y = RN(q r), e = q - y s (exact, one FMA),
// result = RN(y + e r).  Markstein's correction step; for 0 <= q <= 255 and
// every fp32 significand of s it equals the IEEE quotient bit for bit (checked
// exhaustively on the CPU: 2^23 significands x 256 values of q).
__device__ __forceinline__ float exact_quotient(float q, float s, float r) {
  const float y = q * r;
  const float e = __fmaf_rn(-y, s, q);
  return __fmaf_rn(e, r, y);
}

// How scale / min (and, for fp16, the output) are stored.
enum ParamKind { kParamF32 = 0, kParamBF16 = 1, kParamF16 = 2 };

template <int VEC>
__device__ __forceinline__ void store_quad_half(half_t* __restrict__ p, int nv, const float (&v)[4]) {
  if constexpr (VEC == 4) {
    typedef half_t half4 __attribute__((ext_vector_type(4)));
    if (nv > 0) {
      const half4 q = {to_half(v[0]), to_half(v[1]), to_half(v[2]),
                       to_half(v[3])};
      __builtin_nontemporal_store(q, reinterpret_cast<half4*>(p));
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (i < nv) __builtin_nontemporal_store(to_half(v[i]), p + i);
  }
}

// PARAM == kParamF16: scale, min and the output are fp16 and, as in the
// reference's at::Half instantiation (at::Half operators evaluate in fp32 and
// round to fp16), the quotient and the sum are each rounded to fp16
// (quantization_cuda_kernel.cu:182).
//
// ROWS consecutive rows per lane group.  A group issues every load of its rows
// (packed words, scale, min) before the first value is used: with one row per
// group a wavefront has a single 4-byte load in flight, and when the packed
// stream comes from HBM rather than from L2 (backward reads what forward wrote
// long before) the kernel runs at the speed of that latency -- measured 50 us
// instead of 26 at [169343, 256].
template <int BITS, int SLOTS, int VEC, int PARAM, int ROWS>
__global__ __launch_bounds__(kBlock) void unpack_kernel(const UnpackArgs a) {
  constexpr bool BF16P = PARAM == kParamBF16;
  constexpr bool F16 = PARAM == kParamF16;
  constexpr int WPT = 8 / BITS;
  constexpr uint32_t FIELD = ((1u << BITS) - 1u) * 0x01010101u;
  const int t = threadIdx.x;
  const int lpr = 1 << a.lpr_log2;
  const int lane_in_row = t & (lpr - 1);
  const int rows_per_wg = kBlock >> a.lpr_log2;
  const int64_t n_first = (static_cast<int64_t>(blockIdx.x) * rows_per_wg + (t >> a.lpr_log2)) * ROWS;
  if (n_first >= a.N) return;
  const int quad_base = blockIdx.y * (lpr * SLOTS) + lane_in_row;

  float sc[ROWS], mnv[ROWS];
  uint32_t w[ROWS][SLOTS];
#pragma unroll
  for (int rr = 0; rr < ROWS; ++rr) {
    const int64_t n = (n_first + rr < a.N) ? n_first + rr : a.N - 1;  // rows past the end repeat the last one; never stored
    if constexpr (BF16P) {
      sc[rr] = bf16_to_f32(static_cast<const uint16_t*>(a.scale)[n]);
      mnv[rr] = bf16_to_f32(static_cast<const uint16_t*>(a.mn)[n]);
    } else if constexpr (F16) {
      sc[rr] = static_cast<float>(static_cast<const half_t*>(a.scale)[n]);
      mnv[rr] = static_cast<float>(static_cast<const half_t*>(a.mn)[n]);
    } else {
      sc[rr] = static_cast<const float*>(a.scale)[n];
      mnv[rr] = static_cast<const float*>(a.mn)[n];
    }
    const uint8_t* grp = a.packed + (n / WPT) * a.G;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const int c = quad_base + s * lpr;
      w[rr][s] = 0;
      if (c < a.qpr) {
        if (a.in_vec == 4) {
          w[rr][s] = *reinterpret_cast<const uint32_t*>(grp + 4 * c);
        } else {
          const int cnt = min(4, a.G - 4 * c);
          for (int i = 0; i < cnt; ++i) w[rr][s] |= static_cast<uint32_t>(grp[4 * c + i]) << (8 * i);
        }
      }
    }
  }
#pragma unroll
  for (int rr = 0; rr < ROWS; ++rr) {
    const int64_t n = n_first + rr;
    if (n >= a.N) break;
    // One IEEE division per row instead of one per element: with rcp = RN(1/sc),
    // exact_quotient() returns RN(q / sc) for every integer 0 <= q <= 255 as long
    // as sc is a normal number far from the exponent limits; other rows divide.
    const float asc = fabsf(sc[rr]);
    const bool fast_div = asc >= 0x1p-64f && asc <= 0x1p64f;
    const float rcp = 1.0f / sc[rr];
    const int shift = static_cast<int>(n & (WPT - 1)) * BITS;
    float* orow = F16 ? nullptr : a.out + n * a.G;
    half_t* orow_h = F16 ? reinterpret_cast<half_t*>(a.out) + n * a.G : nullptr;
#pragma unroll
    for (int s = 0; s < SLOTS; ++s) {
      const int c = quad_base + s * lpr;
      if (c >= a.qpr) continue;
      const uint32_t f = (w[rr][s] >> shift) & FIELD;
      float r[4];
      if (__builtin_expect(fast_div, 1)) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float quo = exact_quotient(static_cast<float>((f >> (8 * i)) & 0xFFu), sc[rr], rcp);
          r[i] = (F16 ? round_to_half(quo) : quo) + mnv[rr];
        }
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          // quantization_cuda_kernel.cu:182: true division, then add
          const float quo = static_cast<float>((f >> (8 * i)) & 0xFFu) / sc[rr];
          r[i] = (F16 ? round_to_half(quo) : quo) + mnv[rr];
        }
      }
      if constexpr (F16) store_quad_half<VEC>(orow_h + 4 * c, min(4, a.G - 4 * c), r);  // rounds the sum to fp16
      else store_quad<VEC>(orow + 4 * c, min(4, a.G - 4 * c), r);
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct UnpackGeometry {
  int qpr, lpr_log2, grid_y, slots;
};

// Lanes per row for rows of G columns.  One quad per lane (up to 64 lanes per
// row, so a store instruction covers up to 1 KB of one row and a workgroup
// writes 4 KB) is 3 - 9 % faster than two at G = 256 and 1.6 - 3.7x at widths
// that are not a multiple of 64 columns; rows of more than 192 quads keep two
// quads per lane (measured 6 % better at G = 1024).  Rows longer than one pass
// are tiled over grid.y.
static UnpackGeometry plan_unpack(int64_t G) {
  UnpackGeometry g;
  g.qpr = static_cast<int>((G + 3) / 4);
  g.slots = g.qpr <= 192 ? 1 : 2;
  const int lanes_needed = (g.qpr + g.slots - 1) / g.slots;
  const int max_l2 = g.slots == 1 ? 6 : 5;
  int l2 = 1;
  while ((1 << l2) < lanes_needed && l2 < max_l2) ++l2;
  g.lpr_log2 = l2;
  const int quads_per_pass = (1 << l2) * g.slots;
  g.grid_y = (g.qpr + quads_per_pass - 1) / quads_per_pass;
  return g;
}

static bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

template <int BITS, int PARAM, int ROWS>
static void launch_unpack_variant(const UnpackArgs& a, int slots, bool vec4, dim3 grid, hipStream_t s) {
  if (slots == 1) {
    if (vec4)
      hipLaunchKernelGGL((unpack_kernel<BITS, 1, 4, PARAM, ROWS>), grid, dim3(kBlock), 0, s, a);
    else
      hipLaunchKernelGGL((unpack_kernel<BITS, 1, 1, PARAM, ROWS>), grid, dim3(kBlock), 0, s, a);
  } else {
    if (vec4)
      hipLaunchKernelGGL((unpack_kernel<BITS, 2, 4, PARAM, ROWS>), grid, dim3(kBlock), 0, s, a);
    else
      hipLaunchKernelGGL((unpack_kernel<BITS, 2, 1, PARAM, ROWS>), grid, dim3(kBlock), 0, s, a);
  }
}

// Rows per lane group: four once the launch has workgroups to spare (2048 at one row each, eight per compute
// unit), one for small activations, where the number of wavefronts matters more than the loads each has in flight.
constexpr int kUnpackRows = 4;

template <int PARAM>
static int unpack_common(const uint8_t* packed, int bits, const void* scale, const void* mn,
                         int64_t N, int64_t G, float* out, hipStream_t s) {
  if (bits != 1 && bits != 2 && bits != 4 && bits != 8) return EXACT_E_BITS;
  if (N < 0 || G < 0 || N > 0xFFFFFFFFll || G > 0x7FFFFFF0ll) return EXACT_E_SHAPE;
  if (N == 0 || G == 0) return EXACT_OK;
  if (!packed || !scale || !mn || !out) return EXACT_E_NULL;
  const UnpackGeometry g = plan_unpack(G);
  UnpackArgs a;
  a.packed = packed;
  a.scale = scale;
  a.mn = mn;
  a.N = N;
  a.G = static_cast<int>(G);
  a.qpr = g.qpr;
  a.lpr_log2 = g.lpr_log2;
  a.out = out;
  a.in_vec = (G % 4 == 0 && aligned(packed, 4)) ? 4 : 1;
  const bool vec4 = (G % 4 == 0) && aligned(out, PARAM == kParamF16 ? 8 : 16);
  const int rows_per_wg = kBlock >> g.lpr_log2;
  const int64_t wgs_one_row = (N + rows_per_wg - 1) / rows_per_wg;
  if (wgs_one_row * g.grid_y >= 2048) {
    const int64_t rows = static_cast<int64_t>(rows_per_wg) * kUnpackRows;
    const dim3 grid(static_cast<unsigned>((N + rows - 1) / rows), static_cast<unsigned>(g.grid_y));
    switch (bits) {
      case 1: launch_unpack_variant<1, PARAM, kUnpackRows>(a, g.slots, vec4, grid, s); break;
      case 2: launch_unpack_variant<2, PARAM, kUnpackRows>(a, g.slots, vec4, grid, s); break;
      case 4: launch_unpack_variant<4, PARAM, kUnpackRows>(a, g.slots, vec4, grid, s); break;
      default: launch_unpack_variant<8, PARAM, kUnpackRows>(a, g.slots, vec4, grid, s); break;
    }
  } else {
    const dim3 grid(static_cast<unsigned>(wgs_one_row), static_cast<unsigned>(g.grid_y));
    switch (bits) {
      case 1: launch_unpack_variant<1, PARAM, 1>(a, g.slots, vec4, grid, s); break;
      case 2: launch_unpack_variant<2, PARAM, 1>(a, g.slots, vec4, grid, s); break;
      case 4: launch_unpack_variant<4, PARAM, 1>(a, g.slots, vec4, grid, s); break;
      default: launch_unpack_variant<8, PARAM, 1>(a, g.slots, vec4, grid, s); break;
    }
  }
  return launch_status();
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_unpack_f32(const uint8_t* packed, int bits, const float* scale, const float* mn, int64_t N,
                     int64_t G, float* out, void* stream) {
  return unpack_common<kParamF32>(packed, bits, scale, mn, N, G, out, static_cast<hipStream_t>(stream));
}

int exact_unpack_bf16param_f32(const uint8_t* packed, int bits, const uint16_t* scale_bf16,
                               const uint16_t* min_bf16, int64_t N, int64_t G, float* out, void* stream) {
  return unpack_common<kParamBF16>(packed, bits, scale_bf16, min_bf16, N, G, out, static_cast<hipStream_t>(stream));
}

int exact_unpack_f16(const uint8_t* packed, int bits, const uint16_t* scale_f16, const uint16_t* min_f16,
                     int64_t N, int64_t G, uint16_t* out_f16, void* stream) {
  return unpack_common<kParamF16>(packed, bits, scale_f16, min_f16, N, G, reinterpret_cast<float*>(out_f16),
                                  static_cast<hipStream_t>(stream));
}

}  // extern "C"
