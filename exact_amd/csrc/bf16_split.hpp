// fp32 products on the bf16 matrix cores of gfx950 (v_mfma_f32_32x32x16_bf16,
// fp32 accumulate) at fp32 accuracy.  An fp32 number is the exact sum of three
// bf16 numbers: hi = bf16(x), mid = bf16(x - hi), lo = x - hi - mid (each
// difference is exact in fp32 and the last one has at most 8 significant
// bits).  A product of two such sums is formed from the six bf16 products
// hi.hi, hi.mid, mid.hi, hi.lo, lo.hi, mid.mid; the three left out are below
// 2^-24 of the leading one, the rounding of an fp32 product.
//
// Register layout of the instruction (wave64): lane l holds, of the A operand,
// row l % 32 and the eight k-slots 8 * (l / 32) .. + 7 (four 32-bit registers
// of two bf16 each); of the B operand column l % 32 and the same eight k-slots;
// accumulator register v of lane l is C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32],
// as for every 32 x 32 MFMA.
#pragma once

#include "exact_common.hpp"

namespace exact {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// two fp32 -> two bf16 (round to nearest even) in one 32-bit word, `a` in the low half
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const floatx2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
}
__device__ __forceinline__ float low_bf16(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float high_bf16(uint32_t w) { return __uint_as_float(w & 0xFFFF0000u); }

// error-free split of a pair of fp32 numbers into three bf16 pairs
__device__ __forceinline__ void split3(float a, float b, uint32_t& hi, uint32_t& mid, uint32_t& lo) {
  hi = pack_bf16x2(a, b);
  const float ra = a - low_bf16(hi), rb = b - high_bf16(hi);
  mid = pack_bf16x2(ra, rb);
  lo = pack_bf16x2(ra - low_bf16(mid), rb - high_bf16(mid));
}

struct Split8 {
  u32x4 hi, mid, lo;
};
__device__ __forceinline__ Split8 split3x8(const float (&v)[8]) {
  Split8 s;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t h, m, l;
    split3(v[2 * i], v[2 * i + 1], h, m, l);
    s.hi[i] = h;
    s.mid[i] = m;
    s.lo[i] = l;
  }
  return s;
}

__device__ __forceinline__ floatx16 mfma_bf16(u32x4 a, u32x4 b, floatx16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0,
                                                 0);
}

// +-1 (or 0 for a padding entry) as bf16 bits
__device__ __forceinline__ uint32_t sign_bf16(float r, bool inside) {
  return inside ? (0x3F80u | ((__float_as_uint(r) >> 16) & 0x8000u)) : 0u;
}

// acc += A-pieces . B-pieces for one k-step and one column tile.  BP == 1: B is a
// sign matrix (one fragment); BP == 3: B split in three (hi, mid, lo), six products,
// the small ones first.
template <int BP>
__device__ __forceinline__ floatx16 step_product(const Split8& a, const u32x4* b, floatx16 c) {
  if constexpr (BP == 1) {
    c = mfma_bf16(a.lo, b[0], c);
    c = mfma_bf16(a.mid, b[0], c);
    c = mfma_bf16(a.hi, b[0], c);
  } else {
    c = mfma_bf16(a.mid, b[1], c);
    c = mfma_bf16(a.lo, b[0], c);
    c = mfma_bf16(a.hi, b[2], c);
    c = mfma_bf16(a.mid, b[0], c);
    c = mfma_bf16(a.hi, b[1], c);
    c = mfma_bf16(a.hi, b[0], c);
  }
  return c;
}


}  // namespace exact
