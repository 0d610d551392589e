// Shared device helpers for libexact_hip (gfx950 only, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/exact_hip.h"

namespace exact {

constexpr int kWave = 64;
constexpr int kBlock = 256;  // 4 wavefronts per workgroup

// ---- streaming (non-temporal) 16-byte accesses -----------------------------
typedef float f32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ f32x4 nt_load4(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
}
__device__ __forceinline__ void nt_store4(float* p, float a, float b, float c, float d) {
  f32x4 v = {a, b, c, d};
  __builtin_nontemporal_store(v, reinterpret_cast<f32x4*>(p));
}

// ---- launch helpers --------------------------------------------------------
inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? EXACT_OK : static_cast<int>(e);
}

// ---- Philox4x32-10 ---------------------------------------------------------
// Block function of Salmon et al. (SC'11); the reference draws from cuRAND's
// Philox4_32_10 (quantization_cuda_kernel.cu:77-79, 452-453).  The key is
// wave-uniform, so its schedule lives in scalar registers.
// a ^ b ^ c in one instruction (v_bitop3_b32, truth table 0x96 = odd parity)
__device__ __forceinline__ uint32_t xor3(uint32_t a, uint32_t b, uint32_t c) {
  return __builtin_amdgcn_bitop3_b32(a, b, c, 0x96);
}

struct Philox4 {
  uint32_t x, y, z, w;
};

__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2,
                                                 uint32_t c3, uint32_t k0, uint32_t k1) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u;
  constexpr uint32_t W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = static_cast<uint64_t>(M0) * c0;
    const uint64_t p1 = static_cast<uint64_t>(M1) * c2;
    const uint32_t n0 = xor3(static_cast<uint32_t>(p1 >> 32), c1, k0);
    const uint32_t n2 = xor3(static_cast<uint32_t>(p0 >> 32), c3, k1);
    c1 = static_cast<uint32_t>(p1);
    c3 = static_cast<uint32_t>(p0);
    c0 = n0;
    c2 = n2;
    k0 += W0;
    k1 += W1;
  }
  return Philox4{c0, c1, c2, c3};
}

// 16 random bits -> uniform on (0,1): (h + 0.5) * 2^-16, exact in fp32.
__device__ __forceinline__ float u16_to_uniform(uint32_t h) {
  return __fmaf_rn(static_cast<float>(h), 0x1p-16f, 0x1p-17f);
}

// Eight uniforms from one Philox block: word w gives elements 2w (low half)
// and 2w+1 (high half).
__device__ __forceinline__ void philox_uniform8(const Philox4& r, float (&u)[8]) {
  u[0] = u16_to_uniform(r.x & 0xFFFFu);
  u[1] = u16_to_uniform(r.x >> 16);
  u[2] = u16_to_uniform(r.y & 0xFFFFu);
  u[3] = u16_to_uniform(r.y >> 16);
  u[4] = u16_to_uniform(r.z & 0xFFFFu);
  u[5] = u16_to_uniform(r.z >> 16);
  u[6] = u16_to_uniform(r.w & 0xFFFFu);
  u[7] = u16_to_uniform(r.w >> 16);
}

// ---- round and clamp of the quantiser -------------------------------------------
// quantization_cuda_kernel.cu:89-90 turns t = (x - min) * scale + noise into
// uint8(__float2int_rn(fmaxf(t - 0.5f, 0.f))).  When scale and min are the row's
// own, t is below 2^bits + 2, or +inf (a row whose spread is so small that its
// reciprocal overflows), or NaN (0 * inf in a constant row).  For those the same
// byte is the low byte of the bit pattern of  med3(t, 0.5, 511.5) + (2^23 - 0.5):
// t - 0.5 is exact in fp32 whenever t >= 0.5 (a multiple of ulp(t) of smaller
// magnitude), so the sum has the exact value 2^23 + (t - 0.5) in [2^23, 2^24),
// where fp32 holds the integers only -- the one rounding of the addition is the
// round-to-nearest-even onto the integers that __float2int_rn performs, and the
// low mantissa bits are that integer.  t < 0.5 gives 2^23 exactly, code 0, as
// fmaxf(.., 0) does, and so does NaN (v_med3_f32 with a NaN operand returns the
// minimum of the others); +inf is clamped to 511, low byte 0xFF, the low byte of
// the INT_MAX that the saturating conversion returns.  Two instructions instead
// of five.  Callers whose t is not bounded (scale and min supplied from outside)
// keep the written-out form, which saturates at every magnitude.
__device__ __forceinline__ uint32_t code_in_low_byte(float t) {
  return __float_as_uint(__builtin_amdgcn_fmed3f(t, 0.5f, 511.5f) + 8388607.5f);
}
// __float2int_rn of a value that is not negative and not a NaN, every magnitude:
// cvt.rni.s32.f32 clamps to the int32 range (a plain cast of +inf is undefined)
__device__ __forceinline__ uint32_t float2int_rn_sat(float t) {
  return t >= 2147483648.f ? 0x7FFFFFFFu : static_cast<uint32_t>(static_cast<int>(rintf(t)));
}
// the low bytes of four words as one word, a in byte 0 (three v_perm_b32)
__device__ __forceinline__ uint32_t low_bytes4(uint32_t a, uint32_t b, uint32_t c, uint32_t d) {
  const uint32_t ab = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);
  const uint32_t cd = __builtin_amdgcn_perm(d, c, 0x0c0c0400u);
  return __builtin_amdgcn_perm(cd, ab, 0x05040100u);
}

// ---- bf16 ------------------------------------------------------------------
// fp32 -> bf16 bits, round to nearest even (what Tensor.to(torch.bfloat16)
// does at ops.py:80-81 of the reference).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  const uint32_t b = __float_as_uint(f);
  const uint32_t rounded = (b + 0x7FFFu + ((b >> 16) & 1u)) >> 16;
  const uint32_t quiet_nan = ((b >> 16) & 0x8000u) | 0x7FC0u;
  return static_cast<uint16_t>((b & 0x7FFFFFFFu) > 0x7F800000u ? quiet_nan : rounded);
}
__device__ __forceinline__ float bf16_to_f32(uint16_t h) {
  return __uint_as_float(static_cast<uint32_t>(h) << 16);
}

// ---- fp16 ------------------------------------------------------------------
// IEEE binary16 with round-to-nearest-even conversions, as at::Half has them.
//
// at::Half arithmetic rounds twice: the fp32 operation, then the conversion of
// its fp32 result.  Written as cast(a * b) the compiler may select
// v_fma_mixlo_f16, which rounds the exact product ONCE, straight to fp16, and
// differs in the last bit whenever the fp32 rounding lands on a tie of the
// fp16 grid.  to_half() therefore first pins its argument in a register as an
// fp32 value the optimiser cannot look through, so the conversion is always
// a plain v_cvt_f16_f32 of an already rounded fp32 number.
using half_t = _Float16;
#ifndef EXACT_VALUE_BARRIER  // the host build of the tests supplies its own constraint letter
#define EXACT_VALUE_BARRIER(r) asm("" : "+v"(r))
#endif
__device__ __forceinline__ half_t to_half(float x) {
  EXACT_VALUE_BARRIER(x);
  return static_cast<half_t>(x);
}
__device__ __forceinline__ float round_to_half(float x) { return static_cast<float>(to_half(x)); }
__device__ __forceinline__ uint16_t half_bits(float x) {
  const half_t h = to_half(x);
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

// ---- cross-lane ------------------------------------------------------------
// Butterfly min / max over aligned groups of `span` lanes (span a power of two
// <= 64).  Every lane of the group ends with the group's result.
//
// The values travel as order-preserving integer keys (key(f) = bits ^ ((bits >>
// 31) & 0x7FFFFFFF), an involution; -0 sorts below +0 as in v_min_f32): integer
// min / max take a DPP operand directly, so a step is ONE instruction per
// quantity, where the float forms need a move and two canonicalisations more.
// Steps: quad_perm [1,0,3,2] and [2,3,0,1] fold a quad, after which the four
// lanes of a quad agree, so the half-row mirror (lane i <-> 7 - i) delivers "the
// other quad"; row_ror:8 delivers the other half of a 16-lane row; lanes 16
// and 32 apart (rows spread over more than one DPP row) go through ds_bpermute.
__device__ __forceinline__ int order_key(float f) {
  const int b = __float_as_int(f);
  return b ^ ((b >> 31) & 0x7FFFFFFF);
}
__device__ __forceinline__ float key_value(int k) { return __int_as_float(k ^ ((k >> 31) & 0x7FFFFFFF)); }

template <int CTRL>
__device__ __forceinline__ int dpp_lanes(int v) {
  return __builtin_amdgcn_update_dpp(v, v, CTRL, 0xF, 0xF, true);
}

__device__ __forceinline__ void group_minmax(float& mn, float& mx, int span) {
  int lo = order_key(mn), hi = order_key(mx);
  if (span >= 2) {
    lo = min(lo, dpp_lanes<0xB1>(lo));
    hi = max(hi, dpp_lanes<0xB1>(hi));
  }
  if (span >= 4) {
    lo = min(lo, dpp_lanes<0x4E>(lo));
    hi = max(hi, dpp_lanes<0x4E>(hi));
  }
  if (span >= 8) {
    lo = min(lo, dpp_lanes<0x141>(lo));
    hi = max(hi, dpp_lanes<0x141>(hi));
  }
  if (span >= 16) {
    lo = min(lo, dpp_lanes<0x128>(lo));
    hi = max(hi, dpp_lanes<0x128>(hi));
  }
  for (int m = 16; m < span; m <<= 1) {
    lo = min(lo, __shfl_xor(lo, m));
    hi = max(hi, __shfl_xor(hi, m));
  }
  mn = key_value(lo);
  mx = key_value(hi);
}

}  // namespace exact
