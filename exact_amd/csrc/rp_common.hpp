// Pieces shared by the projection kernels (rp_gemm.hip: fp32 matrix cores,
// rp_bf16.hip: bf16 matrix cores on split operands): the 32 x 32 accumulator
// layout and the quantise-and-pack epilogue that works on it.
#pragma once

#include "exact_common.hpp"

namespace exact {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 32;  // MFMA M and N

// Projection and quantisation in one launch: the [N, k] product stays in the
// accumulators, where its per-row min / range, the stochastic rounding and the
// bit-packing of quantize_activation (ops.py:69-83; kernel
// quantization_cuda_kernel.cu:63-94) are applied to it -- what
// exact_rp_fwd_f32 followed by exact_minmax_pack_f32 computes, bit for bit,
// without the [N, k] tensor ever reaching memory.
//
// In the accumulator layout a lane holds, per 32-column tile, one column of 16
// rows: rows 4h .. 4h + 3 of each block of 8 (h = lane / 32).  So the row
// statistics are butterflies over the 32 lanes of a half-wave; the 2, 4 or 8
// rows that share a packed byte sit in one lane (8 rows: in the two lanes
// l and l + 32); and lane l % 32 writes the byte of column l: 32 consecutive
// bytes per row group.
//
// Noise: element (n, d) takes 16-bit half d % 8 of Philox block (d / 8, n), the
// row stream of the pack kernel.  The 8 lanes that share d / 8 compute the
// blocks of four rows at a time between them and hand the words round.
struct RpPackArgs {
  const float* X;
  const float* R;
  const float* noise;  // nullable: [N, k] uniforms
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  int64_t N;
  int D, k, bits;
  uint8_t* packed;
  int64_t pad_index;
  float* scale_f32;
  float* min_f32;
  uint16_t* scale_bf16;
  uint16_t* min_bf16;
};


// The epilogue on the accumulators of one wavefront (rows row0 .. row0 + 31, NT
// tiles of 32 columns), whichever matrix-core path produced them.  The 32 rows
// are handled as four blocks of eight (accumulator registers 4 vg .. 4 vg + 3 of
// both half-waves); the caller may hand a wavefront only some of the blocks
// [vg_begin, vg_end), and then only their registers need to hold values.
template <int NT, bool NOISE_IN>
__device__ __forceinline__ void rp_quantise_and_pack(const RpPackArgs& a, const floatx16 (&acc)[NT], int64_t row0,
                                                     int vg_begin = 0, int vg_end = 4) {
  const int lane = threadIdx.x & (kWave - 1);
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int k = a.k;
  const float B = static_cast<float>((1 << a.bits) - 1);
  // The 16 accumulator rows are handled as four blocks of four consecutive rows
  // (rows 8 * vg + 4 * half + 0 .. 3), the unit in which they share packed bytes;
  // one block at a time keeps the epilogue within the registers of the main loop.
  const int i8 = l32 & 7;            // position in the 8-lane group = element of a Philox block
  const int group_first = lane & ~7;
#pragma unroll
  for (int vg = 0; vg < 4; ++vg) {
    if (vg < vg_begin || vg >= vg_end) continue;     // wave-uniform
    const int64_t rbase = row0 + 8 * vg + 4 * half;  // first of the four rows
    // ---- row statistics: min / max over the k columns, then scale -----------
    float mnv[4], sc[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float lo = __builtin_inff(), hi = -__builtin_inff();
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        if (nt * kTile + l32 < k) {
          lo = fminf(lo, acc[nt][4 * vg + r]);
          hi = fmaxf(hi, acc[nt][4 * vg + r]);
        }
      }
      group_minmax(lo, hi, kTile);
      mnv[r] = lo;
      const float recip = 1.0f / (hi - lo);  // ops.py:39: reciprocal, then * B -- two roundings
      sc[r] = recip * B;
      if (l32 == 0 && rbase + r < a.N) {
        if (a.scale_f32) a.scale_f32[rbase + r] = sc[r];
        if (a.min_f32) a.min_f32[rbase + r] = lo;
        if (a.scale_bf16) a.scale_bf16[rbase + r] = f32_to_bf16_rne(sc[r]);
        if (a.min_bf16) a.min_bf16[rbase + r] = f32_to_bf16_rne(lo);
      }
    }

#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int cj = nt * kTile + l32;
      const bool col_ok = cj < k;
      // ---- noise -------------------------------------------------------------
      float u[4];
      if constexpr (NOISE_IN) {
#pragma unroll
        for (int r = 0; r < 4; ++r) u[r] = (col_ok && rbase + r < a.N) ? a.noise[(rbase + r) * k + cj] : 0.f;
      } else {
        // lane i8 of an 8-lane group computes the block of row i8 % 4 (twice over
        // the group), then every lane fetches the word holding its element
        const Philox4 mine = philox4x32_10(static_cast<uint32_t>(cj >> 3), static_cast<uint32_t>(rbase + (i8 & 3)),
                                           a.off_lo, a.off_hi, a.seed_lo, a.seed_hi);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int src = group_first | r;
          const uint32_t w0 = __shfl(mine.x, src), w1 = __shfl(mine.y, src), w2 = __shfl(mine.z, src),
                         w3 = __shfl(mine.w, src);
          const uint32_t lo_pair = (i8 & 2) ? w1 : w0, hi_pair = (i8 & 2) ? w3 : w2;
          const uint32_t word = (i8 & 4) ? hi_pair : lo_pair;
          u[r] = u16_to_uniform((i8 & 1) ? (word >> 16) : (word & 0xFFFFu));
        }
      }
      // ---- quantise (quantization_cuda_kernel.cu:89, one rounding per operation) --
      uint32_t q[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float tq = acc[nt][4 * vg + r] - mnv[r];
        tq = tq * sc[r];
        tq = tq + u[r];
        const uint32_t qi = code_in_low_byte(tq);  // scale and min are this row's own: tq < 2^bits + 2
        q[r] = (col_ok && rbase + r < a.N) ? (qi & 0xFFu) : 0u;
      }
      // ---- pack: byte (n / wpt) * k + d holds rows n .. n + wpt - 1 of column d ----
      if (a.bits == 8) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (col_ok && rbase + r < a.N) a.packed[(rbase + r) * k + cj] = static_cast<uint8_t>(q[r]);
      } else if (a.bits == 4) {
#pragma unroll
        for (int r = 0; r < 4; r += 2)
          if (col_ok && rbase + r < a.N) a.packed[((rbase + r) >> 1) * k + cj] = static_cast<uint8_t>(q[r] | (q[r + 1] << 4));
      } else if (a.bits == 2) {
        if (col_ok && rbase < a.N)
          a.packed[(rbase >> 2) * k + cj] = static_cast<uint8_t>(q[0] | (q[1] << 2) | (q[2] << 4) | (q[3] << 6));
      } else {
        const uint32_t nib = q[0] | (q[1] << 1) | (q[2] << 2) | (q[3] << 3);  // rows 4 * half .. 4 * half + 3 of the eight
        const uint32_t other = __shfl_xor(nib, 32);
        const uint32_t byte = half ? (other | (nib << 4)) : (nib | (other << 4));
        const int64_t first = row0 + 8 * vg;
        // the two half-waves hold the same byte: they take turns storing
        if (col_ok && first < a.N && (vg & 1) == half) a.packed[(first >> 3) * k + cj] = static_cast<uint8_t>(byte);
      }
    }
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) a.packed[a.pad_index] = 0;
}

static __global__ void rp_zero_byte_kernel(uint8_t* p) { *p = 0; }  // the pad byte of an empty input

__host__ __device__ static inline bool al16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
__host__ __device__ static inline bool al8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }

}  // namespace exact
