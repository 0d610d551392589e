// Per-row min/range and stochastic-rounding quantise + bit-pack for [N, G]
// fp32 activations on gfx950 (the matching unpack lives in quant_unpack.hip).
//
// Algorithm restated from the reference kernels
//   pack_single_precision_kernel    quantization_cuda_kernel.cu:63-94
// and the torch glue around them (ops.py:20-98, qsheme.py:41-48); the
// decomposition below is this library's own.
//
// Work unit: an "oct" = 8 consecutive columns of one row (32 B of fp32, one
// Philox block of noise, 8 quantised bytes before bit-packing).  A row is
// owned by `lpr` adjacent lanes (a power of two <= 32, so a row never leaves
// its wavefront) with OPT octs per lane; a 256-thread workgroup owns
// 256 / lpr consecutive rows (always a multiple of 8, so it owns whole
// row-groups of every bit width).  Row min/max are butterfly reductions in
// registers; the quantised bytes are staged in LDS, where the lane that owns
// the first row of a group ORs the 8/bits rows of that group together and
// writes the packed bytes with one vector store.
//
// All arithmetic that decides a quantised value is written as separate fp32
// operations and this file is compiled with -ffp-contract=off, so the result
// is the unfused expression of the reference source.

#include <cmath>

#include "exact_common.hpp"

namespace exact {

// offsets inside the rows of one workgroup: 32 bits where the rows are known to be short
template <bool NARROW> struct OffsetType { using type = int64_t; };
template <> struct OffsetType<true> { using type = uint32_t; };

// ---------------------------------------------------------------------------
// loads / stores of one oct with `nv` (0..8) valid leading elements
// ---------------------------------------------------------------------------
template <int VEC, bool FULL>
__device__ __forceinline__ void load_oct(const float* __restrict__ p, int nv, float (&v)[8]) {
  if constexpr (VEC == 4) {
    f32x4 a = {0.f, 0.f, 0.f, 0.f}, b = a;
    if (FULL || nv > 0) a = nt_load4(p);
    if (FULL || nv > 4) b = nt_load4(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (i < nv) ? __builtin_nontemporal_load(p + i) : 0.f;
  }
}

template <int VEC, bool FULL>
__device__ __forceinline__ void store_oct(float* __restrict__ p, int nv, const float (&v)[8]) {
  if constexpr (VEC == 4) {
    if (FULL || nv > 0) nt_store4(p, v[0], v[1], v[2], v[3]);
    if (FULL || nv > 4) nt_store4(p + 4, v[4], v[5], v[6], v[7]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < nv) __builtin_nontemporal_store(v[i], p + i);
  }
}

// fp16 activations (the reference's kernels are also instantiated for at::Half,
// quantization_cuda_kernel.cu:132-150): one oct is 16 bytes.  VEC == 4 here
// means "whole octs, 16-byte aligned" (G % 8 == 0).
template <int VEC, bool FULL>
__device__ __forceinline__ void load_oct_half(const half_t* __restrict__ p, int nv, float (&v)[8]) {
  if constexpr (VEC == 4) {
    typedef half_t half8 __attribute__((ext_vector_type(8)));
    half8 q = {0, 0, 0, 0, 0, 0, 0, 0};
    if (FULL || nv > 0) q = __builtin_nontemporal_load(reinterpret_cast<const half8*>(p));
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = static_cast<float>(q[i]);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (i < nv) ? static_cast<float>(__builtin_nontemporal_load(p + i)) : 0.f;
  }
}

// 8 consecutive floats that every workgroup reads again (per-column
// parameters): ordinary cached loads, 16-byte aligned
__device__ __forceinline__ void load_cached8(const float* __restrict__ p, float (&v)[8]) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p);
  const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

// OPT octs of one row segment for a lane, read "row-contiguously": load i of a
// lane fetches quad (16 bytes) i * lpr + lir of the segment, so that every load
// instruction covers lpr * 16 contiguous bytes per row (an oct per lane makes
// the two loads of a lane 16 bytes apart and the instruction skips every other
// 16 bytes: 5 - 10 % slower).  The lanes 2m and 2m + 1 then hold the two halves
// of the octs i * lpr / 2 + m (i < 2 OPT) and trade them: the even lane ends up
// with the octs of even i, the odd lane with those of odd i, i.e. lane lir owns
// oct (2k + lir % 2) * lpr / 2 + lir / 2 as its k-th -- for a given k the lanes
// of a row own lpr consecutive octs, so the packed bytes of a row leave in runs
// of 8 lpr bytes per store instruction.  lpr even; every lane takes part.
template <int OPT>
__device__ __forceinline__ int swizzled_oct(int lir, int lpr, int k) {
  return (2 * k + (lir & 1)) * (lpr >> 1) + (lir >> 1);
}

template <int OPT, typename OFF>
__device__ __forceinline__ void load_octs_swizzled(const float* __restrict__ base, OFF seg, int lpr, int lir,
                                                   float (&v)[OPT][8]) {
  // `base` is the same for the whole workgroup and `seg` (the lane's row segment, in floats from base) is
  // 32 bits wide in the one-launch forms: the addresses then need no 64-bit vector arithmetic
  f32x4 q[2 * OPT];
#pragma unroll
  for (int i = 0; i < 2 * OPT; ++i) q[i] = nt_load4(base + (seg + static_cast<OFF>(4 * (i * lpr + lir))));
  const bool odd = lir & 1;
#pragma unroll
  for (int k = 0; k < OPT; ++k) {
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      // this lane's half of oct 2k' (even_i) and of oct 2k' + 1 (odd_i); the even lane keeps oct 2k' and
      // wants the neighbour's even_i, the odd lane keeps oct 2k' + 1 and wants the neighbour's odd_i
      // (lanes 2m <-> 2m + 1; each select takes the neighbour's value through DPP in the same instruction)
      const float even_i = q[2 * k][c], odd_i = q[2 * k + 1][c];
      const float from_even = __int_as_float(dpp_lanes<0xB1>(__float_as_int(odd_i)));
      const float from_odd = __int_as_float(dpp_lanes<0xB1>(__float_as_int(even_i)));
      v[k][c] = odd ? from_even : even_i;       // first half: columns 0..3 of the oct (held by the even lane)
      v[k][4 + c] = odd ? odd_i : from_odd;     // second half (held by the odd lane)
    }
  }
}

// ---------------------------------------------------------------------------
// pack
// ---------------------------------------------------------------------------
struct PackArgs {
  const float* x;
  const float* noise;     // nullable
  const float* mn_in;     // two-step form only
  const float* scale_in;  // two-step form only
  uint32_t seed_lo, seed_hi, off_lo, off_hi;
  int64_t N;
  int G;
  int opr;        // octs per row
  int lpr_log2;   // log2(lanes per row)
  int out_vec;    // 8, 4 or 1: widest aligned store of packed bytes
  uint8_t* packed;
  int64_t pad_index;  // index of the trailing pad byte
  float* scale_f32;
  float* min_f32;
  uint16_t* scale_bf16;
  uint16_t* min_bf16;
  // ACT form only: ReLU + dropout applied to x before the statistics
  const float* act_noise;  // nullable
  uint32_t act_seed_lo, act_seed_hi, act_off_lo, act_off_hi;
  uint32_t act_keep_from;  // generator noise: an element is kept when its 16 random bits are >= this
  float p, pinv;
  float* y;                // activation output [N, G]
  uint8_t* mask_bytes;     // 1-bit mask of (x > 0) && keep, byte i / 8 holds elements i .. i + 7
  int64_t mask_tail_begin, mask_tail_end;  // bytes of the last mask word no element maps to
  // ACT form, optional: per-column normalisation (x - mean) * mult + shift ahead of the ReLU
  const float* norm_mean;   // nullable: no normalisation
  const float* norm_mult;
  const float* norm_shift;
};

// ACT: x first goes through ReLU and dropout (the arithmetic of
// dropout_fwd_kernel<.., RELU = true>; noise from the flat Philox stream of the
// mask kernels, block = flat index / 8), the result is written to y, its mask
// bits to mask_bytes, and the row statistics / quantisation then work on that
// result -- "ReLU -> dropout -> quantize_activation of the next layer's input"
// in one pass.  Needs G % 8 == 0, so that an oct is one Philox block and one
// mask byte.
//
// HALF: x holds fp16 values and the 16-bit parameter outputs receive fp16 bits.
// The arithmetic follows what the reference's at::Half instantiation computes:
// at::Half operators evaluate in fp32 and round the result to fp16, so
// (x - min) and its product with scale are each rounded to fp16, the noise is
// then added in fp32 (quantization_cuda_kernel.cu:88-89); torch evaluates the
// scale as (mx - mn).reciprocal() * B with an fp16 rounding after every step.
template <int BITS, int OPT, int VEC, bool FULL, bool NOISE_IN, bool FUSED, bool ACT = false, bool HALF = false>
__global__ __launch_bounds__(kBlock) void pack_kernel(const PackArgs a) {
  constexpr int WPT = 8 / BITS;
  constexpr float B = static_cast<float>((1 << BITS) - 1);
  __shared__ uint2 stage[WPT > 1 ? OPT * kBlock : 1];
  __shared__ f32x4 ybuf[ACT ? OPT * kBlock * 2 : 1];  // ACT: the activation output on its way to memory
  // ACT with a normalisation ahead: mean, mult and shift of the G columns (dynamic LDS, 3 G floats, asked for by
  // that launch only).  Every row needs them, so the workgroup fetches them once; read from memory per oct they
  // cost three times the load instructions of x itself
  HIP_DYNAMIC_SHARED(f32x4, norm_quads)  // declared in 16-byte units: the parameters are read as quads
  float* norm_lds = reinterpret_cast<float*>(norm_quads);

  const int t = threadIdx.x;
  const int lpr = 1 << a.lpr_log2;
  const int lane_in_row = t & (lpr - 1);
  const int row_local = t >> a.lpr_log2;
  const int rows_per_wg = kBlock >> a.lpr_log2;
  // Addresses are "first row of this workgroup" (the same for every lane: scalar registers) plus an offset
  // inside the workgroup's rows, which fits 32 bits in the one-launch forms (G <= 1024) -- no 64-bit vector
  // arithmetic there.  The two-step form (any G) keeps 64-bit offsets.
  using off_t = typename OffsetType<FUSED>::type;
  const int64_t row_base = static_cast<int64_t>(blockIdx.x) * rows_per_wg;
  const int64_t rows_left = a.N - row_base;  // >= 1
  const int rows_here = rows_left < rows_per_wg ? static_cast<int>(rows_left) : rows_per_wg;
  const bool row_ok = row_local < rows_here;
  const uint32_t n_lo = static_cast<uint32_t>(row_base) + static_cast<uint32_t>(row_local);  // N < 2^32
  const off_t G = static_cast<off_t>(a.G);
  const off_t row_off = static_cast<off_t>(row_local) * G;
  const float* __restrict__ xw = HALF ? nullptr : a.x + row_base * a.G;
  const half_t* __restrict__ hw = HALF ? reinterpret_cast<const half_t*>(a.x) + row_base * a.G : nullptr;
  const int oct_base = blockIdx.y * (lpr * OPT);  // 0 in the fused form
  // which octs of the row segment a lane owns: lane + k * lpr, or the row-contiguous assignment
  // (whole rows of 16-byte aligned fp32 octs; the host launches those forms with lpr >= 2 only)
  constexpr bool swz = FULL && VEC == 4 && !HALF;
  auto oct_of = [&](int lir, int k) {
    return oct_base + (swz ? swizzled_oct<OPT>(lir, lpr, k) : lir + k * lpr);
  };
  // rows past the end re-read the last row and drop it
  const off_t row_ld_off = static_cast<off_t>(row_ok ? row_local : rows_here - 1) * G + static_cast<off_t>(8 * oct_base);

  if constexpr (ACT) {
    if (a.norm_mean != nullptr) {  // same for every lane of the launch: every wavefront reaches the barrier
      for (int c = t; c < a.G; c += kBlock) {
        norm_lds[c] = a.norm_mean[c];
        norm_lds[a.G + c] = a.norm_mult[c];
        norm_lds[2 * a.G + c] = a.norm_shift[c];
      }
      __syncthreads();
    }
  }

  float v[OPT][8];
  int nv[OPT];
#pragma unroll
  for (int k = 0; k < OPT; ++k) {
    const int j = oct_of(lane_in_row, k);
    const int d0 = 8 * j;
    nv[k] = (row_ok && j < a.opr) ? min(8, a.G - d0) : 0;
    if constexpr (swz) {
      // all OPT octs at once, by every lane (the lanes of a pair trade halves)
      if (k == 0) {
        load_octs_swizzled<OPT, off_t>(xw, row_ld_off, lpr, lane_in_row, v);
        if (!row_ok) {
#pragma unroll
          for (int kk = 0; kk < OPT; ++kk)
#pragma unroll
            for (int i = 0; i < 8; ++i) v[kk][i] = 0.f;
        }
      }
    } else if (FULL && !row_ok) {
#pragma unroll
      for (int i = 0; i < 8; ++i) v[k][i] = 0.f;
    } else {
      if constexpr (HALF) load_oct_half<VEC, FULL>(hw + (row_off + static_cast<off_t>(d0)), nv[k], v[k]);
      else load_oct<VEC, FULL>(xw + (row_off + static_cast<off_t>(d0)), nv[k], v[k]);
    }
    if constexpr (ACT) {
      if (nv[k] > 0) {  // G % 8 == 0: a whole oct or nothing
        // Philox block and mask byte of this oct: flat element index / 8 (G % 8 == 0)
        const uint32_t g8 = static_cast<uint32_t>(a.G) >> 3;
        const uint32_t blk_local = static_cast<uint32_t>(row_local) * g8 + static_cast<uint32_t>(j);
        const int64_t blk = row_base * g8 + blk_local;
        // keep[i]: the element's uniform exceeds p.  Supplied noise is compared as it is; the generator's
        // uniform is (h + 0.5) / 65536 for 16 random bits h, exactly, so u > p  <=>  h >= act_keep_from
        // (the host works the threshold out in double): no conversion per element
        float ud[8];
        uint32_t hd[8];
        if constexpr (NOISE_IN) {
          load_oct<VEC, true>(a.act_noise + row_base * a.G + (row_off + static_cast<off_t>(d0)), 8, ud);
        } else {
          const Philox4 r = philox4x32_10(static_cast<uint32_t>(blk), static_cast<uint32_t>(blk >> 32),
                                          a.act_off_lo, a.act_off_hi, a.act_seed_lo, a.act_seed_hi);
          hd[0] = r.x & 0xFFFFu; hd[1] = r.x >> 16; hd[2] = r.y & 0xFFFFu; hd[3] = r.y >> 16;
          hd[4] = r.z & 0xFFFFu; hd[5] = r.z >> 16; hd[6] = r.w & 0xFFFFu; hd[7] = r.w >> 16;
        }
        if (a.norm_mean != nullptr) {  // same for every lane of the launch
          // training-mode batch norm of the column, statistics given:
          // weight * (x - mean) * invstd + bias with mult = weight * invstd
          float cm[8], cs[8], cb[8];
          load_cached8(norm_lds + d0, cm);
          load_cached8(norm_lds + a.G + d0, cs);
          load_cached8(norm_lds + 2 * a.G + d0, cb);
#pragma unroll
          for (int i = 0; i < 8; ++i) {
            float c = v[k][i] - cm[i];
            c = c * cs[i];
            v[k][i] = c + cb[i];
          }
        }
        uint32_t m = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const bool pos = v[k][i] > 0.f;
          const bool keep = NOISE_IN ? (ud[i] > a.p) : (hd[i] >= a.act_keep_from);
          // (r * keep) * pinv of the separate kernel, keep being 1 or 0: r * pinv or r * 0, the same values
          const float r = pos ? v[k][i] : 0.f;
          v[k][i] = r * (keep ? a.pinv : 0.f);
          m |= static_cast<uint32_t>(pos && keep) << i;
        }
        // y leaves through LDS: an oct per lane would make every 16-byte store
        // instruction skip every other 16 bytes, which halves the store rate
        ybuf[(k * kBlock + t) * 2 + 0] = f32x4{v[k][0], v[k][1], v[k][2], v[k][3]};
        ybuf[(k * kBlock + t) * 2 + 1] = f32x4{v[k][4], v[k][5], v[k][6], v[k][7]};
        (a.mask_bytes + row_base * g8)[blk_local] = static_cast<uint8_t>(m);
      }
    }
  }
  if constexpr (ACT) {
    // Lane l of a wavefront stores quad l, then quad 64 + l, of the wavefront's
    // 64 octs of each k: whole runs of 32 * lpr contiguous bytes per row.
    __syncthreads();
    const int wave_first = t & ~(kWave - 1);
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
#pragma unroll
      for (int s = 0; s < 2; ++s) {
        const int q = s * kWave + (t & (kWave - 1));
        const int src = wave_first + (q >> 1);  // the thread that produced this quad
        const int half = q & 1;
        const int row_src = src >> a.lpr_log2;
        const int j_src = oct_of(src & (lpr - 1), k);
        if (row_src < rows_here && j_src < a.opr) {
          const f32x4 val = ybuf[(k * kBlock + src) * 2 + half];
          nt_store4(a.y + row_base * a.G + (static_cast<off_t>(row_src) * G + static_cast<off_t>(8 * j_src + 4 * half)),
                    val.x, val.y, val.z, val.w);
        }
      }
    }
  }

  float mnv = 0.f, sc = 0.f;
  if constexpr (FUSED) {
    float lo = __builtin_inff(), hi = -__builtin_inff();
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (FULL || i < nv[k]) {
          lo = fminf(lo, v[k][i]);
          hi = fmaxf(hi, v[k][i]);
        }
      }
    }
    group_minmax(lo, hi, lpr);
    mnv = lo;
    // ops.py:39 `(2 ** bits - 1) / (mx - mn)`: torch evaluates int / tensor as
    // tensor.reciprocal() * int, so two roundings
    if constexpr (HALF) {
      const float recip = round_to_half(1.0f / round_to_half(hi - lo));
      sc = round_to_half(recip * B);
    } else {
      const float recip = 1.0f / (hi - lo);
      sc = recip * B;
    }
    if (row_ok && lane_in_row == 0) {
      if (a.scale_f32) (a.scale_f32 + row_base)[row_local] = sc;
      if (a.min_f32) (a.min_f32 + row_base)[row_local] = mnv;
      if (a.scale_bf16) (a.scale_bf16 + row_base)[row_local] = HALF ? half_bits(sc) : f32_to_bf16_rne(sc);
      if (a.min_bf16) (a.min_bf16 + row_base)[row_local] = HALF ? half_bits(mnv) : f32_to_bf16_rne(mnv);
    }
  } else {
    if (row_ok) {
      mnv = (a.mn_in + row_base)[row_local];
      sc = (a.scale_in + row_base)[row_local];
    }
  }

  // supplied noise: read like x (every lane takes part; rows past the end re-read the last row, their
  // codes are dropped below)
  float un[(NOISE_IN && swz) ? OPT : 1][8];
  const float* __restrict__ nw = NOISE_IN ? a.noise + row_base * a.G : nullptr;
  if constexpr (NOISE_IN && swz) load_octs_swizzled<OPT, off_t>(nw, row_ld_off, lpr, lane_in_row, un);
  uint2 codes[OPT];
#pragma unroll
  for (int k = 0; k < OPT; ++k) {
    const int j = oct_of(lane_in_row, k);
    float u[8];
    if constexpr (NOISE_IN) {
      if constexpr (swz) {
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = un[k][i];
      } else if (FULL && !row_ok) {
#pragma unroll
        for (int i = 0; i < 8; ++i) u[i] = 0.f;
      } else {
        load_oct<VEC, FULL>(nw + (row_off + static_cast<off_t>(8 * j)), nv[k], u);
      }
    } else {
      const Philox4 r = philox4x32_10(static_cast<uint32_t>(j), n_lo, a.off_lo, a.off_hi, a.seed_lo, a.seed_hi);
      philox_uniform8(r, u);
    }
    uint32_t q[8];  // the code in the low byte
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // quantization_cuda_kernel.cu:89, one rounding per operation
      float tq = v[k][i] - mnv;
      if constexpr (HALF) tq = round_to_half(tq);
      tq = tq * sc;
      if constexpr (HALF) tq = round_to_half(tq);
      tq = tq + u[i];
      if constexpr (FUSED) {
        // scale and min come from this row: tq < 2^bits + 2
        q[i] = code_in_low_byte(tq);
      } else {
        tq = tq - 0.5f;
        tq = fmaxf(tq, 0.f);
        q[i] = float2int_rn_sat(tq);
      }
      if constexpr (!FULL) q[i] = (i < nv[k]) ? q[i] : 0u;
    }
    codes[k] = make_uint2(low_bytes4(q[0], q[1], q[2], q[3]), low_bytes4(q[4], q[5], q[6], q[7]));
    if constexpr (FULL) {
      if (!row_ok) codes[k] = make_uint2(0u, 0u);
    }
    if constexpr (WPT == 8) {
      // one bit per code: every lane moves its row's bits into place first (bits shifted past bit 7 of a byte
      // vanish, as in the reference's uint8 accumulator), so that the lane that packs only has to OR eight words
      constexpr uint32_t kByte = 0x01010101u;
      const int sh = row_local & 7;
      const uint32_t keep = (0xFFu >> sh) * kByte;
      stage[k * kBlock + t] = make_uint2((codes[k].x & keep) << sh, (codes[k].y & keep) << sh);
    } else if constexpr (WPT > 1) {
      stage[k * kBlock + t] = codes[k];
    }
  }
  if constexpr (WPT > 1) __syncthreads();  // 8-bit codes: one row per byte, nothing to combine

  // The lane holding the first row of a row-group packs the whole group.
  if ((row_local & (WPT - 1)) == 0 && row_ok) {
#pragma unroll
    for (int k = 0; k < OPT; ++k) {
      const int j = oct_of(lane_in_row, k);
      if (j >= a.opr) continue;
      uint32_t w0 = codes[k].x, w1 = codes[k].y;
      if constexpr (WPT == 8) {
#pragma unroll
        for (int i = 1; i < WPT; ++i) {
          const uint2 s = stage[k * kBlock + t + i * lpr];  // already in place
          w0 |= s.x;
          w1 |= s.y;
        }
      } else {
#pragma unroll
      for (int i = 1; i < WPT; ++i) {
        // uint8 accumulator of the reference: bits shifted past bit 7 vanish
        constexpr uint32_t kByte = 0x01010101u;
        const uint32_t keep = (0xFFu >> (i * BITS)) * kByte;
        const uint2 s = stage[k * kBlock + t + i * lpr];
        w0 |= (s.x & keep) << (i * BITS);
        w1 |= (s.y & keep) << (i * BITS);
      }
      }
      const int d0 = 8 * j;
      // row_base is a multiple of 8, hence of WPT
      uint8_t* dst = a.packed + (row_base / WPT) * a.G + (static_cast<off_t>(row_local / WPT) * G + static_cast<off_t>(d0));
      if (a.out_vec == 8) {
        // one 8-byte store: written as two struct members, the compiler hoists the
        // first word's store out of this branch and issues two 4-byte stores
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        const u32x2 both = {w0, w1};
        *reinterpret_cast<u32x2*>(dst) = both;
      } else if (a.out_vec == 4) {
        *reinterpret_cast<uint32_t*>(dst) = w0;
        if (d0 + 4 < a.G) *reinterpret_cast<uint32_t*>(dst + 4) = w1;
      } else {
        const int cnt = min(8, a.G - d0);
        for (int i = 0; i < cnt; ++i)
          dst[i] = static_cast<uint8_t>((i < 4 ? w0 >> (8 * i) : w1 >> (8 * (i - 4))) & 0xFFu);
      }
    }
  }
  if (blockIdx.x == 0 && blockIdx.y == 0 && t == 0) {
    a.packed[a.pad_index] = 0;
    if constexpr (ACT)
      for (int64_t i = a.mask_tail_begin; i < a.mask_tail_end; ++i) a.mask_bytes[i] = 0;
  }
}

// ---------------------------------------------------------------------------
// row statistics for rows longer than the fused kernel holds in registers,
// and the stand-alone a1 entry point: one wavefront per row.
// ---------------------------------------------------------------------------
template <int VEC>
__global__ __launch_bounds__(kBlock) void row_minmax_kernel(const float* __restrict__ x, int64_t N,
                                                            int64_t G, float* __restrict__ mn_out,
                                                            float* __restrict__ mx_out, int bits,
                                                            float* __restrict__ scale_f32,
                                                            uint16_t* __restrict__ scale_bf16,
                                                            uint16_t* __restrict__ min_bf16) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t n = static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + (threadIdx.x >> 6);
  if (n >= N) return;
  const float* row = x + n * G;
  float lo = __builtin_inff(), hi = -__builtin_inff();
  if constexpr (VEC == 4) {
    const float4* r4 = reinterpret_cast<const float4*>(row);
    for (int64_t c = lane; c < G / 4; c += kWave) {
      const float4 q = r4[c];
      lo = fminf(fminf(lo, q.x), fminf(q.y, fminf(q.z, q.w)));
      hi = fmaxf(fmaxf(hi, q.x), fmaxf(q.y, fmaxf(q.z, q.w)));
    }
  } else {
    for (int64_t c = lane; c < G; c += kWave) {
      lo = fminf(lo, row[c]);
      hi = fmaxf(hi, row[c]);
    }
  }
  group_minmax(lo, hi, kWave);
  if (lane == 0) {
    if (mn_out) mn_out[n] = lo;
    if (mx_out) mx_out[n] = hi;
    if (bits > 0) {
      const float recip = 1.0f / (hi - lo);
      const float sc = recip * static_cast<float>((1 << bits) - 1);
      if (scale_f32) scale_f32[n] = sc;
      if (scale_bf16) scale_bf16[n] = f32_to_bf16_rne(sc);
      if (min_bf16) min_bf16[n] = f32_to_bf16_rne(lo);
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct Geometry {
  int opr, lpr_log2, opt, grid_y;
  bool full;
};

// Octs per thread and lanes per row for rows of G columns.  `max_opt` octs fit
// in registers; longer rows are tiled over grid.y (two-step form only).
// `opt_hint` (1, 2 or 4; 0 = none) overrides the default choice when the row
// still fits 32 lanes with it: the caller may have timed the alternatives.
static Geometry plan_rows(int64_t G, int max_opt, int opt_hint = 0) {
  Geometry g;
  g.opr = static_cast<int>((G + 7) / 8);
  // Aim for 16 lanes per row: the per-lane fixed work (row statistics butterfly,
  // the scale division, parameter stores, address set-up) is then shared by
  // two octs at 256 columns and four at 512, and a row never leaves one DPP row.
  int opt = (g.opr + 15) / 16;
  if (opt > max_opt) opt = max_opt;
  if (opt == 3) opt = 4;
  if (opt < 1) opt = 1;
  if ((opt_hint == 1 || opt_hint == 2 || opt_hint == 4) && opt_hint <= max_opt &&
      (g.opr + opt_hint - 1) / opt_hint <= 32)
    opt = opt_hint;
  const int lanes_needed = (g.opr + opt - 1) / opt;
  int l2 = 0;
  while ((1 << l2) < lanes_needed && l2 < 5) ++l2;
  g.lpr_log2 = l2;
  g.opt = opt;
  const int octs_per_pass = (1 << l2) * opt;
  g.grid_y = (g.opr + octs_per_pass - 1) / octs_per_pass;
  // whole rows of whole octs on at least two lanes (the row-contiguous loads pair up neighbouring lanes)
  g.full = (G % 8 == 0) && (g.opr == octs_per_pass * g.grid_y) && l2 >= 1;
  return g;
}

__global__ void zero_byte_kernel(uint8_t* p) { *p = 0; }

static bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

template <int BITS, int OPT, bool NOISE_IN, bool FUSED>
static void launch_pack_variant(const PackArgs& a, bool vec4, bool full, dim3 grid, hipStream_t s) {
  if (vec4 && full)
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 4, true, NOISE_IN, FUSED>), grid, dim3(kBlock), 0, s, a);
  else if (vec4)
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 4, false, NOISE_IN, FUSED>), grid, dim3(kBlock), 0, s, a);
  else
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 1, false, NOISE_IN, FUSED>), grid, dim3(kBlock), 0, s, a);
}

template <int BITS, bool NOISE_IN, bool FUSED>
static void launch_pack_opt(const PackArgs& a, int opt, bool vec4, bool full, dim3 grid, hipStream_t s) {
  if constexpr (FUSED) {
    if (opt == 4) return launch_pack_variant<BITS, 4, NOISE_IN, FUSED>(a, vec4, full, grid, s);
    if (opt == 2) return launch_pack_variant<BITS, 2, NOISE_IN, FUSED>(a, vec4, full, grid, s);
  }
  launch_pack_variant<BITS, 1, NOISE_IN, FUSED>(a, vec4, full, grid, s);
}

template <bool NOISE_IN, bool FUSED>
static void launch_pack_bits(const PackArgs& a, int bits, int opt, bool vec4, bool full, dim3 grid, hipStream_t s) {
  switch (bits) {
    case 1: return launch_pack_opt<1, NOISE_IN, FUSED>(a, opt, vec4, full, grid, s);
    case 2: return launch_pack_opt<2, NOISE_IN, FUSED>(a, opt, vec4, full, grid, s);
    case 4: return launch_pack_opt<4, NOISE_IN, FUSED>(a, opt, vec4, full, grid, s);
    default: return launch_pack_opt<8, NOISE_IN, FUSED>(a, opt, vec4, full, grid, s);
  }
}

static int check_quant_shape(int64_t N, int64_t G, int bits) {
  if (bits != 1 && bits != 2 && bits != 4 && bits != 8) return EXACT_E_BITS;
  if (N < 0 || G < 0 || N > 0xFFFFFFFFll || G > 0x7FFFFFF0ll) return EXACT_E_SHAPE;
  return EXACT_OK;
}

static int pack_common(const float* x, const float* mn, const float* scale, const float* noise,
                       uint64_t seed, uint64_t offset, int64_t N, int64_t G, int bits,
                       uint8_t* packed, float* scale_f32, float* min_f32, uint16_t* scale_bf16,
                       uint16_t* min_bf16, bool fused, hipStream_t s, int opt_hint = 0) {
  if (int rc = check_quant_shape(N, G, bits)) return rc;
  if (!packed) return EXACT_E_NULL;
  const int64_t pad_index = exact_packed_nbytes(N, G, bits) - 1;
  if (N == 0 || G == 0) {
    // nothing but the pad byte (a kernel, not a memset node, so callers may capture it)
    hipLaunchKernelGGL(zero_byte_kernel, dim3(1), dim3(1), 0, s, packed + pad_index);
    return launch_status();
  }
  if (!x || (!fused && (!mn || !scale))) return EXACT_E_NULL;

  bool do_fused = fused;
  if (fused && G > 1024) {
    // rows too long for registers: statistics first, then the two-step form
    float* mn_tmp = min_f32;
    float* sc_tmp = scale_f32;
    if (!mn_tmp || !sc_tmp) return EXACT_E_NULL;  // caller must give fp32 outputs for G > 1024
    const bool v4 = (G % 4 == 0) && aligned(x, 16);
    const dim3 grid(static_cast<unsigned>((N + 3) / 4));
    if (v4)
      hipLaunchKernelGGL((row_minmax_kernel<4>), grid, dim3(kBlock), 0, s, x, N, G, mn_tmp,
                         static_cast<float*>(nullptr), bits, sc_tmp, scale_bf16, min_bf16);
    else
      hipLaunchKernelGGL((row_minmax_kernel<1>), grid, dim3(kBlock), 0, s, x, N, G, mn_tmp,
                         static_cast<float*>(nullptr), bits, sc_tmp, scale_bf16, min_bf16);
    mn = mn_tmp;
    scale = sc_tmp;
    do_fused = false;
  }

  const Geometry g = plan_rows(G, do_fused ? 4 : 1, opt_hint);
  PackArgs a{};
  a.x = x;
  a.noise = noise;
  a.mn_in = mn;
  a.scale_in = scale;
  a.seed_lo = static_cast<uint32_t>(seed);
  a.seed_hi = static_cast<uint32_t>(seed >> 32);
  a.off_lo = static_cast<uint32_t>(offset);
  a.off_hi = static_cast<uint32_t>(offset >> 32);
  a.N = N;
  a.G = static_cast<int>(G);
  a.opr = g.opr;
  a.lpr_log2 = g.lpr_log2;
  a.packed = packed;
  a.pad_index = pad_index;
  a.scale_f32 = do_fused ? scale_f32 : nullptr;
  a.min_f32 = do_fused ? min_f32 : nullptr;
  a.scale_bf16 = do_fused ? scale_bf16 : nullptr;
  a.min_bf16 = do_fused ? min_bf16 : nullptr;
  a.out_vec = (G % 8 == 0 && aligned(packed, 8)) ? 8 : (G % 4 == 0 && aligned(packed, 4)) ? 4 : 1;
  const bool vec4 = (G % 4 == 0) && aligned(x, 16) && (!noise || aligned(noise, 16));
  const int rows_per_wg = kBlock >> g.lpr_log2;
  const dim3 grid(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg), static_cast<unsigned>(g.grid_y));
  const bool full = g.full && vec4;
  if (do_fused) {
    if (noise) launch_pack_bits<true, true>(a, bits, g.opt, vec4, full, grid, s);
    else launch_pack_bits<false, true>(a, bits, g.opt, vec4, full, grid, s);
  } else {
    if (noise) launch_pack_bits<true, false>(a, bits, g.opt, vec4, full, grid, s);
    else launch_pack_bits<false, false>(a, bits, g.opt, vec4, full, grid, s);
  }
  return launch_status();
}

// ---- ReLU + dropout + statistics + pack (ACT form) ---------------------------
template <int BITS, int OPT, bool NOISE_IN>
static void launch_act_variant(const PackArgs& a, bool full, dim3 grid, hipStream_t s) {
  const size_t norm_bytes = a.norm_mean != nullptr ? sizeof(float) * 3 * static_cast<size_t>(a.G) : 0;  // G <= 1024: 12 KB
  if (full)
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 4, true, NOISE_IN, true, true>), grid, dim3(kBlock), norm_bytes, s, a);
  else
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 4, false, NOISE_IN, true, true>), grid, dim3(kBlock), norm_bytes, s, a);
}

template <int BITS, bool NOISE_IN>
static void launch_act_opt(const PackArgs& a, int opt, bool full, dim3 grid, hipStream_t s) {
  if (opt == 4) return launch_act_variant<BITS, 4, NOISE_IN>(a, full, grid, s);
  if (opt == 2) return launch_act_variant<BITS, 2, NOISE_IN>(a, full, grid, s);
  launch_act_variant<BITS, 1, NOISE_IN>(a, full, grid, s);
}

template <bool NOISE_IN>
static void launch_act_bits(const PackArgs& a, int bits, int opt, bool full, dim3 grid, hipStream_t s) {
  switch (bits) {
    case 1: return launch_act_opt<1, NOISE_IN>(a, opt, full, grid, s);
    case 2: return launch_act_opt<2, NOISE_IN>(a, opt, full, grid, s);
    case 4: return launch_act_opt<4, NOISE_IN>(a, opt, full, grid, s);
    default: return launch_act_opt<8, NOISE_IN>(a, opt, full, grid, s);
  }
}

// ---- fp16 activations (HALF form): statistics + pack in one launch, G <= 1024 --
template <int BITS, int OPT, bool NOISE_IN>
static void launch_half_variant(const PackArgs& a, bool whole, bool full, dim3 grid, hipStream_t s) {
  if (whole && full)
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 4, true, NOISE_IN, true, false, true>), grid, dim3(kBlock), 0, s, a);
  else if (whole)
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 4, false, NOISE_IN, true, false, true>), grid, dim3(kBlock), 0, s, a);
  else
    hipLaunchKernelGGL((pack_kernel<BITS, OPT, 1, false, NOISE_IN, true, false, true>), grid, dim3(kBlock), 0, s, a);
}

template <int BITS, bool NOISE_IN>
static void launch_half_opt(const PackArgs& a, int opt, bool whole, bool full, dim3 grid, hipStream_t s) {
  if (opt == 4) return launch_half_variant<BITS, 4, NOISE_IN>(a, whole, full, grid, s);
  if (opt == 2) return launch_half_variant<BITS, 2, NOISE_IN>(a, whole, full, grid, s);
  launch_half_variant<BITS, 1, NOISE_IN>(a, whole, full, grid, s);
}

template <bool NOISE_IN>
static void launch_half_bits(const PackArgs& a, int bits, int opt, bool whole, bool full, dim3 grid, hipStream_t s) {
  switch (bits) {
    case 1: return launch_half_opt<1, NOISE_IN>(a, opt, whole, full, grid, s);
    case 2: return launch_half_opt<2, NOISE_IN>(a, opt, whole, full, grid, s);
    case 4: return launch_half_opt<4, NOISE_IN>(a, opt, whole, full, grid, s);
    default: return launch_half_opt<8, NOISE_IN>(a, opt, whole, full, grid, s);
  }
}

}  // namespace exact

using namespace exact;

extern "C" {

int64_t exact_packed_nbytes(int64_t N, int64_t G, int bits) {
  if (bits != 1 && bits != 2 && bits != 4 && bits != 8) return EXACT_E_BITS;
  const int64_t wpt = 8 / bits;
  const int64_t n_round = N + (wpt - N % wpt) % wpt;
  return (static_cast<int64_t>(bits) * n_round * G + 8) / 8;
}

int exact_row_minmax_f32(const float* x, int64_t N, int64_t G, float* mn, float* mx, void* stream) {
  if (N < 0 || G <= 0) return N == 0 || G == 0 ? (N < 0 || G < 0 ? EXACT_E_SHAPE : EXACT_OK) : EXACT_E_SHAPE;
  if (N == 0) return EXACT_OK;
  if (!x || !mn || !mx) return EXACT_E_NULL;
  const dim3 grid(static_cast<unsigned>((N + 3) / 4));
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (G % 4 == 0 && aligned(x, 16))
    hipLaunchKernelGGL((row_minmax_kernel<4>), grid, dim3(kBlock), 0, s, x, N, G, mn, mx, 0,
                       static_cast<float*>(nullptr), static_cast<uint16_t*>(nullptr),
                       static_cast<uint16_t*>(nullptr));
  else
    hipLaunchKernelGGL((row_minmax_kernel<1>), grid, dim3(kBlock), 0, s, x, N, G, mn, mx, 0,
                       static_cast<float*>(nullptr), static_cast<uint16_t*>(nullptr),
                       static_cast<uint16_t*>(nullptr));
  return launch_status();
}

int exact_pack_f32(const float* x, const float* mn, const float* scale, const float* noise,
                   uint64_t seed, uint64_t offset, int64_t N, int64_t G, int bits, uint8_t* packed,
                   void* stream) {
  return pack_common(x, mn, scale, noise, seed, offset, N, G, bits, packed, nullptr, nullptr, nullptr,
                     nullptr, false, static_cast<hipStream_t>(stream));
}

int exact_minmax_pack_f32(const float* x, const float* noise, uint64_t seed, uint64_t offset,
                          int64_t N, int64_t G, int bits, uint8_t* packed, float* scale_f32,
                          float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16, void* stream) {
  return pack_common(x, nullptr, nullptr, noise, seed, offset, N, G, bits, packed, scale_f32, min_f32,
                     scale_bf16, min_bf16, true, static_cast<hipStream_t>(stream));
}

int exact_minmax_pack_geom_f32(const float* x, const float* noise, uint64_t seed, uint64_t offset,
                               int64_t N, int64_t G, int bits, uint8_t* packed, float* scale_f32,
                               float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16, int octs_per_lane,
                               void* stream) {
  if (octs_per_lane != 0 && octs_per_lane != 1 && octs_per_lane != 2 && octs_per_lane != 4) return EXACT_E_ARG;
  return pack_common(x, nullptr, nullptr, noise, seed, offset, N, G, bits, packed, scale_f32, min_f32,
                     scale_bf16, min_bf16, true, static_cast<hipStream_t>(stream), octs_per_lane);
}

static int act_pack_common(const float* x, const float* norm_mean, const float* norm_mult,
                           const float* norm_shift, float p, const float* act_noise, uint64_t act_seed,
                           uint64_t act_offset, const float* noise, uint64_t seed, uint64_t offset,
                           int64_t N, int64_t G, int bits, float* y, uint32_t* mask, uint8_t* packed,
                           float* scale_f32, float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16,
                           void* stream) {
  if (int rc = check_quant_shape(N, G, bits)) return rc;
  if (!(p >= 0.f && p < 1.f)) return EXACT_E_ARG;
  if ((act_noise == nullptr) != (noise == nullptr)) return EXACT_E_ARG;  // both streams supplied, or neither
  if (G % 8 != 0 || G > 1024 || N * G > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (!packed) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t pad_index = exact_packed_nbytes(N, G, bits) - 1;
  if (N == 0 || G == 0) {
    hipLaunchKernelGGL(zero_byte_kernel, dim3(1), dim3(1), 0, s, packed + pad_index);
    return launch_status();
  }
  if (!x || !y || !mask) return EXACT_E_NULL;
  if (!aligned(x, 16) || !aligned(y, 16) || (noise && (!aligned(noise, 16) || !aligned(act_noise, 16))))
    return EXACT_E_ALIGN;
  if (norm_mean && (!aligned(norm_mean, 16) || !aligned(norm_mult, 16) || !aligned(norm_shift, 16)))
    return EXACT_E_ALIGN;
  const Geometry g = plan_rows(G, 4);
  PackArgs a{};
  a.x = x;
  a.norm_mean = norm_mean;
  a.norm_mult = norm_mult;
  a.norm_shift = norm_shift;
  a.noise = noise;
  a.mn_in = nullptr;
  a.scale_in = nullptr;
  a.seed_lo = static_cast<uint32_t>(seed);
  a.seed_hi = static_cast<uint32_t>(seed >> 32);
  a.off_lo = static_cast<uint32_t>(offset);
  a.off_hi = static_cast<uint32_t>(offset >> 32);
  a.N = N;
  a.G = static_cast<int>(G);
  a.opr = g.opr;
  a.lpr_log2 = g.lpr_log2;
  a.packed = packed;
  a.pad_index = pad_index;
  a.scale_f32 = scale_f32;
  a.min_f32 = min_f32;
  a.scale_bf16 = scale_bf16;
  a.min_bf16 = min_bf16;
  a.out_vec = aligned(packed, 8) ? 8 : aligned(packed, 4) ? 4 : 1;
  a.act_noise = act_noise;
  a.act_seed_lo = static_cast<uint32_t>(act_seed);
  a.act_seed_hi = static_cast<uint32_t>(act_seed >> 32);
  a.act_off_lo = static_cast<uint32_t>(act_offset);
  a.act_off_hi = static_cast<uint32_t>(act_offset >> 32);
  a.p = p;
  // quantization_cuda_kernel.cu:456: float pinv = 1. / (1. - p), evaluated in double
  a.pinv = static_cast<float>(1.0 / (1.0 - static_cast<double>(p)));
  // u = (h + 0.5) / 65536 > p  <=>  h > 65536 p - 0.5  <=>  h >= floor(65536 p - 0.5) + 1   (0 <= p < 1, exact in double)
  a.act_keep_from = static_cast<uint32_t>(static_cast<int>(std::floor(65536.0 * static_cast<double>(p) - 0.5)) + 1);
  a.y = y;
  a.mask_bytes = reinterpret_cast<uint8_t*>(mask);
  a.mask_tail_begin = N * G / 8;
  a.mask_tail_end = (N * G + 31) / 32 * 4;
  const int rows_per_wg = kBlock >> g.lpr_log2;
  const dim3 grid(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg), 1u);
  if (noise) launch_act_bits<true>(a, bits, g.opt, g.full, grid, s);
  else launch_act_bits<false>(a, bits, g.opt, g.full, grid, s);
  return launch_status();
}

int exact_relu_dropout_minmax_pack_f32(const float* x, float p, const float* act_noise, uint64_t act_seed,
                                       uint64_t act_offset, const float* noise, uint64_t seed, uint64_t offset,
                                       int64_t N, int64_t G, int bits, float* y, uint32_t* mask, uint8_t* packed,
                                       float* scale_f32, float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16,
                                       void* stream) {
  return act_pack_common(x, nullptr, nullptr, nullptr, p, act_noise, act_seed, act_offset, noise, seed, offset, N, G,
                         bits, y, mask, packed, scale_f32, min_f32, scale_bf16, min_bf16, stream);
}

int exact_bn_relu_dropout_minmax_pack_f32(const float* x, const float* mean, const float* mult, const float* shift,
                                          float p, const float* act_noise, uint64_t act_seed, uint64_t act_offset,
                                          const float* noise, uint64_t seed, uint64_t offset, int64_t N, int64_t G,
                                          int bits, float* y, uint32_t* mask, uint8_t* packed, float* scale_f32,
                                          float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16, void* stream) {
  if (N > 0 && G > 0 && (!mean || !mult || !shift)) return EXACT_E_NULL;
  return act_pack_common(x, mean, mult, shift, p, act_noise, act_seed, act_offset, noise, seed, offset, N, G, bits, y,
                         mask, packed, scale_f32, min_f32, scale_bf16, min_bf16, stream);
}

int exact_minmax_pack_f16(const uint16_t* x, const float* noise, uint64_t seed, uint64_t offset, int64_t N,
                          int64_t G, int bits, uint8_t* packed, uint16_t* scale_f16, uint16_t* min_f16,
                          void* stream) {
  if (int rc = check_quant_shape(N, G, bits)) return rc;
  if (G > 1024) return EXACT_E_SHAPE;
  if (!packed) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t pad_index = exact_packed_nbytes(N, G, bits) - 1;
  if (N == 0 || G == 0) {
    hipLaunchKernelGGL(zero_byte_kernel, dim3(1), dim3(1), 0, s, packed + pad_index);
    return launch_status();
  }
  if (!x) return EXACT_E_NULL;
  if (!aligned(x, 2)) return EXACT_E_ALIGN;
  const Geometry g = plan_rows(G, 4);
  PackArgs a{};
  a.x = reinterpret_cast<const float*>(x);  // the HALF form reads it as fp16
  a.noise = noise;
  a.seed_lo = static_cast<uint32_t>(seed);
  a.seed_hi = static_cast<uint32_t>(seed >> 32);
  a.off_lo = static_cast<uint32_t>(offset);
  a.off_hi = static_cast<uint32_t>(offset >> 32);
  a.N = N;
  a.G = static_cast<int>(G);
  a.opr = g.opr;
  a.lpr_log2 = g.lpr_log2;
  a.packed = packed;
  a.pad_index = pad_index;
  a.scale_bf16 = scale_f16;
  a.min_bf16 = min_f16;
  a.out_vec = (G % 8 == 0 && aligned(packed, 8)) ? 8 : (G % 4 == 0 && aligned(packed, 4)) ? 4 : 1;
  // whole octs: 16-byte loads of x (and of supplied fp32 noise)
  const bool whole = (G % 8 == 0) && aligned(x, 16) && (!noise || aligned(noise, 16));
  const int rows_per_wg = kBlock >> g.lpr_log2;
  const dim3 grid(static_cast<unsigned>((N + rows_per_wg - 1) / rows_per_wg), 1u);
  if (noise) launch_half_bits<true>(a, bits, g.opt, whole, g.full && whole, grid, s);
  else launch_half_bits<false>(a, bits, g.opt, whole, g.full && whole, grid, s);
  return launch_status();
}

}  // extern "C"
