// Random projection on the bf16 matrix cores of gfx950
// (v_mfma_f32_32x32x16_bf16, fp32 accumulate) with fp32 accuracy:
//   forward   out[N, k] = X[N, D]  . R[D, k]      (input2rp, ops.py:107-118)
//   backward  out[N, D] = Xr[N, k] . R[D, k]^T    (rp2input, ops.py:121-125)
//
// An fp32 number is the exact sum of three bf16 numbers: hi = bf16(x),
// mid = bf16(x - hi), lo = x - hi - mid (each difference is exact in fp32 and
// the last one has at most 8 significant bits).  So
//   * SIGNS: the reference's projection matrix is R = s * c with s = +-1 and
//     one scalar c = 1 / sqrt(k) (ops.py:112-114).  X . R = c * (X . s), and
//     X . s = hi . s + mid . s + lo . s: three bf16 products whose terms are
//     exact, summed in fp32, scaled once at the end.  3 / 16 of the matrix-core
//     time of the fp32 instruction, and one rounding per term less.
//   * SPLIT: any R (e.g. Gaussian) is split the same way and the six products
//     hi.hi, hi.mid, mid.hi, hi.lo, lo.hi, mid.mid are formed; the three left
//     out are below 2^-24 of the leading one, the rounding of an fp32 product.
// Either way the matrix cores are off the critical path and the kernels are
// left with streaming the [N, D] operand, so they are built like streaming
// kernels: many short workgroups, every lane's loads issued at once, no
// prologue.  That needs R in the layout the instruction wants, ready to load:
// exact_rp_prepare_bf16 turns R once into a TABLE of operand fragments (an
// ordinary caller-owned buffer, valid as long as R is), and the kernels read
// 16 bytes per lane from it (it stays in L2).
//
// Register layout of the instruction (wave64): lane l holds, of the A operand,
// row l % 32 and the eight k-slots 8 * (l / 32) .. + 7 (four 32-bit registers
// of two bf16 each); of the B operand column l % 32 and the same eight k-slots;
// accumulator register v of lane l is C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32],
// as for every 32 x 32 MFMA.  A k-step covers 16 consecutive features: lane
// (row, h) reads features 8 h .. 8 h + 7 of the step, 32 contiguous bytes.
//
// Table layout (16-byte units): [0] header {c, 0, 0, 0} with c = |R[0][0]|;
// then the forward fragments [step over D][tile over k][piece][lane], lane
// (col, h) of (step, tile) holding R[16 step + 8 h + i][32 tile + col], i = 0..7;
// then the backward fragments [step over k][tile over D][piece][lane], lane
// (col, h) holding R[32 tile + col][16 step + 8 h + i].  SIGNS: one piece (the
// signs as +-1 in bf16); SPLIT: three (hi, mid, lo).  Padding entries are 0.

#include "bf16_split.hpp"
#include "rp_common.hpp"

namespace exact {

constexpr int kStepFeatures = 16;  // K of one MFMA

// Eight consecutive floats of a row starting at column `col`, zeros from column
// `limit` on; VEC = the widest aligned access (limit % VEC == 0, col % VEC == 0).
// The loads are unconditional (address clamped to the row's first piece): a
// load behind a branch would make the compiler wait for every load in flight.
template <int VEC>
__device__ __forceinline__ void load8(const float* __restrict__ row, int col, int limit, float (&v)[8]) {
#pragma unroll
  for (int p = 0; p < 8; p += VEC) {
    const bool ok = col + p < limit;
    const float* src = row + (ok ? col + p : 0);
    if constexpr (VEC == 4) {
      const f32x4 q = *reinterpret_cast<const f32x4*>(src);
      v[p] = ok ? q.x : 0.f; v[p + 1] = ok ? q.y : 0.f; v[p + 2] = ok ? q.z : 0.f; v[p + 3] = ok ? q.w : 0.f;
    } else if constexpr (VEC == 2) {
      const floatx2 q = *reinterpret_cast<const floatx2*>(src);
      v[p] = ok ? q.x : 0.f; v[p + 1] = ok ? q.y : 0.f;
    } else {
      const float q = *src;
      v[p] = ok ? q : 0.f;
    }
  }
}

// ---- the table ---------------------------------------------------------------
struct TableShape {
  int steps_d, tiles_k, steps_k, tiles_d, pieces;
  __host__ __device__ int64_t fwd_units() const { return static_cast<int64_t>(steps_d) * tiles_k * pieces * kWave; }
  __host__ __device__ int64_t bwd_units() const { return static_cast<int64_t>(steps_k) * tiles_d * pieces * kWave; }
};
__host__ __device__ inline TableShape table_shape(int D, int k, int pieces) {
  return TableShape{(D + kStepFeatures - 1) / kStepFeatures, (k + kTile - 1) / kTile, (k + kStepFeatures - 1) / kStepFeatures,
                    (D + kTile - 1) / kTile, pieces};
}

// one thread per (direction, step, tile, lane): eight entries of R -> one fragment per piece
template <int BP>
__global__ __launch_bounds__(kBlock) void rp_prepare_kernel(const float* __restrict__ R, int D, int k,
                                                            u32x4* __restrict__ table) {
  const TableShape ts = table_shape(D, k, BP);
  const int64_t fwd_frags = static_cast<int64_t>(ts.steps_d) * ts.tiles_k * kWave;
  const int64_t bwd_frags = static_cast<int64_t>(ts.steps_k) * ts.tiles_d * kWave;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx == 0) {
    u32x4 head = {__float_as_uint(fabsf(R[0])), 0u, 0u, 0u};
    table[0] = head;
  }
  if (idx >= fwd_frags + bwd_frags) return;
  const bool fwd = idx < fwd_frags;
  const int64_t f = fwd ? idx : idx - fwd_frags;
  const int l = static_cast<int>(f & (kWave - 1));
  const int tiles = fwd ? ts.tiles_k : ts.tiles_d;
  const int tile = static_cast<int>((f / kWave) % tiles), step = static_cast<int>(f / (static_cast<int64_t>(kWave) * tiles));
  float r[8];
  bool inside[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    // forward: R[16 step + 8 h + i][32 tile + col];  backward: R[32 tile + col][16 step + 8 h + i]
    const int a = step * kStepFeatures + 8 * (l >> 5) + i, b = tile * kTile + (l & 31);
    const int d = fwd ? a : b, c = fwd ? b : a;
    inside[i] = d < D && c < k;
    r[i] = inside[i] ? R[static_cast<int64_t>(d) * k + c] : 0.f;
  }
  u32x4* dst = table + 1 + (fwd ? 0 : ts.fwd_units()) + (static_cast<int64_t>(step) * tiles + tile) * BP * kWave + l;
  if constexpr (BP == 1) {
    u32x4 w;
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = sign_bf16(r[2 * i], inside[2 * i]) | (sign_bf16(r[2 * i + 1], inside[2 * i + 1]) << 16);
    dst[0] = w;
  } else {
    const Split8 s = split3x8(r);
    dst[0] = s.hi;
    dst[kWave] = s.mid;
    dst[2 * kWave] = s.lo;
  }
}

// ---- forward -----------------------------------------------------------------
// One wavefront per 32 rows, one wavefront per workgroup: no workgroup barrier
// anywhere.  The wavefront walks the D features in k-steps of 16, the loads of
// KS steps issued together (two 16-byte loads per lane and step, the steps'
// table fragments beside them), and accumulates in step order.  (A workgroup of
// four wavefronts that split the features and met in LDS was measured against
// this form: equal at 256 -> 32, 15 % slower at 256 -> 64.)
// `frags` holds `tiles` column tiles per k-step; the wavefront multiplies by the NT tiles from `tile0` on.
template <int VEC, int NT, int BP, int KS>
__device__ __forceinline__ void rp_fwd_rows(const float* __restrict__ X, const u32x4* __restrict__ frags, int64_t N,
                                            int D, int64_t row0, floatx16 (&acc)[NT], int tiles = NT, int tile0 = 0) {
  const int lane = threadIdx.x & (kWave - 1);
  const int half = lane >> 5;
  const int64_t my_row = (row0 + (lane & 31) < N) ? row0 + (lane & 31) : N - 1;
  const float* xrow = X + my_row * D;
  const int total = (D + kStepFeatures - 1) / kStepFeatures;

#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

  for (int s0 = 0; s0 < total; s0 += KS) {
    float a[KS][8];
    if ((s0 + KS) * kStepFeatures <= D) {  // wave-uniform: the KS steps lie inside the row, nothing to mask
#pragma unroll
      for (int sb = 0; sb < KS; ++sb) load8<VEC>(xrow, (s0 + sb) * kStepFeatures + 8 * half, 0x7FFFFFFF, a[sb]);
    } else {
#pragma unroll
      for (int sb = 0; sb < KS; ++sb) load8<VEC>(xrow, (s0 + sb) * kStepFeatures + 8 * half, D, a[sb]);  // zeros past the row
    }
#pragma unroll
    for (int sb = 0; sb < KS; ++sb) {
      const int st = (s0 + sb < total) ? s0 + sb : s0;  // a step past the row meets zeros: any valid fragment will do
      const Split8 pieces = split3x8(a[sb]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const u32x4* src = frags + (static_cast<int64_t>(st) * tiles + tile0 + nt) * BP * kWave + lane;
        u32x4 b[BP];
#pragma unroll
        for (int p = 0; p < BP; ++p) b[p] = src[p * kWave];
        acc[nt] = step_product<BP>(pieces, b, acc[nt]);
      }
    }
  }
}

// k-steps in flight: four with one column tile (more wavefronts per SIMD do better than more loads per
// wavefront), eight with several (measured at 256 -> 32 and 256 -> 64)
template <int NT>
constexpr int fwd_steps_in_flight() { return NT == 1 ? 4 : 8; }

template <int VEC, int NT, int BP>
__global__ __launch_bounds__(kWave) void rp_fwd_bf16_kernel(const float* __restrict__ X,
                                                            const u32x4* __restrict__ table, int64_t N, int D,
                                                            int k, float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int half = lane >> 5, l32 = lane & 31;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kTile;
  floatx16 acc[NT];
  rp_fwd_rows<VEC, NT, BP, fwd_steps_in_flight<NT>()>(X, table + 1, N, D, row0, acc);
  const float c = BP == 1 ? __uint_as_float(table[0][0]) : 1.f;
  // accumulator register v of lane l is C[8 (v / 4) + 4 (l / 32) + v % 4][l % 32]: a store instruction writes two
  // rows of 32 consecutive columns
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int64_t n = row0 + 8 * (v / 4) + 4 * half + (v % 4);
      const int col = nt * kTile + l32;
      if (n < N && col < k) __builtin_nontemporal_store(BP == 1 ? acc[nt][v] * c : acc[nt][v], out + n * k + col);
    }
}

__device__ __forceinline__ void wave_sync_lds() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Projection and quantisation in one launch.  The wavefront turns its finished
// tile through LDS: out of the accumulator layout (a lane = one column) into the
// layout the row-wise pack kernel works in, where a lane owns an "oct" -- eight
// consecutive columns of one row, the elements of one Philox block (block
// (d / 8, n) serves columns 8 (d / 8) .. + 7 of row n) -- so the row statistics
// are eight local comparisons and a butterfly over the row's lanes, and no
// random number is computed twice.  The sums are those of rp_fwd_bf16_kernel
// (same loop) and the arithmetic is that of exact_minmax_pack_f32
// (quantization_cuda_kernel.cu:89, one rounding per operation), so the bytes
// equal those of the two launches.  The 8 / bits rows that share a packed byte
// meet through a second LDS array: every lane parks its row's bits of eight
// bytes, then one lane per (row group, oct) ORs the group's rows and stores the
// eight bytes.  Both arrays are private to the wavefront, whose LDS accesses
// complete in order: the hand-overs need no workgroup barrier.
constexpr int kStagePitch = 16;  // octs per row in the hand-over array: k <= 128
template <int NT>
constexpr int fwd_tile_pitch() { return NT * kTile + 4; }  // floats per tile row: 16-byte aligned rows, rows 4 apart on other banks

template <int VEC, int NT, int BP, bool NOISE_IN>
__global__ __launch_bounds__(kWave) void rp_fwd_pack_bf16_kernel(const RpPackArgs a, const u32x4* __restrict__ table) {
  HIP_DYNAMIC_SHARED(float, tile)  // [32][pitch] floats, then uint64 [32][kStagePitch]
  constexpr int PITCH = fwd_tile_pitch<NT>();
  // passes of the 64 lanes over the tile's (row, oct) pairs: 32 rows x (1, 2 or 4 | 8 | 16) lanes per row
  constexpr int PASSES = NT == 1 ? 2 : (NT == 2 ? 4 : 8);
  uint64_t* stage = reinterpret_cast<uint64_t*>(tile + kTile * PITCH);
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kTile;
  {
    floatx16 acc[NT];
    rp_fwd_rows<VEC, NT, BP, fwd_steps_in_flight<NT>()>(a.X, table + 1, a.N, a.D, row0, acc);
    const float c = BP == 1 ? __uint_as_float(table[0][0]) : 1.f;
    const int half = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v)
        tile[(8 * (v / 4) + 4 * half + (v % 4)) * PITCH + nt * kTile + l32] = BP == 1 ? acc[nt][v] * c : acc[nt][v];
  }
  wave_sync_lds();
  uint64_t parked[PASSES];  // this lane's words of the passes below
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) parked[pass] = 0;
  const int k = a.k, bits = a.bits;
  const int wpt = 8 / bits;
  const float B = static_cast<float>((1 << bits) - 1);
  const int octs = (k + 7) >> 3;
  int opr_log = 0;
  while ((1 << opr_log) < octs) ++opr_log;  // lanes per row: the next power of two
  const int opr = 1 << opr_log;

#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    if (pass * kWave >= kTile * opr) break;
    const int t = pass * kWave + lane;
    const int i = (t >> opr_log) & (kTile - 1), oct = t & (opr - 1);  // lanes past the tile (k <= 8 only) mirror a real row
    const bool live = t < kTile * opr && oct < octs;
    const int64_t n = row0 + i;
    const int j0 = live ? 8 * oct : 0;
    // ---- the eight sums ------------------------------------------------------
    float x[8];
    {
      const float* src = tile + i * PITCH + j0;
      const f32x4 lo4 = *reinterpret_cast<const f32x4*>(src), hi4 = *reinterpret_cast<const f32x4*>(src + 4);
      x[0] = lo4.x; x[1] = lo4.y; x[2] = lo4.z; x[3] = lo4.w; x[4] = hi4.x; x[5] = hi4.y; x[6] = hi4.z; x[7] = hi4.w;
    }
    // ---- row statistics --------------------------------------------------------
    float mn = __builtin_inff(), mx = -__builtin_inff();
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (live && j0 + e < k) {
        mn = fminf(mn, x[e]);
        mx = fmaxf(mx, x[e]);
      }
    }
    group_minmax(mn, mx, opr);
    const float recip = 1.0f / (mx - mn);  // ops.py:39: reciprocal, then * B -- two roundings
    const float sc = recip * B;
    if (live && oct == 0 && n < a.N) {
      if (a.scale_f32) a.scale_f32[n] = sc;
      if (a.min_f32) a.min_f32[n] = mn;
      if (a.scale_bf16) a.scale_bf16[n] = f32_to_bf16_rne(sc);
      if (a.min_bf16) a.min_bf16[n] = f32_to_bf16_rne(mn);
    }
    // ---- noise -----------------------------------------------------------------
    float u[8];
    if constexpr (NOISE_IN) {
#pragma unroll
      for (int e = 0; e < 8; ++e) u[e] = (live && j0 + e < k && n < a.N) ? a.noise[n * k + j0 + e] : 0.f;
    } else {
      const Philox4 r = philox4x32_10(static_cast<uint32_t>(oct), static_cast<uint32_t>(n), a.off_lo, a.off_hi, a.seed_lo,
                                      a.seed_hi);
      philox_uniform8(r, u);
    }
    // ---- quantise; this row's bits of the eight bytes ------------------------------
    const int shift = (i & (wpt - 1)) * bits;
    uint32_t q[8];  // the code in the low byte
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float tq = x[e] - mn;
      tq = tq * sc;
      tq = tq + u[e];
      q[e] = code_in_low_byte(tq);  // scale and min are this row's own: tq < 2^bits + 2
    }
    // uint8_t arithmetic of the reference: bits shifted past bit 7 of a byte vanish; columns past k and rows
    // past N contribute nothing
    const uint32_t keep = (0xFFu >> shift) * 0x01010101u;
    const int cols = (live && n < a.N) ? (k - j0 < 8 ? (k - j0 < 0 ? 0 : k - j0) : 8) : 0;
    const uint64_t valid = cols >= 8 ? ~uint64_t{0} : ((uint64_t{1} << (8 * cols)) - 1);
    uint32_t word[2];
    word[0] = ((low_bytes4(q[0], q[1], q[2], q[3]) & keep) << shift) & static_cast<uint32_t>(valid);
    word[1] = ((low_bytes4(q[4], q[5], q[6], q[7]) & keep) << shift) & static_cast<uint32_t>(valid >> 32);
    parked[pass] = static_cast<uint64_t>(word[0]) | (static_cast<uint64_t>(word[1]) << 32);
  }
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
    const int t = pass * kWave + lane;
    if (t < kTile * opr) stage[((t >> opr_log) & (kTile - 1)) * kStagePitch + (t & (opr - 1))] = parked[pass];
  }
  wave_sync_lds();
  // ---- one lane per (row group, oct): OR the group's rows, store eight bytes -----------
  const int groups = kTile / wpt;
  const bool wide = (k & 7) == 0 && (reinterpret_cast<uintptr_t>(a.packed) & 7u) == 0;
  for (int t = lane; t < groups * octs; t += kWave) {
    const int g = t / octs, oct = t - g * octs;
    if (row0 + static_cast<int64_t>(g) * wpt >= a.N) continue;
    uint64_t w = 0;
    for (int r = 0; r < wpt; ++r) w |= stage[(g * wpt + r) * kStagePitch + oct];
    uint8_t* dst = a.packed + (row0 / wpt + g) * k + 8 * oct;
    if (wide) {
      *reinterpret_cast<uint64_t*>(dst) = w;
    } else {
      const int cnt = (k - 8 * oct < 8) ? k - 8 * oct : 8;
      for (int e = 0; e < cnt; ++e) dst[e] = static_cast<uint8_t>(w >> (8 * e));
    }
  }
  if (blockIdx.x == 0 && lane == 0) a.packed[a.pad_index] = 0;
}

// ---- tall operand times a small dense matrix ----------------------------------------
// out[N, K] = X[N, D] . M[D, K] (+ bias[K]) (+ addend[N, K]) for the linear maps of a
// layer (F.linear and the input gradient of linear_backward, backward_func.cc:83-87):
// the forward loop above with M split in three (six bf16 products per fp32
// product, fp32 accuracy), up to four column tiles per wavefront -- wider
// matrices take one launch per slab of 128 columns -- and an epilogue that adds
// a bias row and / or a matrix (which may be `out` itself: every element is read
// and written by the same lane).  The fragments of M come from
// exact_tall_gemm_prepare_bf16, which also takes M transposed (a weight as
// F.linear holds it).  No atomics: the result does not depend on the launch.
constexpr int kGemmXcds = 8;       // accelerator complex dies of an MI355X, each with its own L2
constexpr int kGemmSlabTiles = 4;  // column tiles (of 32) one launch covers
constexpr int kGemmRowTiles = 1;   // row tiles (of 32) per wavefront in the form without LDS
constexpr int kGemmSteps = 4;      // k-steps whose loads are issued together there
// Slabs that fill their launch share the fragments through LDS (tall_gemm_lds_bf16_kernel): results of up to two
// column tiles as one slab with four k-steps per chunk, wider ones in slabs of four tiles with two steps per chunk
// (measured: 64 against 77 us at 256 -> 40, 200 against 230 at 256 -> 256; the other splits tried were slower).

__global__ __launch_bounds__(kBlock) void gemm_prepare_kernel(const float* __restrict__ M, int64_t ld, int transposed,
                                                              int D, int K, u32x4* __restrict__ table) {
  const TableShape ts = table_shape(D, K, 3);
  const int64_t frags = static_cast<int64_t>(ts.steps_d) * ts.tiles_k * kWave;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (idx == 0) {
    u32x4 head = {0u, 0u, 0u, 0u};
    table[0] = head;
  }
  if (idx >= frags) return;
  const int l = static_cast<int>(idx & (kWave - 1));
  const int tile = static_cast<int>((idx / kWave) % ts.tiles_k), step = static_cast<int>(idx / (static_cast<int64_t>(kWave) * ts.tiles_k));
  float r[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int d = step * kStepFeatures + 8 * (l >> 5) + i, c = tile * kTile + (l & 31);
    const bool inside = d < D && c < K;
    r[i] = inside ? (transposed ? M[static_cast<int64_t>(c) * ld + d] : M[static_cast<int64_t>(d) * ld + c]) : 0.f;
  }
  u32x4* dst = table + 1 + (static_cast<int64_t>(step) * ts.tiles_k + tile) * 3 * kWave + l;
  const Split8 s = split3x8(r);
  dst[0] = s.hi;
  dst[kWave] = s.mid;
  dst[2 * kWave] = s.lo;
}

// A wavefront owns RT row tiles (32 RT rows) and NT column tiles, with the loads of KS k-steps of X in flight.
// Measured on [169343 .. 2449029, 100 .. 604] x [.., 40 .. 352]: one row tile, four column tiles and four steps
// is the fastest split (two or three row tiles per wavefront -- every fragment of M then serves several
// products -- cost more in occupancy than they save in fragment loads: 330 against 236 us at 256 x 256).  The
// kernel then equals the framework's fp32 GEMM at 256 output columns and beats it by 20 - 25 % at 40 - 47.
template <int VEC, int RT, int NT, int KS>
__global__ __launch_bounds__(kWave) void tall_gemm_bf16_kernel(const float* __restrict__ X,
                                                               const u32x4* __restrict__ table, int64_t N, int D, int K,
                                                               int tiles, int tile0, const float* __restrict__ bias,
                                                               const float* addend, int64_t ldc, float* out,
                                                               int64_t ldo) {
  const int lane = threadIdx.x & (kWave - 1);
  const int half = lane >> 5, l32 = lane & 31;
  const int64_t row0 = static_cast<int64_t>(blockIdx.x) * (kTile * RT);
  const u32x4* frags = table + 1;
  const float* xrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int64_t r = row0 + rt * kTile + l32;
    xrow[rt] = X + (r < N ? r : N - 1) * D;
  }
  const int total = (D + kStepFeatures - 1) / kStepFeatures;
  floatx16 acc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rt][nt][v] = 0.f;

  for (int s0 = 0; s0 < total; s0 += KS) {
    float a[KS][RT][8];
    if ((s0 + KS) * kStepFeatures <= D) {  // wave-uniform: the KS steps lie inside the row, nothing to mask
#pragma unroll
      for (int sb = 0; sb < KS; ++sb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) load8<VEC>(xrow[rt], (s0 + sb) * kStepFeatures + 8 * half, 0x7FFFFFFF, a[sb][rt]);
    } else {
#pragma unroll
      for (int sb = 0; sb < KS; ++sb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) load8<VEC>(xrow[rt], (s0 + sb) * kStepFeatures + 8 * half, D, a[sb][rt]);
    }
#pragma unroll
    for (int sb = 0; sb < KS; ++sb) {
      const int st = (s0 + sb < total) ? s0 + sb : s0;  // a step past the row meets zeros: any valid fragment will do
      Split8 pieces[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) pieces[rt] = split3x8(a[sb][rt]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const u32x4* src = frags + (static_cast<int64_t>(st) * tiles + tile0 + nt) * 3 * kWave + lane;
        u32x4 b[3];
#pragma unroll
        for (int p = 0; p < 3; ++p) b[p] = src[p * kWave];
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) acc[rt][nt] = step_product<3>(pieces[rt], b, acc[rt][nt]);
      }
    }
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int col = (tile0 + nt) * kTile + l32;
    const float b = (bias != nullptr && col < K) ? bias[col] : 0.f;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t n = row0 + rt * kTile + 8 * (v / 4) + 4 * half + (v % 4);
        if (n < N && col < K) {
          float val = acc[rt][nt][v];
          if (bias != nullptr) val = val + b;
          if (addend != nullptr) val = val + addend[n * ldc + col];
          __builtin_nontemporal_store(val, out + n * ldo + col);
        }
      }
  }
}

// The same product with the fragments of M shared by a workgroup: four wavefronts (128 rows) copy the fragments
// of KS k-steps x NT column tiles into LDS once and all read them from there, so the L2 sees a quarter of the
// fragment traffic and the wavefronts' fragment loads become LDS reads.  For results wider than a few tiles, where
// every wavefront of the form above streams the whole slab of M through the vector memory pipeline.
template <int VEC, int RT, int NT, int KS>
__global__ __launch_bounds__(kBlock) void tall_gemm_lds_bf16_kernel(const float* __restrict__ X,
                                                                    const u32x4* __restrict__ table, int64_t N, int D,
                                                                    int K, int tiles, int slabs,
                                                                    const float* __restrict__ bias, const float* addend,
                                                                    int64_t ldc, float* out, int64_t ldo) {
  HIP_DYNAMIC_SHARED(u32x4, shared_frags)  // [KS][NT][3][64]
  // One launch covers `slabs` column slabs of NT tiles each.  Workgroups are handed to the 8 XCDs (each with its own
  // L2) round-robin by index, so the workgroups of one row block -- one per slab -- take indices 8 apart: they run on
  // the same XCD at about the same time and all but the first find the rows of X in that L2.  The grid is a whole
  // number of such groups; row blocks past the last row leave here, before any barrier.
  const int64_t in_group = blockIdx.x % (kGemmXcds * slabs);
  const int64_t row_block = blockIdx.x / (kGemmXcds * slabs) * kGemmXcds + in_group % kGemmXcds;
  const int tile0 = static_cast<int>(in_group / kGemmXcds) * NT;
  if (row_block * (kBlock / kWave) * (kTile * RT) >= N) return;
  constexpr int kUnits = KS * NT * 3 * kWave;             // 16-byte units per chunk
  constexpr int kPerThread = kUnits / kBlock;             // KS * NT * 3 / 4
  static_assert(kUnits % kBlock == 0, "whole units per thread");
  constexpr int kStepUnits = NT * 3 * kWave;              // contiguous in the table for one k-step
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  // a wavefront owns RT row tiles, so that a fragment read from LDS could serve RT products.  Measured at
  // [169343, 256] x [256, 256]: 201 us with one row tile, 287 with two, 280 with three -- the kernel lives on
  // the number of wavefronts in flight (registers per wavefront), not on fragment reads; RT = 1 is what is launched
  const int64_t row0 = (row_block * (kBlock / kWave) + wave) * (kTile * RT);
  const u32x4* frags = table + 1;
  const float* xrow[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int64_t r = row0 + rt * kTile + l32;
    xrow[rt] = X + (r < N ? r : N - 1) * D;
  }
  const int total = (D + kStepFeatures - 1) / kStepFeatures;
  floatx16 acc[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[rt][nt][v] = 0.f;

  for (int s0 = 0; s0 < total; s0 += KS) {
    float a[KS][RT][8];
    if ((s0 + KS) * kStepFeatures <= D) {  // wave-uniform: the KS steps lie inside the row, nothing to mask
#pragma unroll
      for (int sb = 0; sb < KS; ++sb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) load8<VEC>(xrow[rt], (s0 + sb) * kStepFeatures + 8 * half, 0x7FFFFFFF, a[sb][rt]);
    } else {
#pragma unroll
      for (int sb = 0; sb < KS; ++sb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) load8<VEC>(xrow[rt], (s0 + sb) * kStepFeatures + 8 * half, D, a[sb][rt]);
    }
    // this thread's share of the chunk's fragments: global -> registers -> LDS
    u32x4 mine[kPerThread];
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) {
      const int c = u * kBlock + static_cast<int>(threadIdx.x);  // unit of the chunk
      const int sb = c / kStepUnits, within = c - sb * kStepUnits;
      const int st = (s0 + sb < total) ? s0 + sb : s0;            // a step past the row meets zeros of X
      mine[u] = frags[(static_cast<int64_t>(st) * tiles + tile0) * 3 * kWave + within];
    }
    __syncthreads();  // the previous chunk has been read by every wavefront
#pragma unroll
    for (int u = 0; u < kPerThread; ++u) shared_frags[u * kBlock + threadIdx.x] = mine[u];
    __syncthreads();
#pragma unroll
    for (int sb = 0; sb < KS; ++sb) {
      u32x4 b[NT][3];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int p = 0; p < 3; ++p) b[nt][p] = shared_frags[((sb * NT + nt) * 3 + p) * kWave + lane];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const Split8 pieces = split3x8(a[sb][rt]);
        // the six products of step_product<3>, in its order for every tile, issued tile after tile: consecutive
        // matrix-core instructions write different accumulators and none waits for its predecessor
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = mfma_bf16(pieces.mid, b[nt][1], acc[rt][nt]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = mfma_bf16(pieces.lo, b[nt][0], acc[rt][nt]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = mfma_bf16(pieces.hi, b[nt][2], acc[rt][nt]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = mfma_bf16(pieces.mid, b[nt][0], acc[rt][nt]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = mfma_bf16(pieces.hi, b[nt][1], acc[rt][nt]);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = mfma_bf16(pieces.hi, b[nt][0], acc[rt][nt]);
      }
    }
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int col = (tile0 + nt) * kTile + l32;
    const float b = (bias != nullptr && col < K) ? bias[col] : 0.f;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t n = row0 + rt * kTile + 8 * (v / 4) + 4 * half + (v % 4);
        if (n < N && col < K) {
          float val = acc[rt][nt][v];
          if (bias != nullptr) val = val + b;
          if (addend != nullptr) val = val + addend[n * ldc + col];
          __builtin_nontemporal_store(val, out + n * ldo + col);
        }
      }
  }
}

// ---- backward ----------------------------------------------------------------
// out[N, D] = Xr[N, k] . R^T: the reduction runs over the k kept columns (at most
// 128: 8 k-steps); a wavefront owns 32 rows and a slab of NT * 32 output columns
// (grid.y tiles D), the four wavefronts of a workgroup four consecutive row
// tiles.  They share the slab's fragments, copied from the table into LDS; the
// [N, D] result leaves through a per-wavefront LDS tile of 8 rows as 16-byte
// streaming stores over whole rows of the slab (D % 4 == 0, `out` 16-byte
// aligned), else as 4-byte stores from the accumulator layout.  The tile is
// private to its wavefront, whose LDS accesses complete in order, so the
// hand-over inside it needs no workgroup barrier.
template <int NT>
constexpr int bwd_tile_pitch() { return NT * kTile + 8; }  // 4 * pitch = 32 (mod 64): the two half-waves hit different banks

template <int VEC, int NT, int BP, int KS, bool STAGED>  // KS: k-steps whose loads are issued (2, 4 or 8 >= the steps of k)
__global__ __launch_bounds__(kBlock) void rp_bwd_bf16_kernel(const float* __restrict__ Xr,
                                                             const u32x4* __restrict__ table, int64_t N, int D,
                                                             int k, float* __restrict__ out) {
  HIP_DYNAMIC_SHARED(u32x4, frag)  // the slab's fragments [step][NT][piece][lane], then (STAGED) the four output tiles
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int dbase = blockIdx.y * (NT * kTile);
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kTile;
  const int64_t my_row = (row0 + l32 < N) ? row0 + l32 : N - 1;
  const float* xrow = Xr + my_row * k;
  const TableShape ts = table_shape(D, k, BP);
  const int steps = ts.steps_k;  // <= KS
  const u32x4* bwd = table + 1 + ts.fwd_units();

  // my loads first, then the fragments of this slab: tiles blockIdx.y * NT .. + NT - 1 (past the last tile: zeros)
  float a[KS][8];
#pragma unroll
  for (int sb = 0; sb < KS; ++sb) load8<VEC>(xrow, sb * kStepFeatures + 8 * half, k, a[sb]);
  for (int idx = threadIdx.x; idx < steps * NT * BP * kWave; idx += kBlock) {
    const int l = idx & (kWave - 1), p = (idx / kWave) % BP, nt = (idx / (kWave * BP)) % NT, st = idx / (kWave * BP * NT);
    const int tile = blockIdx.y * NT + nt;
    u32x4 w = {0u, 0u, 0u, 0u};
    if (tile < ts.tiles_d) w = bwd[((static_cast<int64_t>(st) * ts.tiles_d + tile) * BP + p) * kWave + l];
    frag[idx] = w;
  }
  floatx16 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;
  __syncthreads();

#pragma unroll
  for (int sb = 0; sb < KS; ++sb) {
    if (sb < steps) {
      const Split8 pieces = split3x8(a[sb]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const u32x4* src = frag + (sb * NT + nt) * BP * kWave + lane;
        u32x4 b[BP];
#pragma unroll
        for (int p = 0; p < BP; ++p) b[p] = src[p * kWave];
        acc[nt] = step_product<BP>(pieces, b, acc[nt]);
      }
    }
  }
  if constexpr (BP == 1) {
    const float c = __uint_as_float(table[0][0]);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[nt][v] = acc[nt][v] * c;
  }

  if constexpr (STAGED) {
    constexpr int PC = bwd_tile_pitch<NT>();
    constexpr int kQuadsPerRow = NT * kTile / 4;
    float* Ct = reinterpret_cast<float*>(frag + steps * NT * BP * kWave) + wave * (8 * PC);  // [8][PC], this wavefront's own
#pragma unroll
    for (int g = 0; g < 4; ++g) {  // rows 8 g .. 8 g + 7 of the wavefront's 32
      wave_sync_lds();             // the tile's previous contents have been read
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) Ct[(4 * half + r) * PC + nt * kTile + l32] = acc[nt][4 * g + r];
      wave_sync_lds();
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int f = j * kWave + lane;
        const int tr = f / kQuadsPerRow, tq = f - tr * kQuadsPerRow;
        const int64_t rr = row0 + 8 * g + tr;
        const int cj = dbase + 4 * tq;
        const f32x4 q = *reinterpret_cast<const f32x4*>(Ct + tr * PC + 4 * tq);
        if (rr < N && cj < D) __builtin_nontemporal_store(q, reinterpret_cast<f32x4*>(out + rr * D + cj));
      }
    }
  } else {
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
}

// ---- launches ----------------------------------------------------------------
template <int NT>
constexpr size_t fwd_pack_lds_bytes() { return sizeof(float) * kTile * fwd_tile_pitch<NT>() + sizeof(uint64_t) * kTile * kStagePitch; }

template <int VEC, int BP>
static int rp_fwd_bf16_launch(const float* X, const u32x4* table, int64_t N, int D, int k, float* out, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>((N + kTile - 1) / kTile)), block(kWave);
  switch ((k + kTile - 1) / kTile) {
    case 1: hipLaunchKernelGGL((rp_fwd_bf16_kernel<VEC, 1, BP>), grid, block, 0, s, X, table, N, D, k, out); break;
    case 2: hipLaunchKernelGGL((rp_fwd_bf16_kernel<VEC, 2, BP>), grid, block, 0, s, X, table, N, D, k, out); break;
    case 3: hipLaunchKernelGGL((rp_fwd_bf16_kernel<VEC, 3, BP>), grid, block, 0, s, X, table, N, D, k, out); break;
    case 4: hipLaunchKernelGGL((rp_fwd_bf16_kernel<VEC, 4, BP>), grid, block, 0, s, X, table, N, D, k, out); break;
    default: return EXACT_E_SHAPE;
  }
  return launch_status();
}

template <int VEC, int BP, bool NOISE_IN>
static int rp_fwd_pack_bf16_launch(const RpPackArgs& a, const u32x4* table, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>((a.N + kTile - 1) / kTile)), block(kWave);
  switch ((a.k + kTile - 1) / kTile) {
    case 1: hipLaunchKernelGGL((rp_fwd_pack_bf16_kernel<VEC, 1, BP, NOISE_IN>), grid, block, fwd_pack_lds_bytes<1>(), s, a, table); break;
    case 2: hipLaunchKernelGGL((rp_fwd_pack_bf16_kernel<VEC, 2, BP, NOISE_IN>), grid, block, fwd_pack_lds_bytes<2>(), s, a, table); break;
    case 3: hipLaunchKernelGGL((rp_fwd_pack_bf16_kernel<VEC, 3, BP, NOISE_IN>), grid, block, fwd_pack_lds_bytes<3>(), s, a, table); break;
    case 4: hipLaunchKernelGGL((rp_fwd_pack_bf16_kernel<VEC, 4, BP, NOISE_IN>), grid, block, fwd_pack_lds_bytes<4>(), s, a, table); break;
    default: return EXACT_E_SHAPE;
  }
  return launch_status();
}

template <int VEC, int BP, int KS>
static int rp_bwd_bf16_launch(const float* Xr, const u32x4* table, int64_t N, int D, int k, float* out, hipStream_t s) {
  const int steps = (k + kStepFeatures - 1) / kStepFeatures;
  const bool staged = D % 4 == 0 && al16(out);
  // output slab per workgroup: 128 columns; 64 when the fragments of a 128-column slab (and the tiles) pass 64 KB
  const size_t frag4 = static_cast<size_t>(steps) * 4 * BP * kWave * 16;
  const size_t tiles4 = staged ? sizeof(float) * (kBlock / kWave) * 8 * bwd_tile_pitch<4>() : 0;
  const int nt = (frag4 + tiles4 <= 64 * 1024) ? 4 : 2;
  const dim3 grid(static_cast<unsigned>((N + 127) / 128), static_cast<unsigned>((D + nt * kTile - 1) / (nt * kTile)));
  const dim3 block(kBlock);
  if (nt == 4) {
    const size_t lds = frag4 + tiles4;
    if (staged) hipLaunchKernelGGL((rp_bwd_bf16_kernel<VEC, 4, BP, KS, true>), grid, block, lds, s, Xr, table, N, D, k, out);
    else hipLaunchKernelGGL((rp_bwd_bf16_kernel<VEC, 4, BP, KS, false>), grid, block, lds, s, Xr, table, N, D, k, out);
  } else {
    const size_t lds = frag4 / 2 + (staged ? sizeof(float) * (kBlock / kWave) * 8 * bwd_tile_pitch<2>() : 0);
    if (staged) hipLaunchKernelGGL((rp_bwd_bf16_kernel<VEC, 2, BP, KS, true>), grid, block, lds, s, Xr, table, N, D, k, out);
    else hipLaunchKernelGGL((rp_bwd_bf16_kernel<VEC, 2, BP, KS, false>), grid, block, lds, s, Xr, table, N, D, k, out);
  }
  return launch_status();
}

template <int VEC, int BP>
static int rp_bwd_bf16_steps(const float* Xr, const u32x4* table, int64_t N, int D, int k, float* out, hipStream_t s) {
  const int steps = (k + kStepFeatures - 1) / kStepFeatures;
  if (steps <= 2) return rp_bwd_bf16_launch<VEC, BP, 2>(Xr, table, N, D, k, out, s);
  if (steps <= 4) return rp_bwd_bf16_launch<VEC, BP, 4>(Xr, table, N, D, k, out, s);
  return rp_bwd_bf16_launch<VEC, BP, 8>(Xr, table, N, D, k, out, s);
}

static bool rp_shape_ok(int64_t N, int64_t D, int64_t k) {
  return N >= 0 && D > 0 && k > 0 && D <= (1 << 20) && k <= 128;
}
static bool rp_mode_ok(int mode) { return mode == EXACT_RP_BF16_SPLIT || mode == EXACT_RP_BF16_SIGNS; }
static int rp_pieces(int mode) { return mode == EXACT_RP_BF16_SIGNS ? 1 : 3; }

}  // namespace exact

using namespace exact;

extern "C" {

int64_t exact_rp_table_nbytes(int64_t D, int64_t k, int mode) {
  if (!rp_shape_ok(0, D, k) || !rp_mode_ok(mode)) return 0;
  const TableShape ts = table_shape(static_cast<int>(D), static_cast<int>(k), rp_pieces(mode));
  return 16 * (1 + ts.fwd_units() + ts.bwd_units());
}

int exact_rp_prepare_bf16(const float* R, int64_t D, int64_t k, int mode, void* table, void* stream) {
  if (!rp_shape_ok(0, D, k)) return EXACT_E_SHAPE;
  if (!rp_mode_ok(mode)) return EXACT_E_ARG;
  if (!R || !table) return EXACT_E_NULL;
  if (!al16(table)) return EXACT_E_ALIGN;
  const TableShape ts = table_shape(static_cast<int>(D), static_cast<int>(k), rp_pieces(mode));
  const int64_t frags = (ts.fwd_units() + ts.bwd_units()) / ts.pieces;
  const dim3 grid(static_cast<unsigned>((frags + kBlock - 1) / kBlock)), block(kBlock);
  hipStream_t s = static_cast<hipStream_t>(stream);
  u32x4* t = static_cast<u32x4*>(table);
  if (mode == EXACT_RP_BF16_SIGNS) hipLaunchKernelGGL((rp_prepare_kernel<1>), grid, block, 0, s, R, static_cast<int>(D), static_cast<int>(k), t);
  else hipLaunchKernelGGL((rp_prepare_kernel<3>), grid, block, 0, s, R, static_cast<int>(D), static_cast<int>(k), t);
  return launch_status();
}

int exact_rp_fwd_bf16_f32(const float* X, const void* table, int64_t N, int64_t D, int64_t k, int mode, float* out,
                          void* stream) {
  if (!rp_shape_ok(N, D, k)) return EXACT_E_SHAPE;
  if (!rp_mode_ok(mode)) return EXACT_E_ARG;
  if (N == 0) return EXACT_OK;
  if (!X || !table || !out) return EXACT_E_NULL;
  if (!al16(table)) return EXACT_E_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const u32x4* t = static_cast<const u32x4*>(table);
  const int d = static_cast<int>(D), kk = static_cast<int>(k);
#define EXACT_RP_GO(V) \
  (mode == EXACT_RP_BF16_SIGNS ? rp_fwd_bf16_launch<V, 1>(X, t, N, d, kk, out, s) : rp_fwd_bf16_launch<V, 3>(X, t, N, d, kk, out, s))
  if (D % 4 == 0 && al16(X)) return EXACT_RP_GO(4);
  if (D % 2 == 0 && al8(X)) return EXACT_RP_GO(2);
  return EXACT_RP_GO(1);
#undef EXACT_RP_GO
}

int exact_rp_minmax_pack_bf16_f32(const float* X, const void* table, int mode, const float* noise, uint64_t seed,
                                  uint64_t offset, int64_t N, int64_t D, int64_t k, int bits, uint8_t* packed,
                                  float* scale_f32, float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16,
                                  void* stream) {
  if (bits != 1 && bits != 2 && bits != 4 && bits != 8) return EXACT_E_BITS;
  if (!rp_shape_ok(N, D, k) || N > (int64_t{1} << 31) - 64) return EXACT_E_SHAPE;
  if (!rp_mode_ok(mode)) return EXACT_E_ARG;
  if (!packed) return EXACT_E_NULL;
  RpPackArgs a{};
  a.pad_index = exact_packed_nbytes(N, k, bits) - 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (N == 0) {
    hipLaunchKernelGGL(rp_zero_byte_kernel, dim3(1), dim3(1), 0, s, packed + a.pad_index);
    return launch_status();
  }
  if (!X || !table) return EXACT_E_NULL;
  if (!al16(table)) return EXACT_E_ALIGN;
  const u32x4* t = static_cast<const u32x4*>(table);
  a.X = X;
  a.R = nullptr;
  a.noise = noise;
  a.seed_lo = static_cast<uint32_t>(seed);
  a.seed_hi = static_cast<uint32_t>(seed >> 32);
  a.off_lo = static_cast<uint32_t>(offset);
  a.off_hi = static_cast<uint32_t>(offset >> 32);
  a.N = N;
  a.D = static_cast<int>(D);
  a.k = static_cast<int>(k);
  a.bits = bits;
  a.packed = packed;
  a.scale_f32 = scale_f32;
  a.min_f32 = min_f32;
  a.scale_bf16 = scale_bf16;
  a.min_bf16 = min_bf16;
#define EXACT_RP_GO(V, NOISE) \
  (mode == EXACT_RP_BF16_SIGNS ? rp_fwd_pack_bf16_launch<V, 1, NOISE>(a, t, s) : rp_fwd_pack_bf16_launch<V, 3, NOISE>(a, t, s))
  if (D % 4 == 0 && al16(X)) return noise ? EXACT_RP_GO(4, true) : EXACT_RP_GO(4, false);
  if (D % 2 == 0 && al8(X)) return noise ? EXACT_RP_GO(2, true) : EXACT_RP_GO(2, false);
  return noise ? EXACT_RP_GO(1, true) : EXACT_RP_GO(1, false);
#undef EXACT_RP_GO
}

int exact_rp_bwd_bf16_f32(const float* Xr, const void* table, int64_t N, int64_t D, int64_t k, int mode, float* out,
                          void* stream) {
  if (!rp_shape_ok(N, D, k)) return EXACT_E_SHAPE;
  if (!rp_mode_ok(mode)) return EXACT_E_ARG;
  if (N == 0) return EXACT_OK;
  if (!Xr || !table || !out) return EXACT_E_NULL;
  if (!al16(table)) return EXACT_E_ALIGN;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const u32x4* t = static_cast<const u32x4*>(table);
  const int d = static_cast<int>(D), kk = static_cast<int>(k);
#define EXACT_RP_GO(V) \
  (mode == EXACT_RP_BF16_SIGNS ? rp_bwd_bf16_steps<V, 1>(Xr, t, N, d, kk, out, s) : rp_bwd_bf16_steps<V, 3>(Xr, t, N, d, kk, out, s))
  if (k % 4 == 0 && al16(Xr)) return EXACT_RP_GO(4);
  if (k % 2 == 0 && al8(Xr)) return EXACT_RP_GO(2);
  return EXACT_RP_GO(1);
#undef EXACT_RP_GO
}

int64_t exact_tall_gemm_table_nbytes(int64_t D, int64_t K) {
  if (D <= 0 || K <= 0 || D > 4096 || K > 4096) return 0;
  const TableShape ts = table_shape(static_cast<int>(D), static_cast<int>(K), 3);
  return 16 * (1 + ts.fwd_units());
}

int exact_tall_gemm_prepare_bf16(const float* M, int64_t ld, int transposed, int64_t D, int64_t K, void* table,
                                 void* stream) {
  if (D <= 0 || K <= 0 || D > 4096 || K > 4096) return EXACT_E_SHAPE;
  if (transposed != 0 && transposed != 1) return EXACT_E_ARG;
  if (ld < (transposed ? D : K)) return EXACT_E_SHAPE;
  if (!M || !table) return EXACT_E_NULL;
  if (!al16(table)) return EXACT_E_ALIGN;
  const TableShape ts = table_shape(static_cast<int>(D), static_cast<int>(K), 3);
  const int64_t frags = ts.fwd_units() / 3;
  const dim3 grid(static_cast<unsigned>((frags + kBlock - 1) / kBlock)), block(kBlock);
  hipLaunchKernelGGL(gemm_prepare_kernel, grid, block, 0, static_cast<hipStream_t>(stream), M, ld, transposed,
                     static_cast<int>(D), static_cast<int>(K), static_cast<u32x4*>(table));
  return launch_status();
}

int exact_tall_gemm_bf16_f32(const float* X, const void* table, int64_t N, int64_t D, int64_t K, const float* bias,
                             const float* addend, int64_t ldc, float* out, int64_t ldo, void* stream) {
  if (N < 0 || D <= 0 || K <= 0 || D > 4096 || K > 4096 || D % 2 != 0) return EXACT_E_SHAPE;
  if (ldo < K || (addend && ldc < K)) return EXACT_E_SHAPE;
  if (N == 0) return EXACT_OK;
  if (!X || !table || !out) return EXACT_E_NULL;
  if (!al16(table) || !al8(X)) return EXACT_E_ALIGN;
  const bool quads = D % 4 == 0 && al16(X);  // 16-byte loads of X, else 8-byte ones
  hipStream_t s = static_cast<hipStream_t>(stream);
  const u32x4* t = static_cast<const u32x4*>(table);
  const int d = static_cast<int>(D), kk = static_cast<int>(K);
  const int tiles = (kk + kTile - 1) / kTile;
  const int64_t rows_per_wave = static_cast<int64_t>(kTile) * kGemmRowTiles;
  const dim3 grid(static_cast<unsigned>((N + rows_per_wave - 1) / rows_per_wave)), block(kWave);
#ifndef EXACT_GEMM_LDS_ROW_TILES
#define EXACT_GEMM_LDS_ROW_TILES 1
#endif
  constexpr int kLdsRowTiles = EXACT_GEMM_LDS_ROW_TILES;  // row tiles per wavefront in the LDS form
  const int64_t lrows = static_cast<int64_t>(4) * kTile * kLdsRowTiles;  // four wavefronts
  const int64_t lgroups = ((N + lrows - 1) / lrows + kGemmXcds - 1) / kGemmXcds;  // groups of 8 row blocks
  if (lgroups * kGemmXcds * (tiles / kGemmSlabTiles + 1) > 0x7FFFFFFF) return EXACT_E_SHAPE;
  const dim3 lblock(kBlock);
#define EXACT_GEMM_LDS(NTV, KSV)                                                                                    \
  do {                                                                                                              \
    if (quads)                                                                                                      \
      hipLaunchKernelGGL((tall_gemm_lds_bf16_kernel<4, kLdsRowTiles, NTV, KSV>), lgrid, lblock,                     \
                         sizeof(u32x4) * KSV * NTV * 3 * kWave, s, X, t, N, d, kk, tiles, slabs, bias, addend, ldc, out, ldo); \
    else                                                                                                            \
      hipLaunchKernelGGL((tall_gemm_lds_bf16_kernel<2, kLdsRowTiles, NTV, KSV>), lgrid, lblock,                     \
                         sizeof(u32x4) * KSV * NTV * 3 * kWave, s, X, t, N, d, kk, tiles, slabs, bias, addend, ldc, out, ldo); \
  } while (0)
#define EXACT_GEMM_GO(NTV)                                                                                          \
  do {                                                                                                              \
    if (quads)                                                                                                      \
      hipLaunchKernelGGL((tall_gemm_bf16_kernel<4, kGemmRowTiles, NTV, kGemmSteps>), grid, block, 0, s, X, t, N, d, kk, tiles, \
                         tile0, bias, addend, ldc, out, ldo);                                                      \
    else                                                                                                            \
      hipLaunchKernelGGL((tall_gemm_bf16_kernel<2, kGemmRowTiles, NTV, kGemmSteps>), grid, block, 0, s, X, t, N, d, kk, tiles, \
                         tile0, bias, addend, ldc, out, ldo);                                                      \
  } while (0)
  if (tiles == 2) {
    const int slabs = 1;
    const dim3 lgrid(static_cast<unsigned>(lgroups * kGemmXcds));
    EXACT_GEMM_LDS(2, 4);
    return launch_status();
  }
  // every full slab of four tiles in one launch (slabs of two tiles, twice as many sharing an L2 and four
  // wavefronts per SIMD instead of three, measured 5 - 8 % slower: each slab splits X into bf16 pieces again)
  if (const int slabs = tiles / kGemmSlabTiles) {
    const dim3 lgrid(static_cast<unsigned>(lgroups * kGemmXcds * slabs));
    EXACT_GEMM_LDS(4, 2);
  }
  if (const int tile0 = tiles / kGemmSlabTiles * kGemmSlabTiles; tile0 < tiles) {  // a last, narrower slab
    const int nt = tiles - tile0;
    switch (nt) {
      case 1: EXACT_GEMM_GO(1); break;
      case 2: EXACT_GEMM_GO(2); break;
      case 3: EXACT_GEMM_GO(3); break;
      default: EXACT_GEMM_GO(4); break;
    }
  }
#undef EXACT_GEMM_LDS
#undef EXACT_GEMM_GO
  return launch_status();
}

}  // extern "C"
