// Weight gradient of a linear layer over a tall batch:
//   dW[Kout, D] = dY[N, Kout]^T . X[N, D]          (backward_func.cc:88-89,
//                                                   grad_output.t().mm(input))
// N is the number of nodes (10^5 .. 10^6), Kout and D a few hundred at most:
// a GEMM whose reduction dimension is the long one, which general GEMM
// libraries tile poorly (a third of the fp32 matrix-core peak at best here).
//
// v_mfma_f32_32x32x2_f32 takes both operands in exactly the order memory has
// them: the A operand of lane l is A[l % 32][l / 32] = dY[n + l / 32][k0 + l % 32]
// and the B operand is B[l / 32][l % 32] = X[n + l / 32][d0 + l % 32], i.e. each
// half-wave reads 128 consecutive bytes of one row -- no transposition, no LDS.
// A wavefront owns a (32 MK) x (32 MD) block of dW in its accumulators and
// walks a slab of rows two at a time; the four wavefronts of a workgroup hold
// neighbouring blocks, so the fragments they share come out of L1.  The row
// range is cut into slabs, one workgroup each, whose blocks meet in memory
// through fp32 atomic adds into the pre-zeroed dW (the order of those
// additions is not fixed).
//
// Addresses past the last row / column are clamped, not branched around (a
// load behind a branch would make the compiler wait for every outstanding
// load at the join and so undo the prefetch): rows past the slab are zeroed
// by a select, and columns past Kout / D only feed accumulators that are never
// stored.
//
// MFMA 32x32x2 f32 accumulator layout (wave64): register v of lane l is
// C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].

#include "bf16_split.hpp"

namespace exact {

constexpr int kDwPairs = 4;  // row pairs per batch of loads

__global__ __launch_bounds__(kBlock) void dw_zero_kernel(float* __restrict__ out, int64_t n) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kBlock + threadIdx.x;
  if (i < n) out[i] = 0.f;
}

constexpr int kDwXcds = 8;   // accelerator complex dies of an MI355X, each with its own L2

// Workgroup index -> (block of dW, row slab).  Every block of dW reads the same rows of dY and X over a slab, and
// workgroups are handed to the 8 XCDs round-robin by index: the `blocks` workgroups of one slab take indices 8
// apart, so they run on one XCD at about the same time and the rows come from HBM once and from that L2 afterwards.
// The grid is a whole number of groups of 8 slabs; false for a slab past the last one.
__device__ __forceinline__ bool dw_block_and_slab(int blocks, int64_t slabs, int& block, int64_t& slab) {
  const int64_t per_group = static_cast<int64_t>(kDwXcds) * blocks;
  const int64_t in_group = blockIdx.x % per_group;
  block = static_cast<int>(in_group / kDwXcds);
  slab = blockIdx.x / per_group * kDwXcds + in_group % kDwXcds;
  return slab < slabs;
}

// WK x (4 / WK) wavefronts per workgroup along Kout x D.
template <int MK, int MD, int WK>
__global__ __launch_bounds__(kBlock) void linear_dw_kernel(const float* __restrict__ dY, int64_t ldy,
                                                           const float* __restrict__ X, int64_t ldx, int64_t N,
                                                           int Kout, int D, int64_t rows_per_slab, int blocks_d, int blocks, int64_t slabs,
                                                           float* __restrict__ out) {
  constexpr int WD = 4 / WK;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  int block;
  int64_t slab;
  if (!dw_block_and_slab(blocks, slabs, block, slab)) return;  // whole workgroup
  const int bk = block / blocks_d, bd = block % blocks_d;
  const int k0 = (bk * WK + wave / WD) * (32 * MK);
  const int d0 = (bd * WD + wave % WD) * (32 * MD);
  if (k0 >= Kout || d0 >= D) return;  // whole wavefront: no barrier follows
  const int64_t n_begin = slab * rows_per_slab;
  const int64_t n_end = (n_begin + rows_per_slab < N) ? n_begin + rows_per_slab : N;

  int kcol[MK], dcol[MD];
#pragma unroll
  for (int i = 0; i < MK; ++i) kcol[i] = min(k0 + 32 * i + l32, Kout - 1);
#pragma unroll
  for (int j = 0; j < MD; ++j) dcol[j] = min(d0 + 32 * j + l32, D - 1);

  floatx16 acc[MK][MD];
#pragma unroll
  for (int i = 0; i < MK; ++i)
#pragma unroll
    for (int j = 0; j < MD; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  auto load_batch = [&](int64_t n0, float (&a)[kDwPairs][MK], float (&b)[kDwPairs][MD]) {
#pragma unroll
    for (int p = 0; p < kDwPairs; ++p) {
      const int64_t row = n0 + 2 * p + half;
      const int64_t rc = row < N ? row : N - 1;
      const bool ok = row < n_end;
#pragma unroll
      for (int i = 0; i < MK; ++i) {
        const float v = dY[rc * ldy + kcol[i]];
        a[p][i] = ok ? v : 0.f;
      }
#pragma unroll
      for (int j = 0; j < MD; ++j) {
        const float v = X[rc * ldx + dcol[j]];
        b[p][j] = ok ? v : 0.f;
      }
    }
  };
  auto mfma_batch = [&](const float (&a)[kDwPairs][MK], const float (&b)[kDwPairs][MD]) {
#pragma unroll
    for (int p = 0; p < kDwPairs; ++p)
#pragma unroll
      for (int i = 0; i < MK; ++i)
#pragma unroll
        for (int j = 0; j < MD; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[p][i], b[p][j], acc[i][j], 0, 0, 0);
  };

  constexpr int64_t kStep = 2 * kDwPairs;
  float a0[kDwPairs][MK], b0[kDwPairs][MD], a1[kDwPairs][MK], b1[kDwPairs][MD];
  int64_t n0 = n_begin;
  if (n0 < n_end) load_batch(n0, a0, b0);
  while (n0 < n_end) {
    load_batch(n0 + kStep, a1, b1);  // past the slab: clamped addresses, zeroed values
    mfma_batch(a0, b0);
    n0 += kStep;
    if (n0 >= n_end) break;
    load_batch(n0 + kStep, a0, b0);
    mfma_batch(a1, b1);
    n0 += kStep;
  }

#pragma unroll
  for (int i = 0; i < MK; ++i)
#pragma unroll
    for (int j = 0; j < MD; ++j) {
      const int cj = d0 + 32 * j + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ri = k0 + 32 * i + 8 * (v / 4) + 4 * half + (v % 4);
        if (ri < Kout && cj < D) unsafeAtomicAdd(out + static_cast<int64_t>(ri) * D + cj, acc[i][j][v]);
      }
    }
}

// The same product on the bf16 matrix cores at fp32 accuracy (bf16_split.hpp):
// v_mfma_f32_32x32x16_bf16 reduces over 16 rows per instruction, lane (column,
// g) holding rows n + 8 g .. n + 8 g + 7 of its column -- eight 4-byte loads
// per operand fragment, each again 128 consecutive bytes per half-wave.  Both
// operands are split into three bf16 pieces in registers and every 32 x 32
// block takes six instructions per 16 rows, 3 / 8 of the matrix-core time of
// the fp32 instruction.
template <int MK, int MD, int WK>
__global__ __launch_bounds__(kBlock, 2) void linear_dw_bf16_kernel(const float* __restrict__ dY, int64_t ldy,
                                                                const float* __restrict__ X, int64_t ldx, int64_t N,
                                                                int Kout, int D, int64_t rows_per_slab, int blocks_d, int blocks, int64_t slabs,
                                                                float* __restrict__ out) {
  constexpr int WD = 4 / WK;
  constexpr int64_t kRows = 16;  // rows per step
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  int block;
  int64_t slab;
  if (!dw_block_and_slab(blocks, slabs, block, slab)) return;  // whole workgroup
  const int bk = block / blocks_d, bd = block % blocks_d;
  const int k0 = (bk * WK + wave / WD) * (32 * MK);
  const int d0 = (bd * WD + wave % WD) * (32 * MD);
  if (k0 >= Kout || d0 >= D) return;  // whole wavefront: no barrier follows
  const int64_t n_begin = slab * rows_per_slab;
  const int64_t n_end = (n_begin + rows_per_slab < N) ? n_begin + rows_per_slab : N;

  int kcol[MK], dcol[MD];
#pragma unroll
  for (int i = 0; i < MK; ++i) kcol[i] = min(k0 + 32 * i + l32, Kout - 1);
#pragma unroll
  for (int j = 0; j < MD; ++j) dcol[j] = min(d0 + 32 * j + l32, D - 1);

  floatx16 acc[MK][MD];
#pragma unroll
  for (int i = 0; i < MK; ++i)
#pragma unroll
    for (int j = 0; j < MD; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const float* ycol[MK];
  const float* xcol[MD];
#pragma unroll
  for (int i = 0; i < MK; ++i) ycol[i] = dY + kcol[i];
#pragma unroll
  for (int j = 0; j < MD; ++j) xcol[j] = X + dcol[j];
  auto load_step = [&](int64_t n0, float (&a)[MK][8], float (&b)[MD][8]) {
    if (n0 + kRows <= n_end) {  // wave-uniform: the whole step lies inside the slab, nothing to clamp or mask
      const int64_t first = n0 + 8 * half;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
#pragma unroll
        for (int i = 0; i < MK; ++i) a[i][e] = ycol[i][(first + e) * ldy];
#pragma unroll
        for (int j = 0; j < MD; ++j) b[j][e] = xcol[j][(first + e) * ldx];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int64_t row = n0 + 8 * half + e;
        const int64_t rc = row < N ? row : N - 1;
        const bool ok = row < n_end;
#pragma unroll
        for (int i = 0; i < MK; ++i) {
          const float v = ycol[i][rc * ldy];
          a[i][e] = ok ? v : 0.f;
        }
#pragma unroll
        for (int j = 0; j < MD; ++j) {
          const float v = xcol[j][rc * ldx];
          b[j][e] = ok ? v : 0.f;
        }
      }
    }
  };
  // One set of raw registers: a step's values are split into their bf16 pieces first, then the
  // loads of the next step are issued into the same registers and fly during this step's MFMAs.
  float a[MK][8], b[MD][8];
  int64_t n0 = n_begin;
  if (n0 < n_end) load_step(n0, a, b);
  while (n0 < n_end) {
    Split8 sa[MK], sb[MD];
#pragma unroll
    for (int i = 0; i < MK; ++i) sa[i] = split3x8(a[i]);
#pragma unroll
    for (int j = 0; j < MD; ++j) sb[j] = split3x8(b[j]);
    load_step(n0 + kRows, a, b);  // past the slab: clamped addresses, zeroed values
#pragma unroll
    for (int i = 0; i < MK; ++i)
#pragma unroll
      for (int j = 0; j < MD; ++j) {
        const u32x4 pieces[3] = {sb[j].hi, sb[j].mid, sb[j].lo};
        acc[i][j] = step_product<3>(sa[i], pieces, acc[i][j]);
      }
    n0 += kRows;
  }

#pragma unroll
  for (int i = 0; i < MK; ++i)
#pragma unroll
    for (int j = 0; j < MD; ++j) {
      const int cj = d0 + 32 * j + l32;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int ri = k0 + 32 * i + 8 * (v / 4) + 4 * half + (v % 4);
        if (ri < Kout && cj < D) unsafeAtomicAdd(out + static_cast<int64_t>(ri) * D + cj, acc[i][j][v]);
      }
    }
}

template <int MK, int MD, int WK, bool BF16>
static void launch_dw(const float* dY, int64_t ldy, const float* X, int64_t ldx, int64_t N, int Kout, int D, float* out,
                      hipStream_t s) {
  constexpr int WD = 4 / WK;
  const int blocks_k = (Kout + 32 * MK * WK - 1) / (32 * MK * WK);
  const int blocks_d = (D + 32 * MD * WD - 1) / (32 * MD * WD);
  const int blocks = blocks_k * blocks_d;
  // about 1024 workgroups in all, at least 512 rows per slab, whole batches per slab
  int64_t slabs = (1024 + blocks - 1) / blocks;
  int64_t rows = (N + slabs - 1) / slabs;
  if (rows < 512) rows = 512;
  rows = (rows + 15) / 16 * 16;  // whole batches (8 rows) resp. steps (16 rows)
  slabs = (N + rows - 1) / rows;
  const dim3 grid(static_cast<unsigned>((slabs + kDwXcds - 1) / kDwXcds * kDwXcds * blocks));
  if (BF16) hipLaunchKernelGGL((linear_dw_bf16_kernel<MK, MD, WK>), grid, dim3(kBlock), 0, s, dY, ldy, X, ldx, N, Kout, D, rows, blocks_d, blocks, slabs, out);
  else hipLaunchKernelGGL((linear_dw_kernel<MK, MD, WK>), grid, dim3(kBlock), 0, s, dY, ldy, X, ldx, N, Kout, D, rows, blocks_d, blocks, slabs, out);
}

template <bool BF16>
static int linear_dw_any(const float* dY, int64_t ldy, const float* X, int64_t ldx, int64_t N, int64_t Kout, int64_t D,
                         float* out, hipStream_t s) {
  if (N < 0 || Kout < 0 || D < 0 || Kout > 65536 || D > 65536 || N > (int64_t{1} << 40)) return EXACT_E_SHAPE;
  if (ldy < Kout || ldx < D) return EXACT_E_SHAPE;
  if (Kout == 0 || D == 0) return EXACT_OK;
  if (!out || (N > 0 && (!dY || !X))) return EXACT_E_NULL;
  const int64_t total = Kout * D;
  hipLaunchKernelGGL(dw_zero_kernel, dim3(static_cast<unsigned>((total + kBlock - 1) / kBlock)), dim3(kBlock), 0, s, out, total);
  if (N > 0) {
    const int K = static_cast<int>(Kout), Dd = static_cast<int>(D);
    // wavefront block: up to 64 x 64 of dW (wider blocks need more accumulator registers than two wavefronts
    // per SIMD leave); the four wavefronts side by side along the longer extent when the other fits one wavefront
    if (K <= 32) {
      if (Dd <= 128) launch_dw<1, 1, 1, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
      else launch_dw<1, 2, 1, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
    } else if (K <= 64) {
      if (Dd <= 128) launch_dw<2, 1, 1, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
      else launch_dw<2, 2, 1, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
    } else {
      if (Dd <= 32) launch_dw<2, 1, 4, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
      else if (Dd <= 64) launch_dw<2, 2, 4, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
      else launch_dw<2, 2, 2, BF16>(dY, ldy, X, ldx, N, K, Dd, out, s);
    }
  }
  return launch_status();
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_linear_dw_f32(const float* dY, int64_t ldy, const float* X, int64_t ldx, int64_t N, int64_t Kout, int64_t D,
                        float* out, void* stream) {
  return linear_dw_any<false>(dY, ldy, X, ldx, N, Kout, D, out, static_cast<hipStream_t>(stream));
}

int exact_linear_dw_bf16_f32(const float* dY, int64_t ldy, const float* X, int64_t ldx, int64_t N, int64_t Kout, int64_t D,
                             float* out, void* stream) {
  return linear_dw_any<true>(dY, ldy, X, ldx, N, Kout, D, out, static_cast<hipStream_t>(stream));
}

}  // extern "C"
