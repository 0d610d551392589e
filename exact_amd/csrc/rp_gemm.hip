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

#include "rp_common.hpp"

namespace exact {

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

// The product of rp_fwd_kernel for the kernel that goes on to quantise it:
// acc = X[row0 .. row0 + 31, :] . R for the calling wavefront, the MFMA steps in
// the same order (so the same bits).  Rl is the workgroup's LDS staging area
// [kFwdDChunk][NT * 32]; every wavefront of the workgroup must call this (it
// contains workgroup barriers).
//
// Memory-level parallelism: a lane issues the loads of its whole share of a
// 64-column chunk (eight 16-byte loads at VEC = 4: the 128-byte line of its
// row and the next) before the first MFMA consumes them, and the threads that
// stage R fetch eight elements each before the first LDS write -- one exposure
// to memory latency per chunk instead of one per load.
template <int VEC, int NT>
__device__ __forceinline__ void rp_fwd_accumulate(const float* __restrict__ X, const float* __restrict__ R,
                                                  int64_t N, int D, int k, float* Rl, floatx16 (&acc)[NT]) {
  constexpr int KP = NT * kTile;
  constexpr int kBatch = 8;
  constexpr int kStagePerThread = kFwdDChunk * KP / kBlock;  // 8 * NT
  constexpr int kSteps = kFwdDChunk / (2 * VEC);             // k-slices of a lane per chunk
  static_assert(kStagePerThread % kBatch == 0 && kSteps % kBatch == 0, "batches divide the chunk");
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kTile;
  const int64_t my_row = (row0 + l32 < N) ? row0 + l32 : N - 1;
  const float* xrow = X + my_row * D;

#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[nt][v] = 0.f;

  for (int dc = 0; dc < D; dc += kFwdDChunk) {
    __syncthreads();
    for (int b0 = 0; b0 < kStagePerThread; b0 += kBatch) {
      float staged[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        const int idx = threadIdx.x + (b0 + i) * kBlock;
        const int rr = idx / KP, cc = idx - rr * KP;
        staged[i] = (dc + rr < D && cc < k) ? R[static_cast<int64_t>(dc + rr) * k + cc] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < kBatch; ++i) Rl[threadIdx.x + (b0 + i) * kBlock] = staged[i];
    }
    __syncthreads();
    const int dlim = (D - dc < kFwdDChunk) ? D - dc : kFwdDChunk;
    for (int s0 = 0; s0 < kSteps; s0 += kBatch) {
      if (s0 * 2 * VEC >= dlim) break;
      float a[kBatch][VEC];
#pragma unroll
      for (int sb = 0; sb < kBatch; ++sb) {
        const int ks = (s0 + sb) * 2 * VEC + VEC * half;  // this lane's k-slice inside the chunk
        load_k_slice<VEC>(xrow, dc + ks, D, a[sb]);        // zeros past column D
      }
#pragma unroll
      for (int sb = 0; sb < kBatch; ++sb) {
        const int kb = (s0 + sb) * 2 * VEC;
        if (kb < dlim) {
          const int ks = kb + VEC * half;
#pragma unroll
          for (int t = 0; t < VEC; ++t) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
              const float b = Rl[(ks + t) * KP + nt * kTile + l32];
              acc[nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[sb][t], b, acc[nt], 0, 0, 0);
            }
          }
        }
      }
    }
  }
}

// out[N, k] = X[N, D] . R[D, k];  NT * 32 >= k columns per wavefront.
template <int VEC, int NT>
__global__ __launch_bounds__(kBlock) void rp_fwd_kernel(const float* __restrict__ X,
                                                        const float* __restrict__ R, int64_t N, int D,
                                                        int k, float* __restrict__ out) {
  HIP_DYNAMIC_SHARED(float, Rl)  // [kFwdDChunk][NT * 32]
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
  const int l32 = lane & 31;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kTile;

  floatx16 acc[NT];
  rp_fwd_accumulate<VEC, NT>(X, R, N, D, k, Rl, acc);

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

// Projection and quantisation in one launch (the epilogue is rp_quantise_and_pack, rp_common.hpp).
template <int VEC, int NT, bool NOISE_IN>
__global__ __launch_bounds__(kBlock) void rp_fwd_pack_kernel(const RpPackArgs a) {
  HIP_DYNAMIC_SHARED(float, Rl)  // [kFwdDChunk][NT * 32]
  const int wave = threadIdx.x >> 6;
  const int64_t row0 = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + wave) * kTile;
  floatx16 acc[NT];
  rp_fwd_accumulate<VEC, NT>(a.X, a.R, a.N, a.D, a.k, Rl, acc);
  rp_quantise_and_pack<NT, NOISE_IN>(a, acc, row0);
}

// out[N, D] = Xr[N, k] . R[D, k]^T;  grid.y tiles D in slabs of NT * 32 columns.
// The product is bound by writing [N, D].  In the accumulator layout a store
// instruction would write 4 bytes per lane; with STAGED (D % 4 == 0, `out`
// 16-byte aligned) the accumulators leave through a per-wavefront LDS tile of
// 8 rows instead, from which every lane stores 16 bytes and a store instruction
// covers whole rows of the slab (up to 512 contiguous bytes each).
template <int NT>
constexpr int bwd_stage_pitch() { return NT * kTile + 8; }  // 4 * pitch = 32 (mod 64): the two half-waves hit different banks

template <int VEC, int NT, bool STAGED>
__global__ __launch_bounds__(kBlock) void rp_bwd_kernel(const float* __restrict__ Xr,
                                                        const float* __restrict__ R, int64_t N, int D,
                                                        int k, int kpad, float* __restrict__ out) {
  HIP_DYNAMIC_SHARED(float, Rl)  // [NT * 32][kpad + 1], odd pitch: conflict-free column reads; then the staging tiles
  typedef float floatx4 __attribute__((ext_vector_type(4)));
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

  if constexpr (STAGED) {
    constexpr int PC = bwd_stage_pitch<NT>();
    constexpr int kQuadsPerRow = NT * kTile / 4;
    float* Ct = Rl + NT * kTile * pitch + ((-(NT * kTile * pitch)) & 3) + wave * (8 * PC);  // 16-byte aligned [8][PC]
#pragma unroll
    for (int g = 0; g < 4; ++g) {  // rows 8 g .. 8 g + 7 of the wavefront's 32
      __syncthreads();             // the tile's previous contents have been read
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int r = 0; r < 4; ++r) Ct[(4 * half + r) * PC + nt * kTile + l32] = acc[nt][4 * g + r];
      __syncthreads();
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        const int f = j * kWave + lane;
        const int tr = f / kQuadsPerRow, tq = f - tr * kQuadsPerRow;
        const int64_t rr = row0 + 8 * g + tr;
        const int cj = dbase + 4 * tq;
        const floatx4 q = *reinterpret_cast<const floatx4*>(Ct + tr * PC + 4 * tq);
        if (rr < N && cj < D) __builtin_nontemporal_store(q, reinterpret_cast<floatx4*>(out + rr * D + cj));
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

template <int VEC, bool NOISE_IN>
static int rp_fwd_pack_launch(const RpPackArgs& a, hipStream_t s) {
  const int nt = (a.k + kTile - 1) / kTile;
  const dim3 grid(static_cast<unsigned>((a.N + 127) / 128));
  const size_t lds = static_cast<size_t>(kFwdDChunk) * nt * kTile * sizeof(float);
  switch (nt) {
    case 1: hipLaunchKernelGGL((rp_fwd_pack_kernel<VEC, 1, NOISE_IN>), grid, dim3(kBlock), lds, s, a); break;
    case 2: hipLaunchKernelGGL((rp_fwd_pack_kernel<VEC, 2, NOISE_IN>), grid, dim3(kBlock), lds, s, a); break;
    case 3: hipLaunchKernelGGL((rp_fwd_pack_kernel<VEC, 3, NOISE_IN>), grid, dim3(kBlock), lds, s, a); break;
    case 4: hipLaunchKernelGGL((rp_fwd_pack_kernel<VEC, 4, NOISE_IN>), grid, dim3(kBlock), lds, s, a); break;
    default: return EXACT_E_SHAPE;
  }
  return launch_status();
}

template <int VEC>
static int rp_bwd_launch(const float* Xr, const float* R, int64_t N, int D, int k, float* out, hipStream_t s) {
  const int kpad = ((k + 2 * VEC - 1) / (2 * VEC)) * (2 * VEC);
  const bool staged = D % 4 == 0 && al16(out);
  // output slab per workgroup: 128 columns, 64 when R's slab (and the staging tiles) would not fit 64 KB of LDS
  const int nt = (kpad <= (staged ? 64 : 96)) ? 4 : 2;
  const dim3 grid(static_cast<unsigned>((N + 127) / 128), static_cast<unsigned>((D + nt * kTile - 1) / (nt * kTile)));
  const size_t r_floats = static_cast<size_t>(nt) * kTile * (kpad + 1);
  const size_t lds = sizeof(float) * (r_floats + 3 + (staged ? (kBlock / kWave) * 8 * (nt * kTile + 8) : 0));
  if (nt == 4) {
    if (staged) hipLaunchKernelGGL((rp_bwd_kernel<VEC, 4, true>), grid, dim3(kBlock), lds, s, Xr, R, N, D, k, kpad, out);
    else hipLaunchKernelGGL((rp_bwd_kernel<VEC, 4, false>), grid, dim3(kBlock), lds, s, Xr, R, N, D, k, kpad, out);
  } else {
    if (staged) hipLaunchKernelGGL((rp_bwd_kernel<VEC, 2, true>), grid, dim3(kBlock), lds, s, Xr, R, N, D, k, kpad, out);
    else hipLaunchKernelGGL((rp_bwd_kernel<VEC, 2, false>), grid, dim3(kBlock), lds, s, Xr, R, N, D, k, kpad, out);
  }
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

int exact_rp_minmax_pack_f32(const float* X, const float* R, const float* noise, uint64_t seed, uint64_t offset,
                             int64_t N, int64_t D, int64_t k, int bits, uint8_t* packed, float* scale_f32,
                             float* min_f32, uint16_t* scale_bf16, uint16_t* min_bf16, void* stream) {
  if (bits != 1 && bits != 2 && bits != 4 && bits != 8) return EXACT_E_BITS;
  if (N < 0 || D <= 0 || k <= 0 || D > (1 << 20) || k > 128 || N > (int64_t{1} << 31) - 64) return EXACT_E_SHAPE;
  if (!packed) return EXACT_E_NULL;
  RpPackArgs a{};
  a.pad_index = exact_packed_nbytes(N, k, bits) - 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (N == 0) {
    hipLaunchKernelGGL(rp_zero_byte_kernel, dim3(1), dim3(1), 0, s, packed + a.pad_index);
    return launch_status();
  }
  if (!X || !R) return EXACT_E_NULL;
  a.X = X;
  a.R = R;
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
  if (D % 4 == 0 && al16(X)) return noise ? rp_fwd_pack_launch<4, true>(a, s) : rp_fwd_pack_launch<4, false>(a, s);
  if (D % 2 == 0 && al8(X)) return noise ? rp_fwd_pack_launch<2, true>(a, s) : rp_fwd_pack_launch<2, false>(a, s);
  return noise ? rp_fwd_pack_launch<1, true>(a, s) : rp_fwd_pack_launch<1, false>(a, s);
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
