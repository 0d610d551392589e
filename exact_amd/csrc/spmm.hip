// CSR SpMM (sum / mean) for power-law graphs on gfx950:
//   out[r, :] = reduce_{e in row r} val[e] * X[col[e], :]
//
// Semantics restated from the reference (spmm_cuda.cu:27-104 with
// Reducer<SUM|MEAN> reducer.cuh:43-85: fp32 accumulation in CSR order, mean
// divides by max(row length, 1), empty rows give 0).  The reference gives one
// 32-lane warp to each (row, 32-column tile), which serialises hub rows; this
// kernel instead splits the ENTRY stream into chunks of 64 entries and gives
// every wavefront exactly one chunk, so the work per wavefront is the same
// whatever the degree distribution:
//
//   * one coalesced load brings the chunk's 64 column indices (and values)
//     into lanes; a wave-uniform walk over them gathers X rows, the 64 lanes
//     spanning 64 * VEC consecutive feature columns (grid.y tiles wider K);
//   * a row that lies wholly inside one chunk is accumulated in CSR order and
//     written with a plain store; a row that straddles chunks is accumulated
//     per chunk and combined with fp32 atomic adds into rows that a small
//     pre-pass has zeroed (the same pre-pass zeroes empty rows); for the mean a
//     small post-pass divides those rows' totals by the row length.

#include "exact_common.hpp"

namespace exact {

constexpr int kChunk = 64;  // entries per wavefront == lanes per wavefront
constexpr int kGather = 8;  // X rows in flight per lane (4 and 16 measure the same)
constexpr int kXcds = 8;    // accelerator complex dies of an MI355X, each with its own L2
// Mean aggregation, rows cut by chunk boundaries: up to this length every chunk
// divides its partial sum by the row length before the atomic add (at most 32
// rounded terms); longer rows -- the hubs -- add raw partial sums and are
// divided once by spmm_mean_finish_kernel, like the reference's reducer, so
// hundreds of rounded quotients never pile up.  Dividing every split row at
// the end would re-read and re-write most of the output on dense graphs.
constexpr int64_t kMeanFinishLen = 2048;

template <int VEC> struct Vec;
template <> struct Vec<2> { using T = float2; };
template <> struct Vec<1> { using T = float; };

template <int VEC>
__device__ __forceinline__ void load_vec(const float* p, float (&v)[VEC]) {
  if constexpr (VEC == 4) { const float4 q = *reinterpret_cast<const float4*>(p); v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w; }
  else if constexpr (VEC == 2) { const float2 q = *reinterpret_cast<const float2*>(p); v[0] = q.x; v[1] = q.y; }
  else { v[0] = *p; }
}
template <int VEC>
__device__ __forceinline__ void store_vec(float* p, const float (&v)[VEC]) {
  if constexpr (VEC == 4) *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  else if constexpr (VEC == 2) *reinterpret_cast<float2*>(p) = make_float2(v[0], v[1]);
  else *p = v[0];
}

__device__ __forceinline__ int readlane_i(int v, int lane) { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float readlane_f(float v, int lane) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
__device__ __forceinline__ int64_t readlane_i64(int64_t v, int lane) {
  const int lo = __builtin_amdgcn_readlane(static_cast<int>(v), lane);
  const int hi = __builtin_amdgcn_readlane(static_cast<int>(v >> 32), lane);
  return (static_cast<int64_t>(hi) << 32) | static_cast<uint32_t>(lo);
}

// A row needs zeroing before the main kernel when nothing stores to it with a
// plain store: it is empty, or it spans more than one chunk.
template <typename I>
__global__ __launch_bounds__(kBlock) void spmm_zero_rows_kernel(const I* __restrict__ rowptr, int64_t M,
                                                                int64_t K, int64_t ldo, float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + (threadIdx.x >> 6)) * kWave;
  const int64_t r = base + lane;
  bool need = false;
  if (r < M) {
    const int64_t rs = rowptr[r], re = rowptr[r + 1];
    need = (re == rs) || (rs / kChunk != (re - 1) / kChunk);
  }
  uint64_t todo = __ballot(need);
  while (todo) {
    const int l = __builtin_ctzll(todo);
    todo &= todo - 1;
    float* dst = out + (base + l) * ldo;
    for (int64_t c = lane; c < K; c += kWave) dst[c] = 0.f;
  }
}

// Mean aggregation, rows longer than kMeanFinishLen that span more than one
// chunk: the chunk kernel has added up their partial sums; divide by the row
// length (reducer.cuh:75-76).
template <typename I>
__global__ __launch_bounds__(kBlock) void spmm_mean_finish_kernel(const I* __restrict__ rowptr, int64_t M,
                                                                  int64_t K, int64_t ldo, float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t base = (static_cast<int64_t>(blockIdx.x) * (kBlock / kWave) + (threadIdx.x >> 6)) * kWave;
  const int64_t r = base + lane;
  bool split = false;
  float len = 1.f;
  if (r < M) {
    const int64_t rs = rowptr[r], re = rowptr[r + 1];
    split = (re - rs > kMeanFinishLen) && (rs / kChunk != (re - 1) / kChunk);
    len = static_cast<float>(re - rs);
  }
  uint64_t todo = __ballot(split);
  while (todo) {
    const int l = __builtin_ctzll(todo);
    todo &= todo - 1;
    const float d = readlane_f(len, l);
    float* dst = out + (base + l) * ldo;
    for (int64_t c = lane; c < K; c += kWave) dst[c] = dst[c] / d;
  }
}

template <typename I, int VEC, bool HAS_VAL, bool MEAN>
__global__ __launch_bounds__(kBlock) void spmm_chunk_kernel(const I* __restrict__ rowptr,
                                                            const I* __restrict__ col,
                                                            const float* __restrict__ val,
                                                            const float* __restrict__ X, int64_t M,
                                                            int64_t nnz, int64_t K, int64_t ldx, int64_t ldo,
                                                            float* __restrict__ out) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x >> 6));
  // Workgroups are handed to the 8 XCDs round-robin by index; give each XCD a
  // contiguous range of chunks, so that neighbouring CSR rows (which in real
  // graphs share neighbours) gather through the same L2.  gridDim.x is a
  // multiple of kXcds; logical indices past the last chunk fall out below.
  const int64_t per_xcd = gridDim.x / kXcds;
  const int64_t wg = static_cast<int64_t>(blockIdx.x % kXcds) * per_xcd + blockIdx.x / kXcds;
  const int64_t e0 = (wg * (kBlock / kWave) + wave) * kChunk;
  if (e0 >= nnz) return;
  const int cnt = static_cast<int>(nnz - e0 < kChunk ? nnz - e0 : kChunk);
  const int64_t kcol = (static_cast<int64_t>(blockIdx.y) * kWave + lane) * VEC;
  const bool kok = kcol < K;

  // Row that owns entry e0: the last r with rowptr[r] <= e0.  A 64-ary search:
  // every round the 64 lanes probe 64 evenly spaced positions of [lo, hi) at
  // once and a ballot picks the sub-interval, so a graph of M rows costs
  // ceil(log64 M) dependent loads (3 for 169k rows) instead of log2 M.
  // Invariant: rowptr[lo] <= e0, and hi == M or rowptr[hi] > e0.
  int64_t lo = 0, hi = M;
  while (hi - lo > 1) {
    const int64_t step = (hi - lo + kWave - 1) / kWave;
    const int64_t pos = lo + step * lane;
    const bool le = pos < hi && static_cast<int64_t>(rowptr[pos]) <= e0;
    const uint64_t hits = __ballot(le);                 // rowptr is sorted: a run of ones from lane 0
    const int last = 63 - __builtin_clzll(hits | 1u);  // bit 0 is set by the invariant
    lo += step * last;
    hi = (lo + step < hi) ? lo + step : hi;
  }
  int64_t r = lo;

  int my_col = 0;
  float my_val = 1.f;
  if (lane < cnt) {
    my_col = static_cast<int>(col[e0 + lane]);
    if constexpr (HAS_VAL) my_val = val[e0 + lane];
  }
  // row ends for rows r .. r+63, one per lane
  auto load_ends = [&](int64_t first) -> int64_t {
    const int64_t idx = first + 1 + lane;
    return static_cast<int64_t>(rowptr[idx < M ? idx : M]);
  };
  int64_t ends = load_ends(r);
  int rl = 0;
  int64_t row_start = static_cast<int64_t>(rowptr[r]);
  int64_t row_end = readlane_i64(ends, 0);

  float acc[VEC];
#pragma unroll
  for (int c = 0; c < VEC; ++c) acc[c] = 0.f;

  auto flush = [&]() {
    if (row_end > row_start && kok) {
      float* dst = out + r * ldo + kcol;
      if (row_start >= e0 && row_end <= e0 + cnt) {
        float res[VEC];
#pragma unroll
        for (int c = 0; c < VEC; ++c)
          res[c] = MEAN ? acc[c] / static_cast<float>(row_end - row_start) : acc[c];  // reducer.cuh:75-76
        store_vec<VEC>(dst, res);
      } else {
        // a row cut by a chunk boundary: its partial sums meet in memory
        const int64_t len = row_end - row_start;
        const float div = (MEAN && len <= kMeanFinishLen) ? static_cast<float>(len) : 1.f;
#pragma unroll
        for (int c = 0; c < VEC; ++c) unsafeAtomicAdd(dst + c, MEAN ? acc[c] / div : acc[c]);
      }
    }
#pragma unroll
    for (int c = 0; c < VEC; ++c) acc[c] = 0.f;
  };
  auto advance = [&]() {
    ++r;
    ++rl;
    if (rl == kWave) {
      ends = load_ends(r);
      rl = 0;
    }
    row_start = row_end;
    row_end = readlane_i64(ends, rl);
  };

  for (int base = 0; base < cnt; base += kGather) {
    float xv[kGather][VEC];
#pragma unroll
    for (int u = 0; u < kGather; ++u) {
#pragma unroll
      for (int c = 0; c < VEC; ++c) xv[u][c] = 0.f;
      if (base + u < cnt) {  // wave-uniform, so every lane takes part in the broadcast
        const int64_t c = readlane_i(my_col, base + u);
        if (kok) load_vec<VEC>(X + c * ldx + kcol, xv[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < kGather; ++u) {
      if (base + u < cnt) {
        const int64_t e = e0 + base + u;
        while (e >= row_end && r + 1 < M) {  // r + 1 < M: a malformed rowptr cannot spin
          flush();
          advance();
        }
        const float w = HAS_VAL ? readlane_f(my_val, base + u) : 1.f;
#pragma unroll
        for (int c = 0; c < VEC; ++c) acc[c] = __fmaf_rn(w, xv[u][c], acc[c]);
      }
    }
  }
  flush();
}

static bool al(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

template <typename I, int VEC>
static void spmm_dispatch(const I* rowptr, const I* col, const float* val, const float* X, int64_t M,
                          int64_t nnz, int64_t K, int64_t ldx, int64_t ldo, int reduce, float* out, hipStream_t s) {
  const int64_t chunks = (nnz + kChunk - 1) / kChunk;
  const int64_t wgs = (chunks + 3) / 4;
  const dim3 grid(static_cast<unsigned>((wgs + kXcds - 1) / kXcds * kXcds),
                  static_cast<unsigned>((K + kWave * VEC - 1) / (kWave * VEC)));
  const dim3 block(kBlock);
  const bool mean = reduce == EXACT_REDUCE_MEAN;
  if (val) {
    if (mean) hipLaunchKernelGGL((spmm_chunk_kernel<I, VEC, true, true>), grid, block, 0, s, rowptr, col, val, X, M, nnz, K, ldx, ldo, out);
    else hipLaunchKernelGGL((spmm_chunk_kernel<I, VEC, true, false>), grid, block, 0, s, rowptr, col, val, X, M, nnz, K, ldx, ldo, out);
  } else {
    if (mean) hipLaunchKernelGGL((spmm_chunk_kernel<I, VEC, false, true>), grid, block, 0, s, rowptr, col, val, X, M, nnz, K, ldx, ldo, out);
    else hipLaunchKernelGGL((spmm_chunk_kernel<I, VEC, false, false>), grid, block, 0, s, rowptr, col, val, X, M, nnz, K, ldx, ldo, out);
  }
}

}  // namespace exact

using namespace exact;

extern "C" {

int exact_spmm_csr_strided_f32(const void* rowptr, const void* col, const float* val, int idx_bytes,
                               const float* X, int64_t ldx, int64_t M, int64_t n_cols, int64_t K, int64_t nnz,
                               int reduce, float* out, int64_t ldo, void* stream) {
  if (idx_bytes != 4 && idx_bytes != 8) return EXACT_E_ARG;
  if (reduce != EXACT_REDUCE_SUM && reduce != EXACT_REDUCE_MEAN) return EXACT_E_ARG;
  if (M < 0 || K < 0 || nnz < 0 || n_cols < 0 || n_cols > 0x7FFFFFFFll) return EXACT_E_SHAPE;
  if (idx_bytes == 4 && nnz > 0x7FFFFFFFll) return EXACT_E_SHAPE;
  // launch-grid limits: 2^31 - 1 workgroups of 256 rows (pre-pass) resp. 256 entries (main kernel)
  if (M > (int64_t{1} << 38) || nnz > (int64_t{1} << 38) || K > (int64_t{1} << 24)) return EXACT_E_SHAPE;
  if (ldx < K || ldo < K) return EXACT_E_SHAPE;
  if (M == 0 || K == 0) return EXACT_OK;
  if (!rowptr || !out || (nnz > 0 && (!col || !X))) return EXACT_E_NULL;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 zgrid(static_cast<unsigned>((M + kBlock - 1) / kBlock));
  if (idx_bytes == 4)
    hipLaunchKernelGGL((spmm_zero_rows_kernel<int32_t>), zgrid, dim3(kBlock), 0, s,
                       static_cast<const int32_t*>(rowptr), M, K, ldo, out);
  else
    hipLaunchKernelGGL((spmm_zero_rows_kernel<int64_t>), zgrid, dim3(kBlock), 0, s,
                       static_cast<const int64_t*>(rowptr), M, K, ldo, out);
  if (nnz > 0) {
    // Column tile of one wavefront = 64 * vec columns.  Measured on power-law
    // graphs of 170k to 2.4M rows: 8-byte gathers (128-column tiles) beat 16-byte
    // ones (256-column tiles) by 6 to 40 % at every width from 100 to 600 -- twice
    // as many wavefronts share the same gathers -- so 16-byte gathers are not
    // used; rows of at most 64 columns take 4-byte gathers (one tile, more lanes
    // busy than with wider ones).
    const int vec = (K > 64 && K % 2 == 0 && ldx % 2 == 0 && ldo % 2 == 0 && al(X, 8) && al(out, 8)) ? 2 : 1;
    if ((K + kWave * vec - 1) / (kWave * vec) > 65535) return EXACT_E_SHAPE;  // grid.y limit
#define EXACT_SPMM_GO(I, V) \
  spmm_dispatch<I, V>(static_cast<const I*>(rowptr), static_cast<const I*>(col), val, X, M, nnz, K, ldx, ldo, reduce, out, s)
    if (idx_bytes == 4) {
      if (vec == 2) EXACT_SPMM_GO(int32_t, 2); else EXACT_SPMM_GO(int32_t, 1);
    } else {
      if (vec == 2) EXACT_SPMM_GO(int64_t, 2); else EXACT_SPMM_GO(int64_t, 1);
    }
#undef EXACT_SPMM_GO
    if (reduce == EXACT_REDUCE_MEAN) {
      if (idx_bytes == 4)
        hipLaunchKernelGGL((spmm_mean_finish_kernel<int32_t>), zgrid, dim3(kBlock), 0, s,
                           static_cast<const int32_t*>(rowptr), M, K, ldo, out);
      else
        hipLaunchKernelGGL((spmm_mean_finish_kernel<int64_t>), zgrid, dim3(kBlock), 0, s,
                           static_cast<const int64_t*>(rowptr), M, K, ldo, out);
    }
  }
  return launch_status();
}

int exact_spmm_csr_f32(const void* rowptr, const void* col, const float* val, int idx_bytes,
                       const float* X, int64_t M, int64_t n_cols, int64_t K, int64_t nnz, int reduce,
                       float* out, void* stream) {
  return exact_spmm_csr_strided_f32(rowptr, col, val, idx_bytes, X, K, M, n_cols, K, nnz, reduce, out, K, stream);
}

}  // extern "C"
