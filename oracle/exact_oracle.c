/*
 * exact_oracle.c -- plain C restatement of the reference algorithm for the
 * activation pack / unpack, 1-bit masks and CSR SpMM.
 *
 * TEST INFRASTRUCTURE ONLY: the parity checker's second implementation and the
 * CPU baseline that bench.py times next to the GPU kernels.  Nothing in the
 * product (exact_amd/) links, loads or calls it.
 *
 * Each function follows the reference lines it cites (paths relative to
 * exact/exact/cpp_extension/).  Arithmetic that decides a quantised value is
 * written one fp32 operation per statement through `volatile`-free temporaries
 * and the file is compiled with -ffp-contract=off, so nothing is fused.
 * Pinned by tests/test_oracle.py: bit-identical to the NumPy restatement,
 * which in turn is pinned by hand-computed bytes and library routines.
 *
 * Build: make -C oracle      (gcc -O2 -fopenmp -ffp-contract=off)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

int oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ---- Philox4x32-10 (Salmon et al., SC'11) -------------------------------- */
static void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
    c[1] = (uint32_t)p1;
    c[3] = (uint32_t)p0;
    c[0] = n0;
    c[2] = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

void oracle_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  memcpy(out, ctr, 16);
  philox4x32_10(out, key[0], key[1]);
}

/* __float2int_rn = cvt.rni.s32.f32: round half to even, clamped to the int32 range (NaN does not reach it:
 * the fmaxf ahead of it returns 0). */
static inline int32_t float2int_rn(float t) { return t >= 2147483648.0f ? INT32_MAX : (int32_t)rintf(t); }

static inline float u16_to_uniform(uint32_t h) { return ((float)h + 0.5f) * 0x1p-16f; }

/* noise of element (n, d): counter (d / 8, n, offset_lo, offset_hi), key = seed */
static void philox_oct(uint64_t seed, uint64_t offset, uint32_t c0, uint32_t c1, float u[8]) {
  uint32_t c[4] = {c0, c1, (uint32_t)offset, (uint32_t)(offset >> 32)};
  philox4x32_10(c, (uint32_t)seed, (uint32_t)(seed >> 32));
  for (int w = 0; w < 4; ++w) {
    u[2 * w] = u16_to_uniform(c[w] & 0xFFFFu);
    u[2 * w + 1] = u16_to_uniform(c[w] >> 16);
  }
}

/* ---- a1: per-row min / max (qsheme.py:41-48, ops.py:61-66) --------------- */
void oracle_row_minmax(const float *x, int64_t N, int64_t G, float *mn, float *mx) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    const float *row = x + n * G;
    float lo = row[0], hi = row[0];
    for (int64_t d = 1; d < G; ++d) {
      lo = row[d] < lo ? row[d] : lo;
      hi = row[d] > hi ? row[d] : hi;
    }
    mn[n] = lo;
    mx[n] = hi;
  }
}

/* a2: scale = (2^b - 1) / (mx - mn) (ops.py:39): int / tensor is
 * tensor.reciprocal() * int in torch, i.e. two fp32 roundings */
void oracle_scale(const float *mn, const float *mx, int64_t N, int bits, float *scale) {
  const float B = (float)((1 << bits) - 1);
  for (int64_t n = 0; n < N; ++n) {
    const float range = mx[n] - mn[n];
    const float recip = 1.0f / range;
    scale[n] = recip * B;
  }
}

int64_t oracle_packed_nbytes(int64_t N, int64_t G, int bits) {
  const int64_t wpt = 8 / bits;
  const int64_t n_round = N + (wpt - N % wpt) % wpt;
  return ((int64_t)bits * n_round * G + 8) / 8; /* quantization_cuda_kernel.cu:107-113 */
}

/* ---- a3: quantise + pack (quantization_cuda_kernel.cu:63-94) -------------
 * noise == NULL: Philox stream (seed, offset).  The accumulator is a uint8_t
 * exactly as `uint8_t local_packed` in the reference, so a value of 2^bits
 * spills into the next field or off the top of the byte the same way. */
void oracle_pack(const float *x, const float *mn, const float *scale, const float *noise,
                 uint64_t seed, uint64_t offset, int64_t N, int64_t G, int bits, uint8_t *packed) {
  const int wpt = 8 / bits;
  const int64_t groups = (N + wpt - 1) / wpt;
#pragma omp parallel for schedule(static)
  for (int64_t no = 0; no < groups; ++no) {
    for (int64_t d0 = 0; d0 < G; d0 += 8) {
      uint8_t local[8] = {0, 0, 0, 0, 0, 0, 0, 0};
      const int cnt = (int)(G - d0 < 8 ? G - d0 : 8);
      for (int ni = 0; ni < wpt; ++ni) {
        const int64_t n = no * wpt + ni;
        if (n >= N) break;
        float u[8];
        if (noise) {
          for (int i = 0; i < cnt; ++i) u[i] = noise[n * G + d0 + i];
        } else {
          philox_oct(seed, offset, (uint32_t)(d0 / 8), (uint32_t)n, u);
        }
        for (int i = 0; i < cnt; ++i) {
          float t = x[n * G + d0 + i] - mn[n];
          t = t * scale[n];
          t = t + u[i];
          t = t - 0.5f;
          t = fmaxf(t, 0.0f);
          const int32_t val = float2int_rn(t);
          local[i] |= (uint8_t)((uint32_t)val << (ni * bits));
        }
      }
      for (int i = 0; i < cnt; ++i) packed[no * G + d0 + i] = local[i];
    }
  }
  packed[oracle_packed_nbytes(N, G, bits) - 1] = 0;
}

/* ---- a5: unpack + dequantise (quantization_cuda_kernel.cu:158-185) ------- */
void oracle_unpack(const uint8_t *packed, int bits, const float *scale, const float *mn, int64_t N,
                   int64_t G, float *out) {
  const int wpt = 8 / bits;
  const int mask = (1 << bits) - 1;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    const int64_t no = n / wpt;
    const int ni = (int)(n % wpt);
    for (int64_t d = 0; d < G; ++d) {
      const int val = (packed[no * G + d] >> (ni * bits)) & mask;
      const float q = (float)val / scale[n];
      out[n * G + d] = q + mn[n];
    }
  }
}

/* bf16 round-to-nearest-even (ops.py:80-81) and widening (ops.py:94-96) */
uint16_t oracle_f32_to_bf16(float f) {
  uint32_t b;
  memcpy(&b, &f, 4);
  if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)(((b >> 16) & 0x8000u) | 0x7FC0u);
  b += 0x7FFFu + ((b >> 16) & 1u);
  return (uint16_t)(b >> 16);
}

/* quantize_activation + dequantize_activation round trip as the reference
 * chains them (ops.py:69-98): min/max, scale, pack, bf16 detour, unpack. */
void oracle_pack_unpack_roundtrip(const float *x, const float *noise, uint64_t seed, uint64_t offset,
                                  int64_t N, int64_t G, int bits, uint8_t *packed, float *mn, float *mx,
                                  float *scale, float *out) {
  oracle_row_minmax(x, N, G, mn, mx);
  oracle_scale(mn, mx, N, bits, scale);
  oracle_pack(x, mn, scale, noise, seed, offset, N, G, bits, packed);
  for (int64_t n = 0; n < N; ++n) {
    uint32_t s = (uint32_t)oracle_f32_to_bf16(scale[n]) << 16, m = (uint32_t)oracle_f32_to_bf16(mn[n]) << 16;
    memcpy(&scale[n], &s, 4);
    memcpy(&mn[n], &m, 4);
  }
  oracle_unpack(packed, bits, scale, mn, N, G, out);
}

/* ---- a13 / a14: 1-bit masks (quantization_cuda_kernel.cu:237-331, 442-594)
 * linear bit order: bit (i % 32) of word (i / 32) <-> element i. */
void oracle_relu_fwd(const float *x, int64_t n, float *y, uint32_t *mask) {
  const int64_t words = (n + 31) / 32;
#pragma omp parallel for schedule(static)
  for (int64_t w = 0; w < words; ++w) {
    uint32_t m = 0;
    for (int j = 0; j < 32; ++j) {
      const int64_t i = w * 32 + j;
      if (i >= n) break;
      const int bit = x[i] > 0.0f;
      y[i] = bit ? x[i] : 0.0f;
      m |= (uint32_t)bit << j;
    }
    mask[w] = m;
  }
}

void oracle_relu_bwd(const float *dy, const uint32_t *mask, int64_t n, float *dx) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) dx[i] = ((mask[i / 32] >> (i % 32)) & 1u) ? dy[i] : 0.0f;
}

void oracle_dropout_fwd(const float *x, const float *noise, uint64_t seed, uint64_t offset, float p,
                        int64_t n, float *y, uint32_t *mask) {
  const float pinv = (float)(1.0 / (1.0 - (double)p)); /* :456 */
  const int64_t words = (n + 31) / 32;
#pragma omp parallel for schedule(static)
  for (int64_t w = 0; w < words; ++w) {
    uint32_t m = 0;
    for (int o = 0; o < 4; ++o) {
      const int64_t oct = w * 4 + o;
      if (oct * 8 >= n) break;
      float u[8];
      if (!noise) philox_oct(seed, offset, (uint32_t)oct, (uint32_t)(oct >> 32), u);
      for (int j = 0; j < 8; ++j) {
        const int64_t i = oct * 8 + j;
        if (i >= n) break;
        const float ui = noise ? noise[i] : u[j];
        const int keep = ui > p; /* :465-468 */
        float r = x[i] * (keep ? 1.0f : 0.0f);
        r = r * pinv; /* :490 */
        y[i] = r;
        m |= (uint32_t)keep << (o * 8 + j);
      }
    }
    mask[w] = m;
  }
}

void oracle_dropout_bwd(const float *dy, const uint32_t *mask, float p, int64_t n, float *dx) {
  const float p1m = (float)(1.0 - (double)p); /* quantization.cc:121,127 */
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) dx[i] = ((mask[i / 32] >> (i % 32)) & 1u) ? dy[i] / p1m : 0.0f;
}

/* ---- a10 / a11: CSR SpMM (spmm_cuda.cu:27-104, reducer.cuh:43-85) --------
 * sequential CSR order, one multiply and one add per term, fp32. */
void oracle_spmm_csr(const int64_t *rowptr, const int64_t *col, const float *val, const float *X,
                     int64_t M, int64_t K, int mean, float *out) {
#pragma omp parallel for schedule(dynamic, 64)
  for (int64_t r = 0; r < M; ++r) {
    float *o = out + r * K;
    for (int64_t k = 0; k < K; ++k) o[k] = 0.0f;
    for (int64_t e = rowptr[r]; e < rowptr[r + 1]; ++e) {
      const float *xr = X + col[e] * K;
      if (val) {
        const float v = val[e];
        for (int64_t k = 0; k < K; ++k) {
          const float term = v * xr[k];
          o[k] = o[k] + term;
        }
      } else {
        for (int64_t k = 0; k < K; ++k) o[k] = o[k] + xr[k];
      }
    }
    if (mean) {
      const int64_t cnt = rowptr[r + 1] - rowptr[r];
      const float c = (float)(cnt > 0 ? cnt : 1); /* reducer.cuh:75-76 */
      for (int64_t k = 0; k < K; ++k) o[k] = o[k] / c;
    }
  }
}

/* ---- a7: random projection (ops.py:107-125), fp32 accumulate ------------- */
void oracle_rp_fwd(const float *X, const float *R, int64_t N, int64_t D, int64_t k, float *out) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    float *o = out + n * k;
    for (int64_t j = 0; j < k; ++j) o[j] = 0.0f;
    for (int64_t d = 0; d < D; ++d) {
      const float xv = X[n * D + d];
      const float *r = R + d * k;
      for (int64_t j = 0; j < k; ++j) o[j] += xv * r[j];
    }
  }
}

void oracle_rp_bwd(const float *Xr, const float *R, int64_t N, int64_t D, int64_t k, float *out) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; ++n) {
    for (int64_t d = 0; d < D; ++d) {
      float acc = 0.0f;
      for (int64_t j = 0; j < k; ++j) acc += Xr[n * k + j] * R[d * k + j];
      out[n * D + d] = acc;
    }
  }
}

/* ---- division identity used by the GPU unpack kernel ---------------------
 * Counts the (significand of s, q) pairs, over ALL 2^23 significands at the
 * given biased exponent and q = 0..255, for which
 *   y = RN(q r), e = fma(-y, s, q), RN(y + e r)   with r = RN(1 / s)
 * differs from the IEEE quotient q / s.  The kernel relies on the answer
 * being 0; tests/test_oracle.py runs this. */
int64_t oracle_count_fast_division_mismatches(int biased_exponent) {
  int64_t bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (int64_t m = 0; m < (1 << 23); ++m) {
    const uint32_t bits = ((uint32_t)biased_exponent << 23) | (uint32_t)m;
    float s;
    memcpy(&s, &bits, 4);
    const float r = 1.0f / s;
    for (int q = 0; q <= 255; ++q) {
      const float qf = (float)q;
      const float y = qf * r;
      const float e = fmaf(-y, s, qf);
      const float got = fmaf(e, r, y);
      const float want = qf / s;
      bad += memcmp(&got, &want, 4) != 0;
    }
  }
  return bad;
}
