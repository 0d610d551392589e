// AddressSanitizer driver for the SIMT-emulated kernels (TESTS ONLY).
//
// Calls every C-ABI entry point on heap buffers of EXACTLY the documented
// sizes, so that any out-of-bounds load or store of a kernel is reported by
// ASan, and compares the results with the C oracle.  Usage:
//     emu_check [quick|large|full|rp]
// `large` adds grids of thousands of workgroups (20011 x 256, a 20000-node
// graph; minutes); `full` adds the benchmark shapes (169343 x 256 and a
// 169343-node graph; hours under the sanitizer).
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "../../include/exact_hip.h"

extern "C" {
void oracle_row_minmax(const float*, int64_t, int64_t, float*, float*);
void oracle_scale(const float*, const float*, int64_t, int, float*);
void oracle_pack(const float*, const float*, const float*, const float*, uint64_t, uint64_t, int64_t, int64_t, int,
                 uint8_t*);
void oracle_unpack(const uint8_t*, int, const float*, const float*, int64_t, int64_t, float*);
uint16_t oracle_f32_to_bf16(float);
void oracle_relu_fwd(const float*, int64_t, float*, uint32_t*);
void oracle_relu_bwd(const float*, const uint32_t*, int64_t, float*);
void oracle_dropout_fwd(const float*, const float*, uint64_t, uint64_t, float, int64_t, float*, uint32_t*);
void oracle_dropout_bwd(const float*, const uint32_t*, float, int64_t, float*);
void oracle_spmm_csr(const int64_t*, const int64_t*, const float*, const float*, int64_t, int64_t, int, float*);
void oracle_rp_fwd(const float*, const float*, int64_t, int64_t, int64_t, float*);
void oracle_rp_bwd(const float*, const float*, int64_t, int64_t, int64_t, float*);
}

static int g_fail = 0;
#define CHECK(cond, ...)                                   \
  do {                                                     \
    if (!(cond)) {                                         \
      std::fprintf(stderr, "FAIL %s:%d: ", __FILE__, __LINE__); \
      std::fprintf(stderr, __VA_ARGS__);                   \
      std::fprintf(stderr, "\n");                          \
      ++g_fail;                                            \
    }                                                      \
  } while (0)

// malloc'd, exactly sized: ASan puts red zones right behind the last element
template <typename T>
struct Buf {
  T* p;
  size_t n;
  explicit Buf(size_t n_) : p(static_cast<T*>(std::malloc(n_ ? n_ * sizeof(T) : 1))), n(n_) {}
  ~Buf() { std::free(p); }
  T& operator[](size_t i) { return p[i]; }
};

static void check_quant(int64_t N, int64_t G, int bits, bool supplied, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 2.f);
  std::uniform_real_distribution<float> ud(0.f, 1.f);
  Buf<float> x(N * G), u(N * G), mn(N), mx(N), sc(N), mn2(N), sc2(N), out(N * G), want_out(N * G);
  for (int64_t i = 0; i < N * G; ++i) { x[i] = nd(rng); u[i] = ud(rng); if (u[i] >= 1.f) u[i] = 0.5f; }
  const int64_t nb = exact_packed_nbytes(N, G, bits);
  Buf<uint8_t> packed(nb), want(nb), packed2(nb);
  Buf<uint16_t> sbf(N), mbf(N);
  const uint64_t seed = 0x1234abcd5678ull, off = (5ull << 32) + 17;
  oracle_row_minmax(x.p, N, G, mn.p, mx.p);
  oracle_scale(mn.p, mx.p, N, bits, sc.p);
  std::memset(want.p, 0, nb);
  oracle_pack(x.p, mn.p, sc.p, supplied ? u.p : nullptr, seed, off, N, G, bits, want.p);
  int rc = exact_minmax_pack_f32(x.p, supplied ? u.p : nullptr, seed, off, N, G, bits, packed.p, sc2.p, mn2.p, sbf.p,
                                 mbf.p, nullptr);
  CHECK(rc == 0, "minmax_pack rc=%d", rc);
  CHECK(std::memcmp(packed.p, want.p, nb) == 0, "packed bytes differ N=%ld G=%ld bits=%d supplied=%d", (long)N, (long)G, bits, supplied);
  CHECK(std::memcmp(sc2.p, sc.p, N * 4) == 0 && std::memcmp(mn2.p, mn.p, N * 4) == 0, "scale/min differ N=%ld G=%ld", (long)N, (long)G);
  rc = exact_pack_f32(x.p, mn.p, sc.p, supplied ? u.p : nullptr, seed, off, N, G, bits, packed2.p, nullptr);
  CHECK(rc == 0 && std::memcmp(packed2.p, want.p, nb) == 0, "two-step pack differs N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  // unpack with bf16 parameters
  Buf<float> scw(N), mnw(N);
  for (int64_t n = 0; n < N; ++n) {
    CHECK(sbf[n] == oracle_f32_to_bf16(sc[n]) && mbf[n] == oracle_f32_to_bf16(mn[n]), "bf16 params differ row %ld", (long)n);
    uint32_t a = (uint32_t)sbf[n] << 16, b = (uint32_t)mbf[n] << 16;
    std::memcpy(&scw[n], &a, 4);
    std::memcpy(&mnw[n], &b, 4);
  }
  oracle_unpack(want.p, bits, scw.p, mnw.p, N, G, want_out.p);
  rc = exact_unpack_bf16param_f32(packed.p, bits, sbf.p, mbf.p, N, G, out.p, nullptr);
  CHECK(rc == 0 && std::memcmp(out.p, want_out.p, N * G * 4) == 0, "unpack(bf16) differs N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  oracle_unpack(want.p, bits, sc.p, mn.p, N, G, want_out.p);
  rc = exact_unpack_f32(packed.p, bits, sc.p, mn.p, N, G, out.p, nullptr);
  CHECK(rc == 0 && std::memcmp(out.p, want_out.p, N * G * 4) == 0, "unpack(f32) differs N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  Buf<float> rmn(N), rmx(N);
  rc = exact_row_minmax_f32(x.p, N, G, rmn.p, rmx.p, nullptr);
  CHECK(rc == 0 && std::memcmp(rmn.p, mn.p, N * 4) == 0 && std::memcmp(rmx.p, mx.p, N * 4) == 0, "row_minmax differs");
}

static void check_masks(int64_t n, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 1.f);
  std::uniform_real_distribution<float> ud(0.f, 1.f);
  const int64_t words = (n + 31) / 32;
  Buf<float> x(n), u(n), g(n), y(n), wy(n), dx(n), wdx(n);
  Buf<uint32_t> m(words), wm(words);
  for (int64_t i = 0; i < n; ++i) { x[i] = nd(rng); u[i] = ud(rng); g[i] = nd(rng); }
  oracle_relu_fwd(x.p, n, wy.p, wm.p);
  CHECK(exact_relu_fwd_f32(x.p, n, y.p, m.p, nullptr) == 0, "relu rc");
  CHECK(std::memcmp(y.p, wy.p, n * 4) == 0 && std::memcmp(m.p, wm.p, words * 4) == 0, "relu fwd differs n=%ld", (long)n);
  oracle_relu_bwd(g.p, wm.p, n, wdx.p);
  CHECK(exact_relu_bwd_f32(g.p, m.p, n, dx.p, nullptr) == 0 && std::memcmp(dx.p, wdx.p, n * 4) == 0, "relu bwd differs n=%ld", (long)n);
  for (int mode = 0; mode < 2; ++mode) {
    const float p = mode ? 0.1f : 0.5f;
    const float* noise = mode ? nullptr : u.p;
    oracle_dropout_fwd(x.p, noise, 99, 7, p, n, wy.p, wm.p);
    CHECK(exact_dropout_fwd_f32(x.p, noise, 99, 7, p, n, y.p, m.p, nullptr) == 0, "dropout rc");
    CHECK(std::memcmp(y.p, wy.p, n * 4) == 0 && std::memcmp(m.p, wm.p, words * 4) == 0, "dropout fwd differs n=%ld mode=%d", (long)n, mode);
    oracle_dropout_bwd(g.p, wm.p, p, n, wdx.p);
    CHECK(exact_dropout_bwd_f32(g.p, m.p, p, n, dx.p, nullptr) == 0 && std::memcmp(dx.p, wdx.p, n * 4) == 0, "dropout bwd differs n=%ld", (long)n);
  }
}

struct Csr {
  std::vector<int64_t> rowptr, col;
  std::vector<float> val;
};

static Csr powerlaw(int64_t M, int64_t ncols, double avg, int64_t hub, std::mt19937& rng) {
  Csr g;
  g.rowptr.assign(M + 1, 0);
  std::uniform_real_distribution<double> ud(0.0, 1.0);
  std::normal_distribution<float> nd(0.f, 1.f);
  for (int64_t r = 0; r < M; ++r) {
    // Pareto-tailed degree with the requested mean-ish, some empty rows
    double d = avg * 0.5 / std::pow(1.0 - ud(rng), 1.0 / 1.3);
    int64_t deg = ud(rng) < 0.02 ? 0 : std::min<int64_t>((int64_t)d, ncols);
    if (hub && (r == M / 3 || r == M / 2)) deg = std::min(hub, ncols);
    g.rowptr[r + 1] = g.rowptr[r] + deg;
    for (int64_t i = 0; i < deg; ++i) {
      g.col.push_back((int64_t)(ud(rng) * ncols) % ncols);
      g.val.push_back(nd(rng));
    }
  }
  return g;
}

static void check_spmm(int64_t M, int64_t ncols, int64_t K, double avg, int64_t hub, std::mt19937& rng) {
  const Csr g = powerlaw(M, ncols, avg, hub, rng);
  const int64_t nnz = (int64_t)g.col.size();
  std::normal_distribution<float> nd(0.f, 1.f);
  Buf<float> X(ncols * K), out(M * K), want(M * K), val(nnz);
  Buf<int64_t> rp64(M + 1), col64(nnz);
  Buf<int32_t> rp32(M + 1), col32(nnz);
  for (int64_t i = 0; i < ncols * K; ++i) X[i] = nd(rng);
  for (int64_t i = 0; i <= M; ++i) { rp64[i] = g.rowptr[i]; rp32[i] = (int32_t)g.rowptr[i]; }
  for (int64_t i = 0; i < nnz; ++i) { col64[i] = g.col[i]; col32[i] = (int32_t)g.col[i]; val[i] = g.val[i]; }
  for (int reduce = 0; reduce < 2; ++reduce)
    for (int valued = 0; valued < 2; ++valued)
      for (int wide = 0; wide < 2; ++wide) {
        oracle_spmm_csr(rp64.p, col64.p, valued ? val.p : nullptr, X.p, M, K, reduce, want.p);
        const int rc = wide ? exact_spmm_csr_f32(rp64.p, col64.p, valued ? val.p : nullptr, 8, X.p, M, ncols, K, nnz, reduce, out.p, nullptr)
                            : exact_spmm_csr_f32(rp32.p, col32.p, valued ? val.p : nullptr, 4, X.p, M, ncols, K, nnz, reduce, out.p, nullptr);
        CHECK(rc == 0, "spmm rc=%d", rc);
        double worst = 0, scale = 1e-30;
        for (int64_t i = 0; i < M * K; ++i) scale = std::max(scale, (double)std::fabs(want[i]));
        for (int64_t i = 0; i < M * K; ++i) worst = std::max(worst, (double)std::fabs(out[i] - want[i]));
        CHECK(worst <= 1e-5 * scale, "spmm differs M=%ld K=%ld reduce=%d valued=%d wide=%d: %g of %g", (long)M, (long)K, reduce, valued, wide, worst, scale);
        // the reproducible kernel sums in the oracle's order: bit-identical
        const int rc2 = wide ? exact_spmm_csr_rowwise_f32(rp64.p, col64.p, valued ? val.p : nullptr, 8, X.p, M, ncols, K, nnz, reduce, out.p, nullptr)
                             : exact_spmm_csr_rowwise_f32(rp32.p, col32.p, valued ? val.p : nullptr, 4, X.p, M, ncols, K, nnz, reduce, out.p, nullptr);
        CHECK(rc2 == 0 && std::memcmp(out.p, want.p, M * K * 4) == 0, "rowwise spmm differs M=%ld K=%ld reduce=%d valued=%d wide=%d", (long)M, (long)K, reduce, valued, wide);
      }
}

// mode 0: the fp32 instruction; EXACT_RP_BF16_SPLIT on a Gaussian matrix; EXACT_RP_BF16_SIGNS on a +-c matrix
static int rp_fwd_any(int mode, const float* X, const float* R, const void* table, int64_t N, int64_t D, int64_t k, float* out) {
  return mode == 0 ? exact_rp_fwd_f32(X, R, N, D, k, out, nullptr) : exact_rp_fwd_bf16_f32(X, table, N, D, k, mode, out, nullptr);
}
static int rp_bwd_any(int mode, const float* Xr, const float* R, const void* table, int64_t N, int64_t D, int64_t k, float* out) {
  return mode == 0 ? exact_rp_bwd_f32(Xr, R, N, D, k, out, nullptr) : exact_rp_bwd_bf16_f32(Xr, table, N, D, k, mode, out, nullptr);
}

static void check_rp_mode(int mode, int64_t N, int64_t D, int64_t k, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 1.f);
  Buf<float> X(N * D), R(D * k), xr(N * k), wxr(N * k), back(N * D), wback(N * D);
  for (int64_t i = 0; i < N * D; ++i) X[i] = nd(rng);
  const float c = 1.f / std::sqrt((float)k);
  for (int64_t i = 0; i < D * k; ++i) R[i] = mode == EXACT_RP_BF16_SIGNS ? ((rng() & 1) ? c : -c) : nd(rng) * c;
  // the fragment table of the bf16 paths, on a heap buffer of exactly the documented size
  const int64_t tbytes = mode == 0 ? 16 : exact_rp_table_nbytes(D, k, mode);
  CHECK(tbytes > 0 && tbytes % 16 == 0, "rp table size");
  Buf<uint32_t> table(tbytes / 4);
  if (mode != 0) CHECK(exact_rp_prepare_bf16(R.p, D, k, mode, table.p, nullptr) == 0, "rp prepare rc");
  oracle_rp_fwd(X.p, R.p, N, D, k, wxr.p);
  CHECK(rp_fwd_any(mode, X.p, R.p, table.p, N, D, k, xr.p) == 0, "rp fwd rc");
  double worst = 0, scale = 1e-30;
  for (int64_t i = 0; i < N * k; ++i) { scale = std::max(scale, (double)std::fabs(wxr[i])); worst = std::max(worst, (double)std::fabs(xr[i] - wxr[i])); }
  CHECK(worst <= 2e-5 * scale, "rp fwd differs mode=%d N=%ld D=%ld k=%ld: %g of %g", mode, (long)N, (long)D, (long)k, worst, scale);
  oracle_rp_bwd(wxr.p, R.p, N, D, k, wback.p);
  CHECK(rp_bwd_any(mode, wxr.p, R.p, table.p, N, D, k, back.p) == 0, "rp bwd rc");
  worst = 0, scale = 1e-30;
  for (int64_t i = 0; i < N * D; ++i) { scale = std::max(scale, (double)std::fabs(wback[i])); worst = std::max(worst, (double)std::fabs(back[i] - wback[i])); }
  CHECK(worst <= 2e-5 * scale, "rp bwd differs mode=%d N=%ld D=%ld k=%ld: %g of %g", mode, (long)N, (long)D, (long)k, worst, scale);
  // projection + quantisation in one launch == the oracle's quantiser on the kernel's own product
  std::uniform_real_distribution<float> ud(0.f, 1.f);
  Buf<float> u(N * k), mn(N), mx(N), sc(N), mn2(N), sc2(N);
  for (int64_t i = 0; i < N * k; ++i) { u[i] = ud(rng); if (u[i] >= 1.f) u[i] = 0.5f; }
  oracle_row_minmax(xr.p, N, k, mn.p, mx.p);
  for (int bits : {1, 2, 4, 8}) {
    const bool supplied = bits == 2 || bits == 8;
    const int64_t nb = exact_packed_nbytes(N, k, bits);
    Buf<uint8_t> packed(nb), want(nb);
    Buf<uint16_t> sbf(N), mbf(N);
    oracle_scale(mn.p, mx.p, N, bits, sc.p);
    std::memset(want.p, 0, nb);
    oracle_pack(xr.p, mn.p, sc.p, supplied ? u.p : nullptr, 0x99ull, (7ull << 32) + 16, N, k, bits, want.p);
    std::memset(packed.p, 0xEE, nb);
    const int rc = mode == 0
        ? exact_rp_minmax_pack_f32(X.p, R.p, supplied ? u.p : nullptr, 0x99ull, (7ull << 32) + 16, N, D, k, bits,
                                   packed.p, sc2.p, mn2.p, sbf.p, mbf.p, nullptr)
        : exact_rp_minmax_pack_bf16_f32(X.p, table.p, mode, supplied ? u.p : nullptr, 0x99ull, (7ull << 32) + 16, N, D, k, bits,
                                        packed.p, sc2.p, mn2.p, sbf.p, mbf.p, nullptr);
    CHECK(rc == 0 && std::memcmp(packed.p, want.p, nb) == 0, "rp+pack packed differs mode=%d N=%ld D=%ld k=%ld bits=%d rc=%d",
          mode, (long)N, (long)D, (long)k, bits, rc);
    CHECK(std::memcmp(sc2.p, sc.p, N * 4) == 0 && std::memcmp(mn2.p, mn.p, N * 4) == 0, "rp+pack scale/min differ mode=%d N=%ld k=%ld", mode, (long)N, (long)k);
  }
}

static void check_rp(int64_t N, int64_t D, int64_t k, std::mt19937& rng) {
  for (int mode : {0, EXACT_RP_BF16_SPLIT, EXACT_RP_BF16_SIGNS}) check_rp_mode(mode, N, D, k, rng);
}

// LeakyReLU mask, max / min aggregation and the edge-value gradient, against
// straight loops written here (the Python oracle for them is
// oracle/exact_oracle_extra.py, checked by tests/test_more_ops.py).
static void check_extra(int64_t M, int64_t ncols, int64_t K, double avg, std::mt19937& rng) {
  const Csr g = powerlaw(M, ncols, avg, 0, rng);
  const int64_t nnz = (int64_t)g.col.size();
  std::normal_distribution<float> nd(0.f, 1.f);
  Buf<float> X(ncols * K), grad(M * K), out(M * K), val(nnz), ev(nnz);
  Buf<int64_t> rp64(M + 1), col64(nnz), row64(nnz), arg64(M * K);
  Buf<int32_t> rp32(M + 1), col32(nnz), row32(nnz), arg32(M * K);
  for (int64_t i = 0; i < ncols * K; ++i) X[i] = nd(rng);
  for (int64_t i = 0; i < M * K; ++i) grad[i] = nd(rng);
  for (int64_t i = 0; i <= M; ++i) { rp64[i] = g.rowptr[i]; rp32[i] = (int32_t)g.rowptr[i]; }
  for (int64_t r = 0; r < M; ++r)
    for (int64_t e = g.rowptr[r]; e < g.rowptr[r + 1]; ++e) { row64[e] = r; row32[e] = (int32_t)r; }
  for (int64_t i = 0; i < nnz; ++i) { col64[i] = g.col[i]; col32[i] = (int32_t)g.col[i]; val[i] = g.val[i]; }
  for (int is_max = 0; is_max < 2; ++is_max)
    for (int valued = 0; valued < 2; ++valued)
      for (int wide = 0; wide < 2; ++wide) {
        const float* v = valued ? val.p : nullptr;
        const int rc = wide ? exact_spmm_csr_minmax_f32(rp64.p, col64.p, v, 8, X.p, M, ncols, K, nnz, is_max, out.p, arg64.p, nullptr)
                            : exact_spmm_csr_minmax_f32(rp32.p, col32.p, v, 4, X.p, M, ncols, K, nnz, is_max, out.p, arg32.p, nullptr);
        CHECK(rc == 0, "minmax rc=%d", rc);
        int64_t bad = 0;
        for (int64_t r = 0; r < M; ++r)
          for (int64_t k = 0; k < K; ++k) {
            float best = 0.f;
            int64_t arg = nnz;
            for (int64_t e = g.rowptr[r]; e < g.rowptr[r + 1]; ++e) {
              const float t = valued ? g.val[e] * X[g.col[e] * K + k] : X[g.col[e] * K + k];
              if (arg == nnz || (is_max ? t > best : t < best)) { best = t; arg = e; }
            }
            const int64_t got = wide ? arg64[r * K + k] : (int64_t)arg32[r * K + k];
            bad += (out[r * K + k] != best) || (got != arg);
          }
        CHECK(bad == 0, "minmax differs M=%ld K=%ld max=%d valued=%d wide=%d: %ld cells", (long)M, (long)K, is_max, valued, wide, (long)bad);
      }
  for (int reduce = 0; reduce < 2; ++reduce)
    for (int wide = 0; wide < 2; ++wide) {
      const int rc = wide ? exact_sddmm_f32(row64.p, rp64.p, col64.p, 8, X.p, grad.p, nnz, K, reduce, ev.p, nullptr)
                          : exact_sddmm_f32(row32.p, rp32.p, col32.p, 4, X.p, grad.p, nnz, K, reduce, ev.p, nullptr);
      CHECK(rc == 0, "sddmm rc=%d", rc);
      double worst = 0, scale = 1e-30;
      for (int64_t r = 0; r < M; ++r)
        for (int64_t e = g.rowptr[r]; e < g.rowptr[r + 1]; ++e) {
          double acc = 0;
          for (int64_t k = 0; k < K; ++k) acc += (double)X[g.col[e] * K + k] * (double)grad[r * K + k];
          if (reduce) acc /= (double)std::max<int64_t>(g.rowptr[r + 1] - g.rowptr[r], 1);
          scale = std::max(scale, std::fabs(acc));
          worst = std::max(worst, std::fabs(acc - (double)ev[e]));
        }
      CHECK(worst <= 1e-5 * scale, "sddmm differs M=%ld K=%ld reduce=%d wide=%d: %g of %g", (long)M, (long)K, reduce, wide, worst, scale);
    }
}

static void check_leaky(int64_t n, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 1.f);
  const int64_t words = (n + 31) / 32;
  Buf<float> x(n), g(n), y(n), dx(n);
  Buf<uint32_t> m(words);
  for (int64_t i = 0; i < n; ++i) { x[i] = nd(rng); g[i] = nd(rng); }
  const float slope = 0.2f;
  CHECK(exact_leaky_relu_fwd_f32(x.p, n, slope, y.p, m.p, nullptr) == 0, "leaky rc");
  CHECK(exact_leaky_relu_bwd_f32(g.p, m.p, n, slope, dx.p, nullptr) == 0, "leaky bwd rc");
  int64_t bad = 0;
  for (int64_t i = 0; i < n; ++i) {
    const bool pos = x[i] > 0.f;
    bad += y[i] != (pos ? x[i] : x[i] * slope);
    bad += ((m[i / 32] >> (i % 32)) & 1u) != (pos ? 1u : 0u);
    bad += dx[i] != (pos ? g[i] : g[i] * slope);
  }
  for (int64_t i = n; i < words * 32; ++i) bad += (m[i / 32] >> (i % 32)) & 1u;  // tail bits are written as 0
  CHECK(bad == 0, "leaky relu differs n=%ld: %ld", (long)n, (long)bad);
  // ELU derivative on the same data
  CHECK(exact_elu_bwd_f32(g.p, x.p, 1.3f, n, dx.p, nullptr) == 0, "elu bwd rc");
  bad = 0;
  for (int64_t i = 0; i < n; ++i) {
    const float want = x[i] >= 0.f ? g[i] : (1.3f * g[i]) * std::exp(x[i]);
    bad += std::fabs(dx[i] - want) > 4e-7f * std::fabs(want);
  }
  CHECK(bad == 0, "elu backward differs n=%ld: %ld", (long)n, (long)bad);
}

// ReLU -> dropout (-> statistics + pack) in one pass against the chain of the
// oracle's separate functions.
static void check_fused(int64_t N, int64_t G, int bits, bool supplied, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 2.f);
  std::uniform_real_distribution<float> ud(0.f, 1.f);
  const int64_t n = N * G, words = (n + 31) / 32;
  Buf<float> x(n), ua(n), uq(n), y1(n), y2(n), y(n), mn(N), mx(N), sc(N), mn2(N), sc2(N);
  Buf<uint32_t> m1(words), m2(words), m(words);
  for (int64_t i = 0; i < n; ++i) {
    x[i] = nd(rng); ua[i] = ud(rng); uq[i] = ud(rng);
    if (ua[i] >= 1.f) ua[i] = 0.5f;
    if (uq[i] >= 1.f) uq[i] = 0.5f;
  }
  const float p = 0.4f;
  const uint64_t s1 = 0x51ull, o1 = 8, s2 = 0x77ull, o2 = (3ull << 32) + 12;
  oracle_relu_fwd(x.p, n, y1.p, m1.p);
  oracle_dropout_fwd(y1.p, supplied ? ua.p : nullptr, s1, o1, p, n, y2.p, m2.p);
  const int64_t nb = exact_packed_nbytes(N, G, bits);
  Buf<uint8_t> packed(nb), want(nb);
  Buf<uint16_t> sbf(N), mbf(N);
  oracle_row_minmax(y2.p, N, G, mn.p, mx.p);
  oracle_scale(mn.p, mx.p, N, bits, sc.p);
  std::memset(want.p, 0, nb);
  oracle_pack(y2.p, mn.p, sc.p, supplied ? uq.p : nullptr, s2, o2, N, G, bits, want.p);
  int rc = exact_relu_dropout_fwd_f32(x.p, supplied ? ua.p : nullptr, s1, o1, p, n, y.p, m.p, nullptr);
  int64_t bad = 0;
  for (int64_t i = 0; i < words; ++i) bad += m[i] != (m1[i] & m2[i]);
  CHECK(rc == 0 && std::memcmp(y.p, y2.p, n * 4) == 0 && bad == 0, "relu_dropout differs N=%ld G=%ld", (long)N, (long)G);
  if (G % 8 != 0 || G > 1024) return;
  std::memset(y.p, 0xFF, n * 4);
  std::memset(m.p, 0xFF, words * 4);
  rc = exact_relu_dropout_minmax_pack_f32(x.p, p, supplied ? ua.p : nullptr, s1, o1, supplied ? uq.p : nullptr, s2, o2,
                                          N, G, bits, y.p, m.p, packed.p, sc2.p, mn2.p, sbf.p, mbf.p, nullptr);
  bad = 0;
  for (int64_t i = 0; i < words; ++i) bad += m[i] != (m1[i] & m2[i]);
  CHECK(rc == 0 && std::memcmp(y.p, y2.p, n * 4) == 0 && bad == 0, "fused y/mask differ N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  CHECK(std::memcmp(packed.p, want.p, nb) == 0, "fused packed differs N=%ld G=%ld bits=%d supplied=%d", (long)N, (long)G, bits, supplied);
  CHECK(std::memcmp(sc2.p, sc.p, N * 4) == 0 && std::memcmp(mn2.p, mn.p, N * 4) == 0, "fused scale/min differ N=%ld G=%ld", (long)N, (long)G);
  // with batch norm ahead: the same chain on (x - mean) * mult + shift, three roundings
  Buf<float> mean(G), mult(G), shift(G), xn(n);
  for (int64_t d = 0; d < G; ++d) { mean[d] = nd(rng); mult[d] = 0.5f + ud(rng); shift[d] = 0.25f * nd(rng); }
  for (int64_t i = 0; i < n; ++i) {
    volatile float c = x[i] - mean[i % G];
    c = c * mult[i % G];
    xn[i] = c + shift[i % G];
  }
  oracle_relu_fwd(xn.p, n, y1.p, m1.p);
  oracle_dropout_fwd(y1.p, supplied ? ua.p : nullptr, s1, o1, p, n, y2.p, m2.p);
  oracle_row_minmax(y2.p, N, G, mn.p, mx.p);
  oracle_scale(mn.p, mx.p, N, bits, sc.p);
  std::memset(want.p, 0, nb);
  oracle_pack(y2.p, mn.p, sc.p, supplied ? uq.p : nullptr, s2, o2, N, G, bits, want.p);
  std::memset(y.p, 0xFF, n * 4);
  std::memset(m.p, 0xFF, words * 4);
  rc = exact_bn_relu_dropout_minmax_pack_f32(x.p, mean.p, mult.p, shift.p, p, supplied ? ua.p : nullptr, s1, o1,
                                             supplied ? uq.p : nullptr, s2, o2, N, G, bits, y.p, m.p, packed.p, sc2.p,
                                             mn2.p, sbf.p, mbf.p, nullptr);
  bad = 0;
  for (int64_t i = 0; i < words; ++i) bad += m[i] != (m1[i] & m2[i]);
  CHECK(rc == 0 && std::memcmp(y.p, y2.p, n * 4) == 0 && bad == 0, "bn fused y/mask differ N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  CHECK(std::memcmp(packed.p, want.p, nb) == 0, "bn fused packed differs N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  CHECK(std::memcmp(sc2.p, sc.p, N * 4) == 0 && std::memcmp(mn2.p, mn.p, N * 4) == 0, "bn fused scale/min differ N=%ld G=%ld", (long)N, (long)G);
}

// fp16 entry points against straight loops written here with _Float16 (the
// Python oracle for them is oracle/exact_oracle_half.py, checked by
// tests/test_half_kernels.py); supplied noise only.
static float rh(float x) { return (float)(_Float16)x; }

static void check_half(int64_t N, int64_t G, int bits, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 3.f);
  std::uniform_real_distribution<float> ud(0.f, 1.f);
  const int64_t n = N * G, words = (n + 31) / 32;
  Buf<_Float16> x(n), out(n), y(n), dx(n);
  Buf<float> u(n);
  for (int64_t i = 0; i < n; ++i) { x[i] = (_Float16)nd(rng); u[i] = ud(rng); if (u[i] >= 1.f) u[i] = 0.5f; }
  const int64_t nb = exact_packed_nbytes(N, G, bits);
  Buf<uint8_t> packed(nb), want(nb);
  Buf<_Float16> sc(N), mn(N);
  int rc = exact_minmax_pack_f16((const uint16_t*)x.p, u.p, 1, 2, N, G, bits, packed.p, (uint16_t*)sc.p, (uint16_t*)mn.p, nullptr);
  CHECK(rc == 0, "pack f16 rc=%d", rc);
  std::memset(want.p, 0, nb);
  const int wpt = 8 / bits;
  int64_t bad = 0;
  for (int64_t r = 0; r < N; ++r) {
    float lo = INFINITY, hi = -INFINITY;
    for (int64_t d = 0; d < G; ++d) { lo = std::fmin(lo, (float)x[r * G + d]); hi = std::fmax(hi, (float)x[r * G + d]); }
    const float s = rh(rh(1.0f / rh(hi - lo)) * (float)((1 << bits) - 1));
    bad += ((float)sc[r] != s && !(std::isnan(s) && std::isnan((float)sc[r]))) || (float)mn[r] != lo;
    for (int64_t d = 0; d < G; ++d) {
      float t = rh(rh((float)x[r * G + d] - lo) * s);
      t = t + u[r * G + d];
      t = t - 0.5f;
      t = std::fmax(t, 0.f);
      const int q = (int)std::nearbyint(t);
      want[(r / wpt) * G + d] |= (uint8_t)(q << ((r % wpt) * bits));
    }
  }
  CHECK(bad == 0, "f16 scale/min differ N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  CHECK(std::memcmp(packed.p, want.p, nb) == 0, "f16 packed differs N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
  rc = exact_unpack_f16(packed.p, bits, (const uint16_t*)sc.p, (const uint16_t*)mn.p, N, G, (uint16_t*)out.p, nullptr);
  bad = 0;
  for (int64_t r = 0; r < N; ++r)
    for (int64_t d = 0; d < G; ++d) {
      const int q = (want[(r / wpt) * G + d] >> ((r % wpt) * bits)) & ((1 << bits) - 1);
      const _Float16 w = (_Float16)(rh((float)q / (float)sc[r]) + (float)mn[r]);
      const _Float16 g = out[r * G + d];
      bad += std::memcmp(&w, &g, 2) != 0 && !(std::isnan((float)w) && std::isnan((float)g));
    }
  CHECK(rc == 0 && bad == 0, "f16 unpack differs N=%ld G=%ld bits=%d: %ld", (long)N, (long)G, bits, (long)bad);
  // masks
  Buf<uint32_t> m(words);
  const float p = 0.3f, pinv = (float)(1.0 / (1.0 - (double)p)), p1m = (float)(1.0 - (double)p);
  rc = exact_relu_dropout_fwd_f16((const uint16_t*)x.p, u.p, 0, 0, p, n, (uint16_t*)y.p, m.p, nullptr);
  rc |= exact_dropout_bwd_f16((const uint16_t*)x.p, m.p, p, n, (uint16_t*)dx.p, nullptr);
  bad = 0;
  for (int64_t i = 0; i < n; ++i) {
    const bool pos = (float)x[i] > 0.f, keep = u[i] > p;
    const _Float16 wy = (_Float16)(((pos ? (float)x[i] : 0.f) * (keep ? 1.f : 0.f)) * pinv);
    const _Float16 wdx = (pos && keep) ? (_Float16)((float)x[i] / p1m) : (_Float16)0.f;
    bad += (float)y[i] != (float)wy || (float)dx[i] != (float)wdx || (((m[i / 32] >> (i % 32)) & 1u) != (uint32_t)(pos && keep));
  }
  CHECK(rc == 0 && bad == 0, "f16 relu+dropout differs n=%ld: %ld", (long)n, (long)bad);
  rc = exact_relu_fwd_f16((const uint16_t*)x.p, n, (uint16_t*)y.p, m.p, nullptr);
  rc |= exact_leaky_relu_fwd_f16((const uint16_t*)x.p, n, 0.2f, (uint16_t*)y.p, m.p, nullptr);
  rc |= exact_leaky_relu_bwd_f16((const uint16_t*)x.p, m.p, n, 0.2f, (uint16_t*)dx.p, nullptr);
  rc |= exact_relu_bwd_f16((const uint16_t*)x.p, m.p, n, (uint16_t*)dx.p, nullptr);
  rc |= exact_dropout_fwd_f16((const uint16_t*)x.p, nullptr, 3, 4, p, n, (uint16_t*)y.p, m.p, nullptr);
  CHECK(rc == 0, "f16 mask entry points rc=%d", rc);
}

// the traffic probe: exactly sized buffers, the folded words recomputed here
static void check_probe(int64_t n, std::mt19937& rng) {
  std::normal_distribution<float> nd(0.f, 1.f);
  Buf<float> x(n);
  for (int64_t i = 0; i < n; ++i) x[i] = nd(rng);
  const int64_t tiles = n / 4096, lanes = tiles * 256;
  std::vector<uint32_t> w(lanes);
  for (int64_t L = 0; L < lanes; ++L) {
    uint32_t v = 0;
    for (int u = 0; u < 4; ++u)
      for (int c = 0; c < 4; ++c) {
        uint32_t b;
        std::memcpy(&b, &x[((L / 256) * 1024 + u * 256 + L % 256) * 4 + c], 4);
        v ^= b;
      }
    w[L] = v;
  }
  for (int ob : {0, 2, 4, 8, 16}) {
    const int64_t nb = std::max<int64_t>(16, (n / 16) * ob);
    Buf<uint8_t> out(nb);
    std::memset(out.p, 0xA5, nb);
    CHECK(exact_stream_probe_f32(x.p, n, ob, out.p, nullptr) == 0, "probe rc n=%ld ob=%d", (long)n, ob);
    bool ok = true;
    for (int64_t L = 0; L < lanes && ob >= 4; ++L) { uint32_t g; std::memcpy(&g, out.p + L * ob, 4); ok = ok && g == w[L]; }
    for (int64_t L = 0; L < lanes && ob == 2; ++L) { uint16_t g; std::memcpy(&g, out.p + L * 2, 2); ok = ok && g == (uint16_t)w[L]; }
    for (int64_t i = lanes * ob; i < nb; ++i) ok = ok && out[i] == 0xA5;
    CHECK(ok, "probe output differs n=%ld ob=%d", (long)n, ob);
  }
}

static void check_colsum(int64_t N, int64_t K, std::mt19937& rng) {
  std::uniform_int_distribution<int> id(-8, 8);
  Buf<float> x(static_cast<size_t>(N * K)), out(static_cast<size_t>(K));
  std::vector<double> want(static_cast<size_t>(K), 0.0);
  for (int64_t i = 0; i < N * K; ++i) {
    x[i] = static_cast<float>(id(rng));
    want[static_cast<size_t>(i % K)] += x[i];
  }
  const int rc = exact_colsum_f32(x.p, N, K, out.p, nullptr);
  CHECK(rc == 0, "colsum rc %d N=%lld K=%lld", rc, (long long)N, (long long)K);
  for (int64_t k = 0; k < K; ++k)
    CHECK(out[k] == static_cast<float>(want[static_cast<size_t>(k)]), "colsum N=%lld K=%lld col %lld", (long long)N, (long long)K, (long long)k);
  if (K > 256) return;
  // the two-matrix and the centred-moment forms of the same kernel (small integers: exact)
  Buf<float> y(static_cast<size_t>(N * K)), ctr(static_cast<size_t>(K)), a(static_cast<size_t>(K)), b(static_cast<size_t>(K));
  for (int64_t k = 0; k < K; ++k) ctr[k] = static_cast<float>(id(rng) / 4);
  for (int64_t i = 0; i < N * K; ++i) y[i] = static_cast<float>(id(rng) / 2);
  std::vector<double> w1(static_cast<size_t>(K), 0.0), w2(static_cast<size_t>(K), 0.0), m1(static_cast<size_t>(K), 0.0);
  for (int64_t i = 0; i < N * K; ++i) {
    const size_t k = static_cast<size_t>(i % K);
    w1[k] += x[i] * (y[i] - ctr[k]);
    m1[k] += (x[i] - ctr[k]);
    w2[k] += (x[i] - ctr[k]) * (x[i] - ctr[k]);
  }
  CHECK(exact_bn_backward_reduce_f32(x.p, y.p, ctr.p, N, K, a.p, b.p, nullptr) == 0, "bn reduce rc");
  for (int64_t k = 0; k < K; ++k)
    CHECK(a[k] == static_cast<float>(want[static_cast<size_t>(k)]) && b[k] == static_cast<float>(w1[static_cast<size_t>(k)]),
          "bn reduce N=%lld K=%lld col %lld", (long long)N, (long long)K, (long long)k);
  CHECK(exact_col_moments_f32(x.p, ctr.p, N, K, a.p, b.p, nullptr) == 0, "moments rc");
  for (int64_t k = 0; k < K; ++k)
    CHECK(a[k] == static_cast<float>(m1[static_cast<size_t>(k)]) && b[k] == static_cast<float>(w2[static_cast<size_t>(k)]),
          "moments N=%lld K=%lld col %lld", (long long)N, (long long)K, (long long)k);
}

// Unpack alone on random packed bytes, at sizes that take the several-rows-per-lane-group form of the kernel.
static void check_unpack_only(int64_t N, int64_t G, int bits, std::mt19937& rng) {
  const int64_t nb = exact_packed_nbytes(N, G, bits);
  Buf<uint8_t> packed(nb);
  Buf<float> sc(N), mn(N), out(N * G), want(N * G);
  for (int64_t i = 0; i < nb; ++i) packed[i] = static_cast<uint8_t>(rng());
  std::uniform_real_distribution<float> ud(0.5f, 40.f);
  for (int64_t i = 0; i < N; ++i) { sc[i] = ud(rng); mn[i] = ud(rng) - 20.f; }
  oracle_unpack(packed.p, bits, sc.p, mn.p, N, G, want.p);
  const int rc = exact_unpack_f32(packed.p, bits, sc.p, mn.p, N, G, out.p, nullptr);
  CHECK(rc == 0 && std::memcmp(out.p, want.p, N * G * 4) == 0, "unpack alone differs N=%ld G=%ld bits=%d", (long)N, (long)G, bits);
}

static void check_dw(int64_t N, int64_t K, int64_t D, int64_t pad, std::mt19937& rng) {
  std::uniform_int_distribution<int> id(-3, 3);
  const int64_t ldy = K + pad, ldx = D + 2 * pad;
  Buf<float> dy(static_cast<size_t>(N * ldy)), x(static_cast<size_t>(N * ldx)), out(static_cast<size_t>(K * D));
  for (int64_t i = 0; i < N * ldy; ++i) dy[i] = static_cast<float>(id(rng));
  for (int64_t i = 0; i < N * ldx; ++i) x[i] = static_cast<float>(id(rng));
  for (int bf16 = 0; bf16 < 2; ++bf16) {  // the fp32 and the bf16 matrix-core kernel
    const int rc = bf16 ? exact_linear_dw_bf16_f32(dy.p, ldy, x.p, ldx, N, K, D, out.p, nullptr)
                        : exact_linear_dw_f32(dy.p, ldy, x.p, ldx, N, K, D, out.p, nullptr);
    CHECK(rc == 0, "dw rc %d", rc);
    for (int64_t k = 0; k < K; ++k)
      for (int64_t d = 0; d < D; ++d) {
        double want = 0;
        for (int64_t n = 0; n < N; ++n) want += static_cast<double>(dy[n * ldy + k]) * x[n * ldx + d];
        CHECK(out[k * D + d] == static_cast<float>(want), "dw bf16=%d N=%lld K=%lld D=%lld at (%lld, %lld)", bf16, (long long)N,
              (long long)K, (long long)D, (long long)k, (long long)d);
      }
  }
}

// exact_tall_gemm_bf16_f32 on exactly sized buffers: small integers, so the result is the integer product
// bit for bit; the matrix direct with a row stride and transposed; bias, addend and in-place accumulation.
static void check_gemm(int64_t N, int64_t D, int64_t K, int64_t pad, std::mt19937& rng) {
  std::uniform_int_distribution<int> id(-5, 5);
  const int64_t ld = K + pad, ldt = D + pad, ldc = K + 2 * pad, ldo = K + pad;
  Buf<float> X(static_cast<size_t>(N * D)), M(static_cast<size_t>(D * ld)), Mt(static_cast<size_t>(K * ldt)), bias(static_cast<size_t>(K)),
      add(static_cast<size_t>(N * ldc)), out(static_cast<size_t>(N * ldo));
  for (int64_t i = 0; i < N * D; ++i) X[i] = static_cast<float>(id(rng));
  for (int64_t i = 0; i < D * ld; ++i) M[i] = static_cast<float>(id(rng));
  for (int64_t c = 0; c < K; ++c)
    for (int64_t d = 0; d < ldt; ++d) Mt[c * ldt + d] = d < D ? M[d * ld + c] : 99.f;
  for (int64_t i = 0; i < K; ++i) bias[i] = static_cast<float>(id(rng));
  for (int64_t i = 0; i < N * ldc; ++i) add[i] = static_cast<float>(id(rng));
  const int64_t tbytes = exact_tall_gemm_table_nbytes(D, K);
  CHECK(tbytes > 0 && tbytes % 16 == 0, "gemm table size");
  Buf<uint32_t> table(tbytes / 4);
  // variant 4: the rows start 8 bytes into a 16-byte line (and still end where the allocation ends)
  Buf<float> X8(static_cast<size_t>(N * D + 2));
  for (int64_t i = 0; i < N * D; ++i) X8[i + 2] = X[i];
  for (int variant = 0; variant < (D % 2 == 0 ? 5 : 4); ++variant) {
    const bool transposed = variant & 1;
    CHECK(exact_tall_gemm_prepare_bf16(transposed ? Mt.p : M.p, transposed ? ldt : ld, transposed, D, K, table.p, nullptr) == 0,
          "gemm prepare rc");
    const bool with_bias = variant >= 1, with_add = variant == 2 || variant == 3, in_place = variant == 3;
    for (int64_t i = 0; i < N * ldo; ++i) out[i] = -777.f;
    if (in_place)
      for (int64_t n = 0; n < N; ++n)
        for (int64_t c = 0; c < K; ++c) out[n * ldo + c] = add[n * ldc + c];
    const int rc = exact_tall_gemm_bf16_f32(variant == 4 ? X8.p + 2 : X.p, table.p, N, D, K, with_bias ? bias.p : nullptr,
                                            with_add ? (in_place ? out.p : add.p) : nullptr, in_place ? ldo : ldc, out.p, ldo, nullptr);
    CHECK(rc == 0, "gemm rc %d", rc);
    for (int64_t n = 0; n < N; ++n)
      for (int64_t c = 0; c < ldo; ++c) {
        if (c >= K) {
          CHECK(out[n * ldo + c] == -777.f, "gemm wrote into the row padding at (%lld, %lld)", (long long)n, (long long)c);
          continue;
        }
        double want = 0;
        for (int64_t d = 0; d < D; ++d) want += static_cast<double>(X[n * D + d]) * M[d * ld + c];
        if (with_bias) want += bias[c];
        if (with_add) want += add[n * ldc + c];
        CHECK(out[n * ldo + c] == static_cast<float>(want), "gemm variant %d N=%lld D=%lld K=%lld at (%lld, %lld)", variant,
              (long long)N, (long long)D, (long long)K, (long long)n, (long long)c);
      }
  }
}

static void check_gemm_shapes(std::mt19937& rng) {
  check_gemm(1, 4, 1, 0, rng);
  check_gemm(33, 8, 5, 3, rng);
  check_gemm(70, 256, 256, 0, rng);
  check_gemm(40, 128, 40, 1, rng);
  check_gemm(65, 100, 47, 2, rng);
  check_gemm(31, 604, 332, 0, rng);
  check_gemm(64, 256, 300, 4, rng);
  check_gemm(97, 48, 257, 0, rng);
  check_gemm(67, 602, 256, 0, rng);  // D % 4 == 2: the 8-byte-load form
  check_gemm(40, 6, 33, 2, rng);
  check_gemm(35, 50, 70, 0, rng);
}

static const int64_t kRpShapes[][3] = {{1, 256, 32}, {31, 256, 32}, {200, 256, 32}, {130, 602, 76}, {140, 100, 25}, {129, 256, 64},
                                       {64, 128, 64}, {77, 50, 15}, {130, 7, 4}, {100, 256, 126}, {33, 256, 128}, {70, 96, 96},
                                       {133, 97, 13}, {260, 1024, 32}, {2000, 256, 32}, {1700, 100, 25},
                                       {1100, 602, 76}, {900, 64, 128}, {1537, 50, 15}};

int main(int argc, char** argv) {
  std::setvbuf(stdout, nullptr, _IOLBF, 0);
  const std::string mode = argc > 1 ? argv[1] : "quick";
  std::mt19937 rng(12345);
  if (mode == "rp") {  // the projection kernels only
    for (auto& s : kRpShapes) check_rp(s[0], s[1], s[2], rng);
    std::printf("rp shapes ok (failures so far %d)\n", g_fail);
    return g_fail != 0;
  }
  if (mode == "unpack") {  // the several-rows form of the unpack kernel
    for (int bits : {1, 2, 4, 8}) {
      check_unpack_only(8229, 256, bits, rng);
      check_unpack_only(65571, 32, bits, rng);
      check_unpack_only(16397, 100, bits, rng);
      check_unpack_only(131077, 8, bits, rng);
    }
    std::printf("unpack sizes ok (failures so far %d)\n", g_fail);
    return g_fail != 0;
  }
  if (mode == "gemm") {  // the tall-operand GEMM only
    check_gemm_shapes(rng);
    std::printf("gemm shapes ok (failures so far %d)\n", g_fail);
    return g_fail != 0;
  }
  if (mode == "dw") {  // the weight-gradient kernels only
    check_dw(1, 1, 1, 0, rng);
    check_dw(7, 3, 5, 2, rng);
    check_dw(100, 40, 256, 0, rng);
    check_dw(515, 256, 128, 3, rng);
    check_dw(333, 47, 25, 1, rng);
    check_dw(600, 130, 70, 0, rng);
    check_dw(513, 32, 200, 5, rng);
    check_dw(1100, 256, 256, 0, rng);
    std::printf("dw shapes ok (failures so far %d)\n", g_fail);
    return g_fail != 0;
  }
  const int64_t shapes[][2] = {{1, 1}, {5, 3}, {37, 25}, {64, 32}, {100, 76}, {33, 40}, {129, 100}, {300, 128},
                               {203, 256}, {61, 602}, {16, 1024}, {19, 520}, {9, 1500}, {7, 2048}, {8, 8}, {3, 4}};
  for (auto& s : shapes)
    for (int bits : {1, 2, 4, 8})
      for (int supplied = 0; supplied < 2; ++supplied) check_quant(s[0], s[1], bits, supplied, rng);
  std::printf("quant shapes ok (failures so far %d)\n", g_fail);
  for (int64_t n : {1, 3, 4, 7, 8, 31, 32, 33, 255, 256, 257, 1000, 2048, 2049, 4101, 50001}) check_masks(n, rng);
  std::printf("mask sizes ok (failures so far %d)\n", g_fail);
  check_spmm(300, 300, 256, 8, 200, rng);
  check_spmm(200, 200, 40, 5, 0, rng);
  check_spmm(100, 100, 602, 10, 90, rng);
  check_spmm(500, 77, 100, 10, 0, rng);
  check_spmm(64, 64, 1, 3, 0, rng);
  check_spmm(90, 90, 47, 4, 80, rng);
  check_spmm(130, 130, 6, 30, 120, rng);
  check_spmm(4, 9, 8, 0, 0, rng);
  std::printf("spmm shapes ok (failures so far %d)\n", g_fail);
  for (auto& s : kRpShapes) check_rp(s[0], s[1], s[2], rng);
  std::printf("rp shapes ok (failures so far %d)\n", g_fail);
  for (int64_t n : {1, 3, 31, 32, 33, 255, 257, 1000, 2049, 4101, 50001}) check_leaky(n, rng);
  check_extra(120, 120, 256, 6, rng);
  check_extra(80, 50, 40, 5, rng);
  check_extra(60, 60, 602, 4, rng);
  check_extra(70, 33, 7, 8, rng);
  check_extra(40, 40, 1, 3, rng);
  check_extra(50, 50, 1000, 3, rng);
  std::printf("leaky / minmax / sddmm ok (failures so far %d)\n", g_fail);
  const int64_t fs[][2] = {{1, 8}, {5, 16}, {37, 40}, {64, 256}, {203, 256}, {100, 128}, {33, 1024}, {19, 520},
                           {129, 104}, {12, 768}, {7, 12}, {3, 1032}};
  for (auto& f : fs)
    for (int bits : {1, 2, 4, 8})
      for (int supplied = 0; supplied < 2; ++supplied) check_fused(f[0], f[1], bits, supplied, rng);
  std::printf("fused epilogues ok (failures so far %d)\n", g_fail);
  const int64_t hs[][2] = {{1, 1}, {5, 3}, {37, 25}, {64, 32}, {33, 40}, {203, 256}, {61, 602}, {16, 1024}, {19, 520}, {8, 8}};
  for (auto& f : hs)
    for (int bits : {1, 2, 4, 8}) check_half(f[0], f[1], bits, rng);
  std::printf("fp16 entry points ok (failures so far %d)\n", g_fail);
  const int64_t cs[][2] = {{1, 1}, {3, 5}, {7, 47}, {1000, 41}, {4099, 47}, {513, 256}, {33, 602}, {5, 8192}, {20000, 3}};
  for (auto& c : cs) check_colsum(c[0], c[1], rng);
  std::printf("column sums ok (failures so far %d)\n", g_fail);
  for (int64_t n : {100, 4096, 3 * 4096 + 77, 20 * 4096}) check_probe(n, rng);
  std::printf("traffic probe ok (failures so far %d)\n", g_fail);
  const int64_t ds[][4] = {{1, 1, 1, 0}, {7, 3, 5, 1}, {100, 40, 256, 0}, {515, 256, 128, 3}, {333, 47, 25, 0}, {1201, 256, 76, 2},
                           {600, 130, 70, 0}, {513, 32, 200, 5}};
  for (auto& d : ds) check_dw(d[0], d[1], d[2], d[3], rng);
  std::printf("weight gradient ok (failures so far %d)\n", g_fail);
  check_gemm_shapes(rng);
  std::printf("tall gemm ok (failures so far %d)\n", g_fail);
  if (mode == "large" || mode == "full") {
    // a line after every group: this part runs for hours under the sanitizer
    for (int bits : {1, 2, 4, 8}) check_quant(20011, 256, bits, bits == 4, rng);
    check_quant(3001, 1024, 2, false, rng);
    std::printf("  large quant ok (failures so far %d)\n", g_fail);
    check_masks(20011ll * 256 + 3, rng);
    std::printf("  large masks ok (failures so far %d)\n", g_fail);
    check_spmm(20000, 20000, 256, 14, 5000, rng);
    check_spmm(20000, 20000, 100, 14, 5000, rng);
    check_extra(5000, 5000, 64, 10, rng);
    std::printf("  large spmm / minmax / sddmm ok (failures so far %d)\n", g_fail);
    check_rp(20011, 256, 32, rng);
    check_rp(5003, 602, 76, rng);
    std::printf("  large rp ok (failures so far %d)\n", g_fail);
    check_fused(20011, 256, 2, false, rng);
    check_half(20011, 256, 2, rng);
    std::printf("large shapes ok (failures so far %d)\n", g_fail);
  }
  if (mode == "full") {
    for (int bits : {1, 2, 4, 8}) check_quant(169343, 256, bits, bits == 2, rng);
    std::printf("full-size quant ok (failures so far %d)\n", g_fail);
    check_masks(169343ll * 256, rng);
    check_spmm(169343, 169343, 256, 14, 20000, rng);
    check_spmm(169343, 169343, 40, 14, 20000, rng);
    check_rp(169343, 256, 32, rng);
    check_fused(169343, 256, 2, false, rng);
    std::printf("full-size spmm/rp/masks ok (failures so far %d)\n", g_fail);
  }
  std::printf(g_fail ? "FAILED: %d check(s)\n" : "all checks passed\n", g_fail);
  return g_fail ? 1 : 0;
}
