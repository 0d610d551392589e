"""Pins the CPU oracle (oracle/exact_oracle.py and its C twin) WITHOUT the
reference: hand-computed bytes, Random123 known answers, library routines,
brute force and invariants.  The reference's own tests hold no golden vectors
for this path (its inputs are unseeded random tensors), so these are the pins.
"""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import c_oracle as co
import exact_oracle as o

F32 = np.float32


# ---------------------------------------------------------------- Philox ----
PHILOX_KAT = [  # Random123 kat_vectors, philox4x32 10 rounds
    ([0, 0, 0, 0], [0, 0], [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]),
    ([0xFFFFFFFF] * 4, [0xFFFFFFFF] * 2, [0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD]),
    ([0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344], [0xA4093822, 0x299F31D0],
     [0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1]),
]


@pytest.mark.parametrize("ctr,key,want", PHILOX_KAT)
def test_philox_known_answers(ctr, key, want):
    assert o.philox4x32(np.array(ctr), key).tolist() == want
    assert co.philox4x32_10(ctr, key).tolist() == want


def test_philox_noise_layout():
    # element (n, d) <- half (d % 2) of word ((d % 8) // 2) of block (d // 8, n, off_lo, off_hi)
    seed, off = 0x1234567890ABCDEF, (5 << 32) | 9
    u = o.philox_noise_rows(seed, off, 3, 21)
    blk = o.philox4x32(np.array([2, 1, 9, 5]), (seed & 0xFFFFFFFF, seed >> 32))
    h = int(blk[1]) >> 16                      # d = 19 -> oct 2, word (3 // 2) = 1, high half
    assert u[1, 16 + 3] == F32((h + 0.5) / 65536)
    lo = int(blk[0]) & 0xFFFF
    assert u[1, 16] == F32((lo + 0.5) / 65536)
    assert u.min() > 0 and u.max() < 1
    flat = o.philox_noise_flat(seed, off, 21)
    blk = o.philox4x32(np.array([2, 0, 9, 5]), (seed & 0xFFFFFFFF, seed >> 32))
    assert flat[20] == F32(((int(blk[2]) & 0xFFFF) + 0.5) / 65536)


# ------------------------------------------------------------------ bf16 ----
def test_bf16_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(4096).astype(F32) * 10.0 ** rng.integers(-30, 30, 4096),
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.0, 3.0e38, 1.00390625, 1.01171875], dtype=F32)])
    bits, val = o.bf16_round(x)
    t = torch.from_numpy(x).to(torch.bfloat16)
    assert np.array_equal(val, t.float().numpy())
    assert np.array_equal(bits.view(np.int16), t.view(torch.int16).numpy())
    for v, b in zip(x[:64], bits[:64]):
        assert co.lib().oracle_f32_to_bf16(float(v)) == int(b)


# ------------------------------------------------------- pack known answers -
def _pack_both(x, mn, sc, bits, noise):
    a = o.pack_single_precision(x, mn, sc, bits, noise)
    b = co.pack(x, mn, sc, bits, noise)
    assert np.array_equal(a, b)
    return a


def test_pack_kat_0xE4():
    # N=4, G=1, b=2: q=[0,1,2,3] -> 0 | 1<<2 | 2<<4 | 3<<6 = 0xE4
    x = np.array([[0.0], [1.0], [2.0], [3.0]], F32)
    p = _pack_both(x, np.zeros(4, F32), np.ones(4, F32), 2, np.full((4, 1), 0.5, F32))
    assert p.tolist() == [0xE4, 0x00]


def test_pack_kat_alternating_bits():
    # N=8, G=2, b=1: column 0 rows 0,2,4,6 set -> 0x55; column 1 rows 1,3,5,7 -> 0xAA
    x = np.zeros((8, 2), F32)
    x[0::2, 0] = 1.0
    x[1::2, 1] = 1.0
    p = _pack_both(x, np.zeros(8, F32), np.ones(8, F32), 1, np.full((8, 2), 0.5, F32))
    assert p.tolist() == [0x55, 0xAA, 0x00]


def test_pack_kat_ragged_rows():
    # N=5, b=2: second group holds only row 4, in bits 0-1
    x = np.array([[3.0], [2.0], [1.0], [0.0], [2.0]], F32)
    p = _pack_both(x, np.zeros(5, F32), np.ones(5, F32), 2, np.full((5, 1), 0.5, F32))
    assert p.tolist() == [3 | 2 << 2 | 1 << 4 | 0 << 6, 2, 0x00]


@pytest.mark.parametrize("N,G,bits,want", [(169343, 256, 1, 5419009), (169343, 256, 2, 10838017),
                                           (169343, 256, 4, 21676033), (169343, 256, 8, 43351809),
                                           (169343, 32, 1, 677377), (169343, 32, 8, 5418977), (5, 3, 2, 7)])
def test_packed_length(N, G, bits, want):
    assert o.packed_nbytes(N, G, bits) == want
    assert co.lib().oracle_packed_nbytes(N, G, bits) == want


def test_noise_half_is_round_half_even():
    # u == 0.5 makes the rounding deterministic: rint((x - mn) * scale)
    x = np.array([[0.5, 1.5, 2.5, 3.5, 0.49, 2.51, 0.0, 7.0]], F32)
    q = o.quantize_values(x, np.zeros(1, F32), np.ones(1, F32), np.full_like(x, 0.5))
    assert q.tolist() == [[0, 2, 2, 4, 0, 3, 0, 7]]


def _brute_pack(x, mn, sc, bits, noise):
    N, G = x.shape
    wpt = 8 // bits
    out = [0] * o.packed_nbytes(N, G, bits)
    for n in range(N):
        for d in range(G):
            t = F32(F32(F32(F32(x[n, d] - mn[n]) * sc[n]) + noise[n, d]) - F32(0.5))
            t = F32(0.0) if not (t > 0) else t
            val = int(np.rint(t))
            idx = (n // wpt) * G + d
            out[idx] = (out[idx] | (val << ((n % wpt) * bits))) & 0xFF
    return out


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", [(7, 5), (9, 8), (16, 3)])
def test_pack_unpack_brute_force(bits, N, G):
    rng = np.random.default_rng(bits * 100 + N)
    x = rng.standard_normal((N, G)).astype(F32)
    u = rng.random((N, G), dtype=F32)
    mn, mx = o.row_min_max(x)
    sc = o.compute_scale(mn, mx, bits)
    with np.errstate(all="ignore"):
        want = _brute_pack(x, mn, sc, bits, u)
    got = _pack_both(x, mn, sc, bits, u)
    assert got.tolist() == want
    # unpack: brute force
    xh = o.unpack_single_precision(got, bits, sc, mn, N, G)
    assert np.array_equal(xh.view(np.uint32), co.unpack(got, bits, sc, mn, N, G).view(np.uint32))
    wpt = 8 // bits
    for n in range(N):
        for d in range(G):
            q = (int(got[(n // wpt) * G + d]) >> ((n % wpt) * bits)) & (2 ** bits - 1)
            assert xh[n, d] == F32(F32(F32(q) / sc[n]) + mn[n])


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_invariants(bits):
    rng = np.random.default_rng(bits)
    N, G = 257, 76
    x = (rng.standard_normal((N, G)) * rng.uniform(0.01, 50, (N, 1))).astype(F32)
    x[3] = 1.25                                       # constant row
    u = rng.random((N, G), dtype=F32)
    mn, mx = o.row_min_max(x)
    assert np.array_equal(mn, np.array([min(r) for r in x], F32)) and np.array_equal(mx, np.array([max(r) for r in x], F32))
    cmn, cmx = co.row_minmax(x)
    assert np.array_equal(cmn, mn) and np.array_equal(cmx, mx)
    sc = o.compute_scale(mn, mx, bits)
    assert np.array_equal(sc.view(np.uint32), co.scale(mn, mx, bits).view(np.uint32))
    q = o.quantize_values(x, mn, sc, u)
    B = 2 ** bits - 1
    assert q.min() >= 0 and q.max() <= B + 1 and (q > B).mean() < 1e-3   # B+1 only through fp32 rounding
    assert (q[3] == 0).all()                           # scale = inf -> NaN -> fmax -> 0
    packed, b, sbf, mbf, sc32, mn32 = o.quantize_activation(x, bits, u)
    xh = o.dequantize_activation(packed, bits, sbf, mbf, x.shape)
    _, mnb = o.bf16_round(mn)
    assert np.array_equal(xh[3], np.full(G, mnb[3], F32))          # constant row -> bf16(min)
    ok = np.ones(N, bool)
    ok[3] = False
    rng_ = (mx - mn)[ok, None]
    # |x_hat - x| <= one quantisation step + bf16 error of scale (2^-8 relative, on up to B steps) and of min
    err = np.abs(xh[ok] - x[ok])
    bound = rng_ / B * 1.001 + rng_ * 2.0 ** -8 + np.abs(mn[ok, None]) * 2.0 ** -8 + 1e-6
    assert (err <= bound).all()


def test_spill_is_replicated_not_clamped():
    """fp32 rounding can give (mx - mn) * scale = B + ulp; with noise near 1 the
    reference's unclamped value B + 1 then ORs into the neighbouring field
    (bits < 8) or wraps to 0 in its uint8 accumulator (bits == 8)."""
    x = np.array([[0.0], [0.0]], F32)
    x[1, 0] = 1.0
    mn = np.zeros(2, F32)
    # force the situation directly: scale such that x * scale = B + 1 after rounding up
    sc = np.array([4.0, 4.0], F32)                    # b = 2, B = 3: row 1 quantises to rint(4 + u - 0.5) = 4
    p = _pack_both(x, mn, sc, 2, np.full((2, 1), 0.5, F32))
    assert p[0] == (0 | (4 << 2)) & 0xFF == 0x10      # lands in row 2's field, not clamped to 3 (0x0C)
    sc8 = np.array([256.0, 256.0], F32)
    p8 = _pack_both(x, mn, sc8, 8, np.full((2, 1), 0.5, F32))
    assert p8.tolist() == [0, 0, 0]                   # 256 wraps to 0 in a byte
    x4 = np.array([[1.0], [0.0]], F32)
    p4 = _pack_both(x4[::-1].copy(), mn, np.array([16.0, 16.0], F32), 4, np.full((2, 1), 0.5, F32))
    assert p4[0] == 0                                 # 16 << 4 leaves the byte


def test_overflowing_scale_saturates_like_the_conversion():
    """A row whose spread is so small that the reciprocal overflows: scale = inf,
    the minimum gives 0 * inf = NaN -> code 0, every other element inf, which
    __float2int_rn (cvt.rni.s32.f32, clamped to the int32 range) turns into
    INT_MAX; the uint8 accumulator keeps the low byte of INT_MAX << (row * bits)."""
    tiny = F32(1e-45)
    x = np.array([[0, tiny, 0, tiny], [tiny, 0, tiny, tiny]], F32)
    mn, mx = o.row_min_max(x)
    for bits, want in ((8, [0, 0xFF, 0, 0xFF, 0xFF, 0, 0xFF, 0xFF]), (2, [0xFC, 0xFF, 0xFC, 0xFF]),
                       (1, [0xFE, 0xFF, 0xFE, 0xFF]), (4, [0xF0, 0xFF, 0xF0, 0xFF])):
        sc = o.compute_scale(mn, mx, bits)
        assert np.isinf(sc).all()
        p = _pack_both(x, mn, sc, bits, np.full(x.shape, 0.25, F32))
        assert p[:-1].tolist() == want and p[-1] == 0


def test_stochastic_rounding_is_unbiased():
    # E_u[q] = (x - mn) * scale: mean error < 1e-3 over 1e6 draws, supplied and Philox noise
    draws = 1_000_000
    v = F32(1.3)                                       # target value in quantisation units
    x = np.full((1, draws), v, F32)
    for noise in (np.random.default_rng(5).random((1, draws), dtype=F32), o.philox_noise_rows(11, 3, 1, draws)):
        q = o.quantize_values(x, np.zeros(1, F32), np.ones(1, F32), noise)
        assert abs(q.mean() - float(v)) < 1e-3
        assert set(np.unique(q)) == {1, 2}
    u = o.philox_noise_rows(99, 0, 64, 4096)
    assert abs(u.mean() - 0.5) < 1e-3 and abs(u.var() - 1 / 12) < 1e-3


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
def test_scale_is_reciprocal_times_B_like_torch(bits):
    """ops.py:39 is `(2 ** bits - 1) / (mx - mn)` on tensors: torch evaluates
    int / tensor as tensor.reciprocal() * int (two roundings)."""
    rng = np.random.default_rng(bits)
    mn = rng.standard_normal(20000).astype(F32)
    mx = (mn + np.abs(rng.standard_normal(20000)).astype(F32) * F32(3)).astype(F32)
    mx[0] = mn[0]
    want = ((2 ** bits - 1) / (torch.from_numpy(mx) - torch.from_numpy(mn))).numpy()
    assert np.array_equal(o.compute_scale(mn, mx, bits).view(np.uint32), want.view(np.uint32))
    assert np.array_equal(co.scale(mn, mx, bits).view(np.uint32), want.view(np.uint32))
    if bits > 1:   # and it is NOT the single division
        single = (F32(2 ** bits - 1) / (mx[1:] - mn[1:])).astype(F32)
        assert not np.array_equal(single, want[1:])


def test_fast_division_identity_exhaustive():
    """The unpack kernel divides once per row and corrects per element; the
    correction is exact for every significand (one exponent is exhaustive for
    the normal range, two more guard against an exponent dependence)."""
    for e in (127, 64, 190):
        assert co.lib().oracle_count_fast_division_mismatches(e) == 0


# ------------------------------------------------------------------ masks ---
def test_relu_matches_torch_autograd():
    rng = np.random.default_rng(1)
    x = rng.standard_normal(1000 + 7).astype(F32)
    x[:4] = [0.0, -0.0, np.nan, 1e-30]
    g = rng.standard_normal(x.size).astype(F32)
    y, mask = o.relu_fwd(x)
    t = torch.from_numpy(x.copy()).requires_grad_()
    ty = torch.relu(t)
    ty.backward(torch.from_numpy(g))
    ref = ty.detach().numpy().copy()
    ref[2] = 0.0                                       # reference kernel: NaN > 0 is false -> 0
    assert np.array_equal(y, ref)
    dx = o.relu_bwd(g, mask)
    tg = t.grad.numpy().copy()
    tg[2] = 0.0
    assert np.array_equal(dx, tg)
    assert mask.size == (x.size + 31) // 32 and mask.dtype == np.uint32
    cy, cm = co.relu_fwd(x)
    assert np.array_equal(cy, y) and np.array_equal(cm, mask) and np.array_equal(co.relu_bwd(g, mask), dx)
    assert (mask[0] >> 3) & 1 == 1 and (mask[0] & 0b111) == 0


@pytest.mark.parametrize("p", [0.5, 0.1, 0.0])
def test_dropout_closed_form(p):
    rng = np.random.default_rng(2)
    n = 999
    x = rng.standard_normal(n).astype(F32)
    u = rng.random(n, dtype=F32)
    g = rng.standard_normal(n).astype(F32)
    y, mask = o.dropout_fwd(x, p, u)
    keep = u > F32(p)
    assert np.array_equal(y != 0, keep & (x != 0))
    np.testing.assert_allclose(y[keep], x[keep] / (1 - p), rtol=1e-6)
    dx = o.dropout_bwd(g, mask, p)
    assert np.array_equal(dx != 0, keep & (g != 0))   # zero pattern of grad == zero pattern of output
    np.testing.assert_allclose(dx[keep], g[keep] / (1 - p), rtol=1e-6)
    # all-ones input: max(out) == max(grad) == 1/(1-p), as the reference's structural test checks
    y1, m1 = o.dropout_fwd(np.ones(n, F32), p, u)
    assert y1.max() == o.dropout_bwd(np.ones(n, F32), m1, p).max() == F32(1.0) / F32(1.0 - float(F32(p))) or p == 0.1
    cy, cm = co.dropout_fwd(x, p, u)
    assert np.array_equal(cy.view(np.uint32), y.view(np.uint32)) and np.array_equal(cm, mask)
    assert np.array_equal(co.dropout_bwd(g, mask, p), dx)
    # Philox path of the C twin == NumPy noise fed explicitly
    yp, mp = co.dropout_fwd(x, p, None, seed=3, offset=8)
    y2, m2 = o.dropout_fwd(x, p, o.philox_noise_flat(3, 8, n))
    assert np.array_equal(yp.view(np.uint32), y2.view(np.uint32)) and np.array_equal(mp, m2)


# ------------------------------------------------------------------- SpMM ---
def _random_csr(M, N, nnz, seed, valued=True):
    rng = np.random.default_rng(seed)
    A = sp.coo_matrix((rng.standard_normal(nnz).astype(F32), (rng.integers(0, M, nnz), rng.integers(0, N, nnz))),
                      shape=(M, N)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    return A


@pytest.mark.parametrize("valued", [True, False])
@pytest.mark.parametrize("reduce", ["sum", "mean"])
def test_spmm_matches_scipy_and_dense(valued, reduce):
    A = _random_csr(200, 150, 1500, 3)
    A[7, :] = 0
    A.eliminate_zeros()                               # an empty row
    if not valued:
        A.data[:] = 1.0
    X = np.random.default_rng(4).standard_normal((150, 13)).astype(F32)
    val = A.data if valued else None
    got = o.spmm_csr(A.indptr, A.indices, val, X, reduce)
    want = (A.astype(np.float64) @ X.astype(np.float64))
    if reduce == "mean":
        want = want / np.maximum(np.diff(A.indptr), 1)[:, None]
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5)
    dense = A.toarray().astype(np.float64) @ X
    if reduce == "mean":
        dense = dense / np.maximum(np.diff(A.indptr), 1)[:, None]
    np.testing.assert_allclose(got, dense, rtol=1e-5, atol=1e-5)
    assert (got[7] == 0).all()
    assert np.array_equal(got.view(np.uint32), co.spmm_csr(A.indptr, A.indices, val, X, reduce).view(np.uint32))


def test_spmm_backward_is_transpose():
    A = _random_csr(120, 90, 800, 5)
    dY = np.random.default_rng(6).standard_normal((120, 9)).astype(F32)
    row, colptr, csr2csc = o.csr_transpose(A.indptr, A.indices, 90)
    At = A.T.tocsr()
    At.sort_indices()
    assert np.array_equal(colptr, At.indptr) and np.array_equal(row[csr2csc], At.indices)
    np.testing.assert_allclose(o.spmm_sum_bw(row, colptr, csr2csc, A.data, dY), At.astype(np.float64) @ dY,
                               rtol=1e-5, atol=1e-5)
    cnt = np.maximum(np.diff(A.indptr), 1)
    Amean = sp.diags(1.0 / cnt) @ A
    np.testing.assert_allclose(o.spmm_mean_bw(row, np.diff(A.indptr), colptr, csr2csc, A.data, dY),
                               Amean.T.astype(np.float64) @ dY, rtol=1e-5, atol=1e-5)
    ones = sp.csr_matrix((np.ones_like(A.data), A.indices, A.indptr), shape=A.shape)
    np.testing.assert_allclose(o.spmm_mean_bw(row, np.diff(A.indptr), colptr, csr2csc, None, dY),
                               (sp.diags(1.0 / cnt) @ ones).T.astype(np.float64) @ dY, rtol=1e-5, atol=1e-5)


# --------------------------------------------------------------------- RP ---
@pytest.mark.parametrize("frac,D,k", [(0.125, 256, 32), (0.125, 602, 76), (0.25, 100, 25), (0.25, 256, 64)])
def test_kept_acts_table(frac, D, k):
    assert o.kept_acts(frac, D) == k


def test_rp_matrices_and_products():
    rng = np.random.default_rng(7)
    R = o.rademacher_matrix(256, 32, rng)
    assert set(np.unique(R)) == {F32(-1 / 32 ** 0.5), F32(1 / 32 ** 0.5)}
    Gm = o.gaussian_matrix(4096, 32, rng)
    assert abs(Gm.var() - 1 / 32) < 1e-3
    big = o.rademacher_matrix(64, 4096, rng)           # E[R R^T] = I
    np.testing.assert_allclose(big @ big.T, np.eye(64), atol=0.08)
    X = rng.standard_normal((50, 256)).astype(F32)
    np.testing.assert_allclose(o.input2rp(X, R), X @ R, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(co.rp_fwd(X, R), o.input2rp(X, R), rtol=1e-5, atol=1e-5)
    Xr = o.input2rp(X, R)
    np.testing.assert_allclose(o.rp2input(Xr, R), Xr @ R.T, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(co.rp_bwd(Xr, R), o.rp2input(Xr, R), rtol=1e-5, atol=1e-5)
