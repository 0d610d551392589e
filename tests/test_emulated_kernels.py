"""The library's .hip kernels, compiled unchanged for a CPU SIMT emulator
(tests/emu), checked against the oracle: same parity bar as the GPU tests
(bit-exact for bytes, masks and dequantised values; 1e-5 relative for SpMM and
the projection GEMMs), plus sentinel bytes behind every output buffer.  This
is what verifies kernel indexing and arithmetic when no GPU is at hand; the
GPU tests (-m gpu) remain the parity tests proper."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

import emu_util as e
import exact_oracle as o

F32 = np.float32
SHAPES = [(1, 1), (5, 3), (37, 25), (64, 32), (100, 76), (33, 40), (129, 100), (300, 128), (200, 256),
          (61, 602), (16, 1024), (19, 520), (9, 1500), (7, 2048), (8, 8), (24, 16), (3, 4)]


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", SHAPES)
def test_pack_unpack(bits, N, G):
    rng = np.random.default_rng(N * 7 + G + bits)
    x = (rng.standard_normal((N, G)) * 3).astype(F32)
    if N > 4:
        x[2] = 0.75                                          # a constant row
        x[3] = 0.0
        x[3, ::2] = 1e-45                                    # a spread whose reciprocal overflows: scale = inf
    u = rng.random((N, G), dtype=F32)
    want = o.quantize_activation(x, bits, u)
    packed, s32, m32, sbf, mbf = e.minmax_pack(x, bits, u)
    assert np.array_equal(packed, want[0])
    assert np.array_equal(s32.view(np.uint32), want[4].view(np.uint32)) and np.array_equal(m32, want[5])
    assert np.array_equal(sbf, want[2]) and np.array_equal(mbf, want[3])
    xh = e.unpack(packed, bits, sbf, mbf, N, G, bf16=True)
    assert np.array_equal(xh.view(np.uint32), o.dequantize_activation(want[0], bits, want[2], want[3], (N, G)).view(np.uint32))
    xh32 = e.unpack(packed, bits, s32, m32, N, G)
    assert np.array_equal(xh32.view(np.uint32), o.unpack_single_precision(want[0], bits, want[4], want[5], N, G).view(np.uint32))
    # two-step form and the stand-alone row statistics
    mn, mx = e.row_minmax(x)
    assert np.array_equal(mn, want[5]) and np.array_equal(mx, x.max(1))
    assert np.array_equal(e.pack(x, mn, want[4], bits, u), want[0])
    # internal Philox noise == oracle fed with the documented stream
    seed, off = 0xABCDEF0123456789, (9 << 32) + 77
    got = e.minmax_pack(x, bits, None, seed, off)[0]
    assert np.array_equal(got, o.quantize_activation(x, bits, o.philox_noise_rows(seed, off, N, G))[0])
    assert np.array_equal(e.pack(x, mn, want[4], bits, None, seed, off), got)


@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("N,G", [(8229, 256), (65571, 32), (16397, 100), (8195, 1024), (131077, 8)])
def test_unpack_with_several_rows_per_lane_group(bits, N, G):
    """Activations large enough for the kernel form in which a lane group takes
    four consecutive rows (all loads issued first): every value against the
    oracle, with a ragged last group of rows, for fp32 and bf16 scale / min."""
    rng = np.random.default_rng(N + G + bits)
    packed = rng.integers(0, 256, o.packed_nbytes(N, G, bits), dtype=np.uint8)
    scale = (rng.random(N) * 40 + 0.5).astype(F32)
    mn = rng.standard_normal(N).astype(F32)
    got = e.unpack(packed, bits, scale, mn, N, G)
    assert np.array_equal(got.view(np.uint32), o.unpack_single_precision(packed, bits, scale, mn, N, G).view(np.uint32))
    sbf, mbf = o.bf16_round(scale)[0], o.bf16_round(mn)[0]
    got = e.unpack(packed, bits, sbf, mbf, N, G, bf16=True)
    assert np.array_equal(got.view(np.uint32), o.dequantize_activation(packed, bits, sbf, mbf, (N, G)).view(np.uint32))


def test_unpack_extreme_scales_take_the_division_path():
    # scales outside [2^-64, 2^64], inf and nan rows use the per-element IEEE division
    N, G, bits = 16, 24, 8
    rng = np.random.default_rng(3)
    packed = rng.integers(0, 256, o.packed_nbytes(N, G, bits), dtype=np.uint8)
    scale = np.array([1e-30, 1e30, np.inf, 0.0, 3e-39, 1.5, 255.0 / 7, 1e25, 2.0 ** -64, 2.0 ** 64, 1e-20, 1e20,
                      np.nan, -2.5, 1e38, 7e-5], F32)
    mn = rng.standard_normal(N).astype(F32)
    with np.errstate(all="ignore"):
        want = o.unpack_single_precision(packed, bits, scale, mn, N, G)
    got = e.unpack(packed, bits, scale, mn, N, G)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("n", [1, 3, 4, 7, 8, 31, 32, 33, 255, 256, 257, 1000, 2048, 2049, 4096 + 5, 50001])
def test_relu_and_dropout(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(F32)
    x[: min(n, 3)] = [0.0, -0.0, np.nan][: min(n, 3)]
    g = rng.standard_normal(n).astype(F32)
    y, mask = e.relu_fwd(x)
    wy, wm = o.relu_fwd(x)
    assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mask, wm)
    assert np.array_equal(e.relu_bwd(g, mask), o.relu_bwd(g, wm))
    u = rng.random(n, dtype=F32)
    for p in (0.5, 0.1, 0.0, 0.9):
        y, mask = e.dropout_fwd(x, p, u)
        wy, wm = o.dropout_fwd(x, p, u)
        assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mask, wm)
        assert np.array_equal(e.dropout_bwd(g, mask, p).view(np.uint32), o.dropout_bwd(g, wm, p).view(np.uint32))
    seed, off = 1234567, (1 << 40) + 3
    y, mask = e.dropout_fwd(x, 0.5, None, seed, off)
    wy, wm = o.dropout_fwd(x, 0.5, o.philox_noise_flat(seed, off, n))
    assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mask, wm)


def powerlaw_csr(M, avg_deg, seed, n_cols=None, hub=0):
    rng = np.random.default_rng(seed)
    n_cols = n_cols or M
    deg = np.minimum((rng.zipf(2.1, M) * avg_deg / 2.5).astype(np.int64), n_cols)
    deg[rng.integers(0, M, max(1, M // 50))] = 0
    if hub:
        deg[rng.integers(0, M, 3)] = min(hub, n_cols)
    rows = np.repeat(np.arange(M), deg)
    cols = rng.integers(0, n_cols, rows.size)
    A = sp.coo_matrix((rng.standard_normal(rows.size).astype(F32), (rows, cols)), shape=(M, n_cols)).tocsr()
    A.sum_duplicates()
    A.sort_indices()
    return A


@pytest.mark.parametrize("idx", [np.int64, np.int32])
@pytest.mark.parametrize("valued", [True, False])
@pytest.mark.parametrize("reduce", ["sum", "mean"])
@pytest.mark.parametrize("M,K,avg,hub,ncols", [(300, 256, 8, 200, None), (200, 40, 5, 0, None), (100, 602, 10, 90, None),
                                               (500, 100, 10, 0, 77), (64, 1, 3, 0, None), (90, 47, 4, 80, None),
                                               (10, 128, 2, 0, None), (130, 6, 30, 120, None)])
def test_spmm(M, K, avg, hub, ncols, reduce, valued, idx):
    A = powerlaw_csr(M, avg, M + K, n_cols=ncols, hub=hub)
    X = np.random.default_rng(K).standard_normal((A.shape[1], K)).astype(F32)
    val = A.data if valued else None
    want = o.spmm_csr(A.indptr, A.indices, val, X, reduce)
    got = e.spmm(A.indptr, A.indices, val, X, reduce, idx)
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * (np.abs(want).max() + 1e-30))
    assert (got[np.diff(A.indptr) == 0] == 0).all()


def test_spmm_all_empty_and_single_long_row():
    X = np.ones((5, 8), F32)
    z = e.spmm(np.zeros(5, np.int64), np.zeros(0, np.int64), None, X, "mean")
    assert z.shape == (4, 8) and (z == 0).all()
    rowptr = np.array([0, 0, 1000, 1000, 1003], np.int64)
    col = np.random.default_rng(0).integers(0, 5, 1003)
    got = e.spmm(rowptr, col, None, X, "sum")
    assert np.array_equal(got[:, 0], np.array([0, 1000, 0, 3], F32))
    # mean over a hub row (longer than the 2048 entries up to which every chunk divides its own partial sum:
    # its raw partial sums are added up and divided once), next to a split row below that length
    rng = np.random.default_rng(1)
    rowptr = np.array([0, 7, 2600, 2600, 2900, 2903], np.int64)
    col = rng.integers(0, 40, 2903)
    val = rng.standard_normal(2903).astype(F32)
    X = rng.standard_normal((40, 72)).astype(F32)
    for v in (None, val):
        want = o.spmm_csr(rowptr, col, v, X, "mean")
        got = e.spmm(rowptr, col, v, X, "mean")
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-5 * np.abs(want).max())
    ones = e.spmm(rowptr, col, None, np.ones((40, 8), F32), "mean")
    assert np.array_equal(ones[1], np.ones(8, F32)) and np.array_equal(ones[2], np.zeros(8, F32))
    np.testing.assert_allclose(ones[[0, 3, 4]], 1.0, rtol=0, atol=1e-6)


@pytest.mark.parametrize("dist", ["rademacher", "gaussian"])
@pytest.mark.parametrize("N,D,frac", [(1, 256, 0.125), (31, 256, 0.125), (200, 256, 0.125), (130, 602, 0.125),
                                      (140, 100, 0.25), (129, 256, 0.25), (64, 128, 0.5), (77, 50, 0.3), (130, 7, 0.5),
                                      (100, 256, 0.49)])
def test_rp(N, D, frac, dist):
    """Every matrix-core path of the projection (fp32 instruction; bf16
    instruction on operands split in three, for any matrix; bf16 on the signs
    of a +-c matrix) within 1e-5 of the oracle, forward and back."""
    k = o.kept_acts(frac, D)
    rng = np.random.default_rng(N + D)
    R = o.rademacher_matrix(D, k, rng) if dist == "rademacher" else o.gaussian_matrix(D, k, rng)
    X = (rng.standard_normal((N, D)) * np.exp(rng.uniform(-6, 6, (N, 1)))).astype(F32)   # rows of very different size
    want = o.input2rp(X, R)
    for mode in ("fp32", "bf16_split") + (("bf16_signs",) if dist == "rademacher" else ()):
        got = e.rp_fwd(X, R, mode=mode)
        row_scale = np.abs(want).max(1, keepdims=True)
        assert (np.abs(got - want) <= 1e-5 * row_scale + 1e-30).all(), mode
        back = e.rp_bwd(got, R, mode=mode)
        wb = o.rp2input(got, R)
        assert (np.abs(back - wb) <= 1e-5 * np.abs(wb).max(1, keepdims=True) + 1e-30).all(), mode


def test_bf16_split_of_an_fp32_number_is_exact():
    """The identity the bf16 paths rest on: hi = bf16(x), mid = bf16(x - hi),
    lo = bf16(x - hi - mid) reproduce x exactly (x normal, not within 2^16 of
    the smallest normal).  Checked here with torch's bf16 rounding, which is
    the rounding the conversion instruction performs."""
    import torch
    g = torch.Generator().manual_seed(0)
    bits = torch.randint(-2 ** 31, 2 ** 31 - 1, (2_000_000,), generator=g, dtype=torch.int64).to(torch.int32)
    x = bits.view(torch.float32)
    x = x[torch.isfinite(x) & (x.abs() > 1e-30) & (x.abs() < 1e38)]
    hi = x.to(torch.bfloat16).float()
    r1 = x - hi
    mid = r1.to(torch.bfloat16).float()
    r2 = r1 - mid
    lo = r2.to(torch.bfloat16).float()
    assert torch.equal(lo, r2)
    assert torch.equal((hi.double() + mid.double() + lo.double()).float(), x)
    assert torch.equal(hi.double() + mid.double() + lo.double(), x.double())


@pytest.mark.parametrize("N,D,k", [(70, 256, 32), (33, 100, 25), (40, 602, 76), (64, 48, 128)])
def test_rp_signs_path_on_integers_is_exact(N, D, k):
    """Small integers times +-1: every term and every partial sum is exact, so
    the signs path must return c * (integer sum) rounded once -- a wrong
    fragment, a k-slot paired with the wrong feature or a missed tail shows."""
    rng = np.random.default_rng(N + D + k)
    S = (2.0 * rng.integers(0, 2, (D, k)) - 1).astype(F32)
    c = F32(1.0 / np.sqrt(k))
    R = (S * c).astype(F32)
    X = rng.integers(-9, 10, (N, D)).astype(F32) * F32(0.25)
    exact = X.astype(np.float64) @ S.astype(np.float64)
    assert np.array_equal(e.rp_fwd(X, R, mode="bf16_signs"), (exact.astype(F32) * c).astype(F32))
    Xr = rng.integers(-9, 10, (N, k)).astype(F32)
    exact_b = Xr.astype(np.float64) @ S.astype(np.float64).T
    assert np.array_equal(e.rp_bwd(Xr, R, mode="bf16_signs"), (exact_b.astype(F32) * c).astype(F32))
    # the general path on the same integers with an integer matrix: exact as well
    Ri = rng.integers(-5, 6, (D, k)).astype(F32)
    assert np.array_equal(e.rp_fwd(X, Ri, mode="bf16_split"), (X.astype(np.float64) @ Ri.astype(np.float64)).astype(F32))
    assert np.array_equal(e.rp_bwd(Xr, Ri, mode="bf16_split"), (Xr.astype(np.float64) @ Ri.astype(np.float64).T).astype(F32))


@pytest.mark.parametrize("mode", ["fp32", "bf16_split", "bf16_signs"])
@pytest.mark.parametrize("bits", [1, 2, 4, 8])
@pytest.mark.parametrize("supplied", [True, False])
@pytest.mark.parametrize("N,D,frac", [(1, 256, 0.125), (31, 256, 0.125), (200, 256, 0.125), (130, 602, 0.125),
                                      (140, 100, 0.25), (129, 256, 0.25), (64, 128, 0.5), (77, 50, 0.3), (130, 7, 0.5),
                                      (100, 256, 0.49), (261, 602, 0.2)])
def test_projection_and_quantisation_in_one_launch_equal_the_two_launches(N, D, frac, bits, supplied, mode):
    """exact_rp_minmax_pack_f32 == exact_rp_fwd_f32 followed by the oracle's
    quantize_activation of that product, bit for bit (packed bytes, fp32 and
    bf16 scale / min), with supplied noise and with the internal Philox stream."""
    k = o.kept_acts(frac, D)
    rng = np.random.default_rng(N * 7 + D + bits)
    R = o.rademacher_matrix(D, k, rng) if mode == "bf16_signs" else o.gaussian_matrix(D, k, rng)
    X = rng.standard_normal((N, D)).astype(F32)
    if N > 4:
        X[3] = 0.0                                  # a constant (all-zero) projected row: scale = inf
    reduced = e.rp_fwd(X, R, mode=mode)
    noise = rng.random((N, k), dtype=F32) if supplied else o.philox_noise_rows(91, 4 * bits, N, k)
    want_packed, _, want_sbf, want_mbf, want_scale, want_mn = o.quantize_activation(reduced, bits, noise)
    packed, s32, m32, sbf, mbf = e.rp_minmax_pack(X, R, bits, noise if supplied else None, 91, 4 * bits, mode=mode)
    assert np.array_equal(m32.view(np.uint32), want_mn.view(np.uint32))
    assert np.array_equal(s32.view(np.uint32), want_scale.view(np.uint32))
    assert np.array_equal(sbf, want_sbf) and np.array_equal(mbf, want_mbf)
    assert packed[-1] == 0 and np.array_equal(packed[:-1], want_packed[:packed.size - 1])
    # and it is what the stand-alone pack entry point makes of the product
    alone = e.minmax_pack(reduced, bits, noise if supplied else None, 91, 4 * bits)
    assert np.array_equal(alone[0], packed)


def test_projection_and_quantisation_argument_checks():
    X, R = np.zeros((4, 16), F32), np.zeros((16, 4), F32)
    assert e.rp_minmax_pack(X, R, 3, expect_rc=-2) is None
    assert e.rp_minmax_pack(np.zeros((4, 300), F32), np.zeros((300, 129), F32), 2, expect_rc=-3) is None
    got = e.rp_minmax_pack(np.zeros((0, 16), F32), R, 2)
    assert got[0].size == 1 and got[0][0] == 0


def test_pack_unpack_random_shapes():
    """Randomly drawn shapes (any N, any G up to a few thousand, every bit
    width, both noise modes): the fixed list above cannot enumerate every
    remainder of N mod 8 and G mod 8 against every lanes-per-row choice."""
    rng = np.random.default_rng(2024)
    for case in range(60):
        bits = int(rng.choice([1, 2, 4, 8]))
        N = int(rng.integers(1, 70))
        G = int(rng.choice([rng.integers(1, 40), rng.integers(40, 300), rng.integers(300, 1100), rng.integers(1100, 2600)]))
        x = (rng.standard_normal((N, G)) * rng.uniform(0.1, 10)).astype(F32)
        u = rng.random((N, G), dtype=F32)
        want = o.quantize_activation(x, bits, u)
        packed, s32, m32, sbf, mbf = e.minmax_pack(x, bits, u)
        assert np.array_equal(packed, want[0]), (case, bits, N, G)
        assert np.array_equal(sbf, want[2]) and np.array_equal(mbf, want[3]), (case, bits, N, G)
        xh = e.unpack(packed, bits, sbf, mbf, N, G, bf16=True)
        ref = o.dequantize_activation(want[0], bits, want[2], want[3], (N, G))
        assert np.array_equal(xh.view(np.uint32), ref.view(np.uint32)), (case, bits, N, G)
        seed, off = int(rng.integers(0, 2 ** 63)), int(rng.integers(0, 2 ** 63))
        got = e.minmax_pack(x, bits, None, seed, off)[0]
        assert np.array_equal(got, o.quantize_activation(x, bits, o.philox_noise_rows(seed, off, N, G))[0]), (case, bits, N, G)


def test_masks_random_sizes():
    rng = np.random.default_rng(7)
    for n in rng.integers(1, 9000, 25).tolist():
        x = rng.standard_normal(n).astype(F32)
        y, mask = e.relu_fwd(x)
        wy, wm = o.relu_fwd(x)
        assert np.array_equal(y, wy) and np.array_equal(mask, wm), n
        seed, off = int(rng.integers(0, 2 ** 63)), int(rng.integers(0, 2 ** 63))
        y, mask = e.dropout_fwd(x, 0.3, None, seed, off)
        wy, wm = o.dropout_fwd(x, 0.3, o.philox_noise_flat(seed, off, n))
        assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mask, wm), n


def test_spmm_degenerate_row_layouts():
    """Row layouts that stress the search for a chunk's first row: a single
    row, only the last row filled, one hub row among empty ones, M around
    multiples of the wavefront size."""
    rng = np.random.default_rng(7)
    for trial in range(60):
        M = int(rng.choice([1, 2, 3, 63, 64, 65, 129, 1000, 4097]))
        N, K = int(rng.integers(1, 40)), int(rng.choice([1, 4, 7, 64]))
        mode = trial % 3
        if mode == 0:
            deg = rng.integers(0, 4, M)
        elif mode == 1:
            deg = np.zeros(M, np.int64)
            deg[rng.integers(0, M)] = rng.integers(1, 400)
        else:
            deg = np.zeros(M, np.int64)
            deg[-1], deg[0] = rng.integers(1, 200), rng.integers(0, 3)
        rowptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
        col = rng.integers(0, N, int(rowptr[-1]))
        val = rng.standard_normal(col.size).astype(np.float32)
        X = rng.standard_normal((N, K)).astype(np.float32)
        reduce = "sum" if trial % 2 else "mean"
        got = e.spmm(rowptr, col, val, X, reduce, np.int32 if trial % 4 < 2 else np.int64)
        want = o.spmm_csr(rowptr, col, val, X, reduce)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * max(1.0, np.abs(want).max())), (trial, M, N, K, mode)


@pytest.mark.parametrize("N,G", [(203, 256), (64, 128), (37, 40), (19, 520), (16, 1024), (5, 8), (33, 100), (9, 1500)])
def test_every_work_split_of_the_pack_kernel_gives_the_same_bytes(N, G):
    """exact_minmax_pack_geom_f32: 1, 2 or 4 column groups per lane (and hints the
    row length does not allow, which are ignored) -- identical results."""
    rng = np.random.default_rng(N + G)
    x = (rng.standard_normal((N, G)) * 2).astype(np.float32)
    for bits in (1, 2, 4, 8):
        want = o.quantize_activation(x, bits, o.philox_noise_rows(5, 9, N, G))
        for hint in (0, 1, 2, 4):
            if G > 1024:
                continue                      # long rows need the fp32 outputs of the two-step form (covered elsewhere)
            packed, sbf, mbf = e.minmax_pack_geom(x, bits, hint, None, 5, 9)
            assert np.array_equal(packed, want[0]) and np.array_equal(sbf, want[2]) and np.array_equal(mbf, want[3]), (bits, hint)
    assert e.minmax_pack_geom(x[:, :8], 2, 3, expect_rc=-5) is None


def test_pack_geometry_candidates():
    from exact_amd.cpp_extension import quantization as extq
    assert extq.pack_geometry_candidates(256) == [1, 2, 4]
    assert extq.pack_geometry_candidates(8) == [1]
    assert extq.pack_geometry_candidates(16) == [1, 2]
    assert extq.pack_geometry_candidates(520) == [4]          # 65 octs: only 4 per lane fits 32 lanes
    assert extq.pack_geometry_candidates(1024) == [4]
    assert extq.pack_geometry_candidates(2048) == []
    t = torch.zeros(4, 256)
    assert extq._pack_geometry(t, 2) == 0                      # host tensors (emulated runs) are never tuned


@pytest.mark.parametrize("N,D,K", [(1, 4, 1), (33, 8, 5), (70, 256, 256), (40, 128, 40), (65, 100, 47), (31, 604, 332),
                                   (64, 256, 300), (97, 48, 257), (130, 256, 41), (67, 602, 256), (40, 6, 33), (35, 50, 70)])
def test_tall_gemm(N, D, K):
    """exact_tall_gemm_bf16_f32 = X . M (+ bias) (+ addend).  Small integers: every
    bf16 piece, product and partial sum is exact, so the result must be the
    integer product bit for bit -- a wrong fragment, column slab or tile offset
    shows; random data of mixed magnitudes within fp32 accumulation error of
    float64 (a dropped low-order piece would not be); M handed over transposed
    and with a row stride; the output as its own addend."""
    rng = np.random.default_rng(N + D + K)
    X = rng.integers(-6, 7, (N, D)).astype(F32)
    M = rng.integers(-6, 7, (D, K)).astype(F32)
    bias = rng.integers(-9, 10, K).astype(F32)
    add = rng.integers(-9, 10, (N, K)).astype(F32)
    exact = X.astype(np.float64) @ M.astype(np.float64)
    assert np.array_equal(e.tall_gemm(X, M), exact.astype(F32))
    assert np.array_equal(e.tall_gemm(X, M, transposed=True, ld=D + 3), exact.astype(F32))
    assert np.array_equal(e.tall_gemm(X, M, ld=K + 5), exact.astype(F32))
    assert np.array_equal(e.tall_gemm(X, M, bias=bias), (exact + bias).astype(F32))
    assert np.array_equal(e.tall_gemm(X, M, bias=bias, addend=add), (exact + bias + add).astype(F32))
    assert np.array_equal(e.tall_gemm(X, M, addend=add, in_place=True), (exact + add).astype(F32))
    raw = np.zeros(N * D + 8, F32)                       # rows that start 8 bytes into a 16-byte line: 8-byte loads
    first = ((8 - raw.ctypes.data % 16) % 16) // 4
    X8 = raw[first:first + N * D].reshape(N, D); X8[:] = X
    if D % 2 == 0:
        assert X8.ctypes.data % 16 == 8
        assert np.array_equal(e.tall_gemm(X8, M, bias=bias), (exact + bias).astype(F32))
    X = (rng.standard_normal((N, D)) * np.exp(rng.uniform(-4, 4, (N, 1)))).astype(F32)
    M = (rng.standard_normal((D, K)) * np.exp(rng.uniform(-4, 4, (1, K)))).astype(F32)
    want = X.astype(np.float64) @ M.astype(np.float64)
    bound = np.abs(X).astype(np.float64) @ np.abs(M).astype(np.float64)
    assert (np.abs(e.tall_gemm(X, M) - want) <= 1e-6 * bound + 1e-30).all()


def test_tall_gemm_limits():
    X, M = np.zeros((8, 8), F32), np.zeros((8, 8), F32)
    assert e.emu().exact_tall_gemm_table_nbytes(0, 8) == 0 and e.emu().exact_tall_gemm_table_nbytes(8, 5000) == 0
    assert e.emu().exact_tall_gemm_table_nbytes(256, 256) == 16 * (1 + 16 * 8 * 3 * 64)
    assert e.emu().exact_tall_gemm_bf16_f32(e.p(np.zeros((4, 7), F32)), e.p(np.zeros(1024, F32)), 4, 7, 8, None, None, 8,
                                            e.p(np.zeros((4, 8), F32)), 8, None) == -3        # D odd
    assert e.emu().exact_tall_gemm_bf16_f32(e.p(X), e.p(np.zeros(4096, F32)), 8, 8, 8, None, None, 8, e.p(np.zeros((8, 8), F32)), 7,
                                            None) == -3                                              # ldo < K
    assert e.emu().exact_tall_gemm_bf16_f32(None, None, 0, 8, 8, None, None, 8, None, 8, None) == 0   # N == 0: nothing to do
