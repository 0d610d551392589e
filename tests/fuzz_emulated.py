"""Randomised differential run of every entry point on the SIMT emulator against
the oracles (CPU only; tests/test_fuzz_smoke.py runs it for a few seconds, by
hand:  python tests/fuzz_emulated.py <seed> <seconds>).  Any mismatch raises
with the shape that produced it."""
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for _p in (ROOT, os.path.join(ROOT, "tests"), os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

import numpy as np  # noqa: E402

import emu_util as e  # noqa: E402
import exact_oracle as o  # noqa: E402
import exact_oracle_extra as ox  # noqa: E402
import exact_oracle_half as oh  # noqa: E402

F32, F16 = np.float32, np.float16


def quant_case(rng):
    """fp32 and fp16 statistics + pack + unpack, and the fused ReLU / dropout / pack pass."""
    N = int(rng.integers(1, 400))
    G = int(rng.choice([rng.integers(1, 1100), 8 * rng.integers(1, 129), rng.choice([32, 64, 100, 128, 256, 512, 602, 1024])]))
    bits = int(rng.choice([1, 2, 4, 8]))
    supplied = bool(rng.integers(0, 2))
    x = (rng.standard_normal((N, G)) * rng.choice([0.01, 1, 100])).astype(F32)
    if rng.random() < 0.3:
        x[rng.integers(0, N)] = 1.5            # a constant row
    seed, off = int(rng.integers(0, 2**63)), int(rng.integers(0, 2**40))
    noise = rng.random((N, G), dtype=F32) if supplied else o.philox_noise_rows(seed, off, N, G)
    # fp32
    packed, s32, m32, sbf, mbf = e.minmax_pack(x, bits, noise if supplied else None, seed, off)
    want = o.quantize_activation(x, bits, noise)
    assert np.array_equal(packed, want[0]) and np.array_equal(sbf, want[2]) and np.array_equal(mbf, want[3]), ("f32 pack", N, G, bits, supplied)
    out = e.unpack(packed, bits, sbf, mbf, N, G, bf16=True)
    ref = o.dequantize_activation(want[0], bits, want[2], want[3], (N, G))
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32)), ("f32 unpack", N, G, bits)
    # fp16
    if G <= 1024:
        xh = x.astype(F16)
        ph, sh, mh = e.minmax_pack_f16(xh, bits, noise if supplied else None, seed, off)
        wp, ws, wm = oh.quantize_activation(xh, bits, noise)
        assert np.array_equal(ph, wp) and np.array_equal(sh.view(np.uint16), ws.view(np.uint16)), ("f16 pack", N, G, bits, supplied)
        outh = e.unpack_f16(ph, bits, sh, mh, N, G)
        refh = oh.unpack(wp, bits, ws, wm, N, G)
        a, b = outh.view(np.uint16), refh.view(np.uint16)
        nan = np.isnan(outh) & np.isnan(refh)
        assert np.array_equal(a[~nan], b[~nan]), ("f16 unpack", N, G, bits)
    # fused
    if G % 8 == 0 and G <= 1024:
        an = rng.random((N, G), dtype=F32) if supplied else o.philox_noise_flat(seed ^ 5, off + 4, N * G).reshape(N, G)
        got = e.relu_dropout_minmax_pack(x, 0.3, bits, an if supplied else None, noise if supplied else None, seed ^ 5, off + 4, seed, off)
        y1, m1 = o.relu_fwd(x.reshape(-1)); y2, m2 = o.dropout_fwd(y1, 0.3, an.reshape(-1))
        w = o.quantize_activation(y2.reshape(N, G), bits, noise)
        assert np.array_equal(got[0].view(np.uint32), y2.reshape(N, G).view(np.uint32)) and np.array_equal(got[1], m1 & m2) and np.array_equal(got[2], w[0]), ("fused", N, G, bits, supplied)
        # with batch norm ahead of the ReLU
        mean, mult, shift = (rng.standard_normal(G).astype(F32) for _ in range(3))
        got = e.relu_dropout_minmax_pack(x, 0.3, bits, an if supplied else None, noise if supplied else None, seed ^ 5, off + 4, seed, off,
                                         norm=(mean, mult, shift))
        xn = ((x - mean[None, :]) * mult[None, :] + shift[None, :]).astype(F32)
        y1, m1 = o.relu_fwd(xn.reshape(-1)); y2, m2 = o.dropout_fwd(y1, 0.3, an.reshape(-1))
        w = o.quantize_activation(y2.reshape(N, G), bits, noise)
        assert np.array_equal(got[0].view(np.uint32), y2.reshape(N, G).view(np.uint32)) and np.array_equal(got[1], m1 & m2) and np.array_equal(got[2], w[0]), ("bn fused", N, G, bits, supplied)

def other_case(rng, n):
    """masks, max / min aggregation, edge-value gradient, projection, two-step pack."""
    k = int(rng.integers(0, 4))
    if k == 0:      # masks fp32 + fp16
        m = int(rng.integers(1, 5000)); x = rng.standard_normal(m).astype(F32); g = rng.standard_normal(m).astype(F32)
        p = float(rng.choice([0.0, 0.1, 0.5, 0.9])); seed, off = int(rng.integers(0, 2**62)), int(rng.integers(0, 2**40))
        u = o.philox_noise_flat(seed, off, m)
        y, mk = e.dropout_fwd(x, p, None, seed, off); wy, wm = o.dropout_fwd(x, p, u)
        assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mk, wm), ("dropout", m, p)
        assert np.array_equal(e.dropout_bwd(g, mk, p).view(np.uint32), o.dropout_bwd(g, wm, p).view(np.uint32))
        y, mk = e.relu_dropout_fwd(x, p, None, seed, off); y1, m1 = o.relu_fwd(x); y2, m2 = o.dropout_fwd(y1, p, u)
        assert np.array_equal(y.view(np.uint32), y2.view(np.uint32)) and np.array_equal(mk, m1 & m2), ("relu_dropout", m, p)
        y, mk = e.leaky_relu_fwd(x, 0.2); wy, wm = ox.leaky_relu_fwd(x, 0.2)
        assert np.array_equal(y.view(np.uint32), wy.view(np.uint32)) and np.array_equal(mk, wm)
        xh = x.astype(F16)
        y, mk = e.dropout_fwd_f16(xh, p, None, seed, off, relu=True); wy, wm = oh.dropout_fwd(xh, p, u, relu=True)
        assert np.array_equal(y.view(np.uint16), wy.view(np.uint16)) and np.array_equal(mk, wm), ("f16 relu_dropout", m, p)
    elif k == 1:    # minmax / sddmm
        M, N, K = int(rng.integers(1, 200)), int(rng.integers(1, 60)), int(rng.choice([1, 2, 3, 4, 8, 33, 64, 100, 256, 300]))
        deg = rng.integers(0, 6, M); rowptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64); nnz = int(rowptr[-1])
        col = rng.integers(0, N, nnz); val = rng.standard_normal(nnz).astype(F32); X = rng.standard_normal((N, K)).astype(F32)
        for is_max in (True, False):
            for v in (val, None):
                out, arg = e.spmm_minmax(rowptr, col, v, X, is_max, np.int32 if n % 2 else np.int64)
                wout, warg = ox.spmm_minmax(rowptr, col, v, X, is_max)
                assert np.array_equal(out.view(np.uint32), wout.view(np.uint32)) and np.array_equal(arg.astype(np.int64), warg), ("minmax", M, N, K)
        if nnz:
            row = np.repeat(np.arange(M), deg); grad = rng.standard_normal((M, K)).astype(F32)
            for red in ("sum", "mean"):
                got = e.sddmm(row, rowptr, col, X, grad, red); want = ox.sddmm(row, rowptr, col, X, grad, red)
                assert np.allclose(got, want, rtol=1e-5, atol=1e-5 * max(1, np.abs(want).max())), ("sddmm", M, N, K)
    elif k == 2:    # rp
        N, D = int(rng.integers(1, 300)), int(rng.choice([7, 50, 100, 128, 256, 602])); kk = int(rng.integers(1, min(D, 128) + 1))
        # the fp32 matrix-core instruction, or the bf16 one on split operands (any matrix) or on the signs of a +-c matrix
        mode = str(rng.choice(["fp32", "bf16_split", "bf16_signs"]))
        X = rng.standard_normal((N, D)).astype(F32)
        if mode == "bf16_signs":
            R = ((2.0 * rng.integers(0, 2, (D, kk)) - 1) / np.sqrt(kk)).astype(F32)
        else:
            R = (rng.standard_normal((D, kk)) / np.sqrt(kk)).astype(F32)
        a = e.rp_fwd(X, R, mode=mode); w = o.input2rp(X, R)
        assert np.allclose(a, w, rtol=2e-5, atol=2e-5 * np.abs(w).max()), ("rp_fwd", N, D, kk, mode)
        b = e.rp_bwd(w, R, mode=mode); wb = o.rp2input(w, R)
        assert np.allclose(b, wb, rtol=2e-5, atol=2e-5 * np.abs(wb).max()), ("rp_bwd", N, D, kk, mode)
        if rng.integers(0, 2) == 0:     # the tall GEMM on the same operands (D even: 16-byte loads when it is a multiple of 4, else 8-byte ones), with bias and addend
            D4 = max(2, D // 2 * 2); Kg = int(rng.choice([1, 31, 40, 64, 100, 130, 256, 300]))
            Xg = rng.integers(-6, 7, (N, D4)).astype(F32); Mg = rng.integers(-6, 7, (D4, Kg)).astype(F32)
            bias = rng.integers(-9, 10, Kg).astype(F32); add = rng.integers(-9, 10, (N, Kg)).astype(F32)
            want = (Xg.astype(np.float64) @ Mg.astype(np.float64) + bias + add).astype(F32)
            assert np.array_equal(e.tall_gemm(Xg, Mg, bias=bias, addend=add, transposed=bool(rng.integers(0, 2))), want), ("gemm", N, D4, Kg)
        # projection + quantisation in one launch == the oracle's quantiser on the kernel's own product
        bits = int(rng.choice([1, 2, 4, 8])); supplied = bool(rng.integers(0, 2))
        seed, off = int(rng.integers(0, 2**63)), int(rng.integers(0, 2**40))
        noise = rng.random((N, kk), dtype=F32) if supplied else o.philox_noise_rows(seed, off, N, kk)
        got = e.rp_minmax_pack(X, R, bits, noise if supplied else None, seed, off, mode=mode)
        wq = o.quantize_activation(a, bits, noise)
        assert np.array_equal(got[0][:-1], wq[0][:got[0].size - 1]) and np.array_equal(got[3], wq[2]) and np.array_equal(got[4], wq[3]), ("rp_pack", N, D, kk, bits, supplied)
    else:           # two-step pack with given min / scale, row_minmax
        N, G = int(rng.integers(1, 300)), int(rng.integers(1, 2200)); bits = int(rng.choice([1, 2, 4, 8]))
        x = rng.standard_normal((N, G)).astype(F32); mn, mx = o.row_min_max(x); sc = o.compute_scale(mn, mx, bits)
        u = rng.random((N, G), dtype=F32)
        assert np.array_equal(e.pack(x, mn, sc, bits, u), o.pack_single_precision(x, mn, sc, bits, u)), ("pack2", N, G, bits)
        a, b = e.row_minmax(x); assert np.array_equal(a, mn) and np.array_equal(b, mx)
        if G > 1024:
            got = e.minmax_pack(x, bits, u); w = o.quantize_activation(x, bits, u)
            assert np.array_equal(got[0], w[0]) and np.array_equal(got[3], w[2]), ("long rows", N, G, bits)


def run(seed, seconds):
    rng = np.random.default_rng(seed)
    t0, n = time.time(), 0
    while time.time() - t0 < seconds:
        if n % 2:
            quant_case(rng)
        else:
            other_case(rng, n)
        n += 1
    return n


if __name__ == "__main__":
    print("cases:", run(int(sys.argv[1]) if len(sys.argv) > 1 else 0, float(sys.argv[2]) if len(sys.argv) > 2 else 60.0))
