"""Measurements beyond the headline pack+unpack number: the other kernels of
the path at the benchmark shapes, and full-batch training epochs/s of the
INT2 / INT1 GCN and GraphSAGE configurations on synthetic power-law graphs
(the loop of mem_speed_bench/arxiv/train_full_batch.py:256-266 in the
reference: zero_grad, forward on all nodes, nll_loss on the training nodes,
backward, optimizer step).  bench.py calls run(); every number is measured
with HIP events on the stream the kernels are launched on.
"""
from __future__ import annotations

import sys
import time

import torch
import torch.nn.functional as F

from . import ops
from .conf import QuantizationConfig, config
from .cpp_extension import quantization as extq
from .cpp_extension import backward_func as ext_backward_func
from .cpp_extension import spmm as ext_spmm
from .models import GCN, SAGE
from .module import QModule
from .sparse import SparseTensor, gcn_norm

HBM_PEAK_GBS = 8000.0
FP32_MFMA_PEAK_TFLOPS = 157.3


def event_time(fn, reps=20, warm=3):
    """Average seconds per call of fn(), HIP events on the current stream."""
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / reps * 1e-3


def launch_times(fn, reps=40, warm=4):
    """(mean, median) microseconds of fn(i), one HIP event pair around EACH call
    on the current stream -- what a kernel trace reports per dispatch, without
    the overlap of back-to-back launches."""
    for i in range(warm):
        fn(i)
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for i, (e0, e1) in enumerate(pairs):
        e0.record()
        fn(i)
        e1.record()
    torch.cuda.synchronize()
    ts = sorted(e0.elapsed_time(e1) * 1e3 for e0, e1 in pairs)
    return sum(ts) / len(ts), ts[len(ts) // 2]


def bench_device():
    if not torch.cuda.is_available():
        raise RuntimeError("the benchmarks need a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    return dev


def _sync():
    torch.cuda.synchronize()


def _reset_peak(device):
    torch.cuda.reset_peak_memory_stats(device)


def _peak_gb(device):
    return torch.cuda.max_memory_allocated(device) / 1e9


def _trim():
    torch.cuda.empty_cache()


def powerlaw_graph(n, target_directed_edges, seed, device, alpha=2.1, max_degree=None):
    """Synthetic power-law graph: out-degree ~ Pareto tail with exponent alpha
    (the continuous stand-in for Zipf), rescaled to about
    `target_directed_edges` raw edges, uniformly random targets, then
    symmetrised and de-duplicated.  Returns an unvalued SparseTensor (CSR)."""
    g = torch.Generator(device=device).manual_seed(seed)
    u = torch.rand(n, generator=g, device=device).clamp_(min=1e-9)
    raw = u.pow(-1.0 / (alpha - 1.0))
    cap = float(max_degree if max_degree is not None else max(64, n // 16))
    raw.clamp_(max=cap)
    deg = (raw * (target_directed_edges / raw.sum())).round().clamp_(min=1, max=cap).long()
    src = torch.repeat_interleave(torch.arange(n, device=device), deg)
    dst = torch.randint(0, n, (src.numel(),), generator=g, device=device)
    keep = src != dst
    src, dst = src[keep], dst[keep]
    key = torch.cat([src * n + dst, dst * n + src]).unique()        # symmetrise, drop duplicates (sorted)
    row, col = torch.div(key, n, rounding_mode="floor"), key % n
    rowptr = torch.zeros(n + 1, dtype=torch.long, device=device)
    torch.cumsum(torch.bincount(row, minlength=n), 0, out=rowptr[1:])
    adj = SparseTensor(rowptr, col, None, (n, n))
    adj.storage._row = row
    return adj


def spmm_bytes(M, n_cols, nnz, K, idx_bytes, valued):
    """Compulsory traffic: index arrays + values + X once + output once."""
    return (M + 1) * idx_bytes + nnz * (idx_bytes + (4 if valued else 0)) + 4 * n_cols * K + 4 * M * K


def kernel_extras(x, log):
    """Masks, projection GEMMs and supplied-noise pack at the config-2 shape."""
    out = {}
    N, G = x.shape
    n = N * G
    # Three copies of the input, used in turn: the [169343, 256] tensor alone fits the 256 MB
    # memory-side cache, and a kernel timed on one buffer over and over reads it from there.
    import itertools
    xs = [x, x.clone(), x.clone()]
    turn = itertools.count()

    def nx():
        return xs[next(turn) % 3]
    saved = dict(config.__dict__)
    try:
        config.__dict__.update(QuantizationConfig().__dict__)
        # --- 1-bit masks ---------------------------------------------------
        mask_bytes = 8 * n + n // 8
        xr = x.clone().requires_grad_()
        y = extq.act_quantized_relu(xr)
        gys = [torch.ones_like(y) for _ in range(3)]
        gy = gys[0]

        def ngy():
            return gys[next(turn) % 3]
        t = event_time(lambda: extq.act_quantized_relu(nx()))
        out["relu_fwd"] = {"us": t * 1e6, "GB/s": mask_bytes / t / 1e9, "algo_bytes": mask_bytes}
        t = event_time(lambda: torch.autograd.grad(y, xr, ngy(), retain_graph=True))
        out["relu_bwd"] = {"us": t * 1e6, "GB/s": mask_bytes / t / 1e9, "algo_bytes": mask_bytes}
        t = event_time(lambda: extq.act_quantized_dropout(nx(), 0.5, True))
        out["dropout_fwd"] = {"us": t * 1e6, "GB/s": mask_bytes / t / 1e9, "algo_bytes": mask_bytes}
        yd = extq.act_quantized_dropout(xr, 0.5, True)
        t = event_time(lambda: torch.autograd.grad(yd, xr, ngy(), retain_graph=True))
        out["dropout_bwd"] = {"us": t * 1e6, "GB/s": mask_bytes / t / 1e9, "algo_bytes": mask_bytes}
        del y, yd, gy, gys, xr
        # --- fused epilogues: ReLU -> dropout (-> INT2 quantise + pack) in one pass --
        t = event_time(lambda: extq.relu_dropout_fwd(nx(), 0.5))
        out["relu_dropout_fwd"] = {"us": t * 1e6, "GB/s": mask_bytes / t / 1e9, "algo_bytes": mask_bytes,
                                   "replaces_us": out["relu_fwd"]["us"] + out["dropout_fwd"]["us"]}
        if extq.fusable_width(G):
            fused_bytes = mask_bytes + (2 * n) // 8 + 4 * N
            t = event_time(lambda: extq.relu_dropout_minmax_pack(nx(), 0.5, 2))
            t_pack = event_time(lambda: extq.minmax_pack(nx(), 2))
            out["relu_dropout_pack_int2"] = {"us": t * 1e6, "GB/s": fused_bytes / t / 1e9, "algo_bytes": fused_bytes,
                                             "replaces_us": out["relu_fwd"]["us"] + out["dropout_fwd"]["us"] + t_pack * 1e6}
            # batch norm folded in: statistics (torch.var_mean) + the one pass, against
            # native_batch_norm + the ReLU / dropout / pack pass
            try:
                col = torch.ones(G, device=x.device)
                t_fold = event_time(lambda: extq.bn_relu_dropout_minmax_pack(nx(), col, col, col, 0.5, 2))
                t_stats = event_time(lambda: torch.var_mean(nx(), dim=0, unbiased=False))
                t_bn = event_time(lambda: torch.ops.aten.native_batch_norm(nx(), col, col, None, None, True, 0.1, 1e-5))
                out["bn_relu_dropout_pack_int2"] = {"us": t_fold * 1e6, "GB/s": fused_bytes / t_fold / 1e9,
                                                    "algo_bytes": fused_bytes, "stats_us": t_stats * 1e6,
                                                    "replaces_us": t_bn * 1e6 + t * 1e6}
            except RuntimeError as err:          # this entry only; the other timings go on
                out["bn_relu_dropout_pack_int2"] = {"error": str(err)}
        # --- random projection 256 -> 32 (kept_frac 0.125) --------------------------------
        # Three matrix-core paths: the fp32 instruction, and the bf16 instruction on operands split in three --
        # for a Gaussian N(0, 1/k) matrix (six products) and for the +-1/sqrt(k) matrix the reference draws
        # (signs only, three products).  The default entries (rp_fwd, rp_bwd, rp_pack_int2) are what the library
        # runs by default for the reference's matrix: the signs path.
        k = int(0.125 * G + 0.999)
        rp_bytes = 4 * N * G + 4 * G * k + 4 * N * k
        flops = 2.0 * N * G * k
        gauss = torch.randn(G, k, device=x.device) / k ** 0.5
        signs = (2.0 * torch.randint(2, (G, k), device=x.device, dtype=torch.float32) - 1) / k ** 0.5
        signs._exact_sign_matrix = True
        from . import _lib
        from .cpp_extension import _checks
        L = _lib.lib()
        sp = _checks.stream_ptr(x)
        xr_small = torch.empty((N, k), device=x.device)
        backs = [torch.empty((N, G), device=x.device) for _ in range(3)]
        pk = torch.empty(extq.packed_nbytes(N, k, 2), dtype=torch.int8, device=x.device)
        sbf = torch.empty(N, dtype=torch.bfloat16, device=x.device)
        mbf = torch.empty(N, dtype=torch.bfloat16, device=x.device)

        def rp_entry(t, nbytes):
            return {"us": t * 1e6, "GB/s": nbytes / t / 1e9, "TFLOP/s": flops / t / 1e12, "algo_bytes": nbytes}

        fused_bytes = 4 * N * G + 4 * G * k + (2 * N * k) // 8 + 4 * N
        for label, R, mode in (("fp32_gaussian", gauss, 0), ("bf16_split_gaussian", gauss, 1), ("bf16_signs", signs, 2)):
            tb = extq.rp_table(R, mode) if mode else None     # prepared once per matrix (a 3 us launch), not timed
            if mode == 0:
                fw = lambda: L.exact_rp_fwd_f32(nx().data_ptr(), R.data_ptr(), N, G, k, xr_small.data_ptr(), sp)  # noqa: E731
                bw = lambda: L.exact_rp_bwd_f32(xr_small.data_ptr(), R.data_ptr(), N, G, k, backs[next(turn) % 3].data_ptr(), sp)  # noqa: E731
                fp = lambda: L.exact_rp_minmax_pack_f32(nx().data_ptr(), R.data_ptr(), None, 1, 4 * next(turn), N, G, k, 2,  # noqa: E731
                                                        pk.data_ptr(), None, None, sbf.data_ptr(), mbf.data_ptr(), sp)
            else:
                fw = lambda: L.exact_rp_fwd_bf16_f32(nx().data_ptr(), tb.data_ptr(), N, G, k, mode, xr_small.data_ptr(), sp)  # noqa: E731
                bw = lambda: L.exact_rp_bwd_bf16_f32(xr_small.data_ptr(), tb.data_ptr(), N, G, k, mode,  # noqa: E731
                                                     backs[next(turn) % 3].data_ptr(), sp)
                fp = lambda: L.exact_rp_minmax_pack_bf16_f32(nx().data_ptr(), tb.data_ptr(), mode, None, 1, 4 * next(turn), N, G,  # noqa: E731
                                                             k, 2, pk.data_ptr(), None, None, sbf.data_ptr(), mbf.data_ptr(), sp)
            out[f"rp_fwd_{label}"] = rp_entry(event_time(fw), rp_bytes)
            out[f"rp_bwd_{label}"] = rp_entry(event_time(bw), rp_bytes)
            out[f"rp_pack_int2_{label}"] = rp_entry(event_time(fp), fused_bytes)
        for name in ("rp_fwd", "rp_bwd", "rp_pack_int2"):
            out[name] = dict(out[f"{name}_bf16_signs"])
            out[name]["matrix_cores"] = "bf16, signs of the reference's +-1/sqrt(k) matrix"
        del backs
        # compress = project + quantise + pack through the Python layer (what a qlinear pays), and back
        config.kept_frac = 0.125
        t_two = event_time(lambda: ops.quantize_activation(ops.input2rp(nx(), k)[0], None))
        out["rp_compress_int2"] = {"us": t_two * 1e6}
        t_one = event_time(lambda: ops.project_and_quantize(nx(), None))
        out["rp_pack_int2"]["python_us"] = t_one * 1e6
        out["rp_pack_int2"]["replaces_us"] = t_two * 1e6
        q, R, _ = ops.project_and_quantize(x, None)
        t = event_time(lambda: ops.rp2input(ops.dequantize_activation(q, xr_small.shape), x.shape, R))
        out["rp_decompress_int2"] = {"us": t * 1e6}
        # the dense products of a layer: x W^T + b and dY^T x at 256 x 256, library kernels against the framework's GEMM
        w = torch.randn(G, G, device=x.device) / G ** 0.5
        bias = torch.randn(G, device=x.device)
        flops = 2.0 * N * G * G
        gemm_bytes = 8 * N * G + 4 * G * G
        config.tall_gemm_min_depth = 1
        w40 = torch.randn(40, G, device=x.device) / G ** 0.5
        for cores in ("bf16", "fp32"):
            config.matrix_cores = cores
            t = event_time(lambda: ext_backward_func.tall_matmul(nx(), w40, transposed=True))
            out[f"linear_forward_{G}x40_{cores}"] = {"us": t * 1e6, "TFLOP/s": 2.0 * N * G * 40 / t / 1e12,
                                                     "what": "six bf16 matrix-core products per fp32 product (library kernel)"
                                                     if cores == "bf16" else "the framework's fp32 GEMM"}
            t = event_time(lambda: ext_backward_func.tall_matmul(nx(), w, transposed=True, bias=bias))
            out[f"linear_forward_{G}x{G}_{cores}"] = {"us": t * 1e6, "TFLOP/s": flops / t / 1e12, "GB/s": gemm_bytes / t / 1e9,
                                                      "algo_bytes": gemm_bytes,
                                                      "what": "six bf16 matrix-core products per fp32 product (library kernel)"
                                                      if cores == "bf16" else "the framework's fp32 GEMM (addmm)"}
            t = event_time(lambda: ext_backward_func.weight_gradient(nx(), nx()))
            out[f"weight_gradient_{G}x{G}_{cores}"] = {"us": t * 1e6, "TFLOP/s": flops / t / 1e12,
                                                       "what": "library kernel, bf16 instruction on split operands" if cores == "bf16"
                                                       else "library kernel, fp32 instruction"}
        config.matrix_cores = "bf16"
        for name, v in out.items():
            if "GB/s" in v:
                v["frac_hbm_peak"] = v["GB/s"] / HBM_PEAK_GBS
            if "us" in v:
                log(f"  {name:<22s} {v['us']:9.1f} us" + (f"  {v['GB/s']:8.1f} GB/s" if "GB/s" in v else ""))
            else:
                log(f"  {name:<22s} {v}")
    finally:
        config.__dict__.clear()
        config.__dict__.update(saved)
    return out


def spmm_extras(adj, K, log, valued_norm=True):
    """Forward and transpose-backward SpMM on one graph at width K."""
    dev = adj.device()
    rowptr, col, value = adj.csr()
    M = adj.sparse_size(0)
    nnz = col.numel()
    X = torch.randn(M, K, device=dev)
    st = adj.storage
    reduce = "sum" if value is not None else "mean"
    t_fw = event_time(lambda: ext_spmm.spmm_csr(rowptr, col, value, X, reduce), reps=10)
    if reduce == "sum":
        bw = lambda: ext_spmm.spmm_sum_bw(st.row(), rowptr, col, value, st.colptr(), st.csr2csc(), None, X,  # noqa: E731
                                          value is not None, False, True)
    else:
        bw = lambda: ext_spmm.spmm_mean_bw(st.row(), rowptr, col, value, st.rowcount(), st.colptr(), st.csr2csc(),  # noqa: E731
                                           None, X, value is not None, False, True)
    t_bw = event_time(bw, reps=10)
    b = spmm_bytes(M, M, nnz, K, rowptr.element_size(), value is not None)
    b_bw = spmm_bytes(M, M, nnz, K, rowptr.element_size(), True)
    res = {"rows": M, "nnz": nnz, "K": K, "reduce": reduce, "index_bytes": rowptr.element_size(),
           "fwd_us": t_fw * 1e6, "bwd_us": t_bw * 1e6, "compulsory_bytes": b,
           "fwd_GB/s_compulsory": b / t_fw / 1e9, "bwd_GB/s_compulsory": b_bw / t_bw / 1e9,
           "fwd_frac_hbm_peak": b / t_fw / 1e9 / HBM_PEAK_GBS,
           "gather_bytes_no_reuse": 4 * nnz * K, "fwd_GB/s_gather": 4 * nnz * K / t_fw / 1e9,
           "fwd_GFLOP/s": 2.0 * nnz * K / t_fw / 1e9}
    log(f"  spmm {reduce} M={M} nnz={nnz} K={K}: fwd {t_fw * 1e6:.0f} us ({res['fwd_GB/s_compulsory']:.0f} GB/s compulsory, "
        f"{res['fwd_GB/s_gather']:.0f} GB/s gathered), bwd {t_bw * 1e6:.0f} us")
    return res


def train_epochs(model, x, adj, labels, train_idx, epochs, warmup, lr=0.01):
    """The reference's --test_speed loop; returns (epochs/s, last loss).  The
    loss is the mean negative log-likelihood of the training nodes, as
    F.nll_loss(out[train_idx], y[train_idx]) in arxiv/train_full_batch.py:261-262,
    written as a gather of the labelled entries: the framework's nll_loss
    kernels take 4.2 ms per epoch for 1.2 M rows of 47 classes on this GPU,
    forty times what reading those rows costs."""
    opt = torch.optim.Adam(model.parameters(), lr=lr)
    model.train()
    picked = labels[train_idx].unsqueeze(1)

    def one():
        opt.zero_grad()
        out = F.log_softmax(model(x, adj)[train_idx], dim=-1)
        loss = -out.gather(1, picked).mean()
        loss.backward()
        opt.step()
        return loss

    for _ in range(warmup):
        one()
    _sync()
    t0 = time.perf_counter()
    for _ in range(epochs):
        loss = one()
    _sync()
    dt = time.perf_counter() - t0
    return epochs / dt, float(loss.detach())


def epoch_algorithmic_bytes(kind, n, nnz, feat, hidden, classes, layers, bits, kept_frac, batch_norm, idx_bytes=4):
    """Compulsory memory traffic of one training epoch as a list of (what,
    bytes): for every step of the algorithm as this library executes it by
    default (one-node GCN / SAGE layers with the sparse product on the narrower
    side, ReLU + dropout (+ batch norm) + quantise in one pass, projection +
    quantise in one pass, second GEMMs accumulating into the first's result),
    every operand read once and every result written once.  Passes that exist
    only because two kernels were not fused -- adding a bias, adding two GEMM
    results -- are NOT counted: they are not part of the algorithm.  Loss,
    optimiser and the small per-column vectors are left out.  This is the
    numerator of the epoch's roofline fraction."""
    f4 = 4 * n
    widths = [feat] + [hidden] * (layers - 1) + [classes]
    items = []

    def add(what, nbytes):
        items.append((what, int(nbytes)))

    def packed(cols):
        return bits * n * cols / 8 + 8 * n

    def spmm(cols, valued):
        return (n + 1) * idx_bytes + nnz * (idx_bytes + (4 if valued else 0)) + 2 * f4 * cols

    def kept(cols):                                       # columns of the compressed copy of a [n, cols] activation
        return int(kept_frac * cols + 0.999) if kept_frac < 1.0 else cols

    for l in range(layers):
        cin, cout, last = widths[l], widths[l + 1], l == layers - 1
        needs_dx = l > 0
        k = kept(cin)
        if kind == "gcn":
            if l == 0 or kept_frac < 1.0:                 # later layers get their copy from the fused pass before them
                add(f"L{l} quantise input", f4 * cin + packed(k))
            narrow = min(cin, cout)
            add(f"L{l} SpMM forward (width {narrow})", spmm(narrow, True))
            add(f"L{l} GEMM with W^T", f4 * cin + f4 * cout)
            if not last:
                if batch_norm:
                    add(f"L{l} quantise batch-norm input", f4 * cout + packed(cout))
                    add(f"L{l} batch statistics", f4 * cout)
                add(f"L{l} (norm +) ReLU + dropout + quantise", 2 * f4 * cout + n * cout / 8 + (packed(cout) if kept_frac >= 1.0 else 0))
                add(f"L{l} backward: mask", 2 * f4 * cout + n * cout / 8)
                if batch_norm:
                    add(f"L{l} backward: restore norm input", packed(cout) + f4 * cout)
                    add(f"L{l} backward: norm column sums", 2 * f4 * cout)
                    add(f"L{l} backward: norm element-wise", 3 * f4 * cout)
            add(f"L{l} backward: bias gradient", f4 * cout)
            add(f"L{l} backward: restore input", packed(k) + f4 * k)
            if needs_dx or k >= cout:
                add(f"L{l} backward: SpMM transpose (width {cout})", spmm(cout, True))
                add(f"L{l} backward: dW", f4 * cout + f4 * k)
                if needs_dx:
                    add(f"L{l} backward: dX", f4 * cout + f4 * cin)
            else:                                         # first layer: the sparse product runs on the kept copy
                add(f"L{l} backward: SpMM on the kept copy (width {k})", spmm(k, True))
                add(f"L{l} backward: dW", f4 * cout + f4 * k)
        else:
            add(f"L{l} project + quantise input (shared copy)", f4 * cin + packed(k))
            if kept_frac < 1.0 and k + cout < cin:        # aggregate x [R | W_l^T]
                width = k + cout
                add(f"L{l} GEMM x [R | W_l^T]", f4 * cin + f4 * width)
                add(f"L{l} SpMM mean forward (width {width})", spmm(width, False))
                add(f"L{l} quantise aggregate copy", f4 * k + packed(k))
                add(f"L{l} GEMM lin_r (accumulating)", f4 * cin + f4 * cout)
            else:
                add(f"L{l} SpMM mean forward (width {cin})", spmm(cin, False))
                add(f"L{l} project + quantise aggregate", f4 * cin + packed(k))
                add(f"L{l} GEMM lin_l", f4 * cin + f4 * cout)
                add(f"L{l} GEMM lin_r (accumulating)", f4 * cin + f4 * cout)
            if not last:
                add(f"L{l} ReLU + dropout", 2 * f4 * cout + n * cout / 8)
                add(f"L{l} backward: mask", 2 * f4 * cout + n * cout / 8)
            add(f"L{l} backward: bias gradient", f4 * cout)
            for which in ("lin_l", "lin_r"):
                add(f"L{l} backward: restore {which} input", packed(k) + f4 * k)
                add(f"L{l} backward: dW {which}", f4 * cout + f4 * k)
            if needs_dx:
                narrow = min(cin, cout)
                add(f"L{l} backward: SpMM transpose (width {narrow})", spmm(narrow, True))
                add(f"L{l} backward: dX (two GEMMs, the second accumulating)", 2 * f4 * cout + f4 * cin)
    return items


EPOCH_CONFIGS = {
    # name: (model, N, raw directed edges, features, hidden, classes, layers, bits, kept_frac, batch_norm, dropout)
    "cfg3_gcn_int2": ("gcn", 169343, 1_160_000, 128, 256, 40, 3, 2, 1.0, True, 0.5),
    "cfg4_sage_int2_rp0.125": ("sage", 232965, 13_250_000, 602, 256, 41, 2, 2, 0.125, False, 0.5),
    "cfg5_sage_int1_rp0.25": ("sage", 2449029, 65_700_000, 100, 256, 47, 3, 1, 0.25, False, 0.5),
}


def epoch_benchmark(name, device, log, epochs=10, warmup=3, int32_index=True, scale=1.0, with_spmm=True,
                    overrides=None):
    kind, n, edges, feat, hidden, classes, layers, bits, kept_frac, bn, dropout = EPOCH_CONFIGS[name]
    n, edges = int(n * scale), int(edges * scale)
    saved = dict(config.__dict__)
    try:
        config.__dict__.update(QuantizationConfig().__dict__)
        config.activation_compression_bits, config.kept_frac = [bits], kept_frac
        for field, setting in (overrides or {}).items():
            if not hasattr(config, field):
                raise ValueError(f"no config field {field!r}")
            setattr(config, field, setting)
        t0 = time.perf_counter()
        adj = powerlaw_graph(n, edges, seed=1, device=device)
        if kind == "gcn":
            adj = gcn_norm(adj, add_self_loops=True)
        if int32_index:
            adj.to_int32_()
        adj.fill_cache_()
        nnz = adj.nnz()
        g = torch.Generator(device=device).manual_seed(2)
        x = torch.randn(n, feat, generator=g, device=device)
        labels = torch.randint(0, classes, (n,), generator=g, device=device)
        train_idx = torch.randperm(n, generator=g, device=device)[: n // 2]
        torch.manual_seed(3)
        if kind == "gcn":
            net = GCN(feat, hidden, classes, layers, dropout=dropout, batch_norm=bn)
        else:
            net = SAGE(feat, hidden, classes, layers, dropout=dropout, batch_norm=bn)
        model = QModule(net).to(device)
        _sync()
        setup_s = time.perf_counter() - t0
        _reset_peak(device)
        eps, loss = train_epochs(model, x, adj, labels, train_idx, epochs, warmup)
        parts = epoch_algorithmic_bytes(kind, n, nnz, feat, hidden, classes, layers, bits, kept_frac, bn,
                                        4 if int32_index else 8)
        epoch_bytes = sum(b for _, b in parts)
        res = {"epochs_per_s": eps, "ms_per_epoch": 1e3 / eps, "nodes": n, "nnz": nnz, "features": feat,
               "epoch_roofline": {"bound": "hbm", "algo_bytes_per_epoch": epoch_bytes,
                                  "achieved": epoch_bytes * eps / 1e9, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                                  "frac": epoch_bytes * eps / 1e9 / HBM_PEAK_GBS,
                                  "largest_parts": sorted(parts, key=lambda p: -p[1])[:6],
                                  "note": "compulsory traffic of the epoch's compression / aggregation / GEMM kernels "
                                          "(every operand read once, every result written once) over the epoch time"},
               "hidden": hidden, "classes": classes, "layers": layers, "bits": bits, "kept_frac": kept_frac,
               "index_dtype": "int32" if int32_index else "int64", "epochs_timed": epochs, "last_loss": loss,
               "setup_s": setup_s, "peak_mem_GB": _peak_gb(device)}
        log(f"  {name}: {eps:.2f} epochs/s ({1e3 / eps:.1f} ms/epoch), N={n}, nnz={nnz}, peak {res['peak_mem_GB']:.1f} GB, "
            f"compulsory traffic {epoch_bytes / 1e9:.2f} GB/epoch = {100 * res['epoch_roofline']['frac']:.1f}% of HBM peak")
        if with_spmm:
            res["spmm"] = spmm_extras(adj, hidden if kind == "gcn" else feat, log)
        return res
    finally:
        config.__dict__.clear()
        config.__dict__.update(saved)
        ext_spmm.clear_csc_cache()


def run(x, log, budget_s=240.0, epoch_configs=("cfg3_gcn_int2", "cfg4_sage_int2_rp0.125", "cfg5_sage_int1_rp0.25"),
        scale=1.0, epochs=10, warmup=3):
    """Everything beyond the headline number; each part is independent and a
    failure or an exhausted time budget in one only drops that part."""
    t_start = time.perf_counter()
    out = {}
    try:
        out["kernels"] = kernel_extras(x, log)
    except Exception as e:  # noqa: BLE001
        out["kernels"] = {"error": f"{type(e).__name__}: {e}"}
    _trim()
    for name in epoch_configs:
        if time.perf_counter() - t_start > budget_s:
            out[name] = {"skipped": "time budget of the default run exhausted"}
            continue
        try:
            out[name] = epoch_benchmark(name, x.device, log, epochs=epochs, warmup=warmup, scale=scale)
        except Exception as e:  # noqa: BLE001
            out[name] = {"error": f"{type(e).__name__}: {e}"}
        _trim()
    return out


def headline_input(rows, cols, device):
    """The benchmark activation: fp32 [rows, cols] ~ N(0,1), fixed seed."""
    gen = torch.Generator(device=device).manual_seed(1234)
    return torch.randn((rows, cols), generator=gen, device=device, dtype=torch.float32)


def _extras_main(argv):
    """`python -m exact_amd.benchmarks extras`: run() in a process of its own
    and print its result as one JSON line (bench.py starts it as a child, so
    that nothing that happens here can take the headline figure with it)."""
    import argparse
    import json
    ap = argparse.ArgumentParser(prog="python -m exact_amd.benchmarks extras")
    ap.add_argument("--rows", type=int, default=169343)
    ap.add_argument("--cols", type=int, default=256)
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--budget", type=float, default=240.0)
    args = ap.parse_args(argv)

    def log(*a):
        print(*a, file=sys.stderr, flush=True)

    dev = bench_device()
    x = headline_input(args.rows, args.cols, dev)
    print(json.dumps(run(x, log, budget_s=args.budget, scale=args.scale)), flush=True)


def _epoch_main(argv):
    """`python -m exact_amd.benchmarks epoch --config cfg3_gcn_int2 --epochs 5`:
    a few full-batch training epochs of one model configuration, as the target
    of a kernel trace (which kernels an epoch spends its time in)."""
    import argparse
    import json
    ap = argparse.ArgumentParser(prog="python -m exact_amd.benchmarks epoch")
    ap.add_argument("--config", choices=sorted(EPOCH_CONFIGS), default="cfg3_gcn_int2")
    ap.add_argument("--epochs", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--scale", type=float, default=1.0)
    ap.add_argument("--epochs-only", action="store_true", help="leave out the separate SpMM timings after the epochs")
    ap.add_argument("--set", action="append", default=[], metavar="FIELD=VALUE",
                    help="a boolean (0 | 1) or integer field of exact_amd.config to set for the run, e.g. "
                         "--set sage_single_node=0 --set tall_gemm_min_rows=1000000000")
    args = ap.parse_args(argv)
    overrides = {f: (bool(int(v)) if isinstance(getattr(config, f), bool) else int(v))
                 for f, v in (item.split("=", 1) for item in args.set)}

    def log(*a):
        print(*a, file=sys.stderr, flush=True)

    res = epoch_benchmark(args.config, bench_device(), log, epochs=args.epochs, warmup=args.warmup, scale=args.scale,
                          with_spmm=not args.epochs_only, overrides=overrides)
    res["config_overrides"] = overrides
    print(json.dumps(res), flush=True)


def _profile_target(argv=None):
    """One kernel in a loop, as the target of `rocprofv3 --kernel-trace --stats` /
    `--pmc FETCH_SIZE` / `--pmc WRITE_SIZE` runs:

        python -m exact_amd.benchmarks pack --bits 2 --reps 100
        python -m exact_amd.benchmarks {unpack,relu,dropout,relu_dropout_pack,bn_relu_dropout_pack,rp_fwd,rp_bwd,rp_pack,spmm,copy,probe,dw,gemm} ...
        python -m exact_amd.benchmarks epoch --config cfg3_gcn_int2 --epochs 5

    `copy` is a plain device-to-device copy of the same [rows, cols] fp32 tensor
    (4*rows*cols bytes read, as many written) for calibrating the byte counters;
    `probe` is the library's traffic probe with the pack kernel's byte mix at --bits."""
    import argparse

    from . import _lib
    from .cpp_extension import _checks
    if argv is None:
        argv = sys.argv[1:]
    if argv and argv[0] == "extras":
        return _extras_main(argv[1:])
    if argv and argv[0] == "epoch":
        return _epoch_main(argv[1:])
    ap = argparse.ArgumentParser(prog="python -m exact_amd.benchmarks")
    ap.add_argument("kernel", choices=["pack", "unpack", "relu", "dropout", "relu_dropout_pack", "bn_relu_dropout_pack", "rp_fwd", "rp_bwd",
                                      "rp_pack", "spmm", "copy", "probe", "dw", "gemm"])
    ap.add_argument("--fp32-cores", action="store_true", help="dw only: the fp32 matrix-core kernel instead of the bf16 one")
    ap.add_argument("--cold", action="store_true",
                    help="unpack only: every launch reads another copy of the packed stream (48 copies, 0.5 GB at 2 bits: none of it cached)")
    ap.add_argument("--rp-path", choices=["fp32", "split", "signs"], default="signs",
                    help="rp_* only: the fp32 matrix-core instruction on a Gaussian matrix, the bf16 instruction on split "
                         "operands (Gaussian matrix), or on the signs of a +-1/sqrt(k) matrix (the default path)")
    ap.add_argument("--bits", type=int, default=2)
    ap.add_argument("--rows", type=int, default=169343)
    ap.add_argument("--cols", type=int, default=256)
    ap.add_argument("--reps", type=int, default=100)
    ap.add_argument("--supplied-noise", action="store_true")
    ap.add_argument("--config", choices=sorted(EPOCH_CONFIGS), default="cfg3_gcn_int2",
                    help="spmm only: the graph of this model configuration")
    ap.add_argument("--width", type=int, default=0, help="spmm: columns of the dense operand; gemm: columns of the result (0 = --cols)")
    args = ap.parse_args(argv)
    dev = bench_device()
    L = _lib.lib()
    N, G, b = args.rows, args.cols, args.bits
    gen = torch.Generator(device=dev).manual_seed(1234)
    # three input / output sets, used in turn: a launch finds neither its input nor the lines it
    # writes in the 256 MB memory-side cache (one 173 MB output written over and over would stay there)
    xs = [torch.randn((N, G), generator=gen, device=dev) for _ in range(3)]
    outs = [torch.empty_like(xs[0]) for _ in range(3)]
    x, out = xs[0], outs[0]
    sp = _checks.stream_ptr(x)
    packed = torch.empty(int(L.exact_packed_nbytes(N, G, b)), dtype=torch.int8, device=dev)
    sbf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    mbf = torch.empty(N, dtype=torch.bfloat16, device=dev)
    noise = torch.rand((N, G), generator=gen, device=dev) if args.supplied_noise else None
    mask = torch.empty((N * G + 31) // 32, dtype=torch.int32, device=dev)
    L.exact_minmax_pack_f32(x.data_ptr(), None, 1, 1, N, G, b, packed.data_ptr(), None, None, sbf.data_ptr(),
                            mbf.data_ptr(), sp)
    k = int(0.125 * G + 0.999)
    if args.rp_path == "signs":
        R = (2.0 * torch.randint(2, (G, k), generator=gen, device=dev, dtype=torch.float32) - 1) / k ** 0.5
    else:
        R = torch.randn(G, k, generator=gen, device=dev) / k ** 0.5
    rp_mode = {"fp32": 0, "split": 1, "signs": 2}[args.rp_path]
    rp_tb = extq.rp_table(R, rp_mode) if rp_mode else R
    xr = torch.empty((N, k), device=dev)
    packed_k = torch.empty(int(L.exact_packed_nbytes(N, k, b)), dtype=torch.int8, device=dev)
    ones = torch.ones(G, device=dev)
    if args.kernel == "spmm":
        kind, n_nodes, n_edges = EPOCH_CONFIGS[args.config][:3]
        adj = powerlaw_graph(n_nodes, n_edges, seed=1, device=dev)
        adj = (gcn_norm(adj) if kind == "gcn" else adj).to_int32_()
        rowptr, col, value = adj.csr()
        spmm_x = torch.randn((n_nodes, args.width or G), generator=gen, device=dev)
        spmm_reduce = "sum" if kind == "gcn" else "mean"
    packs = [packed] + [packed.clone() for _ in range(47)] if args.cold else [packed]
    dw_out = torch.empty((G, G), device=dev)
    dw_entry = L.exact_linear_dw_f32 if args.fp32_cores else L.exact_linear_dw_bf16_f32
    gemm_w = torch.randn((args.width or G, G), generator=gen, device=dev) / G ** 0.5   # a weight [out, in]
    fns = {
        # x W^T as a layer computes it: the library's bf16 matrix-core kernel where the shim selects it
        "gemm": lambda i: ext_backward_func.tall_matmul(xs[i % 3], gemm_w, transposed=True),
        "dw": lambda i: dw_entry(xs[i % 3].data_ptr(), G, xs[(i + 1) % 3].data_ptr(), G, N, G, G, dw_out.data_ptr(), sp),
        "pack": lambda i: L.exact_minmax_pack_f32(xs[i % 3].data_ptr(), noise.data_ptr() if noise is not None else None, 1,
                                                  i, N, G, b, packed.data_ptr(), None, None, sbf.data_ptr(),
                                                  mbf.data_ptr(), sp),
        "unpack": lambda i: L.exact_unpack_bf16param_f32(packs[i % len(packs)].data_ptr(), b, sbf.data_ptr(), mbf.data_ptr(), N, G,
                                                         outs[i % 3].data_ptr(), sp),
        "relu": lambda i: L.exact_relu_fwd_f32(xs[i % 3].data_ptr(), N * G, outs[i % 3].data_ptr(), mask.data_ptr(), sp),
        "dropout": lambda i: L.exact_dropout_fwd_f32(xs[i % 3].data_ptr(), None, 1, i, 0.5, N * G, outs[i % 3].data_ptr(),
                                                     mask.data_ptr(), sp),
        "relu_dropout_pack": lambda i: L.exact_relu_dropout_minmax_pack_f32(
            xs[i % 3].data_ptr(), 0.5, None, 1, 8 * i, None, 1, 8 * i + 4, N, G, b, outs[i % 3].data_ptr(), mask.data_ptr(),
            packed.data_ptr(), None, None, sbf.data_ptr(), mbf.data_ptr(), sp),
        "bn_relu_dropout_pack": lambda i: L.exact_bn_relu_dropout_minmax_pack_f32(
            xs[i % 3].data_ptr(), ones.data_ptr(), ones.data_ptr(), ones.data_ptr(), 0.5, None, 1, 8 * i, None, 1, 8 * i + 4, N, G,
            b, outs[i % 3].data_ptr(), mask.data_ptr(), packed.data_ptr(), None, None, sbf.data_ptr(), mbf.data_ptr(), sp),
        "rp_pack": (lambda i: L.exact_rp_minmax_pack_f32(xs[i % 3].data_ptr(), R.data_ptr(), None, 1, i, N, G, k, b,
                                                         packed_k.data_ptr(), None, None, sbf.data_ptr(), mbf.data_ptr(),
                                                         sp)) if rp_mode == 0 else
                   (lambda i: L.exact_rp_minmax_pack_bf16_f32(xs[i % 3].data_ptr(), rp_tb.data_ptr(), rp_mode, None, 1, i, N, G, k,
                                                              b, packed_k.data_ptr(), None, None, sbf.data_ptr(),
                                                              mbf.data_ptr(), sp)),
        "rp_fwd": (lambda i: L.exact_rp_fwd_f32(xs[i % 3].data_ptr(), R.data_ptr(), N, G, k, xr.data_ptr(), sp)) if rp_mode == 0
                  else (lambda i: L.exact_rp_fwd_bf16_f32(xs[i % 3].data_ptr(), rp_tb.data_ptr(), N, G, k, rp_mode, xr.data_ptr(), sp)),
        "rp_bwd": (lambda i: L.exact_rp_bwd_f32(xr.data_ptr(), R.data_ptr(), N, G, k, outs[i % 3].data_ptr(), sp)) if rp_mode == 0
                  else (lambda i: L.exact_rp_bwd_bf16_f32(xr.data_ptr(), rp_tb.data_ptr(), N, G, k, rp_mode, outs[i % 3].data_ptr(), sp)),
        "spmm": lambda i: ext_spmm.spmm_csr(rowptr, col, value, spmm_x, spmm_reduce),
        "copy": lambda i: outs[i % 3].copy_(xs[i % 3]),
        # the pack kernel's traffic without its arithmetic: 64 bytes in, 2 * bits bytes out per lane
        "probe": lambda i: L.exact_stream_probe_f32(xs[i % 3].data_ptr(), N * G, 2 * b, outs[i % 3].data_ptr(), sp),
    }
    fn = fns[args.kernel]
    for i in range(args.reps):
        rc = fn(i + 2)
        if isinstance(rc, int) and rc != 0:
            raise RuntimeError(f"{args.kernel}: entry point returned {rc}")
    _sync()
    print(f"{args.kernel}: {args.reps} launches on [{N}, {G}] done")


if __name__ == "__main__":
    _profile_target()
