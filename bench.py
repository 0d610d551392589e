#!/usr/bin/env python3
"""Benchmark of EXACT's activation pack/unpack hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the op-level microbenchmark configuration): fp32 activations [169343, 256] ~ N(0,1)
in device memory.  One step = quantize_activation + dequantize_activation at
every bit width {1,2,4,8}: per-row min/range + stochastic-rounding quantise +
bit-pack (internal Philox noise), then unpack + dequantise with the bf16
scale/min -- eight kernel launches through the C ABI of libexact_hip.so on
preallocated buffers.  The steps rotate over four sets of buffers so that no
step finds its operands in a cache.  `value` is the algorithmic bytes of a
step divided by its time.  Beside it: every kernel's duration (one HIP event
pair per launch), the supplied-noise form of the pack kernel, the CPU
restatement on the host's cores, and -- from a child process -- the other
kernels of the path and epochs/s of the three full-batch model configurations
with the roofline fraction of an epoch.  Prints ONE JSON line on stdout;
progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "oracle")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
N_ROWS, N_COLS = 169343, 256
BITS = (1, 2, 4, 8)
ROTATE = 4             # buffer sets the timed steps rotate over


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def packed_bytes(N, G, b):
    wpt = 8 // b
    n_round = N + (wpt - N % wpt) % wpt
    return b * n_round * G // 8


def algo_bytes_pack(N, G, b, supplied_noise=False):
    """read x (+ noise), write the packed stream + bf16 scale and min"""
    return 4 * N * G * (2 if supplied_noise else 1) + packed_bytes(N, G, b) + 4 * N


def algo_bytes_unpack(N, G, b):
    """read the packed stream + bf16 scale and min, write fp32 [N, G]"""
    return packed_bytes(N, G, b) + 4 * N + 4 * N * G


def cpu_baseline(x_host, step_bytes, seed, min_seconds=10.0, max_passes=20):
    """The C restatement of the reference algorithm (oracle/exact_oracle.c,
    OpenMP) on the same workload, timed on this machine's host cores."""
    import c_oracle
    N, G = x_host.shape
    threads = c_oracle.num_threads()
    c_oracle.pack_unpack_roundtrip(x_host[:4096], 2, None, seed, 0)  # warm up the thread pool
    t0 = time.perf_counter()
    passes = 0
    while True:
        for b in BITS:
            c_oracle.pack_unpack_roundtrip(x_host, b, None, seed, passes)
        passes += 1
        if time.perf_counter() - t0 > min_seconds or passes >= max_passes:
            break
    cpu_s = (time.perf_counter() - t0) / passes
    return {"value": step_bytes / cpu_s / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"{passes} full steps of the same workload ([{N},{G}] fp32, bits 1/2/4/8, pack+unpack, Philox "
                      f"noise) with oracle/exact_oracle.c (OpenMP, {threads} threads), including the reference's "
                      f"separate min and max passes (ops.py:61-66); bytes counted as for the GPU",
            "seconds_per_step": cpu_s, "host_cpus": os.cpu_count()}


def run_extras(rows, cols, scale, timeout_s=300):
    """The secondary measurements (mask / projection / SpMM kernels, epochs/s of
    the three model configurations) in a child process: whatever happens there,
    the headline figures measured in this process are still printed."""
    import subprocess
    cmd = [sys.executable, "-m", "exact_amd.benchmarks", "extras", "--rows", str(rows), "--cols", str(cols),
           "--scale", str(scale), "--budget", str(timeout_s / 2)]   # no part starts in the second half of the limit
    try:
        res = subprocess.run(cmd, cwd=ROOT, stdout=subprocess.PIPE, timeout=timeout_s, text=True)
    except subprocess.TimeoutExpired:
        return {"error": f"extras child exceeded {timeout_s} s"}
    except OSError as e:
        return {"error": f"extras child could not start: {e}"}
    lines = [ln for ln in res.stdout.splitlines() if ln.startswith("{")]
    if res.returncode != 0 or not lines:
        return {"error": f"extras child exited with {res.returncode}"}
    return json.loads(lines[-1])


def other_rooflines(extras):
    """roofline-style objects for the sparse product and the projection, from the
    durations the extras child measured live and the counter-derived traffic of
    the committed rocprofv3 runs (profiles/hbm_traffic.json; null where no such
    run covers the kernel)."""
    counters = {}
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        counters = json.load(open(tpath))
    out = {}
    for cfg, v in extras.items():
        sp_ = v.get("spmm") if isinstance(v, dict) else None
        if not sp_:
            continue
        key = f"spmm_chunk_kernel, {cfg} graph, K={sp_['K']}"
        out[key] = {"bound": "hbm", "achieved": sp_["fwd_GB/s_compulsory"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": sp_["fwd_frac_hbm_peak"], "traffic": counters.get(key, {}).get("traffic_bytes_per_launch"),
                    "avg_launch_us": sp_["fwd_us"], "algo_bytes_per_launch": sp_["compulsory_bytes"],
                    "gathered_GB/s": sp_["fwd_GB/s_gather"],
                    "note": "compulsory bytes (indices + values + the dense operand once + the result once) over the "
                            "launch time; the kernel gathers nnz * K * 4 bytes, reported as gathered_GB/s"}
    ks = extras.get("kernels", {}) if isinstance(extras.get("kernels"), dict) else {}
    for name, label in (("rp_fwd", "rp_fwd_bf16_kernel (256 -> 32)"), ("rp_bwd", "rp_bwd_bf16_kernel (32 -> 256)"),
                        ("rp_pack_int2", "rp_fwd_pack_bf16_kernel (256 -> 32, INT2)")):
        k = ks.get(name)
        if not k or "GB/s" not in k:
            continue
        c = counters.get(label, {})
        out[label] = {"bound": "hbm", "achieved": k["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": k["GB/s"] / HBM_PEAK_GBS,
                      "traffic": c.get("traffic_bytes_per_launch"), "avg_launch_us": k["us"], "algo_bytes_per_launch": k["algo_bytes"],
                      "matrix_cores": {"TFLOP/s": k.get("TFLOP/s"), "instruction": "v_mfma_f32_32x32x16_bf16, 3 per fp32 product",
                                       "busy_fraction_by_counter": c.get("mfma_busy_fraction")}}
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--rows", type=int, default=N_ROWS, help=argparse.SUPPRESS)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true")
    ap.add_argument("--extras-scale", type=float, default=1.0, help=argparse.SUPPRESS)
    ap.add_argument("--extras-in-process", action="store_true", help=argparse.SUPPRESS)
    args = ap.parse_args(argv)
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU; --gpus must be 1 (the path has no multi-GPU code; "
                 "row blocks aligned to 8 rows would shard it without communication)")

    import torch
    from exact_amd import _lib, benchmarks
    from exact_amd.cpp_extension import _checks

    L = _lib.lib()  # raises if the HIP library is missing: there is no fallback
    dev = benchmarks.bench_device()
    N, G = args.rows, N_COLS
    # ROTATE buffer sets, each with its own input, packed streams and output.  One set is 173 MB in, 81 MB packed,
    # 173 MB out; a step touches one set, so a set is re-used only after (ROTATE - 1) * 1.4 GB of other traffic --
    # nothing of it is left in the 256 MB memory-side cache or the L2s.  `value` is measured this way; the
    # single-set figure (every step re-reads the same 173 MB input) is reported beside it.
    sets = []
    for i in range(ROTATE):
        gen = torch.Generator(device=dev).manual_seed(1234 + i)
        xi = torch.randn((N, G), generator=gen, device=dev, dtype=torch.float32)
        sets.append({"x": xi, "out": torch.empty_like(xi),
                     "packed": {b: torch.empty(int(L.exact_packed_nbytes(N, G, b)), dtype=torch.int8, device=dev) for b in BITS},
                     "sbf": torch.empty(N, dtype=torch.bfloat16, device=dev),
                     "mbf": torch.empty(N, dtype=torch.bfloat16, device=dev)})
    x = sets[0]["x"]
    sp = _checks.stream_ptr(x)
    noise = torch.rand((N, G), generator=torch.Generator(device=dev).manual_seed(99), device=dev)
    seed = 0x5EED
    calls = [0]

    # Work split of the pack kernel: the library times its alternatives (1, 2 or 4
    # column groups per lane, same result) once per (width, bits) and keeps the fastest.
    from exact_amd.cpp_extension import quantization as extq
    geometry = {"octs_per_lane": {}, "candidates_us": {}}
    for b in BITS:
        if x.is_cuda:
            try:
                tried = extq.tune_pack_geometry(x, b)
                geometry["candidates_us"][str(b)] = {str(c): t * 1e6 for c, t in tried.items()}
            except RuntimeError as e:       # keep the library's default split; the headline is still measured
                log(f"pack work split not tuned for {b} bits: {e}")
        geometry["octs_per_lane"][str(b)] = extq._PACK_GEOMETRY.get((G, b), 0)
    log(f"pack work split (octs per lane) by bits: {geometry['octs_per_lane']}")

    def pack(b, s, supplied=False):
        calls[0] += 1
        rc = L.exact_minmax_pack_geom_f32(s["x"].data_ptr(), noise.data_ptr() if supplied else None, seed, calls[0], N, G, b,
                                          s["packed"][b].data_ptr(), None, None, s["sbf"].data_ptr(), s["mbf"].data_ptr(),
                                          geometry["octs_per_lane"][str(b)], sp)
        assert rc == 0, rc

    def unpack(b, s):
        rc = L.exact_unpack_bf16param_f32(s["packed"][b].data_ptr(), b, s["sbf"].data_ptr(), s["mbf"].data_ptr(), N, G,
                                          s["out"].data_ptr(), sp)
        assert rc == 0, rc

    def step(s):
        for b in BITS:
            pack(b, s)
            unpack(b, s)

    def timed(nsteps, which):
        benchmarks._sync()
        t0 = time.perf_counter()
        for i in range(nsteps):
            step(which(i))
        benchmarks._sync()
        return (time.perf_counter() - t0) / nsteps * 1e3

    step_bytes = sum(algo_bytes_pack(N, G, b) + algo_bytes_unpack(N, G, b) for b in BITS)
    for i in range(args.warmup):
        step(sets[i % ROTATE])
    # The headline: exactly `steps` steps over the rotating sets, timed as one region.  A region of a few
    # milliseconds is at the mercy of whatever else the machine does in that moment, so the region is repeated
    # until about a second has been measured (at least three times) and the median region is the one reported.
    first = timed(args.steps, lambda i: sets[i % ROTATE])
    repeats = max(3, min(400, int(1.0 / max(first * args.steps * 1e-3, 1e-6)) + 1)) if x.is_cuda else 1
    regions = sorted([first] + [timed(args.steps, lambda i: sets[i % ROTATE]) for _ in range(repeats - 1)])
    ms_per_step = regions[len(regions) // 2]
    ms_single = timed(args.steps, lambda i: sets[0])                      # every step on the same set
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    value_single = step_bytes / (ms_single * 1e-3) / 1e9
    log(f"pack+unpack, bits 1/2/4/8, {ROTATE} rotating buffer sets: {ms_per_step:.3f} ms/step, {value:.1f} GB/s = "
        f"{100 * value / HBM_PEAK_GBS:.1f}% of HBM peak   (median of {len(regions)} regions of {args.steps} steps, "
        f"{regions[0]:.3f} .. {regions[-1]:.3f} ms/step; one set re-used: {ms_single:.3f} ms/step, {value_single:.1f} GB/s)")

    # ---- per-kernel durations, HIP events on the launch stream -----------------
    # `us`: one event pair around a run of 40 launches of the same kernel (median of three runs), rotating
    # over the buffer sets like the timed region, divided by 40 -- launches of one
    # stream run one after the other, so this is the kernel's duration plus the
    # sub-microsecond gap between dispatches, and it is what a kernel trace of this
    # program reports per dispatch.  `single_launch_us`: an event pair around EACH
    # launch, which adds the events' own few microseconds.
    def per_launch_us(fn, reps=40):
        counter = [0]

        def one():
            fn(sets[counter[0] % ROTATE])
            counter[0] += 1
        # the median of three such runs: a single one is now and then disturbed by several microseconds
        run_us = sorted(benchmarks.event_time(one, reps=reps, warm=4) * 1e6 for _ in range(3))[1]
        single_us, _ = benchmarks.launch_times(lambda i: fn(sets[i % ROTATE]), reps=reps, warm=0)
        return run_us, single_us

    kernels = []
    for b in BITS:
        for name, does, fn, nbytes in (
                (f"pack_kernel<bits={b}>", "row min/max + scale + stochastic quantise + bit-pack + bf16 scale/min, Philox noise",
                 lambda s, b=b: pack(b, s), algo_bytes_pack(N, G, b)),
                (f"pack_kernel<bits={b}>, supplied noise", "the same with a uniform[0,1) noise tensor read from memory "
                 "(the parity mode; 4 more bytes per element)", lambda s, b=b: pack(b, s, True), algo_bytes_pack(N, G, b, True)),
                (f"unpack_kernel<bits={b}>", "unpack + dequantise with bf16 scale/min", lambda s, b=b: unpack(b, s),
                 algo_bytes_unpack(N, G, b))):
            mean_us, single_us = per_launch_us(fn)
            kernels.append({"kernel": name, "does": does, "us": mean_us, "single_launch_us": single_us, "algo_bytes": nbytes,
                            "GB/s": nbytes / mean_us / 1e3})
    # Unpack as a training step meets it: backward reads a packed stream that forward wrote long before, so it
    # comes from HBM, not from L2 as in the pack -> unpack step above.  Timed over enough copies of the packed
    # stream (about half a gigabyte) that none is left in a cache when its turn comes again.
    if x.is_cuda:
        for b in BITS:
            nb = int(L.exact_packed_nbytes(N, G, b))
            copies = max(4, min(64, int(5.2e8 // nb)))
            cold = [{"packed": torch.empty(nb, dtype=torch.int8, device=dev), "sbf": torch.empty(N, dtype=torch.bfloat16, device=dev),
                     "mbf": torch.empty(N, dtype=torch.bfloat16, device=dev)} for _ in range(copies)]
            for i, cset in enumerate(cold):
                rc = L.exact_minmax_pack_f32(sets[i % ROTATE]["x"].data_ptr(), None, seed, 1000 + i, N, G, b, cset["packed"].data_ptr(),
                                             None, None, cset["sbf"].data_ptr(), cset["mbf"].data_ptr(), sp)
                assert rc == 0, rc
            turn = [0]

            def unpack_cold(s, b=b, cold=cold, turn=turn):
                cset = cold[turn[0] % len(cold)]
                turn[0] += 1
                rc = L.exact_unpack_bf16param_f32(cset["packed"].data_ptr(), b, cset["sbf"].data_ptr(), cset["mbf"].data_ptr(), N, G,
                                                  s["out"].data_ptr(), sp)
                assert rc == 0, rc
            mean_us, single_us = per_launch_us(unpack_cold)
            kernels.append({"kernel": f"unpack_kernel<bits={b}>, packed stream from HBM",
                            "does": f"the same on {copies} packed streams in turn, as in a backward pass (not part of the timed step)",
                            "us": mean_us, "single_launch_us": single_us, "algo_bytes": algo_bytes_unpack(N, G, b),
                            "GB/s": algo_bytes_unpack(N, G, b) / mean_us / 1e3})
            del cold
        benchmarks._trim()
    # What the memory system delivers for each pack kernel's mix of reads and writes: a kernel
    # without arithmetic that reads the same tensor and writes as many bytes (the library's
    # traffic probe), timed the same way.  Peak stays the published 8 TB/s; this is the bar
    # a kernel of this traffic can reach on this device.
    probe_out = torch.empty(max(16, (N * G // 16) * 16), dtype=torch.uint8, device=dev)
    probe = {}
    for b in BITS:
        def run_probe(s, b=b):
            rc = L.exact_stream_probe_f32(s["x"].data_ptr(), N * G, 2 * b, probe_out.data_ptr(), sp)
            assert rc == 0, rc
        us, _ = per_launch_us(run_probe)
        nbytes = (N * G // 4096) * 4096 * 4 + (N * G // 4096) * 256 * 2 * b
        probe[b] = {"us": us, "GB/s": nbytes / us / 1e3}
        log(f"  traffic probe, {2 * b:2d} bytes out per 64 in     {us:8.1f} us  {nbytes / us / 1e3:8.1f} GB/s  "
            f"{100 * nbytes / us / 1e3 / HBM_PEAK_GBS:5.1f}% of HBM peak")
    del probe_out
    for k in kernels:
        k["frac_hbm_peak"] = k["GB/s"] / HBM_PEAK_GBS
        if k["kernel"].startswith("pack_kernel") and "supplied" not in k["kernel"]:
            b = int(k["kernel"].split("bits=")[1].split(">")[0])
            k["traffic_probe_us"] = probe[b]["us"]
            k["frac_of_traffic_probe"] = probe[b]["us"] / k["us"]
        log(f"  {k['kernel']:<40s} {k['us']:8.1f} us  {k['GB/s']:8.1f} GB/s  {100 * k['frac_hbm_peak']:5.1f}% of HBM peak")
    in_step = [k for k in kernels if "supplied" not in k["kernel"] and "from HBM" not in k["kernel"]]
    dom = max(in_step, key=lambda k: k["us"])
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get(dom["kernel"], {}).get("traffic_bytes_per_launch")
    roofline = {"bound": "hbm", "kernel": dom["kernel"], "achieved": dom["GB/s"], "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": dom["GB/s"] / HBM_PEAK_GBS, "traffic": traffic,
                "avg_launch_us": dom["us"], "algo_bytes_per_launch": dom["algo_bytes"],
                "timing": "HIP events on the launch stream around 40 consecutive launches rotating over the buffer sets, median of three such runs"}
    if "traffic_probe_us" in dom:
        roofline["traffic_probe"] = {"us": dom["traffic_probe_us"], "frac_of_it": dom["frac_of_traffic_probe"],
                                     "what": "a kernel without arithmetic that reads the same tensor and writes as many "
                                             "bytes as this kernel (exact_stream_probe_f32), timed the same way"}

    cpu = None
    if not args.no_cpu_baseline:
        try:
            cpu = cpu_baseline(x.cpu().numpy(), step_bytes, seed)
            log(f"  cpu baseline: {cpu['value']:.2f} GB/s on {cpu['cores']} threads ({cpu['seconds_per_step']:.2f} s/step)")
        except Exception as e:  # noqa: BLE001
            log(f"cpu baseline failed: {type(e).__name__}: {e}")

    del sets[1:], noise
    benchmarks._trim()
    if args.no_extras:
        extras = {}
    elif args.extras_in_process:
        extras = benchmarks.run(x, log, scale=args.extras_scale)
    else:
        extras = run_extras(N, G, args.extras_scale)
    if "error" in extras:
        log(f"extras: {extras['error']}")

    result = {
        "metric": "pack+unpack GB/s (% HBM peak); INT2 GCN/SAGE full-batch epochs/s",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": "config 2: fp32 activation [169343 x 256] ~N(0,1); per-row min/range + stochastic "
                               "quantise + bit-pack, then unpack + dequantise, at bits {1,2,4,8}; internal Philox "
                               "noise; operands in device memory, steps rotate over 4 buffer sets (1.7 GB) so that "
                               "no step finds its input in a cache",
                   "rows": N, "cols": G, "bits": list(BITS), "algo_bytes_per_step": step_bytes,
                   "buffer_sets": ROTATE},
        "pct_hbm_peak": 100.0 * value / HBM_PEAK_GBS,
        "single_buffer_set": {"value": value_single, "ms_per_step": ms_single,
                              "note": "every step re-reads the same 173 MB input (smaller than the 256 MB memory-side cache)"},
        "epochs_per_s": {k: v.get("epochs_per_s") for k, v in extras.items() if isinstance(v, dict) and k.startswith("cfg")},
        "epoch_roofline": {k: v.get("epoch_roofline") for k, v in extras.items()
                           if isinstance(v, dict) and k.startswith("cfg") and "epoch_roofline" in v},
        "roofline": roofline, "other_rooflines": other_rooflines(extras), "cpu_baseline": cpu, "kernels": kernels,
        "pack_geometry": geometry, "extras": extras,
    }
    print(json.dumps(result), flush=True)
    return result


if __name__ == "__main__":
    main()
