"""Benchmark of the SpMM hot path on one MI355X.

One step = one SpMM C = A*B (hspmm_run through the C ABI) on synthetic inputs that
are resident in HBM before the timed region starts.  Prints one JSON line:
effective TFLOP/s (2*nnz*N / t) as `value`, the HBM roofline of the main kernel
(compulsory bytes / its measured duration against 8 TB/s) and a CPU baseline (the
oracle's CSR SpMM on this machine's host cores).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 0..4] [--n N]
                  [--no-cpu-baseline]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
# dense peak of the matrix instruction a kernel issues (hspmm_plan_info.last_mfma_kind)
MFMA = {1: ("v_mfma_f32_16x16x32_f16", 2500.0), 2: ("v_mfma_f32_16x16x32_bf16", 2500.0),
        3: ("v_mfma_f32_16x16x4_f32", 157.3), 4: ("v_mfma_f32_4x4x1_16B_f32", 157.3)}
# which roofline binds each configuration by its compulsory bytes and padded flops: the pruned fp32 weight and the
# block-clustered weight at N = 512 are bound by the matrix cores, the rest by HBM
BOUND = {(3, 256): "mfma", (4, 512): "mfma"}
KERNELS = {1: "spmm_scalar_kernel", 2: "spmm_mfma_kernel", 3: "spmm_panel_kernel"}


def mfma_report(info, useful_flops, kernel_ms):
    """Matrix-core use of the last launch: flops issued (zero padding of tiles and rows included) and useful
    (2 * nnz * N), both against the dense peak of the instruction the kernel issues."""
    kind = info["last_mfma_kind"]
    if kind not in MFMA or kernel_ms <= 0:
        return None
    name, peak = MFMA[kind]
    issued = float(info["last_mfma_instructions"]) * info["last_mfma_flops"]
    t = kernel_ms * 1e-3
    return {"instruction": name, "peak_tflops": peak, "instructions_per_launch": int(info["last_mfma_instructions"]),
            "issued_tflops": issued / t / 1e12, "issued_frac": issued / t / 1e12 / peak,
            "useful_tflops": useful_flops / t / 1e12, "useful_frac": useful_flops / t / 1e12 / peak}


def device_buffers(torch, np, hs, A, B, N):
    if A["dtype"] == hs.FP16:
        return (torch.from_numpy(B.view(np.int16)).cuda(),
                torch.empty((A["rows"], N), dtype=torch.int16, device="cuda"))
    return torch.from_numpy(B).cuda(), torch.empty((A["rows"], N), dtype=torch.float32, device="cuda")


def measure_config(torch, np, hs, G, index, N, steps, warmup, mode=0, matrix=None):
    """One configuration through hspmm_run, timed with device events on the launch stream (the reference's
    convention, src/common.h:48-58: warm-up launches, then timed launches back to back)."""
    cfg = matrix or G.make_config(index, 1)
    A = cfg["A"]
    b = cfg.get("btcf") or hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], A["dtype"])
    cfg["btcf"] = b
    B = G.dense_b(A["cols"], N, cfg["b_seed"], A["dtype"])
    hs.set_kernel_mode(mode)
    try:
        plan = hs.Plan(b)
    finally:
        hs.set_kernel_mode(0)
    dB, dC = device_buffers(torch, np, hs, A, B, N)
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(warmup):
        plan.run(dB.data_ptr(), dC.data_ptr(), N, stream)
    main_ms, fix_ms = plan.profile(dB.data_ptr(), dC.data_ptr(), N, runs=steps, stream=stream)
    main_ms /= steps
    fix_ms /= steps
    info = plan.info()
    flops = 2.0 * int(A["nnzs"]) * N
    bytes_alg = G.algorithmic_bytes(b, N)
    t = (main_ms + fix_ms) * 1e-3
    out = {"workload": "configs[%d]: %s, N=%d" % (index, cfg["name"], N),
           "dtype": "f16 in, f32 accumulate" if A["dtype"] == hs.FP16 else "f32 (tf32 variant)",
           "kernel": KERNELS.get(info["last_kernel_family"], "none"),
           "kernel_ms": main_ms, "fixup_kernel_ms": fix_ms,
           "tflops": flops / t / 1e12, "algorithmic_bytes": bytes_alg,
           "bound": BOUND.get((index, N), "hbm"),
           "hbm_gbps": bytes_alg / t / 1e9, "hbm_frac": bytes_alg / t / 1e9 / HBM_PEAK_GBPS,
           "mfma": mfma_report(info, flops, main_ms)}
    out["frac"] = out["mfma"]["useful_frac"] if out["bound"] == "mfma" and out["mfma"] else out["hbm_frac"]
    if info["last_kernel_family"] == 2 and (N * (2 if A["dtype"] != 1 else 4)) % 128 == 0:
        g_ms, _ = plan.measure_gather(dB.data_ptr(), N, runs=5, stream=stream)
        out["gather_only_ms"] = g_ms
    plan.close()
    del dB, dC
    return out, cfg


def all_configs(torch, np, hs, G, steps, warmup):
    """The other benchmark configurations, one line each: the configuration the CPU check path is quoted on, the
    uniform 65536^2 matrix, the pruned fp32 weight in both arithmetic forms of the tf32 variant (bf16 hi / lo
    parts in three products, the default; fp32 MFMA products, kernel mode 5) and the block-clustered weight at
    N = 16, 64 and 512."""
    rows = []
    for index, n_list in ((0, (64,)), (1, (128,)), (3, (256,)), (4, (16, 64, 512))):
        cfg = None
        for N in n_list:
            r, cfg = measure_config(torch, np, hs, G, index, N, steps, warmup, matrix=cfg)
            if index == 3:
                r["arithmetic"] = "bf16 hi / lo parts of every fp32 factor, three products (a_lo * b_lo left out)"
            rows.append(r)
            if index == 3:
                r5, cfg = measure_config(torch, np, hs, G, index, N, steps, warmup, mode=5, matrix=cfg)
                r5["arithmetic"] = "fp32 MFMA products (hspmm_set_kernel_mode(5))"
                rows.append(r5)
    return rows


def cpu_baseline(A, B, N, flops_full):
    """The oracle's CSR SpMM (test infrastructure used as the measured CPU baseline,
    never as the product path) on a bounded sample of the rows."""
    import numpy as np
    import oracle
    threads = oracle.max_threads()
    rows = A["rows"]
    rp = A["row_ptr"].astype(np.int64)
    # sample: leading rows holding about 1/4 of the stored entries for the single-thread
    # run, the whole matrix for the all-threads run if it is small enough
    def sub(frac):
        r_end = int(np.searchsorted(rp, rp[-1] * frac)) if frac < 1 else rows
        r_end = max(1, min(rows, r_end))
        n = int(rp[r_end])
        return r_end, n
    def run(r_end, n, nthreads):
        t = time.perf_counter()
        if A["dtype"] == 0:
            oracle.spmm_csr_f16(r_end, N, A["row_ptr"][:r_end + 1], A["col_idx"][:n], A["values"][:n], B, threads=nthreads)
        else:
            oracle.spmm_csr_f32(r_end, N, A["row_ptr"][:r_end + 1], A["col_idx"][:n], A["values"][:n], B, threads=nthreads)
        return time.perf_counter() - t
    # size the samples from a tiny probe so that each run stays within ~10-15 s
    r0, n0 = sub(0.01)
    probe = max(run(r0, n0, 1), 1e-4)
    per_nnz_1t = probe / max(n0, 1)
    frac1 = min(1.0, 10.0 / (per_nnz_1t * rp[-1]))
    r1, n1 = sub(frac1)
    t1 = run(r1, n1, 1)
    fracm = min(1.0, 10.0 * threads * 0.7 / (per_nnz_1t * rp[-1]))
    rm, nm = sub(fracm)
    tm = run(rm, nm, threads)
    return {
        "value": 2.0 * nm * N / tm / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": "oracle CSR SpMM (fp32 accumulate), first %d of %d rows (%d of %d stored entries), %d threads, %.2f s"
                  % (rm, rows, nm, int(rp[-1]), threads, tm),
        "single_thread": {"value": 2.0 * n1 * N / t1 / 1e12, "unit": "TFLOP/s", "cores": 1,
                          "sample": "first %d rows (%d stored entries), %.2f s" % (r1, n1, t1)},
    }


def kernel_sources_digest():
    """sha256 over the kernel and host sources libhspmm.so is built from: the counter figures of
    profiles/traffic.json carry the digest they were measured with."""
    import glob
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "hopper_spmm_amd", "csrc")
    for path in sorted(glob.glob(os.path.join(csrc, "*"))):
        if path.endswith((".hip", ".hpp", ".h", ".cpp")) or os.path.basename(path) == "Makefile":
            h.update(os.path.basename(path).encode())
            with open(path, "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def info_family(plan):
    return plan.info()["last_kernel_family"]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2, help="index into the benchmark configurations (default: 2, the 1M-row power-law graph)")
    ap.add_argument("--n", type=int, default=0, help="feature dimension (default: the configuration's)")
    ap.add_argument("--shrink", type=int, default=1)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--mode", type=int, default=0, help="kernel mode (hspmm_set_kernel_mode)")
    ap.add_argument("--stages", type=int, default=0)
    ap.add_argument("--waves-per-group", type=int, default=0)
    ap.add_argument("--ranges-per-simd", type=int, default=0)
    ap.add_argument("--panel-stream", type=int, default=0,
                    help="stream of the LDS-panel kernels (hspmm_set_panel_stream): 0 tiles, 1 two units per wave, 2 packed tiles")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain device copy of 1 GiB (reference point for traffic counters)")
    ap.add_argument("--no-all-configs", action="store_true",
                    help="leave out the lines for the other benchmark configurations (all_configs)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this operator runs on a single MI355X and nothing here uses a "
              "second one (--gpus %d refused)" % args.gpus, file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import hopper_spmm_amd as hs
    from hopper_spmm_amd import generators as G

    if not torch.cuda.is_available():
        print("bench.py needs the GPU", file=sys.stderr)
        sys.exit(3)
    torch.cuda.set_device(0)
    t_gen = time.perf_counter()
    cfg = G.make_config(args.config, args.shrink)
    A = cfg["A"]
    N = args.n or (cfg["N"][0] if args.config != 4 else 64)
    dt = A["dtype"]
    b = hs.csr_to_btcf(A["rows"], A["cols"], A["row_ptr"], A["col_idx"], A["values"], dt)
    B = G.dense_b(A["cols"], N, cfg["b_seed"], dt)
    t_gen = time.perf_counter() - t_gen

    hs.set_kernel_mode(args.mode)
    hs.set_panel_stream(args.panel_stream)
    hs.configure(args.stages, args.waves_per_group, args.ranges_per_simd, 0)
    torch.zeros(1, device="cuda")                    # runtime initialised before anything is timed
    torch.cuda.synchronize()
    t_h2d = time.perf_counter()
    plan = hs.Plan(b)                                # validation, partition, upload of the four format arrays
    if dt == hs.FP16:
        dB = torch.from_numpy(B.view(np.int16)).cuda()
        dC = torch.empty((A["rows"], N), dtype=torch.int16, device="cuda")
    else:
        dB = torch.from_numpy(B).cuda()
        dC = torch.empty((A["rows"], N), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    t_h2d = time.perf_counter() - t_h2d
    stream = torch.cuda.current_stream().cuda_stream
    pB, pC = dB.data_ptr(), dC.data_ptr()

    for _ in range(args.warmup):
        plan.run(pB, pC, N, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        plan.run(pB, pC, N, stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps

    # into pages that exist already, as the host header's operator does it (it touches C's pages on worker
    # threads while the GPU works; a copy into untouched pages takes 4 - 5 times as long)
    host_c = torch.zeros(dC.shape, dtype=dC.dtype)
    t_d2h = time.perf_counter()
    host_c.copy_(dC)
    t_d2h = time.perf_counter() - t_d2h
    del host_c

    # kernel durations with device events on the launch stream
    main_ms, fix_ms = plan.profile(pB, pC, N, runs=args.steps, stream=stream)
    main_ms /= args.steps
    fix_ms /= args.steps
    # the reference's own convention: 3 warm-ups, 5 timed launches (src/common.h:48-49)
    ref_conv_ms = plan.bench(pB, pC, N, warmup=3, runs=5, stream=stream) / 5.0

    # floor of the gather kernels: the same row gathers and nothing else, measured in this run
    gather_floor = None
    if info_family(plan) == 2 and (N * (2 if dt != 1 else 4)) % 128 == 0:
        g_ms, g_bytes = plan.measure_gather(pB, N, runs=5, stream=stream)
        gather_floor = {"ms": g_ms, "bytes": g_bytes}
    # the fp32-storage variant has two arithmetic forms in the LDS-panel kernels: bf16 hi / lo parts in
    # three products (default) and true fp32 MFMA products (kernel mode 5); both are timed
    fp32_products = None
    if dt == 1 and info_family(plan) == 3 and args.mode == 0:
        hs.set_kernel_mode(5)
        try:
            plan5 = hs.Plan(b)
        finally:
            hs.set_kernel_mode(0)
        for _ in range(args.warmup):
            plan5.run(pB, pC, N, stream)
        m5, f5 = plan5.profile(pB, pC, N, runs=args.steps, stream=stream)
        fp32_products = {"kernel_ms": m5 / args.steps, "fixup_kernel_ms": f5 / args.steps,
                         "arithmetic": "v_mfma_f32_4x4x1 / 16x16x4 on fp32 inputs (hspmm_set_kernel_mode(5))"}
        plan5.close()
        plan.run(pB, pC, N, stream)                  # the default plan is the last one that ran
        torch.cuda.synchronize()

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")       # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    nnz = int(A["nnzs"])
    flops = 2.0 * nnz * N
    bytes_alg = G.algorithmic_bytes(b, N)
    bytes_gather = G.gather_bytes(b, N)
    info = plan.info()
    traffic = None
    tfile = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tfile):
        with open(tfile) as f:
            traffic = json.load(f).get("config%d_N%d" % (args.config, N))
        if traffic is not None:
            # false: the kernels' sources have changed since the counters were read
            traffic["measured_with_these_sources"] = traffic.get("kernel_sources_sha256") == kernel_sources_digest()

    kernels_ms = main_ms + fix_ms
    out = {
        "metric": "SpMM effective TFLOP/s (2*nnz*N)",
        "value": flops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 in, f32 accumulate" if dt == hs.FP16 else "f32 (tf32 variant)",
        "data": "synthetic",
        # seeded generators of hopper_spmm_amd/generators.py: raw words of Philox 4x64-10 (numpy's bit generator, a
        # stream numpy keeps stable) through the module's own transforms (Box-Muller normals)
        "data_generator": "Philox 4x64-10 raw words, own transforms (numpy %s)" % np.__version__,
        "config": {"workload": "configs[%d]: %s, N=%d" % (args.config, cfg["name"], N),
                   "rows": A["rows"], "cols": A["cols"], "nnz": nnz, "tiles": int(b["total_tiles"]),
                   "eff_row_windows": int(b["eff_row_windows"]), "ranges": info["n_ranges"],
                   "split_windows": info["n_split_windows"]},
        "effective_gbps": bytes_alg / (ms_per_step * 1e-3) / 1e9,
        # achieved: algorithmic bytes of one launch / (main kernel + partial-sum kernel), device events
        "roofline": {"bound": BOUND.get((args.config, N), "hbm"), "achieved": bytes_alg / (kernels_ms * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": bytes_alg / (kernels_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                     # counter figures stored with the rocprofv3 summary they come from (not measured in this run)
                     "traffic": traffic,
                     "kernel": KERNELS.get(info["last_kernel_family"], "none"),
                     "kernel_ms": main_ms, "fixup_kernel_ms": fix_ms,
                     "algorithmic_bytes": bytes_alg, "gather_bytes": bytes_gather,
                     # every gathered B row counted every time it is gathered, for comparison with the HBM peak
                     "gathered_gbps": bytes_gather / (kernels_ms * 1e-3) / 1e9,
                     "mfma": mfma_report(info, flops, main_ms)},
        "reference_convention_ms": ref_conv_ms,
        # one call of the host-buffer interface (fp16_spmm): plan + upload, one launch, download of C
        "host_buffer_call": {"upload_and_plan_ms": t_h2d * 1e3, "download_ms": t_d2h * 1e3,
                             "tflops_including_transfers": flops / (t_h2d + t_d2h + ms_per_step * 1e-3) / 1e12},
        "setup_seconds": t_gen,
    }
    if gather_floor:
        # every (window, column) pair gathers one B row; this is what loading those rows alone takes
        out["roofline"]["gather_ceiling_gbps"] = gather_floor["bytes"] / (gather_floor["ms"] * 1e-3) / 1e9
        out["roofline"]["gather_only_ms"] = gather_floor["ms"]
        out["roofline"]["frac_of_gather_ceiling"] = gather_floor["ms"] / kernels_ms
    if fp32_products:
        out["tf32_variant"] = {"default": {"kernel_ms": main_ms, "fixup_kernel_ms": fix_ms,
                                           "arithmetic": "bf16 hi / lo parts, three v_mfma_f32_16x16x32_bf16 products"},
                               "fp32_products": fp32_products}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(A, B, N, flops)
    plan.close()
    if args.config == 2 and not args.n and not args.no_all_configs and args.mode == 0:
        del dB, dC
        out["all_configs"] = all_configs(torch, np, hs, G, args.steps, args.warmup)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
