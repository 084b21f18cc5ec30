#!/usr/bin/env python3
"""Benchmark of the ELLPACK compute path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--spinup-ms T] [--no-extras] [--no-cpu]

Headline workload ("step" = one ellpack_matmul launch over the whole dense block):
the large FC configuration, W 4096 x 4096 fp32 N(0, 0.02) with per-row top-10 %
magnitude pruning (uniform r = 410), X 4096 x 256 fp32 N(0,1), bias N(0, 0.1),
operands resident in HBM.  Prints ONE JSON line: nnz-GFLOP/s as `value`, the HBM
roofline of the kernel (algorithmic bytes per launch / HIP-event time), the fp32
VALU fraction, and the same configuration timed on the host cores with the
reference's own kernel (`oracle/_ref`, kind "reference") or, where that cannot run,
the plain-C restatement (kind "port").  `extras` holds the other configurations:
matvec 16384 x 16384 (uniform and Zipf-skewed rows) and the sparse MLP's samples/s.
Every kernel timed on its own is first launched untimed for --spinup-ms (150 ms) so that the
GPU's clocks have settled, then for the W warm-up steps, then timed for exactly K steps (the
two models' chains are timed after their warm-up passes only: they gain nothing from it).
"""
import argparse
import json
import os
import statistics
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (os.path.join(ROOT, "sparse-ops_amd"), os.path.join(ROOT, "sparse-ops_amd", "python"),
           os.path.join(ROOT, "sparse-ops_amd", "bench")):
    sys.path.insert(0, _p)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E
VALU_FP32_PEAK_TF = 157.3    # MI355X vector fp32; plain v_fma_f32 reaches 107 of its 128 multiply-adds per clock and CU, the
                             # register-indexed DPP form of the row-block-merged kernel 77 at three waves per SIMD, the DPP
                             # form of the quad layout 58 (profiles/lds_valu_rates__probe.txt, profiles/indexed_fma_rates__probe.txt)
LDS_OPERAND_PEAK_TF = 78.6   # 256 CUs x 256 B/clk of ds_read_b128 (measured 255) x 2.4 GHz / 4 B per multiply-add x 2 flop
# HBM-side bytes per launch, per kernel: measured with two rocprofv3 --pmc runs (FETCH_SIZE,
# WRITE_SIZE) scaled by a plain copy of known size and kept, keyed by kernel name and together with a
# hash of the kernel's sources, in this table (written by sparse-ops_amd/bench/pmc_summary.py traffic).
# A kernel that is not in the table, or whose sources have changed since, reports null.
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
HEADLINE_KERNEL = "ellpack_matmul_rbm_kernel<0>"
TILED_KERNEL = "ellpack_matmul_tiled_kernel<0>"
MATVEC_KERNELS = {"ellpack_matvec 16384x16384, 95% Bernoulli": ("matvec_binned_kernel<true,true>", "matvec 16384^2 uniform"),
                  "ellpack_matvec 16384x16384, Zipf(1.2) rows capped at 2048": ("matvec_binned_kernel<true,true>", "matvec 16384^2 zipf")}


def measured_traffic(kernel, workload=None):
    from pmc_summary import lookup_traffic
    return lookup_traffic(TRAFFIC_TABLE, kernel, workload)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def alg_bytes(nnz, m, n, C):
    """Compulsory HBM traffic of one launch, every operand once: Wd + idx over the
    stored nonzeros, nnz[], bias, X, Y."""
    return 8 * nnz + 4 * m + 4 * m + 4 * n * C + 4 * m * C


SPINUP_MS = 150.0   # --spinup-ms


def spin_up(ctx, fn):
    """Untimed launches of `fn` for SPINUP_MS of wall time: after an idle spell (an upload, host
    work) the GPU needs some 100 ms of continuous load before its clocks settle, and launches
    timed before that read up to 14 % slow.  Comes before the warm-up steps, not instead of them."""
    t_end = time.perf_counter() + SPINUP_MS * 1e-3
    while time.perf_counter() < t_end:
        for _ in range(32):
            fn()
        ctx.sync()


def time_launches(ctx, fn, steps, warmup):
    """-> (wall seconds for `steps` launches, HIP-event ms per launch)."""
    spin_up(ctx, fn)
    for _ in range(warmup):
        fn()
    ctx.sync()
    t0 = time.perf_counter()
    ctx.timer_begin()
    for _ in range(steps):
        fn()
    ev_ms = ctx.timer_end()           # waits for the last launch
    ctx.sync()
    wall = time.perf_counter() - t0
    return wall, ev_ms / steps


def time_groups(ctx, fn, groups, per_group):
    """-> per-launch microseconds of `groups` event-bracketed groups of `per_group` back-to-back launches
    (the clocks are settled by the caller's earlier time_launches)."""
    for _ in range(per_group):
        fn()
    ctx.sync()
    out = []
    for _ in range(groups):
        ctx.timer_begin()
        for _ in range(per_group):
            fn()
        out.append(ctx.timer_end() * 1e3 / per_group)
    return out


def host_has_avx512f():
    try:
        with open("/proc/cpuinfo") as f:
            return "avx512f" in f.read()
    except OSError:
        return False


def cpu_baseline_matmul(E, X, bias, y_gpu, y_exact, budget_s=15.0):
    """The same matmul on the host cores: the reference's compiled kernel when it
    can run here, else the plain-C restatement.  1 warm-up, then the median of as
    many runs as fit the budget (at least 5, at most 50) -- the reference
    benchmark's protocol (benchmark-mkl/matmul/bench_matmul.cpp:97-116)."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    from oracle import EllpackArrays, Oracle, Ref
    cores = len(os.sched_getaffinity(0))
    threads = max(1, min(cores, int(os.environ.get("OMP_NUM_THREADS", cores))))
    os.environ["OMP_NUM_THREADS"] = str(threads)
    Eo = EllpackArrays(E.m, E.n, E.r, E.Wd, E.idx, E.nnz)
    if Ref.available():
        ref = Ref()
        h = ref.from_arrays(Eo)
        Y = np.empty((E.m, X.shape[1]), dtype=np.float32)
        run, kind = (lambda: ref.matmul(h, X, bias, out=Y)), "reference"
    else:
        orc = Oracle()
        orc.set_num_threads(threads)
        holder = {}
        def run():
            holder["Y"] = orc.matmul(Eo, X, bias)
        kind = "port"
    run()
    times, t_start = [], time.perf_counter()
    while len(times) < 5 or (len(times) < 50 and time.perf_counter() - t_start < budget_s):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    Ycpu = (Y if kind == "reference" else holder["Y"]).copy()
    med = statistics.median(times)
    flops = 2.0 * E.total_nnz * X.shape[1]
    # 1 and 8 threads as well, the thread counts the reference's docs/performance.md quotes
    # (both libraries share one OpenMP runtime, so one call sets the team size for either)
    by_threads = {str(threads): round(flops / med / 1e9, 2)}
    orc_threads = Oracle()
    for t in (1, 8):
        if t >= threads:
            continue
        orc_threads.set_num_threads(t)
        os.environ["OMP_NUM_THREADS"] = str(t)      # the reference kernel re-reads it on every call
        run()
        ts = []
        for _ in range(3):
            t0 = time.perf_counter()
            run()
            ts.append(time.perf_counter() - t0)
        by_threads[str(t)] = round(flops / statistics.median(ts) / 1e9, 2)
    orc_threads.set_num_threads(threads)
    os.environ["OMP_NUM_THREADS"] = str(threads)
    model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {
        "value": round(flops / med / 1e9, 2), "unit": "nnz-GFLOP/s", "cores": threads, "kind": kind,
        "sample": "same 4096x4096 r=410 C=256 matmul, 1 warm-up + median of %d runs (%.2f ms each)" % (len(times), med * 1e3),
        "ms_per_step": round(med * 1e3, 4), "ms_per_step_min": round(min(times) * 1e3, 4), "cpu_model": model,
        "avx512f": host_has_avx512f(),       # without it the reference takes its scalar path (src/ellpack_matmul.cpp:80-90)
        "nnz_gflops_by_threads": by_threads,
        # the headline (row-block-merged) kernel sums in another order: fp32 round-off; the K-tiled kernel gives the CPU's bits
        "gpu_max_rel_err_vs_cpu": float(np.abs(Ycpu.astype(np.float64) - y_gpu).max() / np.abs(Ycpu).max()),
        "gpu_bit_exact_vs_cpu": bool(np.array_equal(Ycpu, y_gpu)),
        "gpu_tiled_kernel_bit_exact_vs_cpu": bool(np.array_equal(Ycpu, y_exact)),
    }


def cpu_baseline_matvec(E, x, b, y_gpu, nbytes):
    """The same matvec on the host cores: the reference's compiled kernel (which also writes its
    E.Xt gather buffer, src/ellpack_matvec.cpp:50-52) or the plain-C restatement; 1 warm-up,
    median of 9."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    from oracle import EllpackArrays, Oracle, Ref
    Eo = EllpackArrays(E.m, E.n, E.r, E.Wd, E.idx, E.nnz)
    if Ref.available():
        ref = Ref()
        h = ref.from_arrays(Eo)
        y = np.empty(E.m, dtype=np.float32)
        run, kind = (lambda: ref.matvec(h, x, b, out=y)), "reference"
    else:
        orc, holder = Oracle(), {}

        def run():
            holder["y"] = orc.matvec(Eo, x, b)
        kind = "port"
    run()
    ts = []
    for _ in range(9):
        t0 = time.perf_counter()
        run()
        ts.append(time.perf_counter() - t0)
    ycpu = y if kind == "reference" else holder["y"]
    med = statistics.median(ts)
    return {"us_per_call": round(med * 1e6, 1), "GBps": round(nbytes / med / 1e9, 1), "kind": kind,
            "cores": int(os.environ.get("OMP_NUM_THREADS", len(os.sched_getaffinity(0)))),
            "gpu_max_rel_err_vs_cpu": float(np.abs(ycpu.astype(np.float64) - y_gpu).max() / max(np.abs(ycpu).max(), 1e-30))}


def bench_matvec(ctx, hipabi, datagen, name, gen, layouts, layout, steps, warmup, with_cpu=True):
    E, x, b = gen()
    # Up to 65536 columns the handle also keeps them in 16 bits (SO_LAYOUT_IDX16) and so_matvec streams 6 bytes
    # per nonzero instead of the format's 8: same bits, a quarter less to read.  `alg_bytes` and `hbm_frac` stay
    # on the reference format's 8 bytes per nonzero; `bytes_read` / `hbm_frac_bytes_read` are what the kernel
    # actually streams, and `idx32` is the same handle with the 32-bit columns.  As the host layer does
    # (ellpack_matvec), compact columns go with the length-class kernel, which on them is the faster one for even
    # rows too while a wave gets only a few rows; `idx32` runs the kernel the host layer takes without them.
    compact = E.n <= 65536
    layout32 = layout
    if compact:
        layouts |= hipabi.LAYOUT_IDX16
        if 4 <= E.m // (16 * ctx.info()[1]) < 6:          # so_matvec's own rule (layout 0): two or three rows per wave
            layouts |= hipabi.LAYOUT_BINS
            layout = hipabi.LAYOUT_BINS
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, layouts)
    dx, dB, dy = ctx.array(x), ctx.array(b), ctx.empty((E.m,))
    _, ms = time_launches(ctx, lambda: ctx.matvec(dE, dx, dB, dy, layout), steps, warmup)
    vectors = 4 * E.m + 4 * E.m + 4 * E.n + 4 * E.m
    nbytes = 8 * E.total_nnz + vectors
    nread = (6 if compact else 8) * E.total_nnz + vectors
    out = {"workload": name, "m": E.m, "n": E.n, "r": E.r, "nnz": E.total_nnz, "us_per_launch": round(ms * 1e3, 2),
           "alg_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1), "hbm_frac": round(nbytes / ms / 1e6 / HBM_PEAK_GBS, 4),
           "column_bits": 16 if compact else 32, "kernel": "length classes" if layout == hipabi.LAYOUT_BINS else "wave per row",
           "bytes_read": nread,
           "hbm_frac_bytes_read": round(nread / ms / 1e6 / HBM_PEAK_GBS, 4),
           "padded_bytes": 8 * E.m * E.r,
           "traffic": measured_traffic(*MATVEC_KERNELS[name]) if name in MATVEC_KERNELS else None}
    if with_cpu:
        out["cpu_baseline"] = cpu_baseline_matvec(E, x, b, dy.download(), nbytes)
    # Cache-cold figure: the streamed arrays (50-108 MB) fit the 256 MB Infinity Cache when the
    # same launch repeats back to back, so also rotate the launches over enough copies of the
    # matrix that a copy has been evicted by the time its turn comes again.
    copies = [dE] + [ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, layouts) for _ in range(5)]
    turn = [0]

    def rotate():
        ctx.matvec(copies[turn[0] % len(copies)], dx, dB, dy, layout)
        turn[0] += 1
    cold_steps = len(copies) * max(2, steps // len(copies))
    _, cold_ms = time_launches(ctx, rotate, cold_steps, len(copies))
    out["us_per_launch_cache_cold"] = round(cold_ms * 1e3, 2)
    out["hbm_frac_cache_cold"] = round(nbytes / cold_ms / 1e6 / HBM_PEAK_GBS, 4)
    out["hbm_frac_bytes_read_cache_cold"] = round(nread / cold_ms / 1e6 / HBM_PEAK_GBS, 4)
    out["cache_cold_copies"] = len(copies)
    if compact:
        y16 = dy.download()
        def rotate32():
            ctx.matvec(copies[turn[0] % len(copies)], dx, dB, dy, layout32)
            turn[0] += 1
        with ctx.tuning(SPARSEOPS_MATVEC_IDX16="0"):
            _, ms32 = time_launches(ctx, lambda: ctx.matvec(dE, dx, dB, dy, layout32), steps, warmup)
            _, cold32 = time_launches(ctx, rotate32, cold_steps, len(copies))
            ctx.matvec(dE, dx, dB, dy, layout)
        out["idx32"] = {"kernel": "length classes" if layout32 == hipabi.LAYOUT_BINS else "wave per row",
                        "us_per_launch": round(ms32 * 1e3, 2), "hbm_frac": round(nbytes / ms32 / 1e6 / HBM_PEAK_GBS, 4),
                        "us_per_launch_cache_cold": round(cold32 * 1e3, 2),
                        "hbm_frac_cache_cold": round(nbytes / cold32 / 1e6 / HBM_PEAK_GBS, 4),
                        "same_bits_as_16_bit_columns": bool(np.array_equal(y16, dy.download()))}
    for c in copies[1:]:
        c.free()
    dE.free()
    for a in (dx, dB, dy):
        a.free()
    return out


def cpu_baseline_mlp(Ws, X, y_gpu, runs=10):
    """The same MLP forward on the host cores with the reference's kernels, as its
    runtime chains them (src/model_run.cpp:28-127): ellpack_matmul_fused with the
    fused ReLU, then the separate scalar Sigmoid / Tanh layers
    (src/layers/activation.cpp:22-62).  Falls back to the plain-C restatement."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    from oracle import Oracle, Ref
    A0 = np.ascontiguousarray(X.T)
    acts = ["relu", "sigmoid", "tanh", None]
    if Ref.available():
        ref, kind = Ref(), "reference"
        hs = [ref.encode(W) for W in Ws]

        def forward():
            A = A0
            for h, act in zip(hs, acts):
                A = ref.matmul_fused(h, A, None, use_mask=False, fuse_relu=(act == "relu"))
                if act in ("sigmoid", "tanh"):
                    A = ref.act_inplace(A, act)
            return A
    else:
        orc, kind = Oracle(), "port"
        Es = [orc.encode(W) for W in Ws]

        def forward():
            A = A0
            for E, act in zip(Es, acts):
                A = orc.matmul(E, A, None, act or "none")
            return A
    Y = forward()
    times = []
    for _ in range(runs):
        t0 = time.perf_counter()
        forward()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {"samples_per_s": round(X.shape[0] / med, 1), "ms_per_batch": round(med * 1e3, 3), "kind": kind,
            "cores": int(os.environ.get("OMP_NUM_THREADS", len(os.sched_getaffinity(0)))),
            "gpu_max_rel_err_vs_cpu": float(np.abs(Y.T.astype(np.float64) - y_gpu).max() / max(np.abs(Y).max(), 1e-30))}


def bench_mlp(steps, warmup, with_cpu=True):
    import datagen
    import onnx_wire as ow
    import sparseops_backend as sb
    Ws = datagen.config4_weights()
    X = datagen.config4_input()
    with tempfile.TemporaryDirectory() as d:
        model = sb.SparseOnnxModel(ow.save(os.path.join(d, "mlp.onnx"), ow.mlp_model(Ws, ["Relu", "Sigmoid", "Tanh", None], 256)))
    Xf = np.asfortranarray(X)
    for _ in range(warmup):
        model.run(Xf)
    t0 = time.perf_counter()
    for _ in range(steps):
        model.run(Xf)                       # includes H2D of the input and D2H of the output
    dt = (time.perf_counter() - t0) / steps
    dev_ms = model.time_device(steps, warmup)   # chain only, activations resident in HBM
    y_gpu = model.run(Xf)
    cpu = cpu_baseline_mlp(Ws, X, y_gpu) if with_cpu else None
    return {"workload": "MLP 784-4096-4096-4096-10, 90% sparse, B=256", "layers": model.describe(), "cpu_baseline": cpu,
            "samples_per_s_device_resident": round(256 / (dev_ms * 1e-3), 1), "us_per_batch_device_resident": round(dev_ms * 1e3, 2),
            "samples_per_s_host_to_host": round(256 / dt, 1), "us_per_batch_host_to_host": round(dt * 1e6, 2),
            "nnz_gflops_device_resident": round(model.nnz_flops_per_sample() * 256 / (dev_ms * 1e-3) / 1e9, 1)}


def cpu_baseline_cnn(payload, model):
    """The same graph on the host cores over the whole batch of 32: every convolution with the
    reference's own conv2d_rbm_fmajor_implicit (its variant that is right for strided layers) and the
    classifier with its ellpack_matmul, both from oracle/_ref; max-pool, residual adds and the global
    average pool with the plain-C port (the reference's versions are private members of a class whose
    constructor needs libprotobuf).  1 warm-up pass, median of 3, kernel time only (the layout shuffles
    between the two libraries' conventions are not counted) -- the reference benchmark's protocol
    (benchmark-mkl/matmul/bench_matmul.cpp:97-116).  Without the compiled reference: the plain-C
    port on 4 images, one pass.  Also compares the GPU's output with the CPU's, bit for bit."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    from graph_oracle import RefGraph, run_graph
    from oracle import Oracle, Ref
    orc = Oracle()
    X = np.random.default_rng(5).standard_normal((32, 3, 224, 224)).astype(np.float32)
    y_gpu = model.run(X)
    if Ref.available():
        G = RefGraph(Ref(), orc, payload, (224, 224))
        y_cpu, _ = G.run(X)
        ts = [G.run(X)[1] for _ in range(3)]
        G.close()
        dt, n, kind = statistics.median(ts), 32, "reference"
        sample = ("all 32 images, 1 warm-up + median of 3 passes, kernel time only; conv + FC layers: the reference's "
                  "conv2d_rbm_fmajor_implicit / ellpack_matmul; max-pool, add, global average pool: plain-C port")
    else:
        n, kind, sample = 4, "port", "4 of the 32 images, one pass"
        t0 = time.perf_counter()
        y_cpu = run_graph(orc, payload, X[:n])
        dt = time.perf_counter() - t0
    return {"samples_per_s": round(n / dt, 2), "ms_per_image": round(dt / n * 1e3, 2), "kind": kind,
            "cores": orc.num_threads(), "sample": sample, "avx512f": host_has_avx512f(),
            "gpu_bit_exact_vs_cpu": bool(np.array_equal(y_cpu, y_gpu[:n])),
            "gpu_max_rel_err_vs_cpu": float(np.abs(y_cpu.astype(np.float64) - y_gpu[:n]).max() / max(np.abs(y_cpu).max(), 1e-30))}


def bench_cnn(steps, warmup, with_cpu=True):
    import datagen
    import onnx_wire as ow
    import sparseops_backend as sb
    payload, _ = datagen.resnet18_onnx(seed=47, batch=32, hw=224, sparsity=0.8)
    with tempfile.TemporaryDirectory() as d:
        model = sb.SparseOnnxModel(ow.save(os.path.join(d, "r18.onnx"), payload))
    dev_ms = model.time_device(steps, warmup)
    flops = model.nnz_flops_per_sample() * 32
    out = {"workload": "ResNet-18-shaped conv stack (no BN), 80% sparse, B=32, 3x224x224, implicit im2col",
           "cpu_baseline": cpu_baseline_cnn(payload, model) if with_cpu else None,
           "layers": len(model.describe()), "ms_per_batch_device_resident": round(dev_ms, 3),
           "samples_per_s_device_resident": round(32 / (dev_ms * 1e-3), 1),
           "nnz_gflop_per_batch": round(flops / 1e9, 2), "nnz_gflops": round(flops / (dev_ms * 1e-3) / 1e9, 1)}
    # the same model at serving-sized batches (latency-bound): resize_buffers re-tunes the convolution plans
    small = {}
    for b in (1, 8):
        model.resize_buffers(b)
        small[str(b)] = round(model.time_device(steps, warmup), 3)
    out["ms_per_batch_by_batch_size"] = small
    return out


def main():
    global SPINUP_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--spinup-ms", type=float, default=SPINUP_MS,
                    help="untimed launches of each measured kernel for this long before its warm-up steps (clock settling)")
    ap.add_argument("--no-extras", action="store_true", help="skip matvec and MLP measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline")
    ap.add_argument("--skip-extra", action="append", default=[], metavar="NAME",
                    help="leave out one entry of `extras` (e.g. matvec_uniform_65536_rows and matvec_zipf, which run the same "
                         "kernel as matvec_uniform: counter passes that average per kernel name need them apart); repeatable")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 256 MiB copy kernel (scale factor for rocprofv3 --pmc byte counters)")
    args = ap.parse_args()
    SPINUP_MS = max(0.0, args.spinup_ms)
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (the path shards over the dense-column axis "
                 "with no exchange: every GPU would take B/N of the batch against its own copy of the weights); run with --gpus 1")

    import datagen
    import hipabi
    ctx = hipabi.Context(0)
    dev_name, cus = ctx.info()
    log("device:", dev_name, cus, "CUs")

    E, X, bias = datagen.config3()
    C = X.shape[1]
    # ROW is the encoder's layout; RBM adds the row-block-merged copy the fastest so_matmul kernel consumes
    # (fp32 round-off accuracy); TILED the K-tiled copy of the LDS-staged kernel (the reference's bits).
    dE = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, hipabi.LAYOUT_ROW | hipabi.LAYOUT_RBM)
    dX, dB, dY = ctx.array(X), ctx.array(bias), ctx.empty((E.m, C))
    step = lambda: ctx.matmul(dE, dX, C, dB, dY, "none")
    wall, ev_ms = time_launches(ctx, step, args.steps, args.warmup)
    group_us = time_groups(ctx, step, 20, max(10, args.steps // 20))
    y_gpu = dY.download()
    # the bit-exact kernels on the same operands, for comparison: K-tiled (LDS-staged) and row-per-wave
    dE_tiled = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, hipabi.LAYOUT_ROW | hipabi.LAYOUT_TILED)
    _, ev_ms_tiled = time_launches(ctx, lambda: ctx.matmul(dE_tiled, dX, C, dB, dY, "none"), max(40, args.steps // 2), 5)
    y_tiled = dY.download()
    dE_tiled.free()
    dE_row = ctx.upload_ellpack(E.Wd, E.idx, E.nnz, E.m, E.n, E.r, hipabi.LAYOUT_ROW)
    _, ev_ms_row = time_launches(ctx, lambda: ctx.matmul(dE_row, dX, C, dB, dY, "none"), max(20, args.steps // 4), 5)
    row_bits_equal = bool(np.array_equal(dY.download(), y_tiled))
    dE_row.free()
    ms_per_step = wall / args.steps * 1e3
    flops = 2.0 * E.total_nnz * C
    nbytes = alg_bytes(E.total_nnz, E.m, E.n, C)
    gbps = nbytes / (ev_ms * 1e-3) / 1e9
    result = {
        "metric": "ellpack_matmul nnz-GFLOP/s", "value": round(flops / (ms_per_step * 1e-3) / 1e9, 1), "unit": "nnz-GFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "ellpack_matmul large FC: W 4096x4096 N(0,0.02) per-row top-10%% (r=410, nnz=%d), "
                               "X 4096x256 N(0,1), bias N(0,0.1), seed 45" % E.total_nnz,
                   "m": E.m, "n": E.n, "r": E.r, "C": C, "sparsity": 0.9, "device": dev_name,
                   "spinup_ms": SPINUP_MS},
        "roofline": {"bound": "hbm", "achieved": round(gbps, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbps / HBM_PEAK_GBS, 4), "traffic": measured_traffic(HEADLINE_KERNEL),
                     "kernel": HEADLINE_KERNEL, "kernel_us": round(ev_ms * 1e3, 2),
                     # 20 event-bracketed groups of max(10, K/20) launches each, per launch
                     "kernel_us_median": round(statistics.median(group_us), 2), "kernel_us_min": round(min(group_us), 2),
                     "alg_bytes_per_launch": nbytes,
                     "tiled_kernel_us": round(ev_ms_tiled * 1e3, 2), "tiled_kernel": TILED_KERNEL,
                     "row_kernel_us": round(ev_ms_row * 1e3, 2), "row_kernel_same_bits_as_tiled": row_bits_equal,
                     "max_rel_diff_vs_tiled_kernel": float(np.abs(y_gpu.astype(np.float64) - y_tiled).max() / np.abs(y_tiled).max()),
                     "valu_fp32_frac_of_157.3TF": round(flops / (ev_ms * 1e-3) / 1e12 / VALU_FP32_PEAK_TF, 4),
                     # without reuse in registers every multiply-add needs a 4-byte X operand from LDS / L1 (what the
                     # row and K-tiled kernels move at that level); the row-block-merged kernel loads an X row segment
                     # once per 128-row block
                     "gather_bytes": 8 * E.total_nnz + 4 * E.total_nnz * C + 4 * E.m * C,
                     "t_hbm_us": round(nbytes / (HBM_PEAK_GBS * 1e9) * 1e6, 2),
                     "t_valu_us": round(flops / (VALU_FP32_PEAK_TF * 1e12) * 1e6, 2),
                     "t_bound_over_t": round(max(nbytes / (HBM_PEAK_GBS * 1e9), flops / (VALU_FP32_PEAK_TF * 1e12)) / (ev_ms * 1e-3), 4),
                     "binding_bound": "not HBM (t_hbm 2.7 us).  From knock-out builds: 3.2 us launch and set-up; ~17 us the loop, bound twice "
                                      "over -- a SIMD issues one scalar instruction per ~4 clk and every nonzero x 64 columns needs an M0 write "
                                      "before its register-indexed v_fmac_f32_dpp (15.5 us with all loads removed), and every iteration of 64 pairs "
                                      "waits one scalar-load round trip (16 us with the multiply-adds removed); 4.8 us the sum of a workgroup's 12 "
                                      "partial tiles through LDS; 2.0 us the exchange of partial tiles between the two workgroups of an output tile"},
    }
    if args.calibrate_copy:
        # A plain copy of known size (act_kernel<NONE>: reads N floats, writes N floats)
        # so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings can be scaled.
        n_cal = 64 * 1024 * 1024
        src, dst = ctx.empty((n_cal,)), ctx.empty((n_cal,))
        ctx.fill_zero(src)
        for _ in range(5):
            ctx.act("none", src, n_cal, dst)
        ctx.sync()
        result["calibration_copy"] = {"kernel": "act_kernel<0, true>", "bytes_read": 4 * n_cal, "bytes_written": 4 * n_cal}
        src.free()
        dst.free()
    if not args.no_cpu:
        log("timing the host-CPU baseline ...")
        result["cpu_baseline"] = cpu_baseline_matmul(E, X, bias, y_gpu, y_tiled)
    else:
        result["cpu_baseline"] = None
    if not args.no_extras:
        extras = {}
        k = max(20, args.steps // 2)
        # what a plain streaming kernel reaches on this box: 1 GiB read + 1 GiB written per launch (nothing of it can
        # stay in the 256 MB Infinity Cache from one launch to the next: an HBM figure), and the same at 256 MiB + 256 MiB
        # (what the calibration copy moves; the source is then served from the cache on repeated launches)
        for key, mib in (("stream_copy", 1024), ("stream_copy_256MiB", 256)):
            if key in args.skip_extra:        # counter passes calibrate on this kernel: its other launches must stay out
                continue
            n_cp = mib * 1024 * 1024 // 4
            src, dst = ctx.empty((n_cp,)), ctx.empty((n_cp,))
            ctx.fill_zero(src)
            _, cp_ms = time_launches(ctx, lambda: ctx.act("none", src, n_cp, dst), 20, 3)
            extras[key] = {"workload": "plain copy kernel, %d MiB in + %d MiB out" % (mib, mib), "us_per_launch": round(cp_ms * 1e3, 1),
                           "GBps": round(8 * n_cp / cp_ms / 1e6, 1), "hbm_frac": round(8 * n_cp / cp_ms / 1e6 / HBM_PEAK_GBS, 4)}
            src.free()
            dst.free()
        # config 1 (1024x1024, C=64): a parity shape whose kernel is shorter than a launch; launches back to back
        E1, X1, b1, _ = datagen.config1()
        dE1 = ctx.upload_ellpack(E1.Wd, E1.idx, E1.nnz, E1.m, E1.n, E1.r, hipabi.LAYOUT_ROW)
        dX1, dB1, dY1 = ctx.array(X1), ctx.array(b1), ctx.empty((E1.m, 64))
        _, ms1 = time_launches(ctx, lambda: ctx.matmul(dE1, dX1, 64, dB1, dY1, "none"), max(100, args.steps), args.warmup)
        extras["matmul_config1"] = {"workload": "ellpack_matmul 1024x1024 Bernoulli(0.1), C=64 (r=%d, nnz=%d), launches back to back"
                                                % (E1.r, E1.total_nnz),
                                    "us_per_launch": round(ms1 * 1e3, 2),
                                    "nnz_gflops": round(2.0 * E1.total_nnz * 64 / ms1 / 1e6, 1)}
        for a in (dX1, dB1, dY1):
            a.free()
        dE1.free()
        if "matvec_uniform" not in args.skip_extra:
            log("matvec 16384^2 uniform ...")
            extras["matvec_uniform"] = bench_matvec(ctx, hipabi, datagen, "ellpack_matvec 16384x16384, 95% Bernoulli",
                                                    datagen.config2a, hipabi.LAYOUT_ROW, hipabi.LAYOUT_ROW, k, args.warmup, not args.no_cpu)
        if "matvec_zipf" not in args.skip_extra:
            log("matvec 16384^2 zipf ...")
            extras["matvec_zipf"] = bench_matvec(ctx, hipabi, datagen, "ellpack_matvec 16384x16384, Zipf(1.2) rows capped at 2048",
                                                 datagen.config2b, hipabi.LAYOUT_ROW | hipabi.LAYOUT_BINS, hipabi.LAYOUT_BINS,
                                                 k, args.warmup, not args.no_cpu)
        if "matvec_uniform_65536_rows" not in args.skip_extra:
            log("matvec 65536x16384 uniform ...")
            # four times the rows of config 2a: what the same kernel streams once its fixed per-launch cost is amortised
            extras["matvec_uniform_65536_rows"] = bench_matvec(ctx, hipabi, datagen, "ellpack_matvec 65536x16384, 95% Bernoulli",
                                                               lambda: datagen.uniform_ellpack(48, 65536, 16384, 0.05),
                                                               hipabi.LAYOUT_ROW, hipabi.LAYOUT_ROW, max(10, k // 4), 3, False)
        if "mlp" not in args.skip_extra:
            log("sparse MLP ...")
            extras["mlp"] = bench_mlp(k, args.warmup, with_cpu=not args.no_cpu)
        if "cnn" not in args.skip_extra:
            log("sparse CNN ...")
            extras["cnn"] = bench_cnn(max(10, args.steps // 10), 5, with_cpu=not args.no_cpu)
        result["extras"] = extras
    ctx.close()
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
