#!/usr/bin/env python3
"""Benchmark of the fused MoE layer on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME]

A "step" is one forward pass of the layer over one batch of synthetic tokens
(inputs already resident in HBM). The default workload is the Qwen3-30B-A3B
decode batch (T=64). Prints ONE JSON line with the whole-job throughput, the
roofline position of the (single) kernel of a step, measured with events on the
launch stream, and the CPU oracle timed on this host beside it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MFMA_F32_PEAK_TFLOPS = 157.3

# which roofline bounds each workload
BOUND = {
    "tiny_f32": "hbm",
    "qwen3_30b_decode": "hbm",
    "qwen3_30b_prefill": "mfma",
    "qwen3_235b_t256": "hbm",
    "qwen3_235b_t4096": "hbm",
    "qwen3_30b_imbalance": "mfma",
}


# HBM bytes per launch as measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch)
# live in profiles/traffic.json, one entry per workload, each with the digest of the kernel
# sources (device code) it was measured on. An entry whose digest differs from the tree's is
# stale: `traffic` is null then and the old figure is shown as `traffic_stale`. `bench.py --record-traffic FETCH_KIB WRITE_KIB` writes the entry
# of --config after a new pair of counter runs. Each counter is scaled by what it reads for a
# plain copy of 1 GiB (bench.py --copy-calibration under the same counters): WRITE_SIZE 1.000,
# FETCH_SIZE 0.500 (this chip reads HBM in 128-byte requests, which the counter's formula
# prices at 64 bytes each).
FETCH_SCALE = 0.5
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")
# device code only: the host launcher does not change what a kernel reads or writes
KERNEL_SOURCES = ["moe_stream_kernel.hip", "moe_tiled_kernel.hip", "moe_device.h", "moe_params.h"]


def kernel_sources_digest():
    import hashlib

    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "flash_distributed_moe_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


WEIGHT_MODES = {
    "in_place": "packed in place by the caller (flashMoePackWeightsInPlace), no second copy",
    "default": "as a caller written against the reference gets them: row-major tensors handed to "
               "create() with no flags, of which the launcher keeps a packed copy (+3*E*H*I elements)",
    "row_major": "caller's row-major tensors read in place (create(..., flags=0))",
}


def traffic_key(workload, weights):
    return workload if weights == "in_place" else workload + ":" + weights


def measured_traffic(workload, weights):
    """(bytes per launch, stale) from profiles/traffic.json: bytes is None if there is no entry
    for this workload and weight layout; stale says the entry was measured on other kernel
    sources than the tree's."""
    try:
        with open(TRAFFIC_FILE) as f:
            entry = json.load(f).get(traffic_key(workload, weights))
    except (OSError, ValueError):
        return None, False
    if not entry:
        return None, False
    nbytes = int((entry["fetch_kib"] / entry["fetch_scale"] + entry["write_kib"]) * 1024)
    return nbytes, entry.get("sources") != kernel_sources_digest()


def record_traffic(workload, weights, fetch_kib, write_kib, kernel):
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        table = {}
    table[traffic_key(workload, weights)] = {"kernel": kernel, "fetch_kib": fetch_kib, "write_kib": write_kib,
                       "fetch_scale": FETCH_SCALE, "weights": weights,
                       "sources": kernel_sources_digest()}
    with open(TRAFFIC_FILE, "w") as f:
        json.dump(table, f, indent=1, sort_keys=True)
        f.write("\n")


def algorithmic_bytes(cfg, active_experts):
    """Weights of the experts actually selected once, router weight once,
    activations in and out once (no scratch traffic)."""
    b = 2 if cfg.dtype == "bf16" else 4
    return (active_experts * 3 * cfg.H * cfg.I + cfg.E * cfg.H + 2 * cfg.T * cfg.H) * b


def algorithmic_flops(cfg):
    return cfg.T * cfg.k * 6 * cfg.H * cfg.I + 2 * cfg.T * cfg.H * cfg.E


def cpu_baseline(cfg, inp, seconds_budget=25.0):
    """The reference's CPU MoE on a bounded sample of the same workload, one thread, as the
    reference ships it: the reference's own headers compiled behind C entry points
    (oracle/_ref, kind "reference") where that library has been built and the workload is one
    it covers (no router bias), else the restatement of it (kind "port"; the two return the
    same bits, tests/test_oracle_vs_ref.py). The restatement with the tokens dealt out over
    all host cores is reported beside it."""
    from oracle import oracle

    gate = inp["gate"].float().cpu().numpy()
    ffn1 = inp["ffn1"].float().cpu().numpy()
    ffn2 = inp["ffn2"].float().cpu().numpy()
    bias = None if inp["bias"] is None else inp["bias"].float().cpu().numpy()
    x = inp["tokens"].float().cpu().numpy()
    use_ref = bias is None and oracle.have_ref()

    def one_thread(rows):
        if use_ref:
            return oracle.ref_full_moe(rows, gate, ffn1, ffn2, cfg.k)
        return oracle.forward(rows, gate, ffn1, ffn2, cfg.k, bias=bias, nthreads=1)[0]

    # cost is linear in tokens: time 2 tokens, then size the sample to the budget
    t0 = time.perf_counter()
    one_thread(x[:2])
    per_tok = (time.perf_counter() - t0) / 2
    n = int(max(2, min(cfg.T, seconds_budget / max(per_tok, 1e-9))))
    # repeat the sample until about 10 s of CPU work have been timed
    reps = int(max(1, min(50, 10.0 / max(per_tok * n, 1e-9))))
    t0 = time.perf_counter()
    for _ in range(reps):
        one_thread(x[:n])
    dt = (time.perf_counter() - t0) / reps
    # the restatement with the tokens dealt out over all host cores (tokens are independent)
    cores = max(1, min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0")) or 64))
    m = int(min(cfg.T, max(n, 4 * cores)))
    t0 = time.perf_counter()
    oracle.forward(x[:m], gate, ffn1, ffn2, cfg.k, bias=bias, nthreads=cores)
    dt_all = time.perf_counter() - t0
    return {
        "value": n / dt,
        "unit": "tokens/s",
        "cores": 1,
        "kind": "reference" if use_ref else "port",
        "sample": "first %d of %d tokens of the workload, %d passes of %.2f s, one thread"
                  % (n, cfg.T, reps, dt),
        "us_per_layer_extrapolated": dt / n * cfg.T * 1e6,
        "all_cores": {"value": m / dt_all, "unit": "tokens/s", "cores": cores, "kind": "port",
                      "sample": "first %d tokens, one pass of %.2f s, tokens sharded over %d threads"
                                % (m, dt_all, cores)},
    }


def cold_cache_us(launcher, x, out, reps=20):
    """Median duration of single launches that each follow a pass over a 1 GiB buffer, which
    evicts the L2s and the 256 MB memory-side cache: the launch as a serving step meets it
    when other layers have run in between."""
    import torch

    flush = torch.empty(1 << 30, dtype=torch.uint8, device=x.device)
    ts = []
    for _ in range(reps):
        flush.add_(1)
        torch.cuda.synchronize()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        launcher.launch(x, out)
        b.record()
        torch.cuda.synchronize()
        ts.append(a.elapsed_time(b) * 1e3)
    del flush
    ts.sort()
    return ts[len(ts) // 2]


def workgroup_balance(launcher, x, out, tokens, waves_per_group):
    """Busy time per workgroup (= per CU: the launch puts one workgroup on each) of one traced
    launch: sum of its tasks' durations as the kernel's own trace facility records them."""
    import numpy as np
    import torch

    launcher.trace_enable(1 << 19)
    launcher.launch(x, out)
    torch.cuda.synchronize()
    rec = launcher.trace_read()
    launcher.trace_enable(0)
    if len(rec) == 0:
        return None
    group = rec["worker"] // waves_per_group
    busy = np.zeros(int(group.max()) + 1)
    np.add.at(busy, group, (rec["t_end"] - rec["t_ready"]) / 100.0 / waves_per_group)
    span = float(rec["t_end"].max() - rec["t_fetch"].min()) / 100.0
    return {"workgroups": int(len(busy)), "busy_us_max": float(busy.max()), "busy_us_mean": float(busy.mean()),
            "busy_us_min": float(busy.min()), "max_over_mean": float(busy.max() / busy.mean()),
            "traced_span_us": span, "tasks": int(len(rec)), "tokens": int(tokens)}


def board_power(name, seed, sched, weights, seconds=2.0):
    """Back-to-back launches of workload `name` for about `seconds`, with the board power the
    driver reports (hwmon power1_input / power1_average, microwatts) sampled every 20 ms from a
    thread of this process: what the launch draws against the board's power cap, next to the
    same reading with the GPU idle."""
    import glob
    import threading

    import torch

    from flash_distributed_moe_amd import synth
    from flash_distributed_moe_amd.flashMoeLauncher import MoeKernelLauncher

    files = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input") +
                   glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_average"))
    caps = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_cap"))
    if not files:
        sys.exit("bench.py --power: the driver exposes no hwmon power reading here")

    def read(path):
        try:
            return int(open(path).read().strip()) / 1e6
        except (OSError, ValueError):
            return None

    launcher = None
    if name == "vendor_gemm_8192":
        # the vendor's bf16 GEMM (torch.matmul) for comparison: 8192 x 8192 x 8192
        a = torch.randn(8192, 8192, device="cuda:0", dtype=torch.bfloat16)
        b = torch.randn(8192, 8192, device="cuda:0", dtype=torch.bfloat16) * 0.02

        def launch():
            torch.matmul(a, b.t())
    else:
        cfg = synth.CONFIGS[name]
        inp = synth.make_inputs_torch(cfg, seed, torch.device("cuda:0"))
        x = inp["tokens"]
        out = torch.empty_like(x)
        launcher = MoeKernelLauncher()
        ffn1, ffn2 = inp["ffn1"], inp["ffn2"]
        if weights == "in_place":
            ffn1, ffn2 = ffn1.clone(), ffn2.clone()
            MoeKernelLauncher.pack_weights_in_place(ffn1, ffn2)
        launcher.create(inp["gate"], ffn1, ffn2, cfg.T, launcher.getDistributedUniqueId(empty=True), 0, 1,
                        top_k=cfg.k, router_bias=inp["bias"], sched=sched, prepacked=weights == "in_place",
                        pack_weights={"in_place": False, "default": None, "row_major": False}[weights])

        def launch():
            launcher.launch(x, out)
    for _ in range(20):
        launch()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(50):
        launch()
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / 50
    launches = max(100, int(seconds * 1e6 / us))
    time.sleep(1.0)

    samples, stop = [], [False]

    def poll():
        while not stop[0]:
            samples.append((time.perf_counter(), read(files[0])))
            time.sleep(0.02)

    th = threading.Thread(target=poll)
    th.start()
    time.sleep(0.4)
    t0 = time.perf_counter()
    for _ in range(launches):
        launch()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    stop[0] = True
    th.join()
    if launcher is not None:
        err, _ = launcher.status()
        launcher.destroy()
        if err:
            sys.exit("bench.py: device error bits %d" % err)
    idle = [w for t, w in samples if t < t0 - 0.05 and w is not None]
    busy = [w for t, w in samples if t0 + 0.3 < t < t1 - 0.05 and w is not None]
    return {"workload": name, "launches": launches, "us_per_launch": (t1 - t0) / launches * 1e6,
            "power_file": files[0], "samples_busy": len(busy),
            "power_w_idle": sum(idle) / len(idle) if idle else None,
            "power_w_busy_mean": sum(busy) / len(busy) if busy else None,
            "power_w_busy_max": max(busy) if busy else None,
            "power_cap_w": read(caps[0]) if caps else None}


def measure(name, seed, steps, warmup, sched, weights, cold=False, balance=False):
    """K timed launches of workload `name`: whole-job wall time, the kernel's launch-to-launch
    duration from events on the launch stream, and where that puts it on its roofline."""
    import torch

    from flash_distributed_moe_amd import synth
    from flash_distributed_moe_amd.flashMoeLauncher import MoeKernelLauncher

    cfg = synth.CONFIGS[name]
    dev = torch.device("cuda:0")
    inp = synth.make_inputs_torch(cfg, seed, dev)
    x = inp["tokens"]
    out = torch.empty_like(x)
    launcher = MoeKernelLauncher()
    ffn1, ffn2 = inp["ffn1"], inp["ffn2"]
    if weights == "in_place":
        # the layout the kernels read fastest, made where the tensors lie: the launcher keeps
        # no copy of the weights (the row-major originals stay in `inp` for the CPU baseline)
        ffn1, ffn2 = ffn1.clone(), ffn2.clone()
        MoeKernelLauncher.pack_weights_in_place(ffn1, ffn2)
    launcher.create(inp["gate"], ffn1, ffn2, cfg.T,
                    launcher.getDistributedUniqueId(empty=True), 0, 1, top_k=cfg.k,
                    router_bias=inp["bias"], sched=sched, prepacked=weights == "in_place",
                    pack_weights={"in_place": False, "default": None, "row_major": False}[weights])
    for _ in range(warmup):
        launcher.launch(x, out)
    torch.cuda.synchronize()

    # whole-job wall time over exactly K steps
    t0 = time.perf_counter()
    for _ in range(steps):
        launcher.launch(x, out)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / steps * 1e3

    # per-launch kernel duration: events on the launch stream around single launches
    n_ev = min(steps, 200)
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
           for _ in range(n_ev)]
    for a, b in evs:
        a.record()
        launcher.launch(x, out)
        b.record()
    torch.cuda.synchronize()
    durs = sorted(a.elapsed_time(b) for a, b in evs)  # ms
    kernel_ms_avg = sum(durs) / len(durs)
    kernel_ms_med = durs[len(durs) // 2]

    err, _ = launcher.status()
    if err:
        sys.exit("bench.py: device error bits %d" % err)
    routing = launcher.routing(cfg.T)
    active = int((routing["counts"] > 0).sum())
    tiled = launcher.sched_for(cfg.T) != 1
    kernel = "moe_tiled_kernel" if tiled else "moe_stream_kernel"
    extra = {}
    if cold:
        extra["cold_cache_us"] = cold_cache_us(launcher, x, out)
    if balance:
        extra["per_cu_busy"] = workgroup_balance(launcher, x, out, cfg.T, 1 if tiled else 8)
        counts = routing["counts"]
        extra["rows_per_expert"] = {"max": int(counts.max()), "mean": float(counts.mean()),
                                    "share_of_4_largest": float(sorted(counts)[-4:] and
                                                                sum(sorted(counts)[-4:]) / max(1, counts.sum()))}
    launcher.destroy()

    bound = BOUND.get(cfg.name, "hbm")
    abytes = algorithmic_bytes(cfg, active)
    aflops = algorithmic_flops(cfg)
    mfma_peak = MFMA_BF16_PEAK_TFLOPS if cfg.dtype == "bf16" else MFMA_F32_PEAK_TFLOPS
    if bound == "hbm":
        achieved = abytes / (kernel_ms_avg * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = aflops / (kernel_ms_avg * 1e-3) / 1e12
        peak, unit = mfma_peak, "TFLOP/s"
    traffic, stale = measured_traffic(cfg.name, weights)
    roofline = {
        "bound": bound, "achieved": achieved, "peak": peak, "unit": unit,
        "frac": achieved / peak,
        "traffic": None if stale else traffic,
        "kernel": kernel,
        "kernel_us_avg": kernel_ms_avg * 1e3, "kernel_us_median": kernel_ms_med * 1e3,
        "algorithmic_bytes": abytes, "algorithmic_flops": aflops, "active_experts": active,
        "hbm_frac": abytes / (kernel_ms_avg * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "mfma_frac": aflops / (kernel_ms_avg * 1e-3) / 1e12 / mfma_peak,
    }
    if stale:
        roofline["traffic_stale"] = traffic   # measured on other kernel sources than the tree's
    roofline.update(extra)
    config = {"workload": cfg.name, "tokens": cfg.T, "hidden": cfg.H, "experts": cfg.E,
              "top_k": cfg.k, "intermediate": cfg.I, "hot_experts": cfg.hot,
              "seed": seed, "packed_weight_copy": weights == "default", "weights": WEIGHT_MODES[weights]}
    return cfg, inp, ms_per_step, roofline, config


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="qwen3_30b_decode")
    ap.add_argument("--seed", type=int, default=7907)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--sched", type=int, default=0)
    ap.add_argument("--weights", default="in_place", choices=sorted(WEIGHT_MODES),
                    help="in_place: weights packed in place by the caller (the headline); default: "
                         "row-major tensors given to create() with no flags (the launcher keeps a "
                         "packed copy); row_major: read in place")
    ap.add_argument("--no-extra-records", action="store_true",
                    help="only the one workload: none of the sub-records of the other configurations")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only copy 1 GiB device to device five times: the known traffic the "
                         "rocprofv3 byte counters are scaled by")
    ap.add_argument("--gemm-calibration", action="store_true",
                    help="time torch.matmul (the vendor GEMM) in bf16 on this box: the matrix-core "
                         "rate reachable in practice, next to the published peak")
    ap.add_argument("--power", action="store_true",
                    help="launch --config back to back for two seconds and report the board power "
                         "the driver reads meanwhile, beside the power cap")
    ap.add_argument("--record-traffic", nargs=2, type=float, metavar=("FETCH_KIB", "WRITE_KIB"),
                    help="no GPU work: write the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings "
                         "(KiB per dispatch) of --config into profiles/traffic.json")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: this build runs the MoE layer on ONE GPU (no collectives, no "
                 "multi-GPU path); run with --gpus 1")
    packed = args.weights
    if args.record_traffic:
        kernel = "moe_tiled_kernel" if BOUND.get(args.config) == "mfma" or "4096" in args.config \
            else "moe_stream_kernel"
        record_traffic(args.config, packed, args.record_traffic[0], args.record_traffic[1], kernel)
        print(json.dumps({args.config: measured_traffic(args.config, packed)[0]}))
        return

    import torch

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    torch.cuda.set_device(0)
    if args.copy_calibration:
        a = torch.randn(1 << 28, device="cuda:0", dtype=torch.float32)
        b = torch.empty_like(a)
        for _ in range(5):
            b.copy_(a)
        torch.cuda.synchronize()
        print(json.dumps({"copy_calibration": {"copies": 5, "kib_read_each": 1 << 20,
                                               "kib_written_each": 1 << 20}}))
        return

    if args.gemm_calibration:
        # What the vendor's GEMM (torch.matmul -> hipBLASLt) reaches on this box, on operands of
        # the same kind (bf16, normal random values): the matrix-core ceiling a kernel meets in
        # practice here, to set beside the published peak the roofline is quoted against.
        out = {}
        for name, (m, n, k) in {"square_8192": (8192, 8192, 8192),
                                "layer_gate_up_as_one_gemm": (65536, 1536, 2048),
                                "layer_down_as_one_gemm": (65536, 2048, 768)}.items():
            a = torch.randn(m, k, device="cuda:0", dtype=torch.bfloat16)
            b = torch.randn(n, k, device="cuda:0", dtype=torch.bfloat16) * 0.02
            for _ in range(5):
                torch.matmul(a, b.t())
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            reps = 30
            e0.record()
            for _ in range(reps):
                torch.matmul(a, b.t())
            e1.record()
            torch.cuda.synchronize()
            us = e0.elapsed_time(e1) * 1e3 / reps
            out[name] = {"m": m, "n": n, "k": k, "us": us, "tflops": 2.0 * m * n * k / us / 1e6,
                         "frac_of_2500": 2.0 * m * n * k / us / 1e6 / 2500.0}
            del a, b
        print(json.dumps({"gemm_calibration": out}))
        return

    if args.power:
        print(json.dumps({"board_power": board_power(args.config, args.seed, args.sched, packed)}))
        return

    headline = args.config == "qwen3_30b_decode"
    cfg, inp, ms_per_step, roofline, config = measure(args.config, args.seed, args.steps,
                                                      args.warmup, args.sched, packed, cold=headline)
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(cfg, inp)
    del inp

    line = {
        "metric": "MoE-layer tokens/s (Qwen3-style fused MoE forward, us/layer alongside)",
        "value": cfg.T / (ms_per_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "us_per_layer": ms_per_step * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": cfg.dtype,
        "data": "synthetic (seeded Irwin-Hall normal weights sigma 0.02, activations sigma 1)",
        "config": config,
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    if not args.no_extra_records and headline:
        # The other configurations the reference's numbers are asked for on, same fields each:
        # the 8192-token prefill (bound by the matrix cores), the decode batch as a caller written
        # against the reference gets it (caller_layout: row-major tensors, create() without flags,
        # the launcher's packed copy) and on the row-major tensors read in place
        # (row_major_weights), the 235B shape at 256 and 4096 tokens (both roofline fractions are
        # in every record: hbm_frac, mfma_frac) and the imbalance stress with the busy time per
        # CU. Each is timed over at least 50 launches, so that ms_per_step is the kernel's
        # time and not the cost of the final synchronisation.
        import torch

        def sub(name, packed_, balance=False):
            steps, warmup = max(50, args.steps), max(5, args.warmup)
            c, i_, ms, roof, conf = measure(name, args.seed, steps, warmup, args.sched, packed_,
                                            balance=balance)
            del i_
            torch.cuda.empty_cache()
            return {"value": c.T / (ms * 1e-3), "unit": "tokens/s", "steps": steps, "warmup": warmup,
                    "ms_per_step": ms, "us_per_layer": ms * 1e3, "dtype": c.dtype, "config": conf,
                    "roofline": roof}

        torch.cuda.empty_cache()
        line["prefill"] = sub("qwen3_30b_prefill", packed)
        line["caller_layout"] = sub("qwen3_30b_decode", "default")
        line["row_major_weights"] = sub("qwen3_30b_decode", "row_major")
        line["c4_t256"] = sub("qwen3_235b_t256", packed)
        line["c4_t4096"] = sub("qwen3_235b_t4096", packed)
        line["imbalance"] = sub("qwen3_30b_imbalance", packed, balance=True)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
