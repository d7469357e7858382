#!/usr/bin/env python3
"""Benchmark of the MoE-layer hot path on one MI355X.

A step is one forward + backward of one MoE layer (gate, routing, dispatch, grouped expert FFN,
combine, and all of their gradients) over one batch of synthetic tokens resident in HBM.  The
default workload is configuration 2 of the benchmark set (the one the headline metric is quoted on): Switch-style layer, bf16 with fp32 accumulation,
16384 tokens x 1024, 16 experts of 1024 -> 4096 -> 1024, top-1, capacity factor 1.25.

Prints ONE JSON line: the metric (tokens/s), the roofline of the dominant kernel measured with HIP
events on the stream the kernel runs on, the same figures for configuration 1 (fp32, the CPU-runnable
case) on the GPU, and the CPU oracle timed on configuration 1 on this box's host cores.

--probe prints a different line: what the matrix cores sustain on their own (zero and random operands)
and what the product's K loop sustains without its epilogue, at the default workload's shape.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: S, M, E, k, F, capacity_factor, dtype, zipf gate bias
    "c1": dict(S=4096, M=512, E=8, k=2, F=2048, cf=1.0, dtype="f32", zipf=False),
    "c2": dict(S=16384, M=1024, E=16, k=1, F=4096, cf=1.25, dtype="bf16", zipf=False),
    "c3": dict(S=8192, M=2048, E=64, k=2, F=8192, cf=0.0, dtype="bf16", zipf=True),
    "c5": dict(S=32768, M=2048, E=256, k=8, F=1024, cf=0.0, dtype="bf16", zipf=False),
}
PEAK_MFMA_TFLOPS = {"bf16": 2500.0, "f32": 157.3}   # MI355X dense peaks
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch (read + write) of the grouped products come from rocprofv3 FETCH_SIZE / WRITE_SIZE runs of
# this script (`--ingest-counters` turns the two counter CSVs into profiles/hbm_traffic.json, which also records the
# hashes of the kernel sources the counters were read from).  A workload whose kernel sources have changed since
# reports "traffic": null rather than a stale figure.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
KERNEL_SOURCES = ("MOLE/cpp/gemm256.hip", "MOLE/cpp/gemm_f32.hip", "MOLE/cpp/ffn_gemm.hip", "MOLE/cpp/gemm.h", "MOLE/cpp/lds_dma.h")
# read bytes = FETCH_SIZE x 2 KiB, written bytes = WRITE_SIZE x 1 KiB on this chip (calibrated against a copy of
# known size in the same runs, see profiles/bench_c2_hbm_traffic.txt)
FETCH_UNIT_BYTES, WRITE_UNIT_BYTES = 2048.0, 1024.0
# a product counts as HBM-bound when the bytes it really moves, over its duration, reach the rate a large copy
# sustains on this chip (4.9-5.4 TB/s of the 8 TB/s peak); below that its duration follows the matrix pipe
HBM_BOUND_FROM = 0.55


def kernel_source_hashes():
    import hashlib
    return {f: hashlib.sha256(open(os.path.join(ROOT, f), "rb").read()).hexdigest()[:16] for f in KERNEL_SOURCES}


def measured_traffic(name):
    """{kernel: bytes per launch} for workload `name`, or {} when no counter run exists for the current kernel sources."""
    try:
        with open(TRAFFIC_FILE) as fh:
            data = json.load(fh)
    except (OSError, ValueError):
        return {}
    entry = data.get("workloads", {}).get(name)
    if not entry or entry.get("kernel_sources") != kernel_source_hashes():
        return {}
    return entry["bytes_per_launch"]


def ingest_counters(args):
    """Reads the counter_collection CSVs of a FETCH_SIZE run and a WRITE_SIZE run of `bench.py --workload W --no-c1
    --no-c35 --no-cpu-baseline` and stores the grouped products' HBM bytes per launch for W in profiles/hbm_traffic.json."""
    import csv
    import re
    import subprocess

    def launches(path, counter):
        """{product: [counter value of every launch, in dispatch order]} of the grouped kernels in one counter CSV"""
        rows = []
        with open(path, newline="") as fh:
            for r in csv.DictReader(fh):
                mt = re.search(r"mole::(?:\(anonymous namespace\)::)?gemm(?:256|_f32)?_kernel<(.*)>\(", r["Kernel_Name"])
                if r.get("Counter_Name") == counter and mt:
                    targs = [a.strip() for a in mt.group(1).split(",")]
                    rows.append((int(r["Dispatch_Id"]), targs, int(r["Grid_Size"]), float(r["Counter_Value"])))
        rows.sort(key=lambda t: t[0])
        # template arguments end in <..., WG, [BM, BN,] EPI>: EPI 2 = h and a, 1 = out, 3 = t, 4 = a weight gradient (g_w2
        # and g_w1 alternate), 0 = gx - or a product of the gate, which has another grid than the launch of `out`
        out = {n: [] for n in ("ffn_fwd1", "ffn_fwd2", "ffn_gw2", "ffn_da", "ffn_gw1", "ffn_gx")}
        grid_fwd2, n_wg = None, 0
        for _, targs, grid, val in rows:
            epi = int(targs[-1])
            if epi == 2: out["ffn_fwd1"].append(val)
            elif epi == 1: out["ffn_fwd2"].append(val); grid_fwd2 = grid
            elif epi == 3: out["ffn_da"].append(val)
            elif epi == 4 and ("true" in targs[:4] or targs[-2] == "true"):
                out["ffn_gw2" if n_wg % 2 == 0 else "ffn_gw1"].append(val); n_wg += 1
            elif epi == 0 and grid == grid_fwd2: out["ffn_gx"].append(val)
        return out
    fetch, write = launches(args.ingest_counters[0], "FETCH_SIZE"), launches(args.ingest_counters[1], "WRITE_SIZE")
    steps = len(fetch["ffn_fwd1"])
    assert steps > 0 and all(len(v) == steps for v in fetch.values()) and all(len(v) == steps for v in write.values()), \
        ({n: len(v) for n, v in fetch.items()}, {n: len(v) for n, v in write.items()})
    first = steps // 3                      # the first third of the launches is warm-up
    out = {}
    for n in fetch:
        rd = sum(fetch[n][first:]) / (steps - first) * FETCH_UNIT_BYTES
        wr = sum(write[n][first:]) / (steps - first) * WRITE_UNIT_BYTES
        out[n] = round(rd + wr)
        out[n + "_read"], out[n + "_written"] = round(rd), round(wr)
    try:
        with open(TRAFFIC_FILE) as fh:
            data = json.load(fh)
    except (OSError, ValueError):
        data = {"what": "HBM bytes per launch of the grouped products, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of "
                        "bench.py (bench.py --ingest-counters); FETCH_SIZE x 2 KiB + WRITE_SIZE x 1 KiB", "workloads": {}}
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        commit = ""
    data["workloads"][args.workload] = {"kernel_sources": kernel_source_hashes(), "measured_after_commit": commit,
                                        "steps_averaged": steps - first, "bytes_per_launch": out}
    with open(TRAFFIC_FILE, "w") as fh:
        json.dump(data, fh, indent=1, sort_keys=True)
        fh.write("\n")
    print(json.dumps({args.workload: out}))


PEAK_HBM_BYTES = PEAK_HBM_GBS * 1e9


def make_layer(w, seed=0):
    import torch
    from mole_amd.moe.layer import MOLEModule
    MOLEModule.reset_instances()
    dt = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    bias = None
    g = torch.Generator().manual_seed(seed)
    if w["zipf"]:
        ranks = torch.randperm(w["E"], generator=g).float() + 1.0
        bias = torch.log(ranks ** -1.2)
    m = MOLEModule(0, w["E"], w["M"], w["F"], -1, w["k"], 4, {"local_rank": 0, "world_size": 1, "rank": 0}, "gelu", 1,
                   False, False, dtype=dt, gate_logit_bias=bias)
    with torch.no_grad():
        m.gate[0].linear.weight.copy_(torch.randn(w["E"], w["M"], generator=g) * (1.0 / w["M"] ** 0.5 if w["name"] == "c5" else 0.02))
        for p in (m.FC1_W_GPU, m.FC1_B_GPU, m.FC2_W_GPU, m.FC2_B_GPU):
            p.all_tensors.normal_(0.0, 0.02)
    x = torch.randn(w["S"], w["M"], generator=g).to(dt).cuda().requires_grad_(True)
    dy = (torch.randn(w["S"], w["M"], generator=g) * 1e-3).to(dt).cuda()
    return m, x, dy


def step(m, x, dy, cf):
    y = m(x, capacity_factor=cf)
    y.backward(dy)
    x.grad = None
    m.gate[0].linear.weight.grad = None


def cpu_baseline(budget_s=12.0):
    """The CPU oracle's layer (fp32 torch on the host cores), forward + backward, on configuration 1 of the benchmark set
    exactly as specified: 4096 tokens x 512 ~N(0,1), gate 512 -> 8 ~N(0,0.02), top-2, experts
    Linear(512 -> 2048) + GELU + Linear(2048 -> 512) ~N(0,0.02), fp32, seed 0, MSE against zero, the reference's
    default capacity factor 1.0.  Three warm-up steps, then at least ten timed ones (until budget_s), median."""
    import torch
    from oracle import moe_oracle as O
    w = WORKLOADS["c1"]
    cores = min(16, os.cpu_count() or 1)
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    S, E, M, F = w["S"], w["E"], w["M"], w["F"]
    x = torch.randn(S, M, generator=g)
    wg = torch.randn(E, M, generator=g) * 0.02
    w1, b1 = torch.randn(E, F, M, generator=g) * 0.02, torch.randn(E, F, generator=g) * 0.02
    w2, b2 = torch.randn(E, F, M, generator=g) * 0.02, torch.randn(E, M, generator=g) * 0.02

    y = O.moe_layer(x, wg, w1, b1, w2, b2, w["k"], w["cf"]).y
    dy = 2.0 * y / y.numel()                      # gradient of mean(y^2); the inputs are fixed, so it is too

    def run():
        return O.moe_layer(x, wg, w1, b1, w2, b2, w["k"], w["cf"], dy=dy)

    for _ in range(3):
        run()
    times = []
    t_start = time.perf_counter()
    while len(times) < 10 or (time.perf_counter() - t_start < budget_s and len(times) < 40):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(S / med, 1), "unit": "tokens/s", "cores": cores, "kind": "port", "ms_per_step": round(med * 1e3, 2),
            "sample": f"{len(times)} steps of configuration c1 exactly (S={S} M={M} E={E} top-{w['k']} F={F} fp32, seed 0, "
                      f"capacity factor {w['cf']}, MSE against zero), forward + backward, "
                      f"fp32 torch-CPU oracle on {cores} threads, median"}


def bench_offloaded_stack(args):
    """Configuration 4 of the benchmark set: a stack of MoE layers whose experts all live in pinned host memory and
    stream through the device slot pool (32 experts of 4096 -> 14336 -> 4096, bf16: 235 MB per expert,
    7.5 GB per layer; 4096 tokens x 4096, top-2, no drop).  The step is PCIe bound by construction, so
    the figures of interest are the copy stream's host-to-device rate and how much of the step the
    copies cover.  --layers sets the depth (12 in the configuration; each layer pins 15 GB of host
    memory for weights and gradients, the default of 2 keeps set-up within a minute or two)."""
    import torch
    from mole_amd import _lib as L, core
    from mole_amd.moe.layer import MOLEModule
    S, M, E, k, F = 4096, 4096, 32, 2, 14336
    n_layers, ebatch = args.layers, 8
    # 64 slots (15 GB of HBM) are the two layers' worth of the configuration; a slot for every expert of the stack
    # (235 MB each: 90 GB at the configuration's 12 layers, of 288 GB) lets the backward passes reuse what the forward
    # passes fetched
    pool = 64 if args.no_resident else max(64, n_layers * E)
    MOLEModule.reset_instances()
    dist = {"local_rank": 0, "world_size": 1, "rank": 0}
    layers = []
    for i in range(n_layers):
        print(f"[c4] building layer {i} (pinned host weights)", file=sys.stderr, flush=True)
        try:
            layers.append(MOLEModule(E, 0, M, F, pool, k, ebatch, dist, "gelu", 1, bool(args.adam), True, dtype=torch.bfloat16,
                                     resident=not args.no_resident))
        except RuntimeError as exc:     # pinned host memory is capped well below the machine's RAM on some boxes
            print(f"[c4] layer {i} could not be built ({str(exc).splitlines()[0]}): lower --layers", file=sys.stderr)
            sys.exit(3)
    for m in layers:
        m.set_prefetch(E, E)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(S, M, generator=g).to(torch.bfloat16).cuda().requires_grad_(True)
    dy = (torch.randn(S, M, generator=g) * 1e-3).to(torch.bfloat16).cuda()
    um = core.get_UniMem()

    step_no = [0]

    def one_step():
        if args.adam:     # the optimizer hands the hyper-parameters and its step counter to every layer
            for m in layers:
                m.MOLECore.set_adam(0.9, 0.999, step_no[0], 1e-4, 0.01, 1e-8, True, -1)
            step_no[0] += 1
        layers[0].prefetch_fwd(E)                 # what the scheduler does before the first layer
        h = x
        for m in layers:
            h = m(h, capacity_factor=0.0, prefetch=True)
        h.backward(dy)
        x.grad = None
        for m in layers:
            m.gate[0].linear.weight.grad = None

    for i in range(args.warmup):
        print(f"[c4] warm-up step {i}", file=sys.stderr, flush=True)
        one_step()
    torch.cuda.synchronize(); core.synchronize_tran()
    um.copy_stats(); um.writeback_stats()         # forget the warm-up's copies
    # a step ends when its gradients have landed in host memory: the optimizer that sits between two steps of a
    # training loop needs them there, so nothing of the next step may hide behind this step's write-back
    t0 = time.perf_counter()
    for i in range(args.steps):
        print(f"[c4] timed step {i}", file=sys.stderr, flush=True)
        one_step()
        torch.cuda.synchronize(); core.synchronize_tran()
    wall = (time.perf_counter() - t0) / args.steps
    # the same steps back to back (the next step's fetches run beside this step's write-back): what a loop whose
    # optimizer keeps up layer by layer could approach; reported beside the headline, never as it
    t1 = time.perf_counter()
    for i in range(args.steps):
        one_step()
    torch.cuda.synchronize(); core.synchronize_tran()
    wall_pipelined = (time.perf_counter() - t1) / args.steps
    h2d_bytes, h2d_ms = um.copy_stats()
    h2d_bytes /= 2 * args.steps; h2d_ms /= 2 * args.steps
    resident = all(m.MOLECore.resident and m.MOLECore._home_base() is not None for m in layers)
    d2h_bytes, d2h_ms = um.writeback_stats()
    d2h_bytes /= 2 * args.steps; d2h_ms /= 2 * args.steps
    L.kernel_timing_enable(True)
    one_step()
    torch.cuda.synchronize(); core.synchronize_tran()
    timing = L.kernel_timing_read()
    L.kernel_timing_enable(False)
    kernel_ms = sum(ms for _, ms in timing.values())
    gemm_ms = sum(ms for n, (_, ms) in timing.items() if n.startswith("ffn_") and n != "ffn_gb")
    R = S * k
    expert_bytes = (2 * F * M + F + M) * 2
    out = {
        "metric": "MoE layer tokens/sec fwd+bwd on 1 MI355X", "value": round(S / wall, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1e3, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": f"c4: {n_layers}-layer offloaded-expert stack fwd+bwd, S={S} M={M} E={E} top-{k} F={F}, "
                               f"experts in pinned host memory, pool {pool} slots, chunks of {ebatch} experts"
                               + (", experts kept in the pool from forward to backward" if resident else ", experts fetched for every pass")
                               + (", in-pipeline AdamW on the GPU (fp32 moments in pinned host memory)" if args.adam else "")},
        "ms_per_step_back_to_back": round(wall_pipelined * 1e3, 2),
        "prefetch": {"h2d_bytes_per_step": int(h2d_bytes), "h2d_busy_ms": round(h2d_ms, 2),
                     "h2d_gbs": round(h2d_bytes / (h2d_ms * 1e-3) / 1e9, 2),
                     "h2d_busy_frac_of_step": round(h2d_ms / (wall * 1e3), 4),
                     # every activated expert once per pass, or once per step when the pool keeps it from the
                     # forward pass to the backward pass (plus the fp32 moments for the in-pipeline optimizer)
                     "expected_h2d_bytes": ((1 if resident else 2) + (4 if args.adam else 0)) * n_layers * E * expert_bytes,
                     "experts_resident_from_forward_to_backward": resident,
                     "d2h_gradient_bytes_per_step": int(d2h_bytes), "d2h_busy_ms": round(d2h_ms, 2),
                     "d2h_gbs": round(d2h_bytes / (d2h_ms * 1e-3) / 1e9, 2)},
        "kernel_ms_per_step": round(kernel_ms, 2),
        "roofline": {"bound": "mfma", "kernel": "all six grouped products", "unit": "TFLOP/s", "peak": 2500.0,
                     "achieved": round(12.0 * R * M * F * n_layers / (gemm_ms * 1e-3) / 1e12, 1),
                     "frac": round(12.0 * R * M * F * n_layers / (gemm_ms * 1e-3) / 1e12 / 2500.0, 4), "traffic": None},
    }
    print(json.dumps(out))


def measure_layer(name, steps, warmup, with_adam=True):
    """Times `steps` forward + backward passes of one MoE layer of workload `name` (inputs resident in HBM), then the
    same steps again with the library's per-kernel events on.  Returns the JSON fields of that workload."""
    import torch
    from mole_amd import _lib as L
    w = dict(WORKLOADS[name], name=name)
    m, x, dy = make_layer(w)
    cf = w["cf"]
    for _ in range(warmup):
        step(m, x, dy, cf)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(m, x, dy, cf)
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    ms_per_step = dt_s / steps * 1e3
    value = w["S"] / (dt_s / steps)

    # per-kernel durations: a second pass of the same steps with start/stop events attached to every kernel
    # launch, on the stream the kernel is launched on
    L.kernel_timing_enable(True)
    for _ in range(steps):
        step(m, x, dy, cf)
    torch.cuda.synchronize()
    timing = L.kernel_timing_read()
    L.kernel_timing_enable(False)

    R = int(m.last_route.offsets[-1].item())       # kept (token, choice) rows
    S, M, F, k = w["S"], w["M"], w["F"], w["k"]
    b = 2 if w["dtype"] == "bf16" else 4
    gemm_flop = 2.0 * R * M * F                     # every one of the six grouped products
    # algorithmic HBM bytes of the products (operands once, results once; kept rows only)
    act, wts = R * (M + 0.0) * b, w["E"] * F * M * b * 1.0
    gemm_bytes = {"ffn_fwd1": act + wts + 2 * R * F * b, "ffn_fwd2": R * F * b + wts + act,
                  "ffn_gw2": R * F * b + act + wts, "ffn_da": act + wts + 2 * R * F * b,
                  "ffn_gw1": R * F * b + act + wts, "ffn_gx": R * F * b + wts + act}
    work = {  # algorithmic work per launch: flop for the GEMMs, bytes for the permutes
        "ffn_fwd1": gemm_flop, "ffn_fwd2": gemm_flop, "ffn_gw2": gemm_flop, "ffn_da": gemm_flop, "ffn_gw1": gemm_flop,
        "ffn_gx": gemm_flop,
        # the combine backward is one fused kernel (d_o scatter and the gate dot products read dy and o once); the
        # dispatch reads a token's row once and writes it to each of its kept pairs' rows (with one choice per token
        # that is the 2 R rows of a read and a write per kept row; with more it is S + R, not 2 R)
        "dispatch_fwd": (min(S, R) + R) * M * b, "combine_fwd": (R + S) * M * b, "combine_bwd": (S + 2.0 * R) * M * b,
        "dispatch_bwd": (R + S) * M * b,
    }
    kernels = {}
    for kname, (cnt, ms) in timing.items():
        if cnt == 0:
            continue
        avg_us = ms / cnt * 1e3
        entry = {"avg_us": round(avg_us, 2), "launches_per_step": cnt / steps}
        if kname in work:
            if kname.startswith("ffn_"):
                entry["tflops"] = round(work[kname] / (avg_us * 1e-6) / 1e12, 1)
            else:
                entry["gbs"] = round(work[kname] / (avg_us * 1e-6) / 1e9, 1)
        kernels[kname] = entry
    gemms = [n for n in kernels if n in gemm_bytes]
    dom = max(gemms, key=lambda n: kernels[n]["avg_us"])
    peak = PEAK_MFMA_TFLOPS[w["dtype"]]
    dom_s = kernels[dom]["avg_us"] * 1e-6
    gemm_total_us = sum(kernels[n]["avg_us"] for n in gemms)
    traffic = measured_traffic(name).get(dom)
    mfma_frac = kernels[dom]["tflops"] / peak
    hbm_alg_frac = gemm_bytes[dom] / dom_s / PEAK_HBM_BYTES
    hbm_meas_frac = traffic / dom_s / PEAK_HBM_BYTES if traffic else None
    # HBM-bound when the bytes the kernel really moves go at the rate of a large copy; without a counter run for the
    # current kernel sources, when its algorithmic bytes are nearer their roof than its flop are to theirs
    hbm_bound = hbm_meas_frac >= HBM_BOUND_FROM if hbm_meas_frac is not None else hbm_alg_frac > mfma_frac
    if hbm_bound:
        roofline = {"bound": "hbm", "kernel": dom, "achieved": round(gemm_bytes[dom] / dom_s / 1e9, 1), "peak": PEAK_HBM_GBS,
                    "unit": "GB/s", "frac": round(hbm_alg_frac, 4)}
    else:
        roofline = {"bound": "mfma", "kernel": dom, "achieved": kernels[dom]["tflops"], "peak": peak, "unit": "TFLOP/s",
                    "frac": round(mfma_frac, 4)}
    # The events attached to a launch put a few microseconds of idle time between the kernels of the event-timed pass,
    # and a chip that runs its matrix products against its power limit clocks them higher after every pause: the
    # products measure 7-9 % shorter there than in the back-to-back steps that `value` is taken from (a rocprofv3
    # trace of both passes shows the same kernels at both durations).  back_to_back = step time / sum of the event-timed
    # kernel durations says by how much; frac_back_to_back is the dominant kernel's fraction at its duration inside a
    # step, if all kernels stretch alike.
    kernel_sum_us = sum(v["avg_us"] * v["launches_per_step"] for v in kernels.values())
    b2b = ms_per_step * 1e3 / kernel_sum_us if kernel_sum_us > 0 else None
    roofline.update({"back_to_back": round(b2b, 4) if b2b else None,
                     "frac_back_to_back": round((hbm_alg_frac if hbm_bound else mfma_frac) / max(b2b, 1.0), 4) if b2b else None})
    roofline.update({"traffic": traffic, "mfma_frac": round(mfma_frac, 4), "hbm_frac_algorithmic_bytes": round(hbm_alg_frac, 4),
                     "hbm_frac_measured_traffic": round(hbm_meas_frac, 4) if hbm_meas_frac is not None else None,
                     "all_ffn_gemms_frac": round(6 * gemm_flop / (gemm_total_us * 1e-6) / 1e12 / peak, 4)})
    out = {
        "value": round(value, 1), "ms_per_step": round(ms_per_step, 4), "dtype": w["dtype"],
        "config": {"workload": f"{name}: single MoE layer fwd+bwd, S={S} M={M} E={w['E']} top-{k} F={F} "
                               f"capacity_factor={cf}, kept rows R={R}"},
        "roofline": roofline,
        "hbm_permutes": {n: {"achieved": kernels[n]["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(kernels[n]["gbs"] / PEAK_HBM_GBS, 4)}
                         for n in ("dispatch_fwd", "combine_fwd", "combine_bwd", "dispatch_bwd") if n in kernels},
        "kernels": kernels,
    }
    if with_adam:
        # the fused Adam update on one weight array of this layer ([E, F, M] parameters and gradients in the
        # layer's dtype, fp32 moments): not part of the step above, measured for its own HBM roofline
        from mole_amd import hip_ops as H
        pdt = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
        n_adam = w["E"] * w["F"] * w["M"]
        ap_, ag_ = (torch.randn(n_adam, device="cuda") * 0.02).to(pdt), (torch.randn(n_adam, device="cuda") * 1e-3).to(pdt)
        am_, av_ = torch.zeros(n_adam, device="cuda"), torch.zeros(n_adam, device="cuda")
        H.adam_step(ap_, ag_, am_, av_, 0.9, 0.999, 1, 1e-3, 0.0, 1e-8, False)
        torch.cuda.synchronize()
        L.kernel_timing_enable(True)
        for i in range(5):
            H.adam_step(ap_, ag_, am_, av_, 0.9, 0.999, 2 + i, 1e-3, 0.0, 1e-8, False)
        torch.cuda.synchronize()
        adam_cnt, adam_ms = L.kernel_timing_read()["adam"]
        L.kernel_timing_enable(False)
        del ap_, ag_, am_, av_
        adam_bytes = n_adam * (22.0 if pdt == torch.bfloat16 else 28.0)   # read p, g, m, v; write p, m, v
        adam_gbs = adam_bytes / (adam_ms / adam_cnt * 1e-3) / 1e9
        out["hbm_optimizer"] = {"adam_step": {"achieved": round(adam_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                              "frac": round(adam_gbs / PEAK_HBM_GBS, 4), "elements": n_adam,
                                              "avg_us": round(adam_ms / adam_cnt * 1e3, 2)}}
    from mole_amd.moe.layer import MOLEModule
    del m, x, dy
    MOLEModule.reset_instances()
    torch.cuda.empty_cache()
    return out


def run_probes(args):
    """What bounds the grouped products at the default workload's shape, from tracked code: the matrix cores alone
    (operands in registers, zero and random data, all CUs), the product's K loop without its epilogue, the full
    first product, and a library GEMM of the same shape as a yardstick."""
    import torch
    from ctypes import byref, c_double
    from mole_amd import _lib as L, hip_ops as H
    w = WORKLOADS["c2"]
    S, M, E, F = w["S"], w["M"], w["E"], w["F"]
    dev = "cuda"
    n_cu = torch.cuda.get_device_properties(0).multi_processor_count
    nb = L.lib().mole_probe_mfma_operand_bytes()
    sink = torch.zeros(n_cu * 512, device=dev)
    res = {}

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        L.kernel_timing_enable(True)
        for _ in range(reps):
            fn()
        torch.cuda.synchronize()
        t = L.kernel_timing_read()
        L.kernel_timing_enable(False)
        return t

    flop = c_double()
    for kind in ("zeros", "random"):
        ops = torch.zeros(nb // 2, dtype=torch.bfloat16, device=dev) if kind == "zeros" else \
            (torch.randn(nb // 2, device=dev) * 0.5).bfloat16()
        iters = 4000
        t = timed(lambda: L.check(L.lib().mole_probe_mfma(L.ptr(ops), n_cu, iters, L.ptr(sink), byref(flop), L.stream()),
                                  "mole_probe_mfma"), 5)
        cnt, ms = t["probe"]
        res[f"mfma_only_{kind}_operands"] = {"avg_us": round(ms / cnt * 1e3, 1), "tflops": round(flop.value / (ms / cnt * 1e-3) / 1e12, 1)}
    xd = torch.randn(S, M, device=dev).bfloat16()
    w1 = (torch.randn(E, F, M, device=dev) * 0.02).bfloat16()
    b1 = (torch.randn(E, F, device=dev) * 0.02).bfloat16()
    w2 = (torch.randn(E, F, M, device=dev) * 0.02).bfloat16()
    b2 = (torch.randn(E, M, device=dev) * 0.02).bfloat16()
    rows = S // E
    kept = torch.full((E,), rows, dtype=torch.int32, device=dev)
    off = torch.arange(E + 1, dtype=torch.int32, device=dev) * rows
    gflop = 2.0 * S * M * F
    # The K loop of the first product without its epilogue, whole and with one ingredient taken out, on random and on
    # zero operands.  The variants without the operand loads multiply whatever the launch before them left in LDS,
    # which is why each follows a whole loop on the same data.  Same instruction stream and (with loads) the same
    # memory traffic on both kinds of data: what zero operands gain is what the power limit takes on real data.
    parts = ((0, "whole"), (1, "without_operand_loads"), (2, "without_fragment_reads"), (3, "without_barriers"),
             (4, "without_loads_reads_and_barriers"))
    for kind, (xa, wa) in (("random", (xd, w1)), ("zeros", (torch.zeros_like(xd), torch.zeros_like(w1)))):
        for part, what in parts:
            try:
                t = timed(lambda: L.check(L.lib().mole_probe_kloop_part(L.ptr(xa), L.ptr(wa), L.ptr(off), L.ptr(kept), E, S, F, M,
                                                                        part, L.ptr(sink), L.stream()), "mole_probe_kloop_part"), 20)
            except RuntimeError:      # only the default tile shape has the variants (MOLE_TMB selects others)
                L.kernel_timing_enable(False)
                continue
            cnt, ms = t["probe"]
            res[f"k_loop_{what}_{kind}_operands"] = {"avg_us": round(ms / cnt * 1e3, 1),
                                                     "tflops": round(gflop / (ms / cnt * 1e-3) / 1e12, 1)}
    del xa, wa
    t = timed(lambda: H.ffn_fwd(xd, off, kept, w1, b1, w2, b2), 20)
    for kname in ("ffn_fwd1", "ffn_fwd2"):
        cnt, ms = t[kname]
        res[kname] = {"avg_us": round(ms / cnt * 1e3, 1), "tflops": round(gflop / (ms / cnt * 1e-3) / 1e12, 1)}
    # yardstick: the vendor library's GEMM of the same shape (not used by the product)
    wt = w1[0].t().contiguous()
    for _ in range(5):
        torch.matmul(xd, wt)
    torch.cuda.synchronize()
    a, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(20):
        torch.matmul(xd, wt)
    b_.record()
    torch.cuda.synchronize()
    us = a.elapsed_time(b_) / 20 * 1e3
    res["library_gemm_same_shape"] = {"avg_us": round(us, 1), "tflops": round(gflop / (us * 1e-6) / 1e12, 1)}
    print(json.dumps({"probe": f"grouped product h = xd . w1^T at S={S} M={M} E={E} F={F}, bf16, {E} experts of {rows} rows",
                      "peak_tflops": PEAK_MFMA_TFLOPS["bf16"], "compute_units": n_cu, "results": res}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS) + ["c4"])
    ap.add_argument("--layers", type=int, default=2, help="depth of the c4 stack (12 in the configuration)")
    ap.add_argument("--adam", action="store_true",
                    help="c4 only: update the offloaded experts with the in-pipeline Adam (adds 30 GB of pinned moments per layer)")
    ap.add_argument("--no-resident", action="store_true",
                    help="c4 only: fetch the experts again for every backward pass, as the reference does")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-c1", action="store_true", help="skip the configuration-1 (fp32) figures beside the headline")
    ap.add_argument("--no-c35", action="store_true", help="skip the configuration-3 and -5 figures beside the headline")
    ap.add_argument("--ingest-counters", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="no GPU work: read the counter_collection CSVs of a FETCH_SIZE and a WRITE_SIZE rocprofv3 run of "
                         "--workload W and store the products' HBM bytes per launch in profiles/hbm_traffic.json")
    ap.add_argument("--probe", action="store_true", help="run the matrix-core and K-loop probes instead of the layer")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU MoE-layer hot path: this build has no multi-GPU path, run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    if args.ingest_counters:
        return ingest_counters(args)
    import torch
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    if args.probe:
        return run_probes(args)
    if args.workload == "c4":
        return bench_offloaded_stack(args)
    res = measure_layer(args.workload, args.steps, args.warmup)
    out = {
        "metric": "MoE layer tokens/sec fwd+bwd on 1 MI355X", "value": res.pop("value"), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": res.pop("ms_per_step"),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": res.pop("dtype"), "data": "synthetic",
    }
    out.update(res)
    if args.workload != "c1" and not args.no_c1:
        # configuration 1 (fp32, the case the CPU baseline runs) on the GPU, beside the headline
        c1 = measure_layer("c1", args.steps, args.warmup, with_adam=False)
        out["c1"] = {"tokens_per_s": c1["value"], "ms_per_step": c1["ms_per_step"], "dtype": c1["dtype"],
                     "workload": c1["config"]["workload"], "roofline": c1["roofline"], "hbm_permutes": c1["hbm_permutes"],
                     "kernels_us": {n: v["avg_us"] for n, v in c1["kernels"].items()}}
    if args.workload == "c2" and not args.no_c35:
        # configurations 3 (Zipf loads, 64 experts) and 5 (256 experts, top-8) beside the headline, a few steps each
        for name in ("c3", "c5"):
            r = measure_layer(name, min(args.steps, 10), min(args.warmup, 3), with_adam=False)
            out[name] = {"tokens_per_s": r["value"], "ms_per_step": r["ms_per_step"], "dtype": r["dtype"],
                         "workload": r["config"]["workload"], "roofline": r["roofline"], "hbm_permutes": r["hbm_permutes"],
                         "kernels_us": {n: v["avg_us"] for n, v in r["kernels"].items()}}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
