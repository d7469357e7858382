#!/usr/bin/env python3
"""Benchmark of the MoE-layer hot path on one MI355X.

A step is one forward + backward of one MoE layer (gate, routing, dispatch, grouped expert FFN,
combine, and all of their gradients) over one batch of synthetic tokens resident in HBM.  The
default workload is BASELINE.json's configuration 2: Switch-style layer, bf16 with fp32 accumulation,
16384 tokens x 1024, 16 experts of 1024 -> 4096 -> 1024, top-1, capacity factor 1.25.

Prints ONE JSON line: the metric (tokens/s), the roofline of the dominant kernel measured with HIP
events on the stream the kernel runs on, and the CPU oracle timed on this box's host cores.
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
# HBM bytes per launch (read + write) of the grouped GEMMs at workload c2, from rocprofv3 FETCH_SIZE and
# WRITE_SIZE runs of this script scaled by the same counters' readings for a copy of known size
# (profiles/bench_c2_hbm_traffic.txt); other workloads have no counter run and report null
MEASURED_TRAFFIC_BYTES = {
    "c2": {"ffn_fwd1": 751.8e6, "ffn_fwd2": 383.9e6, "ffn_gw2": 546.7e6, "ffn_da": 741.5e6, "ffn_gw1": 546.7e6,
           "ffn_gx": 385.0e6},
}


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


def cpu_baseline(w, budget_s=12.0):
    """The CPU oracle's layer (fp32 torch on the host cores), forward + backward, on a bounded
    sample of the workload: the same layer shape at a token count that keeps the run near budget_s."""
    import torch
    from oracle import moe_oracle as O
    cores = min(16, os.cpu_count() or 1)
    torch.set_num_threads(cores)
    S = min(w["S"], 4096)
    g = torch.Generator().manual_seed(0)
    E, M, F = w["E"], w["M"], w["F"]
    x = torch.randn(S, M, generator=g)
    wg = torch.randn(E, M, generator=g) * 0.02
    w1, b1 = torch.randn(E, F, M, generator=g) * 0.02, torch.randn(E, F, generator=g) * 0.02
    w2, b2 = torch.randn(E, F, M, generator=g) * 0.02, torch.randn(E, M, generator=g) * 0.02
    dy = torch.randn(S, M, generator=g) * 1e-3
    run = lambda: O.moe_layer(x, wg, w1, b1, w2, b2, w["k"], w["cf"], dy=dy)
    run()
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 20):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": S / med, "unit": "tokens/s", "cores": cores, "kind": "port",
            "sample": f"{len(times)} steps of the {w['name']} layer shape at {S} tokens, fp32 torch-CPU oracle, median"}


def bench_offloaded_stack(args):
    """BASELINE configuration 4: a stack of MoE layers whose experts all live in pinned host memory and
    stream through the device slot pool (32 experts of 4096 -> 14336 -> 4096, bf16: 235 MB per expert,
    7.5 GB per layer; 4096 tokens x 4096, top-2, no drop).  The step is PCIe bound by construction, so
    the figures of interest are the copy stream's host-to-device rate and how much of the step the
    copies cover.  --layers sets the depth (12 in the configuration; each layer pins 15 GB of host
    memory for weights and gradients, the default of 2 keeps set-up within a minute or two)."""
    import torch
    from mole_amd import _lib as L, core
    from mole_amd.moe.layer import MOLEModule
    S, M, E, k, F = 4096, 4096, 32, 2, 14336
    n_layers, pool, ebatch = args.layers, 64, 8
    MOLEModule.reset_instances()
    dist = {"local_rank": 0, "world_size": 1, "rank": 0}
    layers = []
    for i in range(n_layers):
        print(f"[c4] building layer {i} (pinned host weights)", file=sys.stderr, flush=True)
        try:
            layers.append(MOLEModule(E, 0, M, F, pool, k, ebatch, dist, "gelu", 1, bool(args.adam), True, dtype=torch.bfloat16))
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
    t0 = time.perf_counter()
    for i in range(args.steps):
        print(f"[c4] timed step {i}", file=sys.stderr, flush=True)
        one_step()
    torch.cuda.synchronize(); core.synchronize_tran()
    wall = (time.perf_counter() - t0) / args.steps
    h2d_bytes, h2d_ms = um.copy_stats()
    h2d_bytes /= args.steps; h2d_ms /= args.steps
    d2h_bytes, d2h_ms = um.writeback_stats()
    d2h_bytes /= args.steps; d2h_ms /= args.steps
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
                               + (", in-pipeline AdamW on the GPU (fp32 moments in pinned host memory)" if args.adam else "")},
        "prefetch": {"h2d_bytes_per_step": int(h2d_bytes), "h2d_busy_ms": round(h2d_ms, 2),
                     "h2d_gbs": round(h2d_bytes / (h2d_ms * 1e-3) / 1e9, 2),
                     "h2d_busy_frac_of_step": round(h2d_ms / (wall * 1e3), 4),
                     "expected_h2d_bytes": (2 + (4 if args.adam else 0)) * n_layers * E * expert_bytes,
                     "d2h_gradient_bytes_per_step": int(d2h_bytes), "d2h_busy_ms": round(d2h_ms, 2),
                     "d2h_gbs": round(d2h_bytes / (d2h_ms * 1e-3) / 1e9, 2)},
        "kernel_ms_per_step": round(kernel_ms, 2),
        "roofline": {"bound": "mfma", "kernel": "all six grouped products", "unit": "TFLOP/s", "peak": 2500.0,
                     "achieved": round(12.0 * R * M * F * n_layers / (gemm_ms * 1e-3) / 1e12, 1),
                     "frac": round(12.0 * R * M * F * n_layers / (gemm_ms * 1e-3) / 1e12 / 2500.0, 4), "traffic": None},
    }
    print(json.dumps(out))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS) + ["c4"])
    ap.add_argument("--layers", type=int, default=2, help="depth of the c4 stack (12 in the configuration)")
    ap.add_argument("--adam", action="store_true",
                    help="c4 only: update the offloaded experts with the in-pipeline Adam (adds 30 GB of pinned moments per layer)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures the single-GPU MoE-layer hot path: this build has no multi-GPU path, run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from mole_amd import _lib as L
    assert torch.cuda.is_available(), "bench.py needs an MI355X"
    if args.workload == "c4":
        return bench_offloaded_stack(args)
    w = dict(WORKLOADS[args.workload], name=args.workload)
    m, x, dy = make_layer(w)
    cf = w["cf"]

    for _ in range(args.warmup):
        step(m, x, dy, cf)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(m, x, dy, cf)
    torch.cuda.synchronize()
    dt_s = time.perf_counter() - t0
    ms_per_step = dt_s / args.steps * 1e3
    value = w["S"] / (dt_s / args.steps)

    # per-kernel durations: a second pass of the same steps with an event pair around every kernel,
    # recorded on the stream the kernel is launched on
    L.kernel_timing_enable(True)
    for _ in range(args.steps):
        step(m, x, dy, cf)
    torch.cuda.synchronize()
    timing = L.kernel_timing_read()
    L.kernel_timing_enable(False)

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

    R = int(m.last_route.offsets[-1].item())       # kept (token, choice) rows
    S, M, F, k = w["S"], w["M"], w["F"], w["k"]
    b = 2 if w["dtype"] == "bf16" else 4
    gemm_flop = 2.0 * R * M * F                     # every one of the six grouped products
    work = {  # algorithmic work per launch: flop for the GEMMs, bytes for the permutes
        "ffn_fwd1": gemm_flop, "ffn_fwd2": gemm_flop, "ffn_gw2": gemm_flop, "ffn_da": gemm_flop, "ffn_gw1": gemm_flop,
        "ffn_gx": gemm_flop,
        "dispatch_fwd": 2.0 * R * M * b, "combine_fwd": (R + S) * M * b, "combine_bwd": (S + 3.0 * R) * M * b,
        "dispatch_bwd": (R + S) * M * b,
    }
    kernels = {}
    for name, (cnt, ms) in timing.items():
        if cnt == 0:
            continue
        avg_us = ms / cnt * 1e3
        entry = {"avg_us": round(avg_us, 2), "launches_per_step": cnt / args.steps}
        if name in work:
            if name.startswith("ffn_"):
                entry["tflops"] = round(work[name] / (avg_us * 1e-6) / 1e12, 1)
            else:
                entry["gbs"] = round(work[name] / (avg_us * 1e-6) / 1e9, 1)
        kernels[name] = entry
    gemms = [n for n in kernels if n in ("ffn_fwd1", "ffn_fwd2", "ffn_gw2", "ffn_da", "ffn_gw1", "ffn_gx")]
    dom = max(gemms, key=lambda n: kernels[n]["avg_us"])
    peak = PEAK_MFMA_TFLOPS[w["dtype"]]
    gemm_total_us = sum(kernels[n]["avg_us"] for n in gemms)
    roofline = {"bound": "mfma", "kernel": dom, "achieved": kernels[dom]["tflops"], "peak": peak, "unit": "TFLOP/s",
                "frac": round(kernels[dom]["tflops"] / peak, 4),
                "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload, {}).get(dom),
                "all_ffn_gemms_frac": round(6 * gemm_flop / (gemm_total_us * 1e-6) / 1e12 / peak, 4)}

    out = {
        "metric": "MoE layer tokens/sec fwd+bwd on 1 MI355X", "value": round(value, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic",
        "config": {"workload": f"{args.workload}: single MoE layer fwd+bwd, S={S} M={M} E={w['E']} top-{k} F={F} "
                               f"capacity_factor={cf}, kept rows R={R}"},
        "roofline": roofline,
        "hbm_permutes": {n: {"achieved": kernels[n]["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                             "frac": round(kernels[n]["gbs"] / PEAK_HBM_GBS, 4)}
                         for n in ("dispatch_fwd", "combine_fwd", "combine_bwd", "dispatch_bwd") if n in kernels},
        "hbm_optimizer": {"adam_step": {"achieved": round(adam_gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                        "frac": round(adam_gbs / PEAK_HBM_GBS, 4), "elements": n_adam,
                                        "avg_us": round(adam_ms / adam_cnt * 1e3, 2)}},
        "kernels": kernels,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(w)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
