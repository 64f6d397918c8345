#!/usr/bin/env python3
"""Benchmark of the cascaded low-precision matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One "step" is one pass of the hot path over the SDXL 64x64-stage self-attention
projections on one GPU's patch share: X fp32 [M = 2 x 2048 tokens, K = 640] through four
independent Linear weights W fp32 [640, 640] (to_q, to_k, to_v from X, to_out from a second
activation tensor of the same shape), each as a 2-term bf16 cascade with the three products
hi.hi + hi.lo + lo.hi, fp32 accumulation.  Inputs are synthetic (seeded normal) and resident
in HBM before the timed region.  Both operands are split inside the timed kernels.

Prints ONE JSON line: the whole-job fp32-equivalent throughput (2*M*N*K per GEMM, whatever
the term count), the roofline of the GEMM kernel measured live with events on the stream the
kernels run on, and the CPU oracle timed on this host's cores on a bounded sample.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

M, K, N = 4096, 640, 640
N_PROJ = 4
TERMS, PRODUCTS_PER_ELEMENT = 2, 3  # bf16 hi/lo, tri product set
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
# HBM-side traffic of one launch of the dominant kernel, measured with rocprofv3 counters (the
# summary under profiles/ gives the commands and the calibration); keyed by (--group, GEMMs).
TRAFFIC_BYTES_PER_LAUNCH = {("qkv+o", 3): 2 * 21945.3 * 1024 + 30720.0 * 1024}
SEED = 1


def make_inputs(device):
    import torch

    g = torch.Generator().manual_seed(SEED)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    y = torch.randn(M, K, generator=g, dtype=torch.float32)
    ws = [torch.randn(K, N, generator=g, dtype=torch.float32) * 0.02 for _ in range(N_PROJ)]
    cpu = (x, y, ws)
    dev = (x.to(device), y.to(device), [w.to(device) for w in ws])
    return cpu, dev


def cpu_baseline(cpu_inputs, repeats=5):
    """The oracle's CPU emulation of the same step, timed on this host (rank 0, N = 1)."""
    import torch
    from oracle import cascade as oc

    x, y, ws = cpu_inputs
    torch.set_num_threads(min(os.cpu_count() or 1, 16))

    def step():
        outs = [oc.cascade_matmul_ref(x, ws[i], "bf16", 2, "tri") for i in range(3)]
        outs.append(oc.cascade_matmul_ref(y, ws[3], "bf16", 2, "tri"))
        return outs

    step()
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(N_PROJ * 2.0 * M * N * K / med * 1e-12, 4),
        "unit": "TFLOP/s fp32-equiv",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{repeats} timed repeats (median) of the full 4-projection step, torch CPU emulation: "
                  f"split + 3 fp32 matmuls per projection; {med * 1e3:.1f} ms per step",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch every GEMM from Python instead of replaying a HIP graph")
    ap.add_argument("--group", choices=["qkv+o", "all", "none"], default="qkv+o",
                    help="how the four GEMMs of a step are launched: to_q/to_k/to_v (same input) as one grouped launch "
                         "plus to_out on its own (default), all four in one grouped launch, or four separate launches")
    ap.add_argument("--streams", type=int, default=1,
                    help="number of HIP streams the four independent GEMMs of a step are spread over")
    ap.add_argument("--rotate", type=int, default=1,
                    help="number of distinct input/weight/output buffer sets the steps cycle through (1 = the same "
                         "70 MB every step, resident in the Infinity Cache; 8 = 560 MB, every step reads HBM-cold data)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy three times, as the known-size kernel that scales "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures one GPU only (--gpus 1); the path shards by rows of A with no "
                 "exchange, so N GPUs run N independent copies of this step")

    import torch
    from basedxl_amd import cascaded_lowp_matmul, cascaded_lowp_matmul_grouped, _lib
    from oracle import cascade as oc

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    dev = torch.device("cuda:0")
    cpu_in, (x, y, ws) = make_inputs(dev)
    outs = [torch.empty(M, N, device=dev, dtype=torch.float32) for _ in range(N_PROJ)]

    ins = [x, x, x, y]
    # --rotate R: R - 1 further copies of every buffer; step i uses set i % R
    sets = [(ins, ws, outs)]
    for _ in range(max(1, args.rotate) - 1):
        x2, y2 = x.clone(), y.clone()
        sets.append(([x2, x2, x2, y2], [w.clone() for w in ws], [torch.empty_like(o) for o in outs]))
    step_no = [0]
    extra = [torch.cuda.Stream() for _ in range(max(0, min(args.streams, N_PROJ) - 1))]

    def step():
        # the four projections are independent GEMMs; with --streams > 1 they are enqueued on
        # several streams (forked from and joined back into the current one) so that the tail
        # of one kernel overlaps the start of the next
        ins, ws, outs = sets[step_no[0] % len(sets)]
        step_no[0] += 1
        if args.group == "qkv+o":
            cascaded_lowp_matmul_grouped(ins[:3], ws[:3], outs=outs[:3])
            cascaded_lowp_matmul(ins[3], ws[3], out=outs[3])
            return
        if args.group == "all":
            cascaded_lowp_matmul_grouped(ins, ws, outs=outs)
            return
        cur = torch.cuda.current_stream()
        lanes = [cur] + extra
        for s_ in extra:
            s_.wait_stream(cur)
        for i in range(N_PROJ):
            with torch.cuda.stream(lanes[i % len(lanes)]):
                cascaded_lowp_matmul(ins[i], ws[i], out=outs[i])
        for s_ in extra:
            cur.wait_stream(s_)

    # correctness of what is being timed: error vs fp64 next to the oracle cascade's error
    step()
    torch.cuda.synchronize()
    exp = oc.fp64_matmul(cpu_in[1], cpu_in[2][3])
    err_k = oc.error_metrics(outs[3].cpu(), exp)
    err_o = oc.error_metrics(oc.cascade_matmul_ref(cpu_in[1], cpu_in[2][3], "bf16", 2, "tri"), exp)
    if not (err_k["rel_fro"] <= 1.25 * err_o["rel_fro"] and err_k["max_abs"] <= 1.25 * err_o["max_abs"]):
        sys.exit(f"bench.py: kernel error {err_k} exceeds 1.25x the oracle cascade's {err_o}")

    if args.copy_calibration:
        src = torch.empty(64 * 1024 * 1024, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    graph = None
    if not args.no_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        # one graph holds `per_graph` consecutive steps, as a UNet forward would hold hundreds of
        # layers: the cost of starting a graph is not charged to every step
        per_graph = max(d for d in range(1, 11) if args.steps % d == 0)
        if len(sets) > 1:   # every set appears in the graph
            per_graph = len(sets) if args.steps % len(sets) == 0 else per_graph
        step_no[0] = 0
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(per_graph):
                step()
    else:
        per_graph = 1
    run = graph.replay if graph is not None else step

    # bring the GPU out of its idle clocks first (the input set-up and the CPU-side error check
    # above leave it idle for seconds): untimed replays for about 0.3 s, then the W warm-up steps
    t_spin = time.perf_counter()
    while time.perf_counter() - t_spin < 0.3:
        for _ in range(20):
            run()
        torch.cuda.synchronize()
    for _ in range(max(1, args.warmup // per_graph)):
        run()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps // per_graph):
        run()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = e0.elapsed_time(e1)

    ms_per_step = wall * 1e3 / args.steps
    flops_step = N_PROJ * 2.0 * M * N * K
    value = flops_step / (wall / args.steps) * 1e-12

    # The kernels of a step, each timed on its own: a graph that holds that launch REPS times
    # back to back is replayed between two events on the launch stream (several launches per
    # graph so that the replay overhead of a graph is not charged to the kernel).  The roofline
    # object describes the one that takes most of the step.
    REPS = 10
    l = _lib.lib()
    kinds = {"qkv+o": [("to_q/to_k/to_v grouped", 3, lambda: cascaded_lowp_matmul_grouped(ins[:3], ws[:3], outs=outs[:3])),
                       ("to_out", 1, lambda: cascaded_lowp_matmul(ins[3], ws[3], out=outs[3]))],
             "all": [("q/k/v/out grouped", 4, lambda: cascaded_lowp_matmul_grouped(ins, ws, outs=outs))],
             "none": [("one projection", 1, lambda: cascaded_lowp_matmul(ins[3], ws[3], out=outs[3]))]}[args.group]
    per_kernel = []
    for label, gemms, fn in kinds:
        g1 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g1):
            for _ in range(REPS):
                fn()
        nrep = max(1, args.steps // REPS)
        for _ in range(max(1, args.warmup // REPS)):
            g1.replay()
        torch.cuda.synchronize()
        k0, k1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        k0.record()
        for _ in range(nrep):
            g1.replay()
        k1.record()
        torch.cuda.synchronize()
        us = k0.elapsed_time(k1) * 1e3 / (nrep * REPS)
        vidx = l.cascmm_select_variant_grouped(gemms, M, N, K, K, N, N, 0, 0, 2, 0)
        per_kernel.append({
            "launch": label, "gemms": gemms, "kernel": l.cascmm_variant_name(vidx).decode(), "launch_us": round(us, 3),
            "launches_per_step": (N_PROJ if args.group == "none" else 1),
            "flops_per_launch": PRODUCTS_PER_ELEMENT * 2.0 * M * N * K * gemms,
            "algorithmic_bytes_per_launch": 4 * (M * K + gemms * (K * N + M * N)),
            "mfma_tflops": round(PRODUCTS_PER_ELEMENT * 2.0 * M * N * K * gemms / (us * 1e-6) * 1e-12, 2),
            "fp32_equiv_tflops": round(2.0 * M * N * K * gemms / (us * 1e-6) * 1e-12, 2),
        })
    dom = max(per_kernel, key=lambda r: r["launch_us"] * r["launches_per_step"])
    launches_per_step = {"qkv+o": 2, "all": 1, "none": N_PROJ}[args.group]
    vname = dom["kernel"]

    result = {
        "metric": "fp32-equiv TFLOP/s, 2-term bf16 cascade, SDXL 64x64-stage self-attn projections (one GPU's patch share)",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "cfg2: X fp32 [4096,640] ~N(0,1) x W fp32 [640,640] ~N(0,0.02), q/k/v/out = 4 GEMMs per step, "
                        "hi=bf16(x), lo=bf16(x-hi), products hi.hi+hi.lo+lo.hi, fp32 accumulate, fp32 out",
            "M": M, "N": N, "K": K, "gemms_per_step": N_PROJ, "terms": TERMS, "products": "tri",
            "launch": (f"hip graph replay ({per_graph} steps per graph)" if graph is not None else "python ctypes")
                      + f", {len(extra) + 1} stream(s), "
                      + {"qkv+o": "2 launches per step: to_q/to_k/to_v grouped (3 GEMMs, one activation tensor) + to_out",
                         "all": "1 grouped launch per step (4 GEMMs)", "none": "4 launches per step"}[args.group],
            "launches_per_step": launches_per_step,
            "kernel": vname, "seed": SEED,
            "cache_regime": ("same buffers every step (70 MB working set, resident in the 256 MB Infinity Cache)"
                             if len(sets) == 1 else
                             f"{len(sets)} buffer sets in rotation ({70 * len(sets)} MB: inputs and weights come from HBM)"),
        },
        "roofline": {
            "bound": "mfma",
            "kernel": dom["kernel"] + " (" + dom["launch"] + ", " + str(dom["gemms"]) + " GEMMs per launch)",
            "achieved": dom["mfma_tflops"],
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(dom["mfma_tflops"] / PEAK_BF16_TFLOPS, 4),
            "traffic": TRAFFIC_BYTES_PER_LAUNCH.get((args.group, dom["gemms"])),
            "traffic_is": "HBM-side bytes per launch of this kernel from rocprofv3 --pmc FETCH_SIZE (x2.0) + WRITE_SIZE "
                          "(x1.0), factors from a 256 MiB copy in the same runs; see profiles/",
            "launch_us": dom["launch_us"],
            "launch_us_is": "HIP events on the launch stream around graph replays of this launch alone (10 launches per "
                            "graph) / launches",
            "flops_per_launch": dom["flops_per_launch"],
            "algorithmic_bytes_per_launch": dom["algorithmic_bytes_per_launch"],
            "fp32_equiv_tflops": dom["fp32_equiv_tflops"],
            "frac_of_peak_over_terms": round(dom["fp32_equiv_tflops"] / (PEAK_BF16_TFLOPS / TERMS), 4),
            "step_time_us_from_events": round(ev_ms * 1e3 / args.steps, 3),
            "kernels_of_a_step": per_kernel,
        },
        "error": {"kernel_rel_fro": err_k["rel_fro"], "oracle_rel_fro": err_o["rel_fro"],
                  "kernel_max_abs": err_k["max_abs"], "oracle_max_abs": err_o["max_abs"]},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cpu_in)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
