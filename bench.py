#!/usr/bin/env python3
"""Benchmark of the cascaded low-precision matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload ffn|attn|kv|unet]

One "step" is one pass of the hot path over one batch of synthetic input:

* ``--workload ffn`` (default; the shape the headline metric is quoted on): the GEGLU feed-forward
  block of the SDXL 32x32 stage, full image: X fp32 [M = 2 x 1024 tokens, K = 1280] x W1 fp32
  [1280, 10240], then G fp32 [2048, 5120] x W2 fp32 [5120, 1280] -- two GEMMs per step;
* ``--workload attn``: the self-attention projections of the 64x64 stage on one GPU's patch share:
  X fp32 [M = 2 x 2048 tokens, K = 640] through four Linear weights W fp32 [640, 640] (to_q, to_k,
  to_v from X in one grouped launch, to_out from a second activation tensor).

* ``--workload kv``: the cross-attention key / value projections of the 77 text tokens, X fp32 [154, 2048] x W fp32
  [2048, 1280] and [2048, 640]: the skinny split-K path, reported in HBM GB/s over the algorithmic bytes;
* ``--workload unet``: every Linear layer and 1x1 convolution of one SDXL UNet denoising step (batch 2, 128x128
  latent, random weights), as the patched module tree of basedxl_amd.unet_skeleton calls them, full latent and
  one GPU's half-latent share, 2-term bf16 and 3-term fp8 cascades.

The default (ffn) line also carries the kv and unet figures under ``other_workloads``.
Every GEMM of ffn / attn / kv is a 2-term bf16 cascade with the three products hi.hi + hi.lo + lo.hi and fp32
accumulation.  Inputs are synthetic (seeded normal; weights x 0.02) and resident in HBM before the
timed region.  Both operands are split inside the timed kernels.

Prints ONE JSON line: the whole-job fp32-equivalent throughput (2*M*N*K per GEMM, whatever the term
count), the roofline of the GEMM kernel that takes most of the step, measured live with events on
the stream the kernels run on, and the CPU oracle timed on this host's cores on a bounded sample.
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

TERMS, PRODUCTS_PER_ELEMENT = 2, 3  # bf16 hi/lo, tri product set
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
SEED = 1
METRIC = {"ffn": "fp32-equiv TFLOP/s + % of MFMA roofline at SDXL FFN shape; rel-Frobenius err",
          "attn": "fp32-equiv TFLOP/s + % of MFMA roofline at SDXL self-attention projection shape; rel-Frobenius err"}
TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "counter_traffic.txt")


def counter_traffic():
    """HBM-side traffic per launch as rocprofv3 counter runs measured it: the rows of
    profiles/counter_traffic.txt, keyed by (workload, launch label).  Every row names the kernel variant
    it was measured on, the commit of that build and the summary under profiles/ it comes from; the bench
    reports a figure only for the kernel it actually ran (another kernel: null)."""
    rows = {}
    try:
        with open(TRAFFIC_TABLE) as f:
            for line in f:
                if line.startswith("#") or "|" not in line:
                    continue
                c = [x.strip() for x in line.split("|")]
                if len(c) != 9:
                    continue
                wl, launch, kernel, fetch_kib, f_fac, write_kib, w_fac, commit, profile = c
                rows[(wl, launch)] = {"kernel": kernel, "commit": commit, "profile": profile,
                                      "bytes": (float(fetch_kib) * float(f_fac) + float(write_kib) * float(w_fac)) * 1024.0}
    except OSError:
        pass
    return rows


def traffic_for(workload_name, launch, kernel):
    """(bytes or None, where it comes from) for one launch of `kernel`"""
    row = counter_traffic().get((workload_name, launch))
    if row is None:
        return None, "no counter run recorded for this launch in profiles/counter_traffic.txt"
    if row["kernel"] != kernel:
        return None, f"the recorded counter run ({row['profile']}) is of kernel {row['kernel']}, not of the one that ran"
    return row["bytes"], (f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch, scaled by what the same counters read for a device "
                          f"copy of known size; build {row['commit']}; {row['profile']}")


class Launch:
    """One kernel launch of a step: `gemms` problems of one shape (a_list[i] x w_list[i] -> outs[i])."""

    def __init__(self, label, M, K, N, a_idx, w_idx):
        self.label, self.M, self.K, self.N = label, M, K, N
        self.a_idx, self.w_idx = a_idx, w_idx     # indices into a buffer set's activations / weights
        self.gemms = len(w_idx)

    @property
    def flops(self):            # fp32-equivalent
        return 2.0 * self.M * self.N * self.K * self.gemms

    @property
    def algorithmic_bytes(self):   # every distinct operand once, every result once
        return 4 * (len(set(self.a_idx)) * self.M * self.K + self.gemms * (self.K * self.N + self.M * self.N))


def workload(name, group):
    """(description, activation shapes, weight shapes, launches) of one step."""
    if name == "ffn":
        acts = [(2048, 1280), (2048, 5120)]
        wts = [(1280, 10240), (5120, 1280)]
        launches = [Launch("ff.net.0.proj (W1)", 2048, 1280, 10240, [0], [0]), Launch("ff.net.2 (W2)", 2048, 5120, 1280, [1], [1])]
        desc = ("cfg3: SDXL 32x32-stage GEGLU FFN, full image: X fp32 [2048,1280] ~N(0,1) x W1 fp32 [1280,10240] ~N(0,0.02), "
                "then G fp32 [2048,5120] ~N(0,1) x W2 fp32 [5120,1280] ~N(0,0.02) (a synthetic second input, not the gated "
                "output of the first GEMM); hi=bf16(x), lo=bf16(x-hi), products hi.hi+hi.lo+lo.hi, fp32 accumulate, fp32 out")
        return desc, acts, wts, launches
    acts = [(4096, 640), (4096, 640)]
    wts = [(640, 640)] * 4
    if group == "qkv+o":
        launches = [Launch("to_q/to_k/to_v grouped", 4096, 640, 640, [0, 0, 0], [0, 1, 2]), Launch("to_out", 4096, 640, 640, [1], [3])]
    elif group == "all":
        launches = [Launch("q/k/v/out grouped", 4096, 640, 640, [0, 0, 0, 1], [0, 1, 2, 3])]
    else:
        launches = [Launch(n, 4096, 640, 640, [a], [w]) for n, a, w in (("to_q", 0, 0), ("to_k", 0, 1), ("to_v", 0, 2), ("to_out", 1, 3))]
    desc = ("cfg2: SDXL 64x64-stage self-attention projections on one GPU's patch share: X fp32 [4096,640] ~N(0,1) x W fp32 "
            "[640,640] ~N(0,0.02), q/k/v/out = 4 GEMMs per step; hi=bf16(x), lo=bf16(x-hi), products hi.hi+hi.lo+lo.hi, "
            "fp32 accumulate, fp32 out")
    return desc, acts, wts, launches


def make_inputs(acts, wts, device):
    import torch

    g = torch.Generator().manual_seed(SEED)
    a_cpu = [torch.randn(m, k, generator=g, dtype=torch.float32) for m, k in acts]
    w_cpu = [torch.randn(k, n, generator=g, dtype=torch.float32) * 0.02 for k, n in wts]
    return (a_cpu, w_cpu), ([a.to(device) for a in a_cpu], [w.to(device) for w in w_cpu])


def cpu_baseline(cpu_inputs, launches, repeats=5):
    """The oracle's CPU emulation of the same step, timed on this host (rank 0, N = 1)."""
    import torch
    from oracle import cascade as oc

    a_cpu, w_cpu = cpu_inputs
    torch.set_num_threads(min(os.cpu_count() or 1, 16))

    def step():
        return [oc.cascade_matmul_ref(a_cpu[a], w_cpu[w], "bf16", 2, "tri") for ln in launches for a, w in zip(ln.a_idx, ln.w_idx)]

    step()
    times = []
    for _ in range(repeats):
        t0 = time.perf_counter()
        step()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(sum(ln.flops for ln in launches) / med * 1e-12, 4),
        "unit": "TFLOP/s fp32-equiv",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{repeats} timed repeats (median) of the full step ({sum(ln.gemms for ln in launches)} GEMMs), torch CPU "
                  f"emulation: split + 3 fp32 matmuls per GEMM; {med * 1e3:.1f} ms per step; threads = min(os.cpu_count(), 16): "
                  f"16 is this job's share of the host's cores",
    }



def _graph_time_us(fn, reps, replays=5, spin_s=0.2):
    """Average duration of one call of ``fn`` in microseconds: ``reps`` calls captured in one HIP graph,
    replayed untimed until the clocks are up, then ``replays`` timed replays between two events."""
    import torch

    fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(reps):
            fn()
    t_end = time.perf_counter() + spin_s
    while time.perf_counter() < t_end:
        g.replay()
        torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (replays * reps)


def measured_peaks(dev):
    """What this GPU sustains where the published peaks assume the boost clock: a register-only loop of
    bf16 MFMAs on every SIMD, one streaming read and one copy of 1 GiB (the library's probe kernels,
    events around five launches each after the clocks are up)."""
    import torch
    from basedxl_amd import _lib

    l = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream

    def timed(launch, n=5, spin_s=0.2):
        t_end = time.perf_counter() + spin_s
        while time.perf_counter() < t_end:
            launch()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(n):
            launch()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / n          # seconds per launch

    wgs, iters = 2 * 256, 8000                          # two workgroups of four waves per CU
    out = torch.empty(wgs * 256, device=dev)
    t = timed(lambda: _lib.check(l.cascmm_probe_mfma(wgs, iters, out.data_ptr(), out.numel() * 4, stream), "cascmm_probe_mfma"))
    mfma = wgs * 4 * iters * 4 * 2.0 * 32 * 32 * 16 / t * 1e-12
    n = 1 << 30
    src = torch.empty(n // 4, device=dev).normal_()
    dst = torch.empty_like(src)
    g = 8 * 256
    sums = torch.empty(g * 256, device=dev)
    t_r = timed(lambda: _lib.check(l.cascmm_probe_stream(src.data_ptr(), None, n, g, sums.data_ptr(), sums.numel() * 4, stream),
                                   "cascmm_probe_stream"))
    t_c = timed(lambda: _lib.check(l.cascmm_probe_stream(src.data_ptr(), dst.data_ptr(), n, g, None, 0, stream), "cascmm_probe_stream"))
    del src, dst
    return {"mfma_bf16_tflops": round(mfma, 1), "hbm_read_gbs": round(n / t_r * 1e-9, 1), "hbm_copy_gbs": round(2 * n / t_c * 1e-9, 1),
            "how": "register-only loop of v_mfma_f32_32x32x16_bf16, 8 waves per CU; 1 GiB streamed once (read) / copied (read + write bytes); "
                   "events around 5 launches after 0.2 s of the same launches"}


def bench_kv(dev, check=True):
    """cfg4: the two cross-attention K/V projections of the text tokens; bandwidth-style figures
    over the algorithmic bytes 4 (MK + KN + MN)."""
    import torch
    from basedxl_amd import cascaded_lowp_matmul, _lib
    from oracle import cascade as oc

    out = {"workload": "cfg4: cross-attention K/V projections of 2 x 77 text tokens, X fp32 [154,2048] ~N(0,1) x W fp32 "
                       "[2048,N] ~N(0,0.02), N = 1280 and 640; 2-term bf16 cascade (3 products), one call each",
           "gemms": []}
    g = torch.Generator().manual_seed(SEED + 4)
    x_cpu = torch.randn(154, 2048, generator=g)
    x = x_cpu.to(dev)
    total_bytes = total_us = 0.0
    l = _lib.lib()
    for n in (1280, 640):
        w_cpu = torch.randn(2048, n, generator=g) * 0.02
        w = w_cpu.to(dev)
        res = torch.empty(154, n, device=dev)
        us = _graph_time_us(lambda: cascaded_lowp_matmul(x, w, out=res), reps=20)
        algo = 4 * (154 * 2048 + 2048 * n + 154 * n)
        rec = {"M": 154, "K": 2048, "N": n, "launch_us": round(us, 2), "algorithmic_bytes": algo,
               "hbm_gbs": round(algo / us * 1e-3, 1), "frac_of_8TBs": round(algo / us * 1e-3 / 8000.0, 4),
               "fp32_equiv_tflops": round(2.0 * 154 * 2048 * n / us * 1e-6, 1),
               "kernel": l.cascmm_variant_name(l.cascmm_select_variant(154, n, 2048, 2048, n, n, 0, 0, 2, 0)).decode()}
        if check:
            exp = oc.fp64_matmul(x_cpu, w_cpu)
            ek, eo = oc.error_metrics(res.cpu(), exp), oc.error_metrics(oc.cascade_matmul_ref(x_cpu, w_cpu), exp)
            if not (ek["rel_fro"] <= 1.25 * eo["rel_fro"] and ek["max_abs"] <= 1.25 * eo["max_abs"]):
                sys.exit(f"bench.py: kv kernel error {ek} exceeds 1.25x the oracle cascade's {eo}")
            rec["kernel_rel_fro"], rec["oracle_rel_fro"] = ek["rel_fro"], eo["rel_fro"]
        out["gemms"].append(rec)
        total_bytes += algo
        total_us += us
    out["hbm_gbs"] = round(total_bytes / total_us * 1e-3, 1)
    out["us_both"] = round(total_us, 2)
    return out


def bench_unet(dev, cascades=(("bf16", 2, None, False), ("fp8", 3, None, False), ("bf16", 2, True, False), ("fp8", 3, True, False),
                              ("bf16", 2, False, True), ("bf16", 2, True, True), ("bf16", 2, True, "chain"),
                              ("bf16", 2, True, True, True)),
               latents=(("full latent", None), ("half-latent share", 64)), forward=True):
    """cfg5: the routed layers of one UNet step.  The module tree is built on the GPU with random
    weights and patched through the config switch; one forward pass records every routed call; those
    calls are then replayed in call order on resident inputs from ONE HIP graph, so the figure is the
    Linear / 1x1-convolution path alone (the convolutions, normalisations and attention of the
    surrounding model are not part of it; the time of a whole eager forward pass is given beside it).
    A fifth element of a cascade tuple asks for a LATER step of a sample: the reference projects the text tokens
    to cross-attention keys and values on a sample's first denoising step only and keeps them for the other 49
    (basedxl/modules/attn.py:57,74-78); with it the modules keep theirs, the first pass fills them and the
    recorded step no longer has those calls (neither their time nor their flops)."""
    import torch
    from basedxl_amd.unet import BasedXLUnet
    from basedxl_amd.unet_skeleton import SDXLUNetSkeleton, distinct_shapes, routed_calls, synthetic_inputs
    from basedxl_amd.utils import BasedXLConfig

    rows = []
    for lowp, terms, prepared, geglu, *later in cascades:
        kv_kept = bool(later and later[0])
        model = SDXLUNetSkeleton(device=dev, seed=SEED)
        chain = geglu == "chain"     # the two GEMMs of every feed-forward block chained (gate in the first one's store, result as slots)
        unet = BasedXLUnet(model, BasedXLConfig(fp16_acc_matmul=True, lowp=lowp, terms=terms, prepared=prepared,
                                                fuse_geglu=bool(geglu) and not chain, chain_ffn=chain, cache_cross_kv=kv_kept))
        for label, latent_rows in latents:
            inp = synthetic_inputs(model, latent=128, latent_rows=latent_rows, seed=SEED, device=dev)
            if kv_kept:
                for m in unet.modules():
                    if hasattr(m, "kv_cache"):
                        m.reset()
                with torch.no_grad():
                    unet(*inp)                      # a sample's first step: fills every cross-attention layer's K/V
            calls = routed_calls(unet, *inp)
            shapes = distinct_shapes(calls)
            gen = torch.Generator(device=dev).manual_seed(SEED)
            xs = {k: torch.randn(c["input_shape"], device=dev, generator=gen) for k, c in shapes.items()}
            plan = [(c["module"], xs[(type(c["module"]).__name__, c["M"], c["K"], c["N"])]) for c in calls]

            def path():
                for mod, x in plan:
                    mod(x)

            with torch.no_grad():
                us = _graph_time_us(path, reps=1, replays=3, spin_s=0.3)
                fwd_ms = None
                if forward and not prepared:
                    unet(*inp)
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(2):
                        unet(*inp)
                    torch.cuda.synchronize()
                    fwd_ms = (time.perf_counter() - t0) * 1e3 / 2
            flops = sum(2.0 * c["M"] * c["K"] * c["N"] + c.get("extra_flops", 0.0) for c in calls)
            rows.append({"cascade": f"{lowp}x{terms} tri", "weights": "kept split (prepared once)" if prepared else "split in every call",
                         "geglu": "feed-forward blocks chained: value * gelu(gate) in the store of the projection's GEMM, written as the operand "
                                  "slots of the block's second GEMM (this figure includes the gate)" if chain
                         else "value * gelu(gate) in the store of the projection's GEMM (this figure includes the gate)" if geglu
                         else "projection routed as a Linear; the gate stays with torch (two elementwise kernels, in no figure but "
                              "whole_forward_ms_eager)",
                         "step_of_a_sample": "a later one: text-token keys / values kept from the first step" if kv_kept
                         else "the first: text tokens projected to keys / values (49 of the reference's 50 steps skip this)",
                         "latent": label, "routed_calls": len(calls), "distinct_shapes": len(shapes),
                         "gflop_fp32_equiv": round(flops * 1e-9, 1), "linear_path_ms_per_step": round(us * 1e-3, 3),
                         "fp32_equiv_tflops": round(flops / us * 1e-6, 1),
                         "whole_forward_ms_eager": None if fwd_ms is None else round(fwd_ms, 1)})
            del plan, xs
        del unet, model
        torch.cuda.empty_cache()
    return {"workload": "cfg5: every nn.Linear and 1x1 convolution of one SDXL UNet denoising step (latent 2x4x128x128, text "
                        "context 2x77x2048, weights ~N(0,0.02)) through the patched module tree (to_q/to_k/to_v of self-attention as one "
                        "GEMM, to_k/to_v of cross-attention as one, bias in the "
                        "store, fp8 activation scale found in every call, weight scales kept); one HIP graph of all routed calls; "
                        "activations are split in every call, weights either in every call too or once (a labelled mode)",
            "configs": rows}


def bench_attn(dev, check=True):
    """cfg2: the four self-attention projections of the 64x64 stage on one GPU's patch share, as the step of
    `--workload attn` runs them (to_q / to_k / to_v of the same tokens in one grouped launch, to_out on a
    second activation tensor), each launch timed on its own and the two together."""
    import torch
    from basedxl_amd import cascaded_lowp_matmul, cascaded_lowp_matmul_grouped, _lib
    from oracle import cascade as oc

    l = _lib.lib()
    g = torch.Generator().manual_seed(SEED + 2)
    x_cpu, x2_cpu = torch.randn(4096, 640, generator=g), torch.randn(4096, 640, generator=g)
    w_cpu = [torch.randn(640, 640, generator=g) * 0.02 for _ in range(4)]
    x, x2, w = x_cpu.to(dev), x2_cpu.to(dev), [t.to(dev) for t in w_cpu]
    outs = [torch.empty(4096, 640, device=dev) for _ in range(4)]
    qkv = lambda: cascaded_lowp_matmul_grouped([x, x, x], w[:3], outs=outs[:3])      # noqa: E731
    o = lambda: cascaded_lowp_matmul(x2, w[3], out=outs[3])                          # noqa: E731

    def step():
        qkv()
        o()

    us_qkv, us_o, us_step = _graph_time_us(qkv, reps=10), _graph_time_us(o, reps=10), _graph_time_us(step, reps=10)
    flop = 2.0 * 4096 * 640 * 640
    names = _lib.variant_names()
    k_qkv = names[l.cascmm_select_variant_grouped(3, 4096, 640, 640, 640, 640, 640, 0, 0, 2, 0) & 0xFFFF]
    k_o = names[l.cascmm_select_variant(4096, 640, 640, 640, 640, 640, 0, 0, 2, 0) & 0xFFFF]
    rec = {"workload": "cfg2: SDXL 64x64-stage self-attention projections on one GPU's patch share: X fp32 [4096,640] ~N(0,1) x W fp32 "
                       "[640,640] ~N(0,0.02), to_q/to_k/to_v as one grouped launch + to_out; 2-term bf16 cascade (3 products), both "
                       "operands split inside the kernels",
           "us_per_step": round(us_step, 2), "fp32_equiv_tflops": round(4 * flop / us_step * 1e-6, 1),
           "launches": [
               {"launch": "to_q/to_k/to_v grouped", "kernel": k_qkv, "launch_us": round(us_qkv, 2),
                "mfma_tflops": round(9 * flop / us_qkv * 1e-6, 1), "frac_of_mfma_peak": round(9 * flop / us_qkv * 1e-6 / PEAK_BF16_TFLOPS, 4),
                "traffic": traffic_for("attn", "to_q/to_k/to_v grouped", k_qkv)[0]},
               {"launch": "to_out", "kernel": k_o, "launch_us": round(us_o, 2), "mfma_tflops": round(3 * flop / us_o * 1e-6, 1),
                "frac_of_mfma_peak": round(3 * flop / us_o * 1e-6 / PEAK_BF16_TFLOPS, 4),
                "traffic": traffic_for("attn", "to_out", k_o)[0]}]}
    if check:
        exp = oc.fp64_matmul(x2_cpu, w_cpu[3])
        ek, eo = oc.error_metrics(outs[3].cpu(), exp), oc.error_metrics(oc.cascade_matmul_ref(x2_cpu, w_cpu[3]), exp)
        if not (ek["rel_fro"] <= 1.25 * eo["rel_fro"] and ek["max_abs"] <= 1.25 * eo["max_abs"]):
            sys.exit(f"bench.py: attn kernel error {ek} exceeds 1.25x the oracle cascade's {eo}")
        rec["kernel_rel_fro"], rec["oracle_rel_fro"] = ek["rel_fro"], eo["rel_fro"]
    return rec


def bench_ffn_modes(dev, check=True):
    """cfg3 as the model runs it -- the gate between the two GEMMs is real: h = X W1 + b1, G = value x
    gelu(gate), Y = G W2 + b2 -- in the modes the library offers for it.  The headline step multiplies a
    synthetic G and applies no gate; these are labelled modes beside it, with the same 80.5 GFLOP
    (fp32-equivalent) of GEMM work per step:
      * layer by layer: the gated store writes G as fp32, the second GEMM reads and splits it;
      * chained: the gated store writes G as the second GEMM's operand slots, the second GEMM multiplies slots
        by slots (its weight split once: the chained GEMM has no other form); W1 split in every call, or
        kept split as well."""
    import torch
    from basedxl_amd import (ChainedWeight, LeftSlots, PreparedWeight, cascaded_lowp_matmul, cascaded_lowp_matmul_chained,
                             cascaded_lowp_matmul_glu_chained)
    from basedxl_amd.cascaded_lowp_matmul import cascaded_lowp_matmul_glu
    from oracle import cascade as oc

    M, K, inner, N2 = 2048, 1280, 5120, 1280
    g = torch.Generator().manual_seed(SEED + 3)
    x_cpu = torch.randn(M, K, generator=g)
    w1_cpu, b1_cpu = torch.randn(K, 2 * inner, generator=g) * 0.02, torch.randn(2 * inner, generator=g) * 0.1
    w2_cpu, b2_cpu = torch.randn(inner, N2, generator=g) * 0.02, torch.randn(N2, generator=g) * 0.1
    x, w1, b1, w2, b2 = (t.to(dev) for t in (x_cpu, w1_cpu, b1_cpu, w2_cpu, b2_cpu))
    pw1, pw2, cw2 = PreparedWeight(w1, glu=True), PreparedWeight(w2), ChainedWeight(w2)
    gbuf, y = torch.empty(M, inner, device=dev), torch.empty(M, N2, device=dev)
    slots = LeftSlots.empty((M,), inner, dev)
    modes = [
        ("geglu, layer by layer, weights split in every call",
         lambda: cascaded_lowp_matmul_glu(x, w1, bias=b1, out=gbuf), lambda: cascaded_lowp_matmul(gbuf, w2, bias=b2, out=y)),
        ("geglu, layer by layer, weights kept split",
         lambda: cascaded_lowp_matmul(x, pw1, bias=b1, out=gbuf), lambda: cascaded_lowp_matmul(gbuf, pw2, bias=b2, out=y)),
        ("geglu, chained (slots), W1 split in every call, W2 kept split",
         lambda: cascaded_lowp_matmul_glu_chained(x, w1, bias=b1, out=slots), lambda: cascaded_lowp_matmul_chained(slots, cw2, bias=b2, out=y)),
        ("geglu, chained (slots), weights kept split",
         lambda: cascaded_lowp_matmul_glu_chained(x, pw1, bias=b1, out=slots), lambda: cascaded_lowp_matmul_chained(slots, cw2, bias=b2, out=y)),
    ]
    flops = 2.0 * M * K * 2 * inner + 2.0 * M * inner * N2
    exp = ref_err = None
    if check:
        h = x_cpu.double() @ w1_cpu.double() + b1_cpu.double()
        gate = h[:, inner:]
        exp = (h[:, :inner] * (0.5 * gate * (1.0 + torch.erf(gate / 2.0 ** 0.5)))) @ w2_cpu.double() + b2_cpu.double()
        ref_err = oc.error_metrics(oc.cascade_matmul_ref(oc.gated_projection_ref(x_cpu, w1_cpu, b1_cpu), w2_cpu) + b2_cpu, exp)
    rows = []
    for label, first, second in modes:
        def step():
            first()
            second()
        step()
        torch.cuda.synchronize()
        row = {"mode": label}
        if check:
            ek = oc.error_metrics(y.cpu(), exp)
            if not (ek["rel_fro"] <= 1.25 * ref_err["rel_fro"] and ek["max_abs"] <= 1.25 * ref_err["max_abs"]):
                sys.exit(f"bench.py: ffn mode '{label}': error {ek} exceeds 1.25x the oracle composition's {ref_err}")
            row.update(kernel_rel_fro=ek["rel_fro"], oracle_rel_fro=ref_err["rel_fro"], kernel_max_abs=ek["max_abs"],
                       oracle_max_abs=ref_err["max_abs"])
        us1, us2, us = _graph_time_us(first, reps=10), _graph_time_us(second, reps=10), _graph_time_us(step, reps=10)
        row.update(us_per_step=round(us, 2), first_gemm_us=round(us1, 2), second_gemm_us=round(us2, 2),
                   fp32_equiv_tflops=round(flops / us * 1e-6, 1),
                   second_gemm_mfma_tflops=round(3 * 2.0 * M * inner * N2 / us2 * 1e-6, 1))
        rows.append(row)
    return {"workload": "cfg3 with the real gate: X fp32 [2048,1280] ~N(0,1) x W1 [1280,10240] ~N(0,0.02) + b1, value x gelu(gate), "
                        "x W2 [5120,1280] ~N(0,0.02) + b2; 2-term bf16 cascades; the gate is applied in the first GEMM's store in every "
                        "mode; checked against the oracle's gated projection followed by its cascade (1.25x on both metrics vs fp64)",
            "gflop_fp32_equiv_per_step": round(flops * 1e-9, 2), "modes": rows}


def bench_sweep(dev, sizes=(256, 512, 1024, 2048, 4096, 8192)):
    """The reference's self-benchmark (basedxl/triton/cascaded_lowp_matmul.py:204-242): square
    problems M = N = K against the vendor GEMM.  Here: the two-term bf16 cascade on fp32 tensors
    (three products, both operands split inside the timed kernel) next to torch.matmul on the same
    fp32 tensors and on their bf16 roundings (one product, no split); HIP-graph replay."""
    import torch
    from basedxl_amd import cascaded_lowp_matmul, _lib

    rows = []
    l = _lib.lib()
    for n in sizes:
        g = torch.Generator(device=dev).manual_seed(SEED + n)
        a = torch.randn(n, n, device=dev, generator=g)
        b = torch.randn(n, n, device=dev, generator=g) * 0.02
        a16, b16 = a.bfloat16(), b.bfloat16()
        o, o16 = torch.empty(n, n, device=dev), torch.empty(n, n, device=dev, dtype=torch.bfloat16)
        reps = 20 if n <= 2048 else 5
        us = _graph_time_us(lambda: cascaded_lowp_matmul(a, b, out=o), reps=reps)
        us32 = _graph_time_us(lambda: torch.matmul(a, b, out=o), reps=reps)
        us16 = _graph_time_us(lambda: torch.matmul(a16, b16, out=o16), reps=reps)
        flop = 2.0 * n ** 3
        ref = a.double() @ b.double()
        err = lambda x: float((x.double() - ref).norm() / ref.norm())   # noqa: E731
        e_c, e_32, e_16 = err(cascaded_lowp_matmul(a, b)), err(torch.matmul(a, b)), err(torch.matmul(a16, b16))
        rows.append({"n": n, "kernel": l.cascmm_variant_name(l.cascmm_select_variant(n, n, n, n, n, n, 0, 0, 2, 0)).decode(),
                     "cascade_bf16x2_us": round(us, 2), "cascade_fp32_equiv_tflops": round(flop / us * 1e-6, 1),
                     "cascade_mfma_tflops": round(3 * flop / us * 1e-6, 1), "cascade_rel_fro": e_c,
                     "torch_fp32_us": round(us32, 2), "torch_fp32_tflops": round(flop / us32 * 1e-6, 1), "torch_fp32_rel_fro": e_32,
                     "torch_bf16_us": round(us16, 2), "torch_bf16_tflops": round(flop / us16 * 1e-6, 1), "torch_bf16_rel_fro": e_16})
        del a, b, a16, b16, o, o16, ref
    return {"workload": "square sweep M = N = K: two-term bf16 cascade of fp32 tensors vs torch.matmul (fp32 tensors; bf16 tensors)",
            "sizes": rows}


def bench_eager_launch(dev):
    """Host cost of the eager path the reference runs (no graph): back-to-back eager calls of one
    cfg2-sized GEMM (16 us of GPU work), wall time per call."""
    import torch
    from basedxl_amd import cascaded_lowp_matmul

    g = torch.Generator(device=dev).manual_seed(SEED)
    x = torch.randn(4096, 640, device=dev, generator=g)
    w = torch.randn(640, 640, device=dev, generator=g) * 0.02
    res = torch.empty(4096, 640, device=dev)
    for _ in range(50):
        cascaded_lowp_matmul(x, w, out=res)
    torch.cuda.synchronize()
    n = 2000
    t0 = time.perf_counter()
    for _ in range(n):
        cascaded_lowp_matmul(x, w, out=res)
    t_issue = time.perf_counter() - t0
    torch.cuda.synchronize()
    t_all = time.perf_counter() - t0
    us_graph = _graph_time_us(lambda: cascaded_lowp_matmul(x, w, out=res), reps=20)
    return {"gemm": "4096x640x640 bf16x2", "eager_us_per_call_wall": round(t_all / n * 1e6, 2),
            "host_issue_us_per_call": round(t_issue / n * 1e6, 2), "graph_replay_us_per_call": round(us_graph, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", choices=["ffn", "attn", "kv", "unet", "sweep", "ffn-modes"], default="ffn",
                    help="ffn: the two GEMMs of the 32x32-stage GEGLU feed-forward block (the shape the metric is quoted on); "
                         "attn: the four 64x64-stage self-attention projections of one GPU's patch share; kv: the skinny "
                         "cross-attention K/V projections (GB/s); unet: the Linear path of one whole UNet step; sweep: square "
                         "problems 256 .. 8192 against torch.matmul")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="ffn only: leave the kv / unet / eager-launch figures out of the line (they add about a minute)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch every GEMM from Python instead of replaying a HIP graph")
    ap.add_argument("--group", choices=["qkv+o", "all", "none"], default="qkv+o",
                    help="attn only: how the four GEMMs of a step are launched: to_q/to_k/to_v (same input) as one grouped "
                         "launch plus to_out on its own (default), all four in one grouped launch, or four separate launches")
    ap.add_argument("--streams", type=int, default=1,
                    help="number of HIP streams the launches of a step are spread over (attn --group none: the four "
                         "GEMMs are independent)")
    ap.add_argument("--rotate", type=int, default=1,
                    help="number of distinct input/weight/output buffer sets the steps cycle through (1 = the same buffers "
                         "every step, resident in the Infinity Cache; 8 = every step reads HBM-cold data)")
    ap.add_argument("--unet-select", default="",
                    help="unet only: run one configuration instead of all ten, as cascade:weights:latent, e.g. "
                         "bf16x2:raw:full, fp8x3:prepared:half, bf16x2:raw+geglu:full, bf16x2:prepared+geglu:full, bf16x2:prepared+geglu+kvkept:full (a later step of a sample: text-token K/V kept from the first) or bf16x2:prepared+chain:full (what a profiler run wants)")
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
    if args.workload in ("kv", "unet", "sweep", "ffn-modes"):
        base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
                "vs_baseline": None, "dtype": "bf16", "data": "synthetic"}
        if args.workload == "kv":
            kv = bench_kv(dev)
            worst = min(kv["gemms"], key=lambda r: r["hbm_gbs"])
            print(json.dumps(dict(base, metric="achieved HBM GB/s over algorithmic bytes at the cross-attention K/V shapes",
                                  value=kv["hbm_gbs"], unit="GB/s", ms_per_step=round(kv["us_both"] * 1e-3, 5),
                                  config={"workload": kv["workload"], "launch": "hip graph replay (20 launches per graph)"},
                                  roofline={"bound": "hbm", "kernel": worst["kernel"], "achieved": worst["hbm_gbs"], "peak": 8000.0,
                                            "unit": "GB/s", "frac": worst["frac_of_8TBs"],
                                            "traffic": traffic_for("kv", f"N={worst['N']}", worst["kernel"])[0],
                                            "traffic_is": traffic_for("kv", f"N={worst['N']}", worst["kernel"])[1],
                                            "launch_us": worst["launch_us"], "algorithmic_bytes_per_launch": worst["algorithmic_bytes"]},
                                  gemms=kv["gemms"])))
        elif args.workload == "ffn-modes":
            fm = bench_ffn_modes(dev)
            head = fm["modes"][-1]
            print(json.dumps(dict(base, metric="fp32-equiv TFLOP/s of the SDXL FFN block with its gate, chained GEMMs",
                                  value=head["fp32_equiv_tflops"], unit="TFLOP/s", ms_per_step=round(head["us_per_step"] * 1e-3, 5),
                                  config={"workload": fm["workload"], "launch": "hip graph replay (10 steps per graph); mode: " + head["mode"]},
                                  modes=fm["modes"])))
        elif args.workload == "sweep":
            sw = bench_sweep(dev)
            head = sw["sizes"][-1]
            print(json.dumps(dict(base, metric="fp32-equiv TFLOP/s of the two-term bf16 cascade on square problems",
                                  value=head["cascade_fp32_equiv_tflops"], unit="TFLOP/s", ms_per_step=round(head["cascade_bf16x2_us"] * 1e-3, 5),
                                  config={"workload": sw["workload"], "headline": f"n = {head['n']}"}, sizes=sw["sizes"])))
        else:
            if args.unet_select:
                casc, wts, lat = args.unet_select.split(":")
                lowp, terms = casc.split("x")
                un = bench_unet(dev, cascades=((lowp, int(terms), True if wts in ("prepared", "prepared+chain", "prepared+geglu", "prepared+geglu+kvkept") else False if wts == "raw+geglu" else None,
                                                "chain" if wts == "prepared+chain" else wts in ("raw+geglu", "prepared+geglu", "prepared+geglu+kvkept"),
                                                wts == "prepared+geglu+kvkept"),),
                                latents=(("full latent", None),) if lat == "full" else (("half-latent share", 64),), forward=False)
            else:
                un = bench_unet(dev)
            head = un["configs"][0]
            print(json.dumps(dict(base, metric="fp32-equiv TFLOP/s of the Linear / 1x1-convolution path of one SDXL UNet step",
                                  value=head["fp32_equiv_tflops"], unit="TFLOP/s", ms_per_step=head["linear_path_ms_per_step"],
                                  config={"workload": un["workload"], "headline": head["cascade"] + ", " + head["latent"]},
                                  configs=un["configs"])))
        return
    desc, acts, wts, launches = workload(args.workload, args.group)
    cpu_in, (a_dev, w_dev) = make_inputs(acts, wts, dev)

    def out_buffers():
        return [[torch.empty(ln.M, ln.N, device=dev, dtype=torch.float32) for _ in range(ln.gemms)] for ln in launches]

    # --rotate R: R - 1 further copies of every buffer; step i uses set i % R
    sets = [(a_dev, w_dev, out_buffers())]
    for _ in range(max(1, args.rotate) - 1):
        sets.append(([a.clone() for a in a_dev], [w.clone() for w in w_dev], out_buffers()))
    set_bytes = sum(t.numel() * 4 for t in a_dev + w_dev) + sum(o.numel() * 4 for lo in sets[0][2] for o in lo)
    step_no = [0]
    extra = [torch.cuda.Stream() for _ in range(max(0, min(args.streams, len(launches)) - 1))]

    def run_launch(i, bufs):
        a, w, o = bufs
        ln = launches[i]
        if ln.gemms == 1:
            cascaded_lowp_matmul(a[ln.a_idx[0]], w[ln.w_idx[0]], out=o[i][0])
        else:
            cascaded_lowp_matmul_grouped([a[j] for j in ln.a_idx], [w[j] for j in ln.w_idx], outs=o[i])

    def step():
        # with --streams > 1 the launches are enqueued on several streams (forked from and joined
        # back into the current one) so that the tail of one kernel overlaps the start of the next
        bufs = sets[step_no[0] % len(sets)]
        step_no[0] += 1
        if not extra:
            for i in range(len(launches)):
                run_launch(i, bufs)
            return
        cur = torch.cuda.current_stream()
        lanes = [cur] + extra
        for s_ in extra:
            s_.wait_stream(cur)
        for i in range(len(launches)):
            with torch.cuda.stream(lanes[i % len(lanes)]):
                run_launch(i, bufs)
        for s_ in extra:
            cur.wait_stream(s_)

    # correctness of what is being timed: error vs fp64 next to the oracle cascade's error, on
    # the last GEMM of the step (the smaller one of the ffn workload: the CPU side takes seconds)
    step()
    torch.cuda.synchronize()
    chk = launches[-1]
    a_chk, w_chk = cpu_in[0][chk.a_idx[-1]], cpu_in[1][chk.w_idx[-1]]
    exp = oc.fp64_matmul(a_chk, w_chk)
    err_k = oc.error_metrics(sets[0][2][-1][-1].cpu(), exp)
    err_o = oc.error_metrics(oc.cascade_matmul_ref(a_chk, w_chk, "bf16", 2, "tri"), exp)
    del exp
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
        for _ in range(5):
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
    flops_step = sum(ln.flops for ln in launches)
    value = flops_step / (wall / args.steps) * 1e-12

    # The kernels of a step, each timed on its own: a graph that holds that launch REPS times
    # back to back is replayed between two events on the launch stream (several launches per
    # graph so that the replay overhead of a graph is not charged to the kernel).  The roofline
    # object describes the one that takes most of the step.
    REPS = 10
    l = _lib.lib()
    per_kernel = []
    seen = {}
    for i, ln in enumerate(launches):
        key = (ln.M, ln.K, ln.N, ln.gemms)
        if key in seen:      # same shape and group size: the same kernel (attn --group none)
            seen[key]["launches_per_step"] += 1
            continue
        g1 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g1):
            for _ in range(REPS):
                run_launch(i, sets[0])
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
        vidx = l.cascmm_select_variant_grouped(ln.gemms, ln.M, ln.N, ln.K, ln.K, ln.N, ln.N, 0, 0, 2, 0)
        rec = {
            "launch": ln.label, "gemms": ln.gemms, "M": ln.M, "K": ln.K, "N": ln.N,
            "kernel": l.cascmm_variant_name(vidx).decode(), "launch_us": round(us, 3), "launches_per_step": 1,
            "flops_per_launch": PRODUCTS_PER_ELEMENT * ln.flops,
            "algorithmic_bytes_per_launch": ln.algorithmic_bytes,
            "mfma_tflops": round(PRODUCTS_PER_ELEMENT * ln.flops / (us * 1e-6) * 1e-12, 2),
            "fp32_equiv_tflops": round(ln.flops / (us * 1e-6) * 1e-12, 2),
        }
        seen[key] = rec
        per_kernel.append(rec)
    dom = max(per_kernel, key=lambda r: r["launch_us"] * r["launches_per_step"])
    cache = (f"same buffers every step ({set_bytes / 1e6:.0f} MB working set, resident in the 256 MB Infinity Cache)"
             if len(sets) == 1 else
             f"{len(sets)} buffer sets in rotation ({set_bytes * len(sets) / 1e6:.0f} MB: inputs and weights come from HBM)")

    result = {
        "metric": METRIC[args.workload],
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
            "workload": desc,
            "gemms": [{"M": ln.M, "K": ln.K, "N": ln.N, "count": ln.gemms} for ln in launches],
            "gemms_per_step": sum(ln.gemms for ln in launches), "terms": TERMS, "products": "tri",
            "launch": (f"hip graph replay ({per_graph} steps per graph)" if graph is not None else "python ctypes")
                      + f", {len(extra) + 1} stream(s), {len(launches)} launches per step: " + " + ".join(ln.label for ln in launches),
            "launches_per_step": len(launches),
            "kernel": dom["kernel"], "seed": SEED,
            "cache_regime": cache,
        },
        "roofline": {
            "bound": "mfma",
            "kernel": dom["kernel"] + " (" + dom["launch"] + ", " + str(dom["gemms"]) + " GEMM(s) per launch)",
            "achieved": dom["mfma_tflops"],
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(dom["mfma_tflops"] / PEAK_BF16_TFLOPS, 4),
            "traffic": traffic_for(args.workload, dom["launch"], dom["kernel"])[0],
            "traffic_is": traffic_for(args.workload, dom["launch"], dom["kernel"])[1],
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
        "error": {"checked_gemm": chk.label, "kernel_rel_fro": err_k["rel_fro"], "oracle_rel_fro": err_o["rel_fro"],
                  "kernel_max_abs": err_k["max_abs"], "oracle_max_abs": err_o["max_abs"]},
    }
    if args.workload == "ffn" and not args.no_graph:
        # cfg3 also names the 3-term fp16 cascade, and the fp8 comparison of cfg5 starts at this shape: the
        # same two GEMMs with six products each, reported beside the headline, not part of `value`.  fp8:
        # both operands raw fp32, the weight's scale kept (found once, as a layer does), the activation's
        # found inside every call; its MFMA rate is priced against the fp8 peak.
        from basedxl_amd import tensor_scale_exp
        others = []
        for lowp, peak in (("fp16", PEAK_BF16_TFLOPS), ("fp8", 5000.0)):
            other = {"cascade": f"{lowp}x3 tri", "mfma_peak_tflops": peak, "gemms": []}
            for i, ln in enumerate(launches):
                a, w, o = sets[0][0][ln.a_idx[0]], sets[0][1][ln.w_idx[0]], sets[0][2][i][0]
                kw = {"b_exp": tensor_scale_exp(w)} if lowp == "fp8" else {}
                us = _graph_time_us(lambda: cascaded_lowp_matmul(a, w, out=o, lowp=lowp, terms=3, **kw), reps=REPS, spin_s=0.05)
                other["gemms"].append({"launch": ln.label, "launch_us": round(us, 2), "fp32_equiv_tflops": round(ln.flops / us * 1e-6, 1),
                                       "mfma_tflops": round(6 * ln.flops / us * 1e-6, 1),
                                       "frac_of_mfma_peak": round(6 * ln.flops / us * 1e-6 / peak, 4)})
            exp = oc.fp64_matmul(a_chk, w_chk)
            e3 = oc.error_metrics(sets[0][2][-1][-1].cpu(), exp)
            e3o = oc.error_metrics(oc.cascade_matmul_ref(a_chk, w_chk, lowp, 3, "tri"), exp)
            del exp
            other["error"] = {"checked_gemm": chk.label, "kernel_rel_fro": e3["rel_fro"], "oracle_rel_fro": e3o["rel_fro"],
                              "kernel_max_abs": e3["max_abs"], "oracle_max_abs": e3o["max_abs"]}
            others.append(other)
        result["other_cascades"] = others
    elif args.workload == "ffn":
        # (--no-graph is how the counter runs of a profiler are made: let them see the other cascades' kernels too)
        from basedxl_amd import tensor_scale_exp
        for lowp in ("fp16", "fp8"):
            for i, ln in enumerate(launches):
                a, w, o = sets[0][0][ln.a_idx[0]], sets[0][1][ln.w_idx[0]], sets[0][2][i][0]
                kw = {"b_exp": tensor_scale_exp(w)} if lowp == "fp8" else {}
                for _ in range(3):
                    cascaded_lowp_matmul(a, w, out=o, lowp=lowp, terms=3, **kw)
        torch.cuda.synchronize()
    if args.workload == "ffn" and not args.no_graph and not args.no_other_workloads:
        del sets, a_dev, w_dev
        torch.cuda.empty_cache()
        result["ffn_modes"] = bench_ffn_modes(dev)
        result["other_workloads"] = {"attn": bench_attn(dev), "kv": bench_kv(dev), "unet": bench_unet(dev),
                                     "eager_launch": bench_eager_launch(dev)}
    if args.workload == "ffn" and not args.no_graph:
        # the published peak beside what the board holds: `peak` and `frac` stay the published ones
        torch.cuda.empty_cache()
        mp = measured_peaks(dev)
        result["roofline"]["measured_peaks"] = mp
        result["roofline"]["frac_of_measured_mfma"] = round(dom["mfma_tflops"] / mp["mfma_bf16_tflops"], 4)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(cpu_in, launches)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
