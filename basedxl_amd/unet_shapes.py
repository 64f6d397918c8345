"""The Linear-layer workload of one SDXL UNet step, as a shape table plus a timing harness.

The reference gets the UNet from diffusers (basedxl/model.py:17-22) and swaps its ``nn.Linear``
children (basedxl/unet.py:81-87); diffusers and the checkpoint are not available offline, so
this module carries the layer table itself (SDXL base architecture: channels 320/640/1280,
transformer depth 2 at 640 channels and 10 at 1280, 5 + 6 Transformer2D blocks, cross-attention
width 2048, 77 text tokens) and runs every distinct GEMM shape with random weights.  1x1
convolutions (resnet shortcuts), which the reference does not route (unet.py:85), are listed as
GEMMs over channels-last pixels and can be included with ``--convs``.

    python -m basedxl_amd.unet_shapes [--half-latent] [--convs] [--cascades bf16x2,fp8x3] [--prepared]
                                      [--geglu off|unfused|fused]
"""
from __future__ import annotations

import argparse
import json
from dataclasses import dataclass
from typing import List


@dataclass(frozen=True)
class LinearShape:
    name: str
    count: int      # occurrences per UNet step
    M: int
    K: int
    N: int
    group: int = 1  # GEMMs that share one activation tensor and can share one launch (to_q/k/v)
    routed_by_reference: bool = True
    gated: bool = False  # the projection of a GEGLU block: value * gelu(gate) follows

    @property
    def flops(self) -> float:
        return 2.0 * self.M * self.K * self.N * self.count * self.group


def sdxl_linear_shapes(batch: int = 2, latent: int = 128, half_latent: bool = False, text_tokens: int = 77,
                       convs: bool = False) -> List[LinearShape]:
    """GEMM shapes of one UNet forward.  ``half_latent``: one GPU's share under 2-way patch
    parallelism (image tokens halved; text tokens and embeddings are not split)."""
    div = 2 if half_latent else 1
    t64 = batch * (latent // 2) ** 2 // div      # tokens at the 640-channel stage
    t32 = batch * (latent // 4) ** 2 // div      # tokens at the 1280-channel stage
    t128 = batch * latent ** 2 // div
    txt = batch * text_tokens
    out: List[LinearShape] = []
    for d, tok, blocks, t2d in ((640, t64, 10, 5), (1280, t32, 60, 6)):
        out += [
            LinearShape(f"attn1.to_q/k/v d={d}", blocks, tok, d, d, group=3),
            LinearShape(f"attn1.to_out d={d}", blocks, tok, d, d),
            LinearShape(f"attn2.to_q d={d}", blocks, tok, d, d),
            # key and value of the text tokens as ONE [2048, 2 d] projection, the way the reference's
            # attention wrapper fuses them (basedxl/modules/attn.py:23-39) and BasedXLFusedKV does here
            LinearShape(f"attn2.to_kv d={d}", blocks, txt, 2048, 2 * d),
            LinearShape(f"attn2.to_out d={d}", blocks, tok, d, d),
            LinearShape(f"ff.geglu_proj d={d}", blocks, tok, d, 8 * d, gated=True),
            LinearShape(f"ff.out d={d}", blocks, tok, 4 * d, d),
            LinearShape(f"transformer.proj_in/out d={d}", 2 * t2d, tok, d, d),
        ]
    out += [
        LinearShape("time_embedding.linear_1", 1, batch, 320, 1280),
        LinearShape("time_embedding.linear_2 + add_embedding.linear_2", 2, batch, 1280, 1280),
        LinearShape("add_embedding.linear_1", 1, batch, 2816, 1280),
        LinearShape("resnet.time_emb_proj -> 320", 5, batch, 1280, 320),
        LinearShape("resnet.time_emb_proj -> 640", 5, batch, 1280, 640),
        LinearShape("resnet.time_emb_proj -> 1280", 7, batch, 1280, 1280),
    ]
    if convs:
        c = dict(routed_by_reference=False)
        out += [
            LinearShape("conv_shortcut 320->640 @64^2", 1, t64, 320, 640, **c),
            LinearShape("conv_shortcut 640->1280 @32^2", 1, t32, 640, 1280, **c),
            LinearShape("conv_shortcut 2560->1280 @32^2", 2, t32, 2560, 1280, **c),
            LinearShape("conv_shortcut 1920->1280 @32^2", 1, t32, 1920, 1280, **c),
            LinearShape("conv_shortcut 1920->640 @64^2", 1, t64, 1920, 640, **c),
            LinearShape("conv_shortcut 1280->640 @64^2", 1, t64, 1280, 640, **c),
            LinearShape("conv_shortcut 960->640 @64^2", 1, t64, 960, 640, **c),
            LinearShape("conv_shortcut 960->320 @128^2", 1, t128, 960, 320, **c),
            LinearShape("conv_shortcut 640->320 @128^2", 2, t128, 640, 320, **c),
        ]
    return out


def total_flops(shapes: List[LinearShape]) -> float:
    return sum(s.flops for s in shapes)


def time_shapes(shapes: List[LinearShape], lowp: str, terms: int, prepared: bool = False, iters: int = 10,
                seed: int = 0, static_scales: bool = False, geglu: str = "off", dtype: str = "fp32",
                torch_matmul: bool = False) -> List[dict]:
    """Times every shape on cuda:0 (HIP-graph replay of `iters` launches, random fp32 operands:
    activations N(0,1), weights 0.02 N(0,1)); returns one record per shape.  ``geglu``: what is
    timed for the gated projections: "off" the GEMM alone, "unfused" the GEMM plus torch's
    ``value * gelu(gate)``, "fused" the kernel that applies the gate in its store.  ``dtype``: element
    type of the tensors ("fp16" is what the reference runs its UNet in); ``torch_matmul``: time
    ``torch.matmul`` (the vendor GEMM library) on the same tensors instead of the cascade kernels."""
    import torch

    from . import PreparedWeight, cascaded_lowp_matmul, cascaded_lowp_matmul_grouped, cascaded_lowp_matmul_prepared

    dev = torch.device("cuda:0")
    tdt = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}[dtype]
    g = torch.Generator(device="cpu").manual_seed(seed)
    rows = []
    for s in shapes:
        a = torch.randn(s.M, s.K, generator=g).to(dev).to(tdt)
        ws = [(torch.randn(s.K, s.N, generator=g) * 0.02).to(dev).to(tdt) for _ in range(s.group)]
        outs = [torch.empty(s.M, s.N, device=dev, dtype=tdt) for _ in range(s.group)]
        use_prepared = prepared and s.K % 64 == 0 and s.N % 4 == 0
        gate = geglu if s.gated else "off"
        if torch_matmul:
            use_prepared = False
            gate = "unfused" if gate == "fused" else gate

            def run():
                for i in range(s.group):
                    torch.matmul(a, ws[i], out=outs[i])
        elif gate == "fused":
            pw = PreparedWeight(ws[0], lowp=lowp, terms=terms, glu=True)
            gated_out = torch.empty(s.M, s.N // 2, device=dev, dtype=tdt)
            use_prepared = True

            def run():
                cascaded_lowp_matmul(a, pw, out=gated_out)
        elif lowp == "fp8" and static_scales:
            # fp8 tensor scales found once (as a calibrated deployment would), not in every call
            from . import tensor_scale_exp
            ea = tensor_scale_exp(a)
            exps = [torch.cat([ea, tensor_scale_exp(w)]) for w in ws]

            def run():
                for i in range(s.group):
                    cascaded_lowp_matmul(a, ws[i], out=outs[i], lowp=lowp, terms=terms, tensor_exps=exps[i])
        elif use_prepared:
            pw = [PreparedWeight(w, lowp=lowp, terms=terms) for w in ws]

            def run():
                cascaded_lowp_matmul_prepared([a] * s.group, pw, outs=outs)
        elif s.group > 1:
            # fp8: a layer keeps the scale of its constant weight (modules/lowp_linear.py); the scale of
            # the activations is found in every call
            from . import tensor_scale_exp
            wexp = [tensor_scale_exp(w) for w in ws] if lowp == "fp8" else None

            def run():
                cascaded_lowp_matmul_grouped([a] * s.group, ws, outs=outs, lowp=lowp, terms=terms, b_exps=wexp)
        else:
            from . import tensor_scale_exp
            wexp = tensor_scale_exp(ws[0]) if lowp == "fp8" else None

            def run():
                cascaded_lowp_matmul(a, ws[0], out=outs[0], lowp=lowp, terms=terms, b_exp=wexp)
        if gate == "unfused":
            gemm, gated_out = run, torch.empty(s.M, s.N // 2, device=dev, dtype=tdt)

            def run():
                gemm()
                torch.mul(outs[0][:, : s.N // 2], torch.nn.functional.gelu(outs[0][:, s.N // 2:]), out=gated_out)
        for _ in range(2):
            run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(iters):
                run()
        # the GPU leaves its idle clocks only after some 0.3 s of work (and drops back between
        # shapes while the host builds the next operands): replay untimed until it has
        import time
        t_end = time.perf_counter() + (0.3 if not rows else 0.05)
        while time.perf_counter() < t_end:
            graph.replay()
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(3):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (3 * iters)
        rows.append({"name": s.name, "count": s.count, "group": s.group, "M": s.M, "K": s.K, "N": s.N,
                     "launch_us": round(us, 2), "prepared": use_prepared, "gate": gate,
                     "tflops_fp32_equiv": round(2.0 * s.M * s.K * s.N * s.group / us * 1e-6, 1),
                     "us_per_step": round(us * s.count, 1)})
        del a, ws, outs
    return rows


def main(argv=None) -> None:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--batch", type=int, default=2)
    ap.add_argument("--latent", type=int, default=128)
    ap.add_argument("--half-latent", action="store_true")
    ap.add_argument("--convs", action="store_true", help="include the 1x1 shortcut convolutions as GEMMs")
    ap.add_argument("--cascades", default="bf16x2,fp8x3")
    ap.add_argument("--prepared", action="store_true", help="split the weights once (PreparedWeight)")
    ap.add_argument("--static-scales", action="store_true", help="fp8: the activation scale too is found once, not in every call (the weight scale always is)")
    ap.add_argument("--geglu", choices=["off", "unfused", "fused"], default="off",
                    help="gated projections: time the GEMM alone, with torch's gate after it, or the fused kernel")
    ap.add_argument("--dtype", choices=["fp32", "fp16", "bf16"], default="fp32",
                    help="element type of activations, weights and results (use --cascades fp16x1 / bf16x1 with 16-bit tensors)")
    ap.add_argument("--torch-matmul", action="store_true", help="time torch.matmul on the same tensors instead")
    ap.add_argument("--json", action="store_true")
    args = ap.parse_args(argv)
    shapes = sdxl_linear_shapes(args.batch, args.latent, args.half_latent, convs=args.convs)
    flops = total_flops(shapes)
    summary = {"batch": args.batch, "latent": args.latent, "half_latent": args.half_latent, "convs": args.convs,
               "prepared": args.prepared, "gflop_fp32_equiv_per_step": round(flops * 1e-9, 1), "cascades": {}}
    for casc in args.cascades.split(","):
        lowp, terms = casc.split("x")
        rows = time_shapes(shapes, lowp, int(terms), prepared=args.prepared, static_scales=args.static_scales,
                           geglu=args.geglu, dtype=args.dtype, torch_matmul=args.torch_matmul)
        total_us = sum(r["us_per_step"] for r in rows)
        summary["cascades"][casc] = {"linear_ms_per_step": round(total_us * 1e-3, 3),
                                     "tflops_fp32_equiv": round(flops / total_us * 1e-6, 1), "shapes": rows}
        if not args.json:
            label = f"torch.matmul {args.dtype}" if args.torch_matmul else f"{casc} on {args.dtype} tensors"
            print(f"== {label}{' (prepared weights)' if args.prepared else ''}: {total_us * 1e-3:.3f} ms of Linear work per "
                  f"UNet step, {flops / total_us * 1e-6:.1f} TFLOP/s fp32-equivalent")
            for r in rows:
                print(f"  {r['name']:50s} x{r['count']:3d}  [{r['M']:6d} x {r['K']:5d}] x [{r['K']:5d} x {r['N']:5d}]"
                      f"{' x' + str(r['group']) if r['group'] > 1 else '   '}  {r['launch_us']:9.2f} us  "
                      f"{r['tflops_fp32_equiv']:7.1f} TFLOP/s")
    if args.json:
        print(json.dumps(summary))


if __name__ == "__main__":
    main()
