"""Error study of the cascades against an fp64 product, in the format of the reference's
extras/measure_cascaded_lowp_matmul_error.py (:8-9 EPS and percentiles, :27-31 metrics): L1, MSE,
max error and percentiles of the relative error, per shape and cascade, next to torch's own fp32
matmul.  Runs on the GPU; the fp64 product is torch's.

    python -m basedxl_amd.measure_error [--shapes llm|sdxl|all] [--cascades bf16x1,bf16x2,...] [--csv results.csv]
"""
from __future__ import annotations

import argparse

EPS = 1e-6
QUANTILES = (0.01, 0.2, 0.5, 0.8, 0.99)
LLM_SHAPES = [(4096, 4096, 4096), (4096, 14336, 4096), (14336, 4096, 4096), (4096, 4096, 14336)]   # (M, N, K) of the reference
SDXL_SHAPES = [(4096, 640, 640), (2048, 10240, 1280), (2048, 1280, 5120), (154, 1280, 2048)]
QUANTILE_SAMPLE = 4_000_000   # relative-error percentiles are taken over an evenly strided sample of this many elements


def metrics(out, expected):
    import torch

    diff = (expected - out.double()).abs()
    rel = diff / (expected.abs() + EPS)
    flat = rel.flatten()
    step = max(1, flat.numel() // QUANTILE_SAMPLE)
    q = torch.quantile(flat[::step], torch.tensor(QUANTILES, dtype=torch.float64, device=flat.device))
    return {"L1": diff.mean().item(), "MSE": (diff * diff).mean().item(), "Max": diff.max().item(),
            "rel_fro": (diff.norm() / expected.norm()).item(), "quantiles": [v.item() for v in q]}


def main(argv=None) -> None:
    import torch

    from . import cascaded_lowp_matmul

    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--shapes", choices=["llm", "sdxl", "all"], default="all")
    ap.add_argument("--cascades", default="bf16x1,bf16x2,bf16x3,fp16x2,fp16x3,fp8x3")
    ap.add_argument("--w-std", type=float, default=None, help="std of B (default: 1 for the llm shapes, 0.02 for sdxl)")
    ap.add_argument("--csv", default=None)
    args = ap.parse_args(argv)
    shapes = {"llm": [(s, 1.0) for s in LLM_SHAPES], "sdxl": [(s, 0.02) for s in SDXL_SHAPES]}
    todo = shapes["llm"] + shapes["sdxl"] if args.shapes == "all" else shapes[args.shapes]
    rows = []
    for (M, N, K), std in todo:
        torch.manual_seed(42)
        a = torch.randn(M, K, device="cuda", dtype=torch.float32)
        b = torch.randn(K, N, device="cuda", dtype=torch.float32) * (args.w_std if args.w_std is not None else std)
        expected = a.double() @ b.double()
        outs = [("torch fp32 matmul", a @ b)]
        for casc in args.cascades.split(","):
            lowp, terms = casc.split("x")
            outs.append((casc + " tri", cascaded_lowp_matmul(a, b, lowp=lowp, terms=int(terms))))
        for label, out in outs:
            m = metrics(out, expected)
            print(M, K, N, "-" * 20, label, "-" * 20)
            print(f"\tL1 error: {m['L1']:.3e}")
            print(f"\tMSE error: {m['MSE']:.3e}")
            print(f"\tMax error: {m['Max']:.3e}")
            print(f"\trel. Frobenius: {m['rel_fro']:.3e}")
            print(f"\t          PERCENTILES: {' '.join(f'{q:10}' for q in QUANTILES)}")
            print(f"\t       relative error: {' '.join(f'{q:10.3e}' for q in m['quantiles'])}", flush=True)
            rows.append([M, K, N, label, m["L1"], m["MSE"], m["Max"], m["rel_fro"], m["quantiles"][2]])
        del expected, outs
    print("-" * 100)
    head = ["M", "K", "N", "method", "L1", "MSE", "Max", "rel Fro", "Median rel"]
    print(" | ".join(head))
    for r in rows:
        print(" | ".join(str(v) if not isinstance(v, float) else f"{v:.3e}" for v in r))
    if args.csv:
        with open(args.csv, "w") as f:
            f.write(",".join(head) + "\n")
            for r in rows:
                f.write(",".join(str(v) for v in r) + "\n")


if __name__ == "__main__":
    main()
