"""Writes tests/golden/oracle_fixture.json from the CPU oracle (oracle/cascade.py).

The reference holds no vectors for the operand-split cascade (its kernel is an fp16-accumulate
GEMM), so this fixture does not pin the oracle to the reference; the oracle is pinned by the
closed forms and invariants in tests/test_oracle_*.py.  The fixture freezes what the pinned
oracle produces on small seeded inputs, to detect drift (a different torch build, an edited
oracle) and to give the GPU tests data-only vectors:
  * split: 96 fp32 inputs (bit patterns) and the bit patterns of every term for bf16 / fp16 / fp8;
  * cascade: error metrics versus fp64 of six cascades on two small seeded problems.

    python tests/golden/make_oracle_fixture.py
"""
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import cascade as oc  # noqa: E402

CASCADES = [("bf16", 1, "tri"), ("bf16", 2, "tri"), ("bf16", 2, "full"), ("bf16", 3, "tri"), ("fp16", 3, "tri"),
            ("fp8", 3, "tri")]
PROBLEMS = [(96, 128, 80, 0.02, 101), (154, 256, 64, 1.0, 102)]   # M, K, N, w_std, seed


def bits(t):
    return [int(v) for v in t.contiguous().view(torch.int32).tolist()]


def main():
    g = torch.Generator().manual_seed(7)
    x = torch.cat([torch.randn(64, generator=g), torch.randn(16, generator=g) * 1e-3, torch.randn(12, generator=g) * 200.0,
                   torch.tensor([0.0, 1.0, -1.0, 1.00390625])]).float()
    split = {"x_bits": bits(x), "terms": {}}
    for fmt in ("bf16", "fp16", "fp8"):
        e = oc.tensor_scale_exp(x, fmt)
        terms, _ = oc.split_terms(x, fmt, 3, tensor_exp=e)
        split["terms"][fmt] = {"tensor_exp": e, "bits": [bits(t) for t in terms]}
    cascade = []
    for (M, K, N, w_std, seed) in PROBLEMS:
        a, b = oc.make_operands(M, K, N, seed=seed, w_std=w_std)
        exp = oc.fp64_matmul(a, b)
        for fmt, terms, products in CASCADES:
            m = oc.error_metrics(oc.cascade_matmul_ref(a, b, fmt, terms, products), exp)
            cascade.append({"M": M, "K": K, "N": N, "w_std": w_std, "seed": seed, "fmt": fmt, "terms": terms,
                            "products": products, "rel_fro": m["rel_fro"], "max_abs": m["max_abs"]})
    out = {"torch": torch.__version__, "split": split, "cascade": cascade}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_fixture.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=0)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
