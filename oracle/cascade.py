"""CPU oracle for the cascaded low-precision matmul.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the product package never does (it raises when its HIP library is missing).

What is restated here and from where
------------------------------------
* The operand-split cascade itself has no counterpart in the reference: the reference
  kernel (basedxl/triton/cascaded_lowp_matmul.py:55-136) is an fp16-in / fp16-accumulate
  GEMM whose "cascade" is a K-chunk loop clamped to one chunk (:8-9, :23-26).  The
  arithmetic below is the one the target states in words: ``hi = lowp(x)``,
  ``lo = lowp(x - hi)`` (optionally a third term), every partial product accumulated in
  fp32.  Its pins are therefore mathematical (tests/test_oracle_*.py): bit-level closed
  forms of the roundings against two independent library casts, exactness invariants of
  the residuals, brute-force integer matmuls that must match bit for bit, special cases
  that collapse to a plain library matmul, and error bands against an fp64 product.
* Wrapper semantics (batch flattening, the two asserts, output dtype/shape) follow
  basedxl/triton/cascaded_lowp_matmul.py:139-173.
* The gated projection (``gated_projection_ref``) restates diffusers' ``GEGLU.forward``
  (``hidden_states, gate = proj(x).chunk(2, dim=-1); return hidden_states * gelu(gate)``,
  gelu in the exact erf form).  diffusers is a third-party dependency of the reference
  (README.md:17 installs it unpinned; model.py:3-4 imports it) and is absent here, so its
  published formula is restated; pins: math.erf in double precision on a grid, torch's own
  gelu (a library routine) and the identities gelu(x) - gelu(-x) = x, gelu(0) = 0.
* Error metrics follow extras/measure_cascaded_lowp_matmul_error.py:8-9,21,27-31 and the
  TFLOP/s formula follows basedxl/triton/cascaded_lowp_matmul.py:237-238.

Parity status: every function here is pinned by at least one check that does not retype
its formula (see tests/test_oracle_split.py, tests/test_oracle_cascade.py).  Nothing of
the target arithmetic is pinned by a reference golden vector, because the reference
holds none for it.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

# --------------------------------------------------------------------------------------
# formats
# --------------------------------------------------------------------------------------

#: low-precision formats of the cascade.  ``term_shift`` is log2 of the factor by which
#: residual i is scaled up before rounding (term i is scaled by 2**(term_shift*i));
#: ``sig_bits`` counts the implicit bit.
FORMATS: Dict[str, dict] = {
    "bf16": dict(dtype=torch.bfloat16, term_shift=0, sig_bits=8, tensor_scaled=False),
    "fp16": dict(dtype=torch.float16, term_shift=11, sig_bits=11, tensor_scaled=False),
    "fp8": dict(dtype=torch.float8_e4m3fn, term_shift=4, sig_bits=4, tensor_scaled=True),
}

#: largest finite float8_e4m3fn value
FP8_E4M3_MAX = 448.0


def product_set(terms: int, products: str = "tri") -> List[Tuple[int, int]]:
    """Index pairs (i, j) of the partial products ``A_i . B_j`` that are summed.

    ``tri`` keeps i + j <= terms - 1 (3 products for two terms, 6 for three); ``full``
    keeps all terms**2.  Ordered by decreasing i + j, i.e. smallest magnitude first.
    """
    if products not in ("tri", "full"):
        raise ValueError(f"products must be 'tri' or 'full', got {products!r}")
    pairs = [(i, j) for i in range(terms) for j in range(terms)
             if products == "full" or i + j <= terms - 1]
    pairs.sort(key=lambda p: (-(p[0] + p[1]), p[0]))
    return pairs


def tensor_scale_exp(x: torch.Tensor, fmt: str) -> int:
    """Power-of-two exponent e such that max|x| * 2**e lies in (224, 448] (fp8 only).

    Formats without a tensor scale return 0, and so does an all-zero tensor.
    """
    if not FORMATS[fmt]["tensor_scaled"]:
        return 0
    amax = float(x.detach().abs().max()) if x.numel() else 0.0
    if amax == 0.0 or not math.isfinite(amax):
        return 0
    m, ex = math.frexp(amax)  # amax = m * 2**ex, m in [0.5, 1)
    # 448 = 0.875 * 2**9
    return (9 - ex) if m <= 0.875 else (8 - ex)


def split_terms(x: torch.Tensor, fmt: str = "bf16", terms: int = 2,
                tensor_exp: Optional[int] = None) -> Tuple[List[torch.Tensor], List[float]]:
    """Split fp32 ``x`` into ``terms`` low-precision terms.

    r_0 = x;  t_i = lowp(r_i * s_i);  r_{i+1} = r_i - t_i / s_i
    with s_i = 2**(tensor_exp + term_shift * i).  Returns the terms upcast to fp32 (their
    values are exactly representable in the low-precision format) and the scales s_i.
    Every operation is an fp32 operation; s_i are powers of two so the scalings are
    exact, and r_i - t_i/s_i is exact in fp32 unless it underflows.
    """
    if x.dtype != torch.float32:
        raise TypeError("oracle splits fp32 operands only")
    spec = FORMATS[fmt]
    if tensor_exp is None:
        tensor_exp = tensor_scale_exp(x, fmt)
    out: List[torch.Tensor] = []
    scales: List[float] = []
    r = x.clone()
    for i in range(terms):
        s = math.ldexp(1.0, tensor_exp + spec["term_shift"] * i)
        t = (r * s).to(spec["dtype"]).to(torch.float32)
        out.append(t)
        scales.append(s)
        if i + 1 < terms:
            r = r - t / s
    return out, scales


def cascade_matmul_ref(a: torch.Tensor, b: torch.Tensor, fmt: str = "bf16", terms: int = 2,
                       products: str = "tri", a_exp: Optional[int] = None,
                       b_exp: Optional[int] = None) -> torch.Tensor:
    """2-D cascade: fp32 A[M,K] . fp32 B[K,N] through split terms, fp32 accumulation.

    One fp32 matmul per kept product on the upcast terms (each elementwise product is
    exact in fp32: 8+8, 11+11 or 4+4 significand bits), products of one scale class
    (i + j) summed first, classes combined from the smallest to the largest magnitude.
    ``a_exp`` / ``b_exp``: tensor-scale exponents to use instead of the operands' own
    (fp8; for checking a sample of the rows or columns of a larger product, whose scale
    comes from the whole tensor).
    """
    assert a.dim() == 2 and b.dim() == 2 and a.shape[1] == b.shape[0]
    ta, sa = split_terms(a, fmt, terms, a_exp)
    tb, sb = split_terms(b, fmt, terms, b_exp)
    classes: Dict[int, torch.Tensor] = {}
    inv: Dict[int, float] = {}
    for (i, j) in product_set(terms, products):
        p = torch.matmul(ta[i], tb[j])
        c = i + j
        classes[c] = p if c not in classes else classes[c] + p
        inv[c] = 1.0 / (sa[i] * sb[j])
    total = None
    for c in sorted(classes, reverse=True):
        part = classes[c] * inv[c]
        total = part if total is None else total + part
    return total


def cascaded_lowp_matmul_ref(a: torch.Tensor, b: torch.Tensor, *,
                             out: Optional[torch.Tensor] = None, fmt: str = "bf16",
                             terms: int = 2, products: str = "tri") -> torch.Tensor:
    """Wrapper semantics of basedxl/triton/cascaded_lowp_matmul.py:139-173 on the CPU.

    Same asserts (:146-148), leading dims of ``a`` flattened into M (:150-151,158),
    result in ``a.dtype`` (:161) reshaped to ``[*batch, N]`` (:173).  A batched ``b``
    (reachable in the reference only through its torch.matmul fallback, :155-156)
    broadcasts like torch.matmul.
    """
    assert a.shape[-1] == b.shape[-2], "Incompatible dimensions"
    assert b.is_contiguous(), "Matrix B must be contiguous"
    K, N = b.shape[-2], b.shape[-1]
    if b.dim() > 2:
        batch = torch.broadcast_shapes(a.shape[:-2], b.shape[:-2])
        a_b = a.expand(*batch, *a.shape[-2:]).reshape(-1, a.shape[-2], K)
        b_b = b.expand(*batch, K, N).reshape(-1, K, N)
        res = torch.stack([
            cascade_matmul_ref(a_b[i].float().contiguous(), b_b[i].float().contiguous(),
                               fmt, terms, products) for i in range(a_b.shape[0])])
        res = res.reshape(*batch, a.shape[-2], N).to(a.dtype)
    else:
        batch_dims = a.shape[:-1]
        a2 = a.reshape(-1, K).float().contiguous()
        res = cascade_matmul_ref(a2, b.float(), fmt, terms, products).to(a.dtype)
        res = res.reshape(*batch_dims, N)
    if out is not None:
        out.copy_(res.reshape(out.shape))
        return out.reshape(res.shape)
    return res


def gelu_erf(x: torch.Tensor) -> torch.Tensor:
    """Exact GELU, x * Phi(x) = 0.5 x (1 + erf(x / sqrt 2)), evaluated in the dtype of ``x``."""
    return 0.5 * x * (1.0 + torch.erf(x * (1.0 / math.sqrt(2.0))))


def gated_projection_ref(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, fmt: str = "bf16",
                         terms: int = 2, products: str = "tri") -> torch.Tensor:
    """``h = a . w (+ bias)`` through the cascade, then ``h[:, :inner] * gelu(h[:, inner:])``
    in fp32: what diffusers' GEGLU computes around its ``proj`` Linear."""
    assert w.shape[1] % 2 == 0
    h = cascade_matmul_ref(a, w, fmt, terms, products)
    if bias is not None:
        h = h + bias
    inner = w.shape[1] // 2
    return h[:, :inner] * gelu_erf(h[:, inner:])


# --------------------------------------------------------------------------------------
# reference results and metrics
# --------------------------------------------------------------------------------------

def fp64_matmul(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """The fp64 product used as ground truth (extras/measure_cascaded_lowp_matmul_error.py:21)."""
    return a.double() @ b.double()


EPS = 1e-6  # extras/measure_cascaded_lowp_matmul_error.py:8
QUANTILES = (0.01, 0.2, 0.5, 0.8, 0.99)  # extras/measure_cascaded_lowp_matmul_error.py:9


def error_metrics(out: torch.Tensor, expected: torch.Tensor) -> Dict[str, object]:
    """Error of ``out`` against an fp64 ``expected``.

    l1 / mse / max_abs / relative-error quantiles as in
    extras/measure_cascaded_lowp_matmul_error.py:27-31, plus the relative Frobenius norm
    ``||out - expected||_F / ||expected||_F`` used for the acceptance bound.
    """
    e = expected.double()
    d = (out.double().reshape(e.shape) - e)
    ad = d.abs()
    rel = ad / (e.abs() + EPS)
    denom = float(torch.linalg.norm(e))
    return {
        "l1": float(ad.mean()) if ad.numel() else 0.0,
        "mse": float((d * d).mean()) if ad.numel() else 0.0,
        "max_abs": float(ad.max()) if ad.numel() else 0.0,
        "rel_fro": float(torch.linalg.norm(d)) / denom if denom > 0 else 0.0,
        "rel_quantiles": [float(q) for q in np.quantile(rel.numpy().ravel(), QUANTILES)]
        if ad.numel() else [0.0] * len(QUANTILES),
    }


def fp32_equiv_tflops(M: int, N: int, K: int, seconds: float) -> float:
    """2*M*N*K / t in TFLOP/s, independent of the term count
    (basedxl/triton/cascaded_lowp_matmul.py:237-238)."""
    return 2.0 * M * N * K * 1e-12 / seconds


# --------------------------------------------------------------------------------------
# bit-level closed forms of the roundings (numpy, integer arithmetic only)
# --------------------------------------------------------------------------------------

def f32_bits(x: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)


def bits_f32(u: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(u, dtype=np.uint32).view(np.float32)


def rne_bf16_closed_form(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 -> fp32 by round-to-nearest-even on the bit pattern.

    Finite inputs: ``u + 0x7FFF + ((u >> 16) & 1)`` then clear the low 16 bits (a carry
    out of the mantissa correctly bumps the exponent, up to inf).  NaN stays a quiet NaN.
    """
    u = f32_bits(x).astype(np.uint64)
    rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    is_nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = np.where(is_nan, (u | 0x00400000) & 0xFFFF0000, rounded)
    return bits_f32((rounded & 0xFFFFFFFF).astype(np.uint32))


def _rne_to_grid(x: np.ndarray, sig_bits: int, emin: int, max_finite: float,
                 overflow_to: float) -> np.ndarray:
    """Round fp32 to a binary grid with ``sig_bits`` significant bits (implicit bit
    included), minimum normal exponent ``emin`` (gradual underflow below it), ties to
    even.  Magnitudes that round above ``max_finite`` become ``overflow_to``.

    Works in exact integer arithmetic on the fp32 bit pattern: x = m * 2**e with an
    integer 24-bit m; the result keeps q = m >> drop bits with RNE on the dropped part.
    """
    u = f32_bits(x).astype(np.int64)
    sign = np.where((u >> 31) & 1, -1.0, 1.0)
    expf = (u >> 23) & 0xFF
    frac = u & 0x7FFFFF
    is_nan = (expf == 0xFF) & (frac != 0)
    is_inf = (expf == 0xFF) & (frac == 0)
    # integer significand and exponent of the fp32 value: |x| = m * 2**e
    m = np.where(expf == 0, frac, frac | 0x800000)
    e = np.where(expf == 0, -149, expf - 150)
    # exponent of the top bit of |x| (floor(log2|x|)) for normals; subnormal fp32 are far
    # below every target grid so their exact msb does not matter.
    top = np.where(expf == 0, -127, expf - 127)
    # spacing of the target grid at this magnitude: 2**(max(top, emin) - (sig_bits - 1))
    ulp_e = np.maximum(top, emin) - (sig_bits - 1)
    drop = np.clip(ulp_e - e, 0, 62)  # how many low bits of m fall below the grid
    q = m >> drop
    rem = m - (q << drop)
    half = np.where(drop > 0, np.int64(1) << np.maximum(drop - 1, 0), 0)
    round_up = (drop > 0) & ((rem > half) | ((rem == half) & ((q & 1) == 1)))
    q = q + round_up
    val = q.astype(np.float64) * np.exp2((e + drop).astype(np.float64))
    val = np.where(val > max_finite, overflow_to, val)
    val = np.where(is_inf, overflow_to, val)
    out = (sign * val).astype(np.float32)
    out = np.where(is_nan, np.float32(np.nan), out)
    return out.astype(np.float32)


def rne_fp16_closed_form(x: np.ndarray) -> np.ndarray:
    """fp32 -> IEEE binary16 -> fp32 (11 significant bits, emin -14, overflow to inf)."""
    return _rne_to_grid(x, 11, -14, 65504.0, np.inf)


def rne_e4m3_closed_form(x: np.ndarray) -> np.ndarray:
    """fp32 -> float8 e4m3 (OCP "fn": 4 significant bits, emin -6, max 448, no inf;
    anything that rounds above 448 is NaN, as torch.float8_e4m3fn does) -> fp32."""
    return _rne_to_grid(x, 4, -6, FP8_E4M3_MAX, np.nan)


LOWP_CLOSED_FORMS = {
    "bf16": rne_bf16_closed_form,
    "fp16": rne_fp16_closed_form,
    "fp8": rne_e4m3_closed_form,
}


# --------------------------------------------------------------------------------------
# brute force for tiny cases (pure Python / numpy integer loops)
# --------------------------------------------------------------------------------------

def int_matmul_bruteforce(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    """Exact integer matmul by explicit loops over K (int64), for small known-answer tests."""
    a = np.asarray(a, dtype=np.int64)
    b = np.asarray(b, dtype=np.int64)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    c = np.zeros((M, N), dtype=np.int64)
    for k in range(K):
        c += a[:, k:k + 1] * b[k:k + 1, :]
    return c


# --------------------------------------------------------------------------------------
# synthetic workloads named by the baseline configs
# --------------------------------------------------------------------------------------

def make_operands(M: int, K: int, N: int, seed: int, w_std: float = 1.0,
                  x_std: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Seeded fp32 operands generated on the CPU: A ~ N(0, x_std), B ~ N(0, w_std)."""
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g, dtype=torch.float32) * x_std
    b = torch.randn(K, N, generator=g, dtype=torch.float32) * w_std
    return a, b
