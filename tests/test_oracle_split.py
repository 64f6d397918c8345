"""Pins for the oracle's roundings and operand split (CPU only).

None of these retype the oracle's formula: the library casts the oracle uses are checked
against integer-arithmetic closed forms and against a second library (numpy), and the
split is checked through exactness invariants a wrong split would break.
"""
import math

import numpy as np
import pytest
import torch
from hypothesis import given, settings, strategies as st

from oracle import cascade as oc


def _edge_values():
    vals = [0.0, -0.0, 1.0, -1.0, 1.5, 3.0, 0.1, -0.1, 1e-3, 448.0, 449.0, 464.0, 240.0, 15.5,
            65504.0, 65519.9, 65520.0, 70000.0, 1e-8, 6e-8, 5.96e-8, 2.98e-8, 2.99e-8,
            6.1e-5, 6.0e-5, 2 ** -14, 2 ** -24, 2 ** -25, 2 ** -6, 2 ** -9, 2 ** -10,
            1.17e-38, 1e-40, 3.0e38, 3.4e38, float("inf"), -float("inf")]
    # exact ties for each format: 1 + (odd or even) * half ulp
    for sig in (4, 8, 11):
        ulp = 2.0 ** -(sig - 1)
        for base in (1.0, 1.0 + ulp, 2.0 - ulp, 1.0 + 2 * ulp):
            for sgn in (1.0, -1.0):
                vals.append(sgn * (base + ulp / 2))
                vals.append(sgn * (base + ulp / 2) * 2 ** -5)
                vals.append(sgn * np.nextafter(np.float32(base + ulp / 2), np.float32(4.0)))
                vals.append(sgn * np.nextafter(np.float32(base + ulp / 2), np.float32(0.0)))
    return np.array(vals, dtype=np.float32)


def _random_bits(n, seed):
    rng = np.random.default_rng(seed)
    return rng.integers(0, 2 ** 32, size=n, dtype=np.uint64).astype(np.uint32).view(np.float32)


def _same(a, b):
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.all(both_nan | (a.view(np.uint32) == b.view(np.uint32)))


@pytest.mark.parametrize("fmt", ["bf16", "fp16", "fp8"])
def test_library_cast_matches_bit_level_closed_form(fmt):
    x = np.concatenate([_edge_values(), _random_bits(200_000, 1),
                        np.random.default_rng(2).standard_normal(200_000).astype(np.float32),
                        (np.random.default_rng(3).standard_normal(100_000) * 1e-4).astype(np.float32)])
    if fmt == "fp8":
        # torch's e4m3fn cast is only specified (non-NaN) up to 464; keep finite inputs in
        # range and check the overflow -> NaN rule separately below
        x = np.where(np.abs(x) > 1e6, np.float32(3.0), x)
    lib = torch.from_numpy(x.copy()).to(oc.FORMATS[fmt]["dtype"]).to(torch.float32).numpy()
    closed = oc.LOWP_CLOSED_FORMS[fmt](x)
    assert _same(lib, closed)


def test_fp16_cast_matches_numpy_too():
    x = np.concatenate([_edge_values(), _random_bits(100_000, 4)])
    with np.errstate(over="ignore"):
        via_np = x.astype(np.float16).astype(np.float32)
    via_torch = torch.from_numpy(x.copy()).to(torch.float16).to(torch.float32).numpy()
    assert _same(via_np, via_torch)
    assert _same(via_np, oc.rne_fp16_closed_form(x))


def test_e4m3_known_values():
    x = np.array([448.0, 464.0, 465.0, 1e9, 2 ** -9, 2 ** -10, 0.875 * 2 ** -6, 17.0, 18.0, 19.0, 21.0],
                 dtype=np.float32)
    got = oc.rne_e4m3_closed_form(x)
    # 464 is the tie between 448 and the (absent) 480 -> even mantissa 448; above -> NaN;
    # 2**-10 is the tie between 0 and the smallest subnormal 2**-9 -> 0;
    # spacing is 2 in [16,32): 17 -> 16 (tie to even), 19 -> 20, 21 -> 20
    want = np.array([448.0, 448.0, np.nan, np.nan, 2 ** -9, 0.0, 0.875 * 2 ** -6, 16.0, 18.0, 20.0, 20.0],
                    dtype=np.float32)
    assert _same(got, want)


def test_bf16_known_values():
    x = np.array([1.0, 1.00390625, 1.005859375, 1.01171875, 3.4e38], dtype=np.float32)
    # 1 + 2^-8 is a tie -> 1.0 (even); 1 + 1.5*2^-8 -> 1 + 2^-7; 1+3*2^-8 tie -> 1 + 2^-6 (even)
    want = np.array([1.0, 1.0, 1.0078125, 1.015625, np.inf], dtype=np.float32)
    assert _same(oc.rne_bf16_closed_form(x), want)


@pytest.mark.parametrize("fmt,terms", [("bf16", 2), ("bf16", 3), ("fp16", 2), ("fp16", 3), ("fp8", 3)])
def test_split_terms_are_representable_and_reconstruct(fmt, terms):
    g = torch.Generator().manual_seed(5)
    for std in (1.0, 0.02):
        x = torch.randn(4096, generator=g) * std
        ts, ss = oc.split_terms(x, fmt, terms)
        assert len(ts) == terms and len(ss) == terms
        acc = torch.zeros_like(x, dtype=torch.float64)
        sig = oc.FORMATS[fmt]["sig_bits"]
        for i, (t, s) in enumerate(zip(ts, ss)):
            # each term is a fixed point of the format's rounding
            assert _same(oc.LOWP_CLOSED_FORMS[fmt](t.numpy()), t.numpy())
            acc += t.double() / s
            resid = (x.double() - acc).abs()
            # after i+1 terms the residual is below half an ulp of the last term, i.e.
            # 2**-(sig*(i+1)) relative for values clear of the subnormal range
            bound = x.double().abs() * 2.0 ** (-sig * (i + 1)) + (1e-30 if fmt != "fp8" else 0)
            if fmt == "fp8":
                # e4m3 subnormals (below 2**-6 after scaling): absolute bound half a subnormal step
                bound = torch.maximum(bound, torch.full_like(bound, 2.0 ** -10 / s))
            if fmt == "fp16":
                bound = torch.maximum(bound, torch.full_like(bound, 2.0 ** -25 / s))
            assert bool((resid <= bound).all()), (fmt, terms, i, float((resid - bound).max()))


@settings(max_examples=300, deadline=None)
@given(st.floats(min_value=-1e4, max_value=1e4, allow_nan=False, width=32))
def test_bf16_residual_is_exact_in_fp32(v):
    x = torch.tensor([v], dtype=torch.float32)
    (hi, lo), _ = oc.split_terms(x, "bf16", 2)
    # x - hi must be exactly representable: computing it in fp64 and in fp32 agrees
    r64 = x.double() - hi.double()
    assert float((x - hi).double() - r64) == 0.0
    assert abs(float(r64)) <= abs(v) * 2.0 ** -8 + 2.0 ** -134  # half a bf16 subnormal step
    assert abs(float(r64 - lo.double())) <= abs(v) * 2.0 ** -16 + 2.0 ** -134


@pytest.mark.parametrize("fmt,keep_bits", [("bf16", 8), ("fp16", 11), ("fp8", 4)])
def test_inputs_with_few_significant_bits_have_zero_low_terms(fmt, keep_bits):
    # values with <= keep_bits significant bits are exactly representable -> lo terms are 0
    rng = np.random.default_rng(6)
    mant = rng.integers(2 ** (keep_bits - 1), 2 ** keep_bits, size=2000)
    expo = rng.integers(-3, 4, size=2000)
    x = torch.tensor(mant * 2.0 ** expo * rng.choice([-1, 1], size=2000), dtype=torch.float32)
    ts, ss = oc.split_terms(x, fmt, 3)
    assert torch.equal(ts[0] / ss[0], x)
    assert float(ts[1].abs().max()) == 0.0 and float(ts[2].abs().max()) == 0.0
    # and 2*keep_bits significant bits are captured exactly by two terms
    mant2 = rng.integers(2 ** (2 * keep_bits - 1), 2 ** (2 * keep_bits), size=2000)
    x2 = torch.tensor(mant2 * 2.0 ** -(2 * keep_bits - 4) * rng.choice([-1, 1], size=2000), dtype=torch.float32)
    ts2, ss2 = oc.split_terms(x2, fmt, 3)
    assert torch.equal((ts2[0].double() / ss2[0] + ts2[1].double() / ss2[1]).float(), x2)
    assert float(ts2[2].abs().max()) == 0.0


def test_fp8_tensor_scale_exponent():
    for amax in [1.0, 0.02, 3.9, 447.0, 448.0, 449.0, 1e-5, 7.0, 0.875, 0.876]:
        x = torch.tensor([amax, -amax / 3], dtype=torch.float32)
        e = oc.tensor_scale_exp(x, "fp8")
        scaled = float(np.float32(amax)) * 2.0 ** e
        assert 224.0 < scaled <= 448.0, (amax, e, scaled)
    assert oc.tensor_scale_exp(torch.zeros(4), "fp8") == 0
    assert oc.tensor_scale_exp(torch.ones(4), "bf16") == 0
    assert oc.tensor_scale_exp(torch.ones(4), "fp16") == 0


def test_fp16_term_scaling_beats_unscaled_on_small_weights():
    # N(0, 0.02) weights: unscaled lo terms fall into fp16 subnormals; the scaled split must
    # keep ~22 bits with two terms
    g = torch.Generator().manual_seed(7)
    w = torch.randn(20000, generator=g) * 0.02
    ts, ss = oc.split_terms(w, "fp16", 2)
    rec = ts[0].double() / ss[0] + ts[1].double() / ss[1]
    rel = ((rec - w.double()).abs() / w.double().abs().clamp_min(1e-12))
    big = w.abs() > 1e-3
    assert float(rel[big].max()) <= 2.0 ** -22
    hi = w.half()
    lo_unscaled = (w - hi.float()).half()
    rec_u = hi.double() + lo_unscaled.double()
    rel_u = ((rec_u - w.double()).abs() / w.double().abs().clamp_min(1e-12))
    assert float(rel_u[big].max()) > 4 * float(rel[big].max())
