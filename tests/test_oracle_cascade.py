"""Pins for the oracle's cascade matmul, wrapper semantics and metrics (CPU only)."""
import numpy as np
import pytest
import torch

from oracle import cascade as oc

ALL_VARIANTS = [("bf16", 1), ("bf16", 2), ("bf16", 3), ("fp16", 2), ("fp16", 3), ("fp8", 3)]


def test_product_sets():
    assert sorted(oc.product_set(2, "tri")) == [(0, 0), (0, 1), (1, 0)]
    assert len(oc.product_set(3, "tri")) == 6 and (1, 1) in oc.product_set(3, "tri")
    assert (1, 2) not in oc.product_set(3, "tri")
    assert len(oc.product_set(2, "full")) == 4 and len(oc.product_set(3, "full")) == 9
    assert oc.product_set(1, "tri") == [(0, 0)]
    # smallest magnitude first
    ps = oc.product_set(3, "tri")
    assert [i + j for i, j in ps] == sorted([i + j for i, j in ps], reverse=True)
    with pytest.raises(ValueError):
        oc.product_set(2, "all")


@pytest.mark.parametrize("fmt,terms", ALL_VARIANTS)
@pytest.mark.parametrize("shape", [(16, 32, 16), (17, 33, 19), (154, 64, 48), (1, 7, 1)])
def test_small_integer_inputs_equal_bruteforce_integer_matmul(fmt, terms, shape):
    """Every partial product is exact and all partial sums stay below 2**24, so the
    cascade must equal the integer matmul bit for bit, whatever the summation order."""
    M, K, N = shape
    rng = np.random.default_rng(M * 1000 + K)
    hi = 7 if fmt == "fp8" else 100  # fp8 first term holds 4 bits; more bits spill into later terms
    a = rng.integers(-hi, hi + 1, size=(M, K))
    b = rng.integers(-hi, hi + 1, size=(K, N))
    want = oc.int_matmul_bruteforce(a, b)
    assert np.abs(want).max() < 2 ** 24
    got = oc.cascade_matmul_ref(torch.tensor(a, dtype=torch.float32), torch.tensor(b, dtype=torch.float32),
                                fmt, terms, "full")
    assert np.array_equal(got.numpy().astype(np.int64), want)
    if terms == 1 or hi < 2 ** oc.FORMATS[fmt]["sig_bits"]:
        # operands fit the first term: tri equals full
        got_tri = oc.cascade_matmul_ref(torch.tensor(a, dtype=torch.float32),
                                        torch.tensor(b, dtype=torch.float32), fmt, terms, "tri")
        assert np.array_equal(got_tri.numpy().astype(np.int64), want)


def test_integers_needing_two_terms_full_exact_tri_drops_lo_lo():
    """16-bit integers need hi and lo bf16 terms.  The full product set is exact; the tri
    set differs from it by exactly the lo.lo product (computed independently in int64)."""
    rng = np.random.default_rng(11)
    a = rng.integers(-2000, 2001, size=(8, 12))
    b = rng.integers(-2000, 2001, size=(12, 8))
    at, bt = torch.tensor(a, dtype=torch.float32), torch.tensor(b, dtype=torch.float32)
    want = oc.int_matmul_bruteforce(a, b)
    assert np.abs(want).max() < 2 ** 27
    # partial sums < 2**24 are needed for exactness: shrink K contribution check
    full = oc.cascade_matmul_ref(at, bt, "bf16", 2, "full").numpy().astype(np.int64)
    (a_hi, a_lo), _ = oc.split_terms(at, "bf16", 2)
    (b_hi, b_lo), _ = oc.split_terms(bt, "bf16", 2)
    assert torch.equal(a_hi + a_lo, at) and torch.equal(b_hi + b_lo, bt)
    lolo = oc.int_matmul_bruteforce(a_lo.numpy().astype(np.int64), b_lo.numpy().astype(np.int64))
    tri = oc.cascade_matmul_ref(at, bt, "bf16", 2, "tri").numpy().astype(np.int64)
    small = np.abs(want) < 2 ** 24
    assert small.any()
    assert np.array_equal(full[small], want[small])
    assert np.array_equal((full - tri)[small], lolo[small])


def test_one_term_equals_library_matmul_on_rounded_operands():
    a, b = oc.make_operands(64, 96, 80, seed=3)
    got = oc.cascade_matmul_ref(a, b, "bf16", 1)
    want = torch.matmul(a.bfloat16().float(), b.bfloat16().float())
    assert torch.equal(got, want)


@pytest.mark.parametrize("fmt", ["bf16", "fp16"])
def test_representable_inputs_make_extra_terms_a_no_op(fmt):
    a, b = oc.make_operands(48, 64, 40, seed=4)
    dt = oc.FORMATS[fmt]["dtype"]
    a, b = a.to(dt).float(), b.to(dt).float()
    one = oc.cascade_matmul_ref(a, b, fmt, 1)
    assert torch.equal(oc.cascade_matmul_ref(a, b, fmt, 2), one)
    assert torch.equal(oc.cascade_matmul_ref(a, b, fmt, 3, "full"), one)


def test_linearity_in_power_of_two_scaling():
    a, b = oc.make_operands(32, 128, 32, seed=5)
    base = oc.cascade_matmul_ref(a, b, "bf16", 2)
    assert torch.equal(oc.cascade_matmul_ref(a * 4.0, b * 0.5, "bf16", 2), base * 2.0)
    base3 = oc.cascade_matmul_ref(a, b, "fp8", 3)  # tensor scale absorbs powers of two exactly
    assert torch.equal(oc.cascade_matmul_ref(a * 8.0, b * 0.25, "fp8", 3), base3 * 2.0)


# error bands against fp64: wide enough for any seed / BLAS summation order, tight enough
# that a dropped product, a missing term or a wrong scale falls outside
BANDS = {
    ("bf16", 1, "tri"): (1.5e-3, 3.5e-3),
    ("bf16", 2, "tri"): (3.3e-6, 5.5e-6),
    ("bf16", 2, "full"): (2.6e-6, 4.3e-6),
    ("bf16", 3, "tri"): (0.5e-7, 4.5e-7),
    ("fp16", 2, "tri"): (0.8e-7, 6e-7),
    ("fp16", 3, "tri"): (0.8e-7, 6e-7),
    ("fp8", 3, "tri"): (2.3e-5, 4.0e-5),
    ("fp8", 3, "full"): (1.5e-5, 2.7e-5),
}


@pytest.mark.parametrize("key", sorted(BANDS))
@pytest.mark.parametrize("w_std,shape", [(1.0, (256, 512, 192)), (0.02, (154, 640, 128))])
def test_error_vs_fp64_lies_in_band(key, w_std, shape):
    fmt, terms, products = key
    M, K, N = shape
    a, b = oc.make_operands(M, K, N, seed=0, w_std=w_std)
    exp = oc.fp64_matmul(a, b)
    m = oc.error_metrics(oc.cascade_matmul_ref(a, b, fmt, terms, products), exp)
    lo, hi = BANDS[key]
    assert lo <= m["rel_fro"] <= hi, (key, m["rel_fro"])


def test_tri_is_worse_than_full_by_the_expected_factor():
    a, b = oc.make_operands(512, 512, 256, seed=1)
    exp = oc.fp64_matmul(a, b)
    tri = oc.error_metrics(oc.cascade_matmul_ref(a, b, "bf16", 2, "tri"), exp)["rel_fro"]
    full = oc.error_metrics(oc.cascade_matmul_ref(a, b, "bf16", 2, "full"), exp)["rel_fro"]
    assert 1.15 < tri / full < 1.45


# ---- wrapper semantics (shape cases of tests/test_cascaded_lowp_matmul.py:9-14) ----

@pytest.mark.parametrize("shape_a,shape_b", [
    ((10, 20), (20, 30)), ((5, 10, 20), (20, 30)), ((10, 20), (5, 20, 30)), ((5, 10, 20), (5, 20, 30)),
    ((128, 512), (512, 128)),
])
def test_wrapper_shapes_and_values(shape_a, shape_b):
    g = torch.Generator().manual_seed(8)
    a = torch.randn(*shape_a, generator=g)
    b = torch.randn(*shape_b, generator=g)
    out = oc.cascaded_lowp_matmul_ref(a, b)
    want = torch.matmul(a.double(), b.double())
    assert out.shape == want.shape and out.dtype == a.dtype
    assert oc.error_metrics(out, want)["rel_fro"] < 1e-5


def test_wrapper_asserts_and_out():
    a = torch.randn(4, 8)
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        oc.cascaded_lowp_matmul_ref(a, torch.randn(9, 4))
    with pytest.raises(AssertionError, match="Matrix B must be contiguous"):
        oc.cascaded_lowp_matmul_ref(a, torch.randn(4, 8).t())
    out = torch.empty(4, 5)
    b = torch.randn(8, 5)
    r = oc.cascaded_lowp_matmul_ref(a, b, out=out)
    assert r.data_ptr() == out.data_ptr()
    assert torch.equal(out, oc.cascaded_lowp_matmul_ref(a, b))
    h = oc.cascaded_lowp_matmul_ref(a.half(), b.half())
    assert h.dtype == torch.float16


def test_metrics_on_a_known_case():
    exp = torch.tensor([[1.0, 2.0], [0.0, -4.0]], dtype=torch.float64)
    out = torch.tensor([[1.5, 2.0], [0.0, -3.0]], dtype=torch.float32)
    m = oc.error_metrics(out, exp)
    assert m["max_abs"] == 1.0
    assert m["l1"] == pytest.approx(0.375)
    assert m["mse"] == pytest.approx((0.25 + 1.0) / 4)
    assert m["rel_fro"] == pytest.approx(np.sqrt(1.25) / np.sqrt(21.0))
    # relative errors |d| / (|e| + 1e-6) of the four elements: 0.5 / 1.000001, 0, 0, 1 / 4.000001;
    # numpy's linear interpolation on the sorted values [0, 0, 0.25, 0.5] at 1 / 20 / 50 / 80 / 99 %
    r = sorted([0.5 / 1.000001, 0.0, 0.0, 1.0 / 4.000001])
    def interp(q):
        pos = q * 3
        lo = int(pos)
        return r[lo] + (r[min(lo + 1, 3)] - r[lo]) * (pos - lo)
    assert m["rel_quantiles"] == pytest.approx([interp(q) for q in (0.01, 0.2, 0.5, 0.8, 0.99)], rel=1e-12, abs=1e-15)
    assert m["rel_quantiles"][2] == pytest.approx(0.125, rel=1e-5) and m["rel_quantiles"][0] == 0.0
    # a larger known case: out = 1.01 x expected everywhere -> every relative error is 0.01 / (1 + 1e-6 / |e|)
    e = torch.arange(1, 1001, dtype=torch.float64).reshape(10, 100)
    q = oc.error_metrics((e * 1.01).float(), e)["rel_quantiles"]
    assert all(abs(v - 0.01) < 1e-6 for v in q) and q == sorted(q)
    assert oc.fp32_equiv_tflops(1024, 1024, 1024, 1e-3) == pytest.approx(2.147483648)


# ---------------------------------------------------------------------------------------
# drift check against the committed fixture (tests/golden/make_oracle_fixture.py)
# ---------------------------------------------------------------------------------------
def _fixture():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "oracle_fixture.json")) as f:
        return json.load(f)


def test_oracle_split_reproduces_the_fixture_bit_for_bit():
    fx = _fixture()["split"]
    x = torch.tensor(fx["x_bits"], dtype=torch.int32).view(torch.float32)
    for fmt, rec in fx["terms"].items():
        assert oc.tensor_scale_exp(x, fmt) == rec["tensor_exp"]
        terms, _ = oc.split_terms(x, fmt, 3, tensor_exp=rec["tensor_exp"])
        for t, want in zip(terms, rec["bits"]):
            assert t.view(torch.int32).tolist() == want, fmt


def test_oracle_cascade_errors_match_the_fixture():
    for rec in _fixture()["cascade"]:
        a, b = oc.make_operands(rec["M"], rec["K"], rec["N"], seed=rec["seed"], w_std=rec["w_std"])
        m = oc.error_metrics(oc.cascade_matmul_ref(a, b, rec["fmt"], rec["terms"], rec["products"]), oc.fp64_matmul(a, b))
        # the fp32 matmuls inside the oracle may sum in another order on another torch build
        assert m["rel_fro"] == pytest.approx(rec["rel_fro"], rel=0.02), rec
        assert m["max_abs"] == pytest.approx(rec["max_abs"], rel=0.25), rec


def test_gelu_erf_against_double_precision_erf_and_identities():
    """The oracle's gate: double-precision math.erf on a grid (an independent evaluation), torch's
    own gelu (library routine), and what the definition x * Phi(x) fixes: gelu(0) = 0,
    gelu(x) - gelu(-x) = x, gelu(x) -> x and gelu(-x) -> 0 for large x."""
    import math

    xs = torch.linspace(-6.0, 6.0, 481, dtype=torch.float64)
    want = torch.tensor([0.5 * v * (1.0 + math.erf(v / math.sqrt(2.0))) for v in xs.tolist()], dtype=torch.float64)
    got64 = oc.gelu_erf(xs)
    assert torch.allclose(got64, want, rtol=1e-13, atol=1e-15)
    got32 = oc.gelu_erf(xs.float())
    assert torch.allclose(got32.double(), want, rtol=0, atol=1e-6)   # ulp(6) = 4.8e-7
    assert torch.allclose(got32, torch.nn.functional.gelu(xs.float()), rtol=0, atol=1e-6)
    assert oc.gelu_erf(torch.zeros(3)).abs().max() == 0
    x = torch.linspace(0.0, 5.0, 101, dtype=torch.float64)
    assert torch.allclose(oc.gelu_erf(x) - oc.gelu_erf(-x), x, rtol=0, atol=1e-15)
    assert oc.gelu_erf(torch.tensor([40.0]))[0] == 40.0 and oc.gelu_erf(torch.tensor([-40.0]))[0] == 0.0


def test_gated_projection_is_the_cascade_followed_by_the_gate():
    """Integer operands make the cascade exact, so the gated projection must equal the gate applied
    to the integer product (computed in int64), bias included; the value half must come from the
    first half of the columns and the gate from the second (a swapped pair changes the result)."""
    g = torch.Generator().manual_seed(5)
    a = torch.randint(-4, 5, (9, 16), generator=g).float()
    w = torch.randint(-3, 4, (16, 12), generator=g).float()
    bias = torch.randint(-2, 3, (12,), generator=g).float()
    h = (a.long() @ w.long() + bias.long()).double()
    want = h[:, :6] * torch.nn.functional.gelu(h[:, 6:])
    got = oc.gated_projection_ref(a, w, bias)
    assert got.shape == (9, 6)
    assert torch.allclose(got.double(), want, rtol=1e-6, atol=1e-6)
    swapped = h[:, 6:] * torch.nn.functional.gelu(h[:, :6])
    assert not torch.allclose(got.double(), swapped, rtol=1e-3, atol=1e-3)
