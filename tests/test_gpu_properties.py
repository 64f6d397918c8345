"""Properties of the cascade GEMM that hold at any size, checked at the full sizes of the baseline
configurations (where the CPU oracle would take minutes): they need no reference values, only the
kernels' own results on related inputs, and every one of them is EXACT (bit for bit), because each
output element is a fixed-order fp32 accumulation over k of exact products:

* permuting the rows of A permutes the rows of C; permuting the columns of B permutes its columns
  (a wrong tile-to-row / tile-to-column map, a clamped or repeated row, a mis-stored block shows);
* multiplying A and B by powers of two scales C by their product (bf16: the split of 2^k x is 2^k
  times the split of x; fp8: the tensor scale absorbs the factor) -- term scaling / tensor-scale
  mistakes show;
* appending zero columns to A and zero rows to B (a longer K) changes nothing (the K loop bounds and
  the staging of the extra steps show);
* B = I returns the sum of the terms of A (the product set and the order of the classes show).
"""
import pytest
import torch

from basedxl_amd import PreparedWeight, _lib, cascaded_lowp_matmul

pytestmark = pytest.mark.gpu

FULL_SIZES = [
    pytest.param(4096, 640, 640, id="cfg2-4096x640x640"),
    pytest.param(2048, 1280, 10240, id="cfg3-2048x1280x10240"),
    pytest.param(2048, 5120, 1280, id="cfg3-2048x5120x1280"),
    pytest.param(154, 2048, 1280, id="cfg4-154x2048x1280"),
    pytest.param(1024, 1024, 1024, id="cfg1-1024x1024x1024"),
]
CASCADES = [("bf16", 2), ("bf16", 3), ("fp16", 3), ("fp8", 3)]


def _operands(M, K, N, seed):
    g = torch.Generator(device="cuda:0").manual_seed(seed)
    a = torch.randn(M, K, device="cuda:0", generator=g)
    b = torch.randn(K, N, device="cuda:0", generator=g) * 0.02
    return a, b


@pytest.mark.parametrize("M,K,N", FULL_SIZES)
@pytest.mark.parametrize("lowp,terms", CASCADES)
def test_row_and_column_permutations_commute_with_the_product(gpu_device, M, K, N, lowp, terms):
    print("permutations", M, K, N, lowp, terms, flush=True)
    a, b = _operands(M, K, N, 1)
    c = cascaded_lowp_matmul(a, b, lowp=lowp, terms=terms)
    g = torch.Generator(device="cuda:0").manual_seed(2)
    pr = torch.randperm(M, device="cuda:0", generator=g)
    pc = torch.randperm(N, device="cuda:0", generator=g)
    # fp8: the tensor scales depend only on max |x|, which a permutation keeps
    assert torch.equal(cascaded_lowp_matmul(a[pr].contiguous(), b, lowp=lowp, terms=terms), c[pr])
    assert torch.equal(cascaded_lowp_matmul(a, b[:, pc].contiguous(), lowp=lowp, terms=terms), c[:, pc])


@pytest.mark.parametrize("M,K,N", FULL_SIZES)
@pytest.mark.parametrize("lowp,terms", [("bf16", 2), ("bf16", 3), ("fp8", 3)])
def test_powers_of_two_factor_out_exactly(gpu_device, M, K, N, lowp, terms):
    print("powers of two", M, K, N, lowp, terms, flush=True)
    a, b = _operands(M, K, N, 3)
    c = cascaded_lowp_matmul(a, b, lowp=lowp, terms=terms)
    c2 = cascaded_lowp_matmul(a * 8.0, b * 2.0 ** -5, lowp=lowp, terms=terms)
    assert torch.equal(c2, c * 2.0 ** -2)


@pytest.mark.parametrize("M,K,N", FULL_SIZES)
@pytest.mark.parametrize("lowp,terms", [("bf16", 2), ("fp16", 3)])
def test_zero_padding_of_k_changes_nothing(gpu_device, M, K, N, lowp, terms):
    """Same kernel on both sides (forced), K and K + 128."""
    print("zero padding", M, K, N, lowp, terms, flush=True)
    l = _lib.lib()
    a, b = _operands(M, K, N, 4)
    ap = torch.cat([a, torch.zeros(M, 128, device="cuda:0")], dim=1).contiguous()
    bp = torch.cat([b, torch.zeros(128, N, device="cuda:0")], dim=0).contiguous()
    v = l.cascmm_select_variant(M, N, K + 128, K + 128, N, N, _lib.DT_F32, _lib.FMT_BY_NAME[lowp], terms, 0)
    assert v >= 0
    if "splitk" in l.cascmm_variant_name(v).decode() or "skinny" in l.cascmm_variant_name(v).decode():
        pytest.skip("the split-K kernels cut K differently for the two lengths: sums are regrouped, not bit-equal")
    c = cascaded_lowp_matmul(a, b, lowp=lowp, terms=terms, variant=v)
    assert torch.equal(cascaded_lowp_matmul(ap, bp, lowp=lowp, terms=terms, variant=v), c)


@pytest.mark.parametrize("M,K", [(4096, 640), (2048, 1280), (154, 2048)])
@pytest.mark.parametrize("lowp,terms,products", [("bf16", 2, "tri"), ("bf16", 3, "tri"), ("bf16", 2, "full"), ("fp16", 2, "tri")])
def test_identity_returns_the_sum_of_the_terms(gpu_device, M, K, lowp, terms, products):
    """B = I has the terms (1, 0, 0): of the kept products only t_i(A) x hi(I) are non-zero, so
    C = sum_i t_i(A) / s_i, every partial sum exactly representable (it is A minus a residual)."""
    print("identity", M, K, lowp, terms, products, flush=True)
    a = torch.randn(M, K, device="cuda:0", generator=torch.Generator(device="cuda:0").manual_seed(5))
    c = cascaded_lowp_matmul(a, torch.eye(K, device="cuda:0"), lowp=lowp, terms=terms, products=products)
    t = torch.empty(terms, a.numel(), dtype=torch.float32, device="cuda:0")
    assert _lib.lib().cascmm_split_terms(a.data_ptr(), t.data_ptr(), a.numel(), _lib.DT_F32, _lib.FMT_BY_NAME[lowp], terms, 0,
                                         torch.cuda.current_stream().cuda_stream) == 0
    shift = {"bf16": 0, "fp16": 11}[lowp]
    want = sum((t[i].double() * 2.0 ** (-shift * i) for i in range(terms))).float().reshape(M, K)
    assert torch.equal(c, want)


@pytest.mark.parametrize("M,K,N", FULL_SIZES[:3])
def test_prepared_weight_has_the_same_properties(gpu_device, M, K, N):
    print("prepared permutations", M, K, N, flush=True)
    a, b = _operands(M, K, N, 6)
    pr = torch.randperm(M, device="cuda:0", generator=torch.Generator(device="cuda:0").manual_seed(7))
    pw = PreparedWeight(b)
    c = cascaded_lowp_matmul(a, pw)
    assert torch.equal(cascaded_lowp_matmul(a[pr].contiguous(), pw), c[pr])
    assert torch.equal(cascaded_lowp_matmul(a * 4.0, pw), c * 4.0)
