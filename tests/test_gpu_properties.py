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


@pytest.mark.parametrize("M,K,N", [(1024, 1280, 1280), (1024, 5120, 1280), (300, 2560, 200)])
def test_the_small_tile_of_the_k_over_waves_kernel_has_the_same_properties(gpu_device, M, K, N):
    """The 64 x 80 tile, forced by name, on the half-latent share's shapes and a ragged one: rows and columns may be
    permuted, powers of two factor out, and 32 more k of zeros (one more stage, for one of the four waves) change nothing."""
    print("64 x 80 tile properties", M, K, N, flush=True)
    from basedxl_amd import _lib
    v = _lib.variant_names().index("k64x80x32_wk4_bf16x2_tri_bpre")
    a, b = _operands(M, K, N, 16)
    g = torch.Generator(device="cuda:0").manual_seed(17)
    pr, pc = torch.randperm(M, device="cuda:0", generator=g), torch.randperm(N, device="cuda:0", generator=g)
    c = cascaded_lowp_matmul(a, PreparedWeight(b), variant=v)
    assert torch.equal(cascaded_lowp_matmul(a[pr].contiguous(), PreparedWeight(b), variant=v), c[pr])
    assert torch.equal(cascaded_lowp_matmul(a, PreparedWeight(b[:, pc].contiguous()), variant=v), c[:, pc])
    assert torch.equal(cascaded_lowp_matmul(a * 4.0, PreparedWeight(b * 0.5), variant=v), c * 2.0)
    a2 = torch.cat([a, torch.zeros(M, 32, device="cuda:0")], dim=1).contiguous()
    b2 = torch.cat([b, torch.zeros(32, N, device="cuda:0")], dim=0).contiguous()
    assert torch.equal(cascaded_lowp_matmul(a2, PreparedWeight(b2), variant=v), c)


def test_prepared_weight_takes_rows_that_are_not_16_byte_aligned(gpu_device):
    """A view whose rows start at odd element offsets (row stride K + 3, first element shifted by
    one) gives the same bits as its contiguous copy: the wrapper copies what the prepared kernels
    cannot load, as the reference copies every ``a`` (basedxl/triton/cascaded_lowp_matmul.py:158)."""
    g = torch.Generator(device="cuda:0").manual_seed(11)
    K, N, M = 512, 320, 130
    store = torch.randn(M, K + 3, device="cuda:0", generator=g)
    b = torch.randn(K, N, device="cuda:0", generator=g) * 0.02
    pw = PreparedWeight(b)
    a = store[:, 1:K + 1]
    assert a.data_ptr() % 16 != 0 and a.stride(0) % 4 != 0
    want = cascaded_lowp_matmul(a.contiguous(), pw)
    assert torch.equal(cascaded_lowp_matmul(a, pw), want)
    # the raw weight gives the same sum of the same products, in the summation order of its own kernel
    torch.testing.assert_close(want, cascaded_lowp_matmul(a, b), rtol=1e-5, atol=1e-5)


def test_random_shapes_strides_and_cascades_integer_exact(gpu_device):
    """Seeded sweep over what a caller can vary at once -- M, N, K (odd sizes included), row
    strides of A and of the result, leading batch dims, bias, dtype, cascade and product set -- with
    the kernel left to the library's own selection.  Operands are small integers, so every cascade
    that keeps enough products equals the integer matmul exactly (for 16-bit outputs: after one
    rounding), whatever kernel, tile edge or K tail the case lands on."""
    import numpy as np

    from basedxl_amd import cascaded_lowp_matmul_grouped

    rng = np.random.default_rng(20240607)
    cascades = [("bf16", 1, "tri"), ("bf16", 2, "tri"), ("bf16", 2, "full"), ("bf16", 3, "tri"), ("fp16", 1, "tri"),
                ("fp16", 2, "tri"), ("fp16", 3, "tri"), ("fp8", 3, "full"), ("fp8", 3, "tri"), ("fp8", 2, "full")]
    sizes = [1, 2, 3, 7, 16, 31, 32, 33, 64, 77, 96, 128, 154, 160, 200, 256, 320]
    for case in range(120):
        M, N, K = (int(rng.choice(sizes)) for _ in range(3))
        lowp, terms, products = cascades[case % len(cascades)]
        dtype = [torch.float32, torch.float32, torch.float16, torch.bfloat16][case % 4]
        if dtype != torch.float32:
            lowp, terms, products = ("fp16" if dtype == torch.float16 else "bf16"), 1, "tri"
        # fp8 keeps 4 significand bits per term: 'tri' with three terms is exact only on one-term operands
        hi = 7 if (lowp == "fp8" and products == "tri") or dtype != torch.float32 else 15
        pad_a, pad_c = int(rng.integers(0, 3)) * 4, int(rng.integers(0, 3)) * 4
        a = torch.tensor(rng.integers(-hi, hi + 1, (M, K)), dtype=torch.float32)
        b = torch.tensor(rng.integers(-hi, hi + 1, (K, N)), dtype=torch.float32)
        bias = torch.tensor(rng.integers(-hi, hi + 1, (N,)), dtype=torch.float32) if case % 3 == 0 else None
        want = a.long() @ b.long() + (bias.long() if bias is not None else 0)
        print("fuzz", case, M, N, K, lowp, terms, products, dtype, pad_a, pad_c, bias is not None, flush=True)
        a_full = torch.full((M, K + pad_a), 99.0, device="cuda:0", dtype=dtype)      # rows padded with junk
        a_full[:, :K] = a.to("cuda:0").to(dtype)
        ad, bd = a_full[:, :K], b.to("cuda:0").to(dtype)
        bias_d = None if bias is None else bias.to("cuda:0").to(dtype)
        out_full = torch.full((M, N + pad_c), -77.0, device="cuda:0", dtype=dtype)   # result rows padded too
        kw = dict(lowp=lowp, terms=terms, products=products)
        if case % 5 == 0 and M % 2 == 0 and pad_a == 0:
            got = cascaded_lowp_matmul(ad.reshape(2, M // 2, K), bd, bias=bias_d, **kw).reshape(M, N)
        elif case % 7 == 0:
            got = cascaded_lowp_matmul_grouped([ad, ad], [bd, bd], biases=None if bias is None else [bias_d] * 2, **kw)[1]
        else:
            got = cascaded_lowp_matmul(ad, bd, bias=bias_d, out=out_full[:, :N], **kw)
            assert got.data_ptr() == out_full.data_ptr()
            assert bool((out_full[:, N:] == -77.0).all())                            # nothing written past a row's N columns
        want_t = want.to(torch.float32).to(dtype)      # 16-bit results: the exact integer rounded once
        assert torch.equal(got.cpu(), want_t), (case, M, N, K, lowp, terms, products, dtype)


def test_every_kind_of_launch_replays_from_a_captured_graph(gpu_device):
    """The reference compiles its UNet (unet.py:76-78), and compiled models are commonly replayed
    from device graphs: every launch path of the library -- LDS-tiled kernel, K split with its
    reduction pass, skinny split-K kernel, grouped launch, 16-bit tensors (weights re-laid into the
    workspace), prepared and gated weights, fp8 with the scale found on the device -- is captured
    once and replayed with fresh operand values; each replay must return the bits of the eager call
    on the same values.  The library records only kernels; the Python operator allocates its results
    (and the small fp8 exponent tensors) from the graph's pool during the capture, but no workspace:
    the eager warm-up has sized the per-device workspace that captured launches use, which the test
    checks by comparing the memory allocated during the capture with the size of the results."""
    from basedxl_amd import cascaded_lowp_matmul_grouped

    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(5)
    rn = lambda *s, dtype=torch.float32: torch.randn(*s, device=dev, generator=g).to(dtype)
    w = {
        "tile": rn(640, 640) * 0.02, "ksplit": rn(5120, 1280) * 0.02, "skinny": rn(2048, 640) * 0.02,
        "h": (rn(640, 640) * 0.02).half(), "glu": rn(640, 1280) * 0.02, "fp8": rn(320, 640) * 0.02,
        "kwave": rn(1280, 1280) * 0.02,     # with 2048 rows: one 64 x 160 tile per CU, K split over the waves of a workgroup
    }
    x = {"tile": rn(2048, 640), "ksplit": rn(1024, 5120), "skinny": rn(154, 2048), "h": rn(1024, 640).half(),
         "glu": rn(512, 640), "fp8": rn(512, 320), "kwave": rn(2048, 1280)}
    pw, pg, pk = PreparedWeight(w["tile"]), PreparedWeight(w["glu"], glu=True), PreparedWeight(w["kwave"])
    pk8 = PreparedWeight(w["kwave"], lowp="fp8", terms=3)
    p8 = PreparedWeight(w["fp8"], lowp="fp8", terms=3)   # (holds the weight's kept scale exponent too)

    def run():
        return [
            cascaded_lowp_matmul(x["tile"], w["tile"]),
            cascaded_lowp_matmul(x["ksplit"], w["ksplit"]),
            cascaded_lowp_matmul(x["skinny"], w["skinny"]),
            cascaded_lowp_matmul_grouped([x["tile"]] * 3, [w["tile"]] * 3)[2],
            cascaded_lowp_matmul_grouped([x["h"]] * 2, [w["h"]] * 2)[1],
            cascaded_lowp_matmul(x["tile"], pw),
            cascaded_lowp_matmul(x["glu"], pg),
            cascaded_lowp_matmul(x["fp8"], w["fp8"], lowp="fp8", terms=3),
            # the activation scale found inside the call (maxima, split, GEMM: all on the stream), weight raw / kept split
            cascaded_lowp_matmul(x["fp8"], w["fp8"], lowp="fp8", terms=3, b_exp=p8.exp),
            cascaded_lowp_matmul(x["fp8"], p8),
            cascaded_lowp_matmul(x["kwave"], w["kwave"]),      # both operands raw
            cascaded_lowp_matmul(x["kwave"], pk),              # raw rows through the LDS ring, weight as slots
            cascaded_lowp_matmul(x["kwave"], pk8),             # three fp8 terms: scale search, split of the rows, K over the waves
            # three fp16 terms on operand slots: both scale searches, both splits, K over the waves
            cascaded_lowp_matmul(x["kwave"], w["kwave"], lowp="fp16", terms=3),
        ]

    run()                                            # warm-up: workspaces exist before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                        # and on a side stream, as torch's capture recipe asks
    torch.cuda.current_stream().wait_stream(side)
    from basedxl_amd.cascaded_lowp_matmul import _workspaces
    ws_before = {k: v.data_ptr() for k, v in _workspaces.items()}
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    with torch.cuda.graph(graph):
        outs = run()
    grown = torch.cuda.memory_allocated() - before
    assert {k: v.data_ptr() for k, v in _workspaces.items()} == ws_before        # no workspace was created or replaced
    # what the capture allocated: the fourteen results plus the grouped launches' other results and the
    # two-int exponent tensor, each rounded up to the allocator's 512-byte granule -- far below the
    # 21 MB K-split workspace a capture-time allocation would add
    results = sum(o.numel() * o.element_size() for o in outs)
    others = 2 * x["tile"].shape[0] * 640 * 4 + x["h"].shape[0] * 640 * 2
    assert results <= grown <= results + others + 64 * 1024, (grown, results, others)
    for rep in range(3):
        for k in x:                                  # new values in the captured buffers
            x[k].copy_(rn(*x[k].shape, dtype=x[k].dtype) * (1.0 + rep))
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs]
        want = run()                                 # eager work between the replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), (rep, i)


def test_a_captured_graph_keeps_its_workspace_when_a_later_call_needs_a_larger_one(gpu_device):
    """A graph has the address of the K-split workspace baked into its launches.  An eager call with a
    larger problem makes the package replace that buffer; the old one must stay the package's, or the
    caching allocator hands it to the next tensor and the graph's replays write partial results into
    it.  Capture a small K-split GEMM, run a larger one eagerly, allocate tensors of the old buffer's
    size class, replay: the replay equals the eager result and none of the new tensors was touched."""
    from basedxl_amd.cascaded_lowp_matmul import _retired_capture_buffers, _workspaces

    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(9)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    # start from a capture buffer of exactly this problem's need, so that the next problem must grow it
    x1, w1 = rn(154, 2048), rn(2048, 640) * 0.02          # skinny: K split with partial results in the workspace
    need1 = _lib.lib().cascmm_workspace_bytes(154, 640, 2048, _lib.DT_F32, _lib.FMT_BF16, 2, _lib.PROD_TRI)
    assert need1 > 0
    saved = dict(_workspaces)
    _workspaces.clear()
    try:
        want1 = cascaded_lowp_matmul(x1, w1)              # eager warm-up sizes the capture buffer
        torch.cuda.synchronize()
        old = _workspaces[(0, "capture")]
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            out1 = cascaded_lowp_matmul(x1, w1)
        x2, w2 = rn(1024, 5120), rn(5120, 1280) * 0.02    # needs 4 x 1024 x 1280 x 4 bytes: far more
        cascaded_lowp_matmul(x2, w2)
        torch.cuda.synchronize()
        new = _workspaces[(0, "capture")]
        assert new.data_ptr() != old.data_ptr() and new.numel() > old.numel()
        old_ptr, old_bytes = old.data_ptr(), old.numel()
        del old
        # tensors of the old buffer's size: the allocator would reuse a freed block of that size at once
        canaries = [torch.full((old_bytes,), 0x5A, dtype=torch.uint8, device=dev) for _ in range(4)]
        assert all(c.data_ptr() != old_ptr for c in canaries)
        for rep in range(2):
            out1.fill_(float("nan"))
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(out1, want1), rep
            assert all(bool((c == 0x5A).all()) for c in canaries)
    finally:
        _workspaces.clear()
        _workspaces.update(saved)
    assert _retired_capture_buffers


def test_operands_beyond_two_gib_are_addressed_correctly(gpu_device):
    """The fast kernels address rows through 32-bit offsets from a per-tile buffer descriptor, the
    bounds-checked ones through 64-bit pointers: a left operand and a result of 2.3 GB each (row offsets
    cross 2^31 bytes inside the matrix) and a right operand of 2.4 GB must give the exact integer
    products in the rows on both sides of every boundary.  Operands are made on the device; only the
    sampled rows are recomputed (in float64, exact for these integers)."""
    from basedxl_amd import cascaded_lowp_matmul_grouped

    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(3)
    ints = lambda *shape, hi=7: torch.randint(-hi, hi + 1, shape, device=dev, generator=g).to(torch.float32)
    M, K, N = 900_000, 640, 640
    a, b, bias = ints(M, K), ints(K, N), ints(N)
    edge = (2 ** 31) // (K * 4)                    # first row that starts beyond 2^31 bytes
    rows = torch.tensor([0, 1, 255, 256, edge - 1, edge, edge + 1, edge + 300, M - 257, M - 2, M - 1], device=dev)
    want = a[rows].double() @ b.double() + bias.double()
    for kw in (dict(), dict(lowp="fp16", terms=3), dict(lowp="fp8", terms=3, products="full")):
        c = cascaded_lowp_matmul(a, b, bias=bias, **kw)
        assert torch.equal(c[rows].double(), want), kw
        del c
    c = cascaded_lowp_matmul(a, PreparedWeight(b), bias=bias)
    assert torch.equal(c[rows].double(), want)
    del c
    second = cascaded_lowp_matmul_grouped([a, a], [b, b.clone()])[1]
    assert torch.equal(second[rows].double(), want - bias.double())
    del second, a
    torch.cuda.empty_cache()
    # a right operand beyond 2 GiB takes the kernels with 64-bit addressing
    M, K, N = 96, 16384, 36864
    a, b = ints(M, K, hi=3), ints(K, N, hi=3)
    assert b.numel() * 4 > 2 ** 31
    assert torch.equal(cascaded_lowp_matmul(a, b).double(), a.double() @ b.double())
    b2 = b[:, :32000].contiguous()                 # just under 2 GiB: the fast split-K kernels for few rows
    assert torch.equal(cascaded_lowp_matmul(a, b2).double(), a.double() @ b2.double())
    del a, b, b2
    torch.cuda.empty_cache()


def test_two_streams_do_not_share_scratch(gpu_device):
    """The library keeps no state; the Python operator keeps one workspace (K-split partials, re-laid
    16-bit weights) and one scale-search scratch PER STREAM.  Launches that need them, issued
    alternately on two streams with different operands, must give what each gives alone."""
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(9)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)
    jobs = []
    for i in range(2):
        jobs.append(dict(x=rn(1024, 5120), w=rn(5120, 1280) * 0.02,                       # K split: partials in the workspace
                         xh=rn(1024, 640).half(), wh=(rn(640, 640) * 0.02).half(),        # 16-bit: weight re-laid into it
                         x8=rn(512, 320) * (1 + 10 * i), w8=rn(320, 640) * 0.02))         # fp8: scale found on the device

    def run(j):
        return [cascaded_lowp_matmul(j["x"], j["w"]), cascaded_lowp_matmul(j["xh"], j["wh"]),
                cascaded_lowp_matmul(j["x8"], j["w8"], lowp="fp8", terms=3)]

    alone = [run(j) for j in jobs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = [[], []]
    for rep in range(8):
        for i, s in enumerate(streams):
            with torch.cuda.stream(s):
                got[i].append(run(jobs[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for outs in got[i]:
            for a, b in zip(outs, alone[i]):
                assert torch.equal(a, b)
