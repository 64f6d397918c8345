"""The chained feed-forward path: operand slots of the left operand, the GEMM of slots by slots, the
gated store that writes slots, and the module that chains the two GEMMs of a feed-forward block.

CPU part: the patcher and the argument checks of the C entry points.  GPU part (through the C ABI):
* the stand-alone split of the left operand against the oracle's split, bit for bit, and its layout
  (the documented order of k) through a matrix whose entries name their own position;
* slots x slots on integer operands: exact, for whole and ragged tiles, K tails of every length modulo
  the four waves' stages, with and without bias, nothing written outside the result;
* the error bound against the oracle cascade at the feed-forward shape;
* the slot-writing gated store against the fp32 gated store of the same kernel: the slots are the split
  of exactly those fp32 values; and against exact integers with a gate that is a power of two;
* the chain against the oracle composed layer by layer (1.25x on both metrics against fp64).
"""
import numpy as np
import pytest
import torch

from basedxl_amd import _lib
from oracle import cascade as oc

DEV = "cuda:0"


def _stream():
    return torch.cuda.current_stream().cuda_stream


# ---------------------------------------------------------------------------------- CPU
class _GEGLU(torch.nn.Module):
    def __init__(self, d_in, d_out):
        super().__init__()
        self.proj = torch.nn.Linear(d_in, 2 * d_out)

    def forward(self, x):
        v, g = self.proj(x).chunk(2, dim=-1)
        return v * torch.nn.functional.gelu(g)


_GEGLU.__name__ = "GEGLU"


class _FF(torch.nn.Module):
    def __init__(self, p=0.0):
        super().__init__()
        self.net = torch.nn.ModuleList([_GEGLU(8, 32), torch.nn.Dropout(p), torch.nn.Linear(32, 8)])

    def forward(self, x):
        for m in self.net:
            x = m(x)
        return x


def test_patcher_replaces_only_inactive_dropout_feed_forwards():
    from basedxl_amd import BasedXLChainedFeedForward, chain_feed_forward_layers
    from basedxl_amd.unet import patch_unet
    from basedxl_amd.utils import BasedXLConfig

    model = torch.nn.ModuleDict({"a": _FF(), "b": _FF(0.5), "c": _FF(0.5).eval()})
    model["a"].train()
    model["b"].train()
    chain_feed_forward_layers(model)
    assert isinstance(model["a"].net[0], BasedXLChainedFeedForward)
    assert isinstance(model["a"].net[1], torch.nn.Identity) and isinstance(model["a"].net[2], torch.nn.Identity)
    assert type(model["b"].net[0]).__name__ == "GEGLU" and isinstance(model["b"].net[2], torch.nn.Linear)   # live dropout
    assert isinstance(model["c"].net[0], BasedXLChainedFeedForward)                                         # eval(): inactive
    ff = model["a"].net[0]
    assert (ff.in_features, ff.inner, ff.out_features) == (8, 32, 8) and ff.chainable
    assert ff.geglu.weight.shape == (8, 64) and ff.linear.weight.shape == (32, 8)
    # other cascades keep the module (it falls back layer by layer) but never chain
    other = _FF()
    chain_feed_forward_layers(other, lowp="fp16", terms=3)
    assert not other.net[0].chainable
    # the install hook: chain first, then the Linear walk finds nothing left inside the block
    m2 = torch.nn.ModuleDict({"ff": _FF(), "lin": torch.nn.Linear(4, 4)})
    patch_unet(m2, BasedXLConfig(fp16_acc_matmul=True, chain_ffn=True))
    assert isinstance(m2["ff"].net[0], BasedXLChainedFeedForward) and type(m2["lin"]).__name__ == "BasedXLLowPLinear"
    m3 = torch.nn.ModuleDict({"ff": _FF()})
    patch_unet(m3, BasedXLConfig(fp16_acc_matmul=True))
    assert type(m3["ff"].net[0]).__name__ == "GEGLU" and type(m3["ff"].net[2]).__name__ == "BasedXLLowPLinear"


def test_chained_entry_points_check_their_arguments():
    l = _lib.lib()
    assert l.cascmm_left_slots_bytes(2048, 5120) == 4 * 2048 * 5120
    assert l.cascmm_left_slots_bytes(64, 40) == 0 and l.cascmm_left_slots_bytes(0, 64) == 0     # K % 16, empty
    assert l.cascmm_left_slots_bytes(2 ** 40, 2 ** 30) == 0                                      # overflow
    assert l.cascmm_chained_supported(2048, 1280, 5120) == 1 and l.cascmm_chained_supported(100, 84, 80) == 1
    assert l.cascmm_chained_supported(64, 160, 48) == 1 and l.cascmm_chained_supported(64, 160, 72) == 0   # K % 16
    assert l.cascmm_chained_supported(1 << 20, 160, 1 << 12) == 0                                # slots beyond 2 GiB
    p = 0x100000
    assert l.cascmm_prepare_left(p, 64, 40, 40, p, 1 << 20, None) == -2
    assert l.cascmm_prepare_left(p, 64, 64, 64, None, 1 << 20, None) == -1
    assert l.cascmm_prepare_left(p + 4, 64, 64, 64, p, 1 << 20, None) == -6
    assert l.cascmm_prepare_left(p, 64, 64, 66, p, 1 << 20, None) == -6                          # rows not 16-byte aligned
    assert l.cascmm_prepare_left(p, 64, 64, 64, p, 100, None) == -5
    assert l.cascmm_prepare_left(p, 0, 64, 64, None, 0, None) == 0
    assert l.cascmm_prepare_weight_chained(p, 72, 64, 64, p, 1 << 20, None) == -2
    assert l.cascmm_prepare_weight_chained(p, 64, 64, 64, p, 100, None) == -5
    assert l.cascmm_gemm_chained(p, p, p, None, 64, 160, 40, 160, None) == -4
    assert l.cascmm_gemm_chained(p, p, p, None, 64, 160, 64, 100, None) == -2
    assert l.cascmm_gemm_chained(None, p, p, None, 64, 160, 64, 160, None) == -1
    assert l.cascmm_gemm_chained(p, p + 8, p, None, 64, 160, 64, 160, None) == -6
    assert l.cascmm_gemm_chained(p, p, p, None, 0, 160, 64, 160, None) == 0
    assert l.cascmm_gemm_glu_chained(p, p, 0, p, 1 << 30, None, 256, 330, 64, 64, 330, None) == -2      # N % 64
    assert l.cascmm_gemm_glu_chained(p, p, 0, p, 100, None, 256, 640, 64, 64, 640, None) == -5          # slots too small
    assert l.cascmm_gemm_glu_chained(p, p, 0, None, 1 << 30, None, 256, 640, 64, 64, 640, None) == -1
    assert l.cascmm_gemm_glu_chained(p, p, 0, p, 1 << 30, None, 128, 640, 64, 64, 640, None) == -4      # no kernel: rows % 256


# ---------------------------------------------------------------------------------- GPU
def _left_slots(a):
    from basedxl_amd import LeftSlots
    return LeftSlots.from_tensor(a)


@pytest.mark.gpu
def test_left_slots_are_the_oracle_split_in_the_documented_order(gpu_device):
    g = torch.Generator().manual_seed(3)
    M, K = 100, 80
    a = torch.randn(M, K, generator=g)
    a[0, :8] = torch.tensor([0.0, -0.0, 1e-39, 3.0e38, 1.00390625, -1.00390625, 1.01171875, 2.0 ** -126])   # zeros, subnormal, ties
    a[1, :4] = torch.tensor([float("inf"), float("-inf"), float("nan"), 1.0])
    sl = _left_slots(a.to(DEV))
    t = sl.terms().cpu()
    want, _ = oc.split_terms(a, "bf16", 2)
    for i in range(2):
        assert torch.equal(t[i].view(torch.int32), want[i].view(torch.int32)) or \
            torch.equal(torch.nan_to_num(t[i], nan=7.0), torch.nan_to_num(want[i], nan=7.0)), i
    # the raw layout, decoded by hand: slot (term, kg, m), position p holds k = 16 (kg / 2) + 8 (p / 4) + 4 (kg % 2) + p % 4
    pos = torch.arange(M * K, dtype=torch.float32).reshape(M, K) % 251        # bf16-exact values that name (m, k) up to 251
    raw = _left_slots(pos.to(DEV)).slots.cpu().view(torch.bfloat16).view(2, K // 8, M, 8).float()
    for kg, m, p in [(0, 0, 0), (1, 5, 2), (3, 99, 7), (9, 42, 4), (6, 17, 3)]:
        k = 16 * (kg // 2) + 8 * (p // 4) + 4 * (kg % 2) + p % 4
        assert raw[0, kg, m, p] == pos[m, k] and raw[1, kg, m, p] == 0


CHAIN_SHAPES = [(64, 16, 160), (33, 48, 32), (64, 64, 160), (128, 256, 320), (100, 80, 96), (70, 112, 36), (257, 144, 164), (256, 272, 480), (2048, 5120, 1280),
                (512, 2560, 640), (30, 1040, 20)]


@pytest.mark.gpu
@pytest.mark.parametrize("shape", CHAIN_SHAPES)
def test_slots_by_slots_integer_exact_through_the_c_abi(gpu_device, shape):
    M, K, N = shape
    print("chained int-exact", shape, flush=True)
    l = _lib.lib()
    rng = np.random.default_rng(M + K + N)
    hi = 100 if K <= 256 else (40 if K <= 1280 else 20)
    a = rng.integers(-hi, hi + 1, size=(M, K))
    b = rng.integers(-hi, hi + 1, size=(K, N))
    bias = rng.integers(-50, 51, size=(N,))
    want = a @ b
    assert np.abs(want).max() + 50 < 2 ** 24
    ad, bd = torch.tensor(a, dtype=torch.float32, device=DEV), torch.tensor(b, dtype=torch.float32, device=DEV)
    biasd = torch.tensor(bias, dtype=torch.float32, device=DEV)
    asl = torch.empty(l.cascmm_left_slots_bytes(M, K), dtype=torch.uint8, device=DEV)
    bsl = torch.empty(l.cascmm_prepared_bytes(K, N, _lib.FMT_BF16, 2), dtype=torch.uint8, device=DEV)
    assert l.cascmm_prepare_left(ad.data_ptr(), M, K, K, asl.data_ptr(), asl.numel(), _stream()) == 0
    assert l.cascmm_prepare_weight_chained(bd.data_ptr(), K, N, N, bsl.data_ptr(), bsl.numel(), _stream()) == 0
    for with_bias in (False, True):
        ldc = N + 3
        c = torch.full((M + 1, ldc), -77.0, device=DEV)
        st = l.cascmm_gemm_chained(asl.data_ptr(), bsl.data_ptr(), c.data_ptr(), biasd.data_ptr() if with_bias else None, M, N, K, ldc,
                                   _stream())
        assert st == 0, l.cascmm_strerror(st)
        got = c.cpu().numpy()
        assert np.array_equal(got[:M, :N].astype(np.int64), want + (bias if with_bias else 0)), (shape, with_bias)
        assert (got[:M, N:] == -77.0).all() and (got[M] == -77.0).all()            # nothing outside the result


@pytest.mark.gpu
def test_slots_by_slots_meets_the_bound_at_the_feed_forward_shape_and_repeats(gpu_device):
    from basedxl_amd import ChainedWeight, LeftSlots, cascaded_lowp_matmul_chained
    M, K, N = 2048, 5120, 1280
    a, b = oc.make_operands(M, K, N, seed=21, w_std=0.02)
    sl, w = LeftSlots.from_tensor(a.to(DEV)), ChainedWeight(b.to(DEV))
    bias = torch.randn(N)
    c = cascaded_lowp_matmul_chained(sl, w, bias=bias.to(DEV))
    c2 = cascaded_lowp_matmul_chained(sl, w, bias=bias.to(DEV))
    assert torch.equal(c, c2)                                        # fixed order of summation: bit-reproducible
    exp = oc.fp64_matmul(a, b) + bias.double()
    ek = oc.error_metrics(c.cpu(), exp)
    eo = oc.error_metrics(oc.cascade_matmul_ref(a, b) + bias, exp)
    print("chained W2", ek["rel_fro"], eo["rel_fro"], ek["max_abs"], eo["max_abs"], flush=True)
    assert ek["rel_fro"] <= 1.25 * eo["rel_fro"] and ek["max_abs"] <= 1.25 * eo["max_abs"]


def _glu_chained(x, w, bias, prepared):
    """(fp32 gated result of the same kernel, slots written by the slot store) through the C ABI"""
    from basedxl_amd import PreparedWeight
    l = _lib.lib()
    M, K = x.shape
    N = w.shape[1]
    inner = N // 2
    y = torch.empty(M, inner, device=DEV)
    slots = torch.full((l.cascmm_left_slots_bytes(M, inner),), 0xEE, dtype=torch.uint8, device=DEV)
    bptr = bias.data_ptr() if bias is not None else None
    # the fp32 store is forced onto the large-tile kernel, the only one with the slot store: another tile
    # would add the same products in another order
    big = _lib.variant_names().index("t256x320x32_w512_bf16x2_tri" + ("_bpre" if prepared else ""))
    if prepared:
        pw = PreparedWeight(w, glu=True)
        import ctypes
        arr = ctypes.c_void_p * 1
        st = l.cascmm_gemm_prepared_glu(1, arr(x.data_ptr()), arr(pw.slots.data_ptr()), arr(y.data_ptr()), arr(bptr) if bias is not None else None,
                                        M, N, K, K, inner, _lib.DT_F32, _lib.FMT_BF16, 2, _lib.PROD_TRI, None, _stream(), big)
        assert st == 0, l.cascmm_strerror(st)
        st = l.cascmm_gemm_glu_chained(x.data_ptr(), pw.slots.data_ptr(), 1, slots.data_ptr(), slots.numel(), bptr, M, N, K, K, N, _stream())
    else:
        st = l.cascmm_gemm_glu(x.data_ptr(), w.data_ptr(), y.data_ptr(), bptr, M, N, K, K, N, inner, _lib.DT_F32, _lib.FMT_BF16, 2,
                               _lib.PROD_TRI, _stream(), big)
        assert st == 0, l.cascmm_strerror(st)
        st = l.cascmm_gemm_glu_chained(x.data_ptr(), w.data_ptr(), 0, slots.data_ptr(), slots.numel(), bptr, M, N, K, K, N, _stream())
    assert st == 0, l.cascmm_strerror(st)
    return y, slots


@pytest.mark.gpu
@pytest.mark.parametrize("prepared", [False, True])
@pytest.mark.parametrize("M,K,N,with_bias", [(256, 64, 640, True), (512, 96, 1280, False), (2048, 1280, 10240, True)])
def test_slot_store_writes_the_split_of_the_fp32_gated_store(gpu_device, M, K, N, with_bias, prepared):
    """Same kernel, same accumulators, same gate: the slots must be the two-term split of exactly the
    fp32 values the fp32 store writes (pinned by the stand-alone split, itself pinned by the oracle)."""
    print("slot store", M, K, N, with_bias, prepared, flush=True)
    l = _lib.lib()
    g = torch.Generator(device=DEV).manual_seed(M + N)
    x = torch.randn(M, K, device=DEV, generator=g)
    w = torch.randn(K, N, device=DEV, generator=g) * 0.05
    bias = torch.randn(N, device=DEV, generator=g) if with_bias else None
    y, slots = _glu_chained(x, w, bias, prepared)
    want = torch.empty_like(slots)
    assert l.cascmm_prepare_left(y.data_ptr(), M, N // 2, N // 2, want.data_ptr(), want.numel(), _stream()) == 0
    assert torch.equal(slots, want)


@pytest.mark.gpu
def test_slot_store_on_integers_with_a_power_of_two_gate(gpu_device):
    """Gate columns of the weight zero and a gate bias of 8: gelu(8) is 8 exactly in this
    implementation's arithmetic (0.5 x 8 x 2), so the result is 8 (x . w_value + b_value), an integer: every slot is known
    exactly, whatever the order of the accumulation."""
    from basedxl_amd import LeftSlots
    l = _lib.lib()
    M, K, N = 512, 96, 1280
    inner = N // 2
    rng = np.random.default_rng(5)
    x = rng.integers(-60, 61, size=(M, K))
    wv = rng.integers(-60, 61, size=(K, inner))
    bv = rng.integers(-99, 100, size=(inner,))
    w = np.concatenate([wv, np.zeros((K, inner), dtype=np.int64)], axis=1)
    bias = np.concatenate([bv, np.full(inner, 8)])
    want = 8 * (x @ wv + bv)
    assert np.abs(want).max() < 2 ** 24
    xd = torch.tensor(x, dtype=torch.float32, device=DEV)
    wd = torch.tensor(w, dtype=torch.float32, device=DEV)
    bd = torch.tensor(bias, dtype=torch.float32, device=DEV)
    slots = LeftSlots.empty((M,), inner, DEV)
    st = l.cascmm_gemm_glu_chained(xd.data_ptr(), wd.data_ptr(), 0, slots.slots.data_ptr(), slots.slots.numel(), bd.data_ptr(), M, N, K, K, N,
                                   _stream())
    assert st == 0, l.cascmm_strerror(st)
    t = slots.terms().cpu()
    wt, _ = oc.split_terms(torch.tensor(want, dtype=torch.float32), "bf16", 2)
    assert torch.equal(t[0], wt[0]) and torch.equal(t[1], wt[1])


@pytest.mark.gpu
@pytest.mark.parametrize("prepared", [False, True])
def test_chain_against_the_oracle_composed_layer_by_layer(gpu_device, prepared):
    """configs[2] of the baseline as the model runs it: X [2048, 1280] -> W1 [1280, 10240] -> gate ->
    W2 [5120, 1280].  Ground truth: the same composition in fp64.  The oracle: its gated projection
    followed by its cascade on that result.  1.25x on both metrics."""
    from basedxl_amd import ChainedWeight, PreparedWeight, cascaded_lowp_matmul_chained, cascaded_lowp_matmul_glu_chained
    M, K, inner, out = 2048, 1280, 5120, 1280
    g = torch.Generator().manual_seed(11)
    x = torch.randn(M, K, generator=g)
    w1 = torch.randn(K, 2 * inner, generator=g) * 0.02
    b1 = torch.randn(2 * inner, generator=g) * 0.1
    w2 = torch.randn(inner, out, generator=g) * 0.02
    b2 = torch.randn(out, generator=g) * 0.1
    xd, w1d, w2d = x.to(DEV), w1.to(DEV), w2.to(DEV)
    slots = cascaded_lowp_matmul_glu_chained(xd, PreparedWeight(w1d, glu=True) if prepared else w1d, bias=b1.to(DEV))
    y = cascaded_lowp_matmul_chained(slots, ChainedWeight(w2d), bias=b2.to(DEV)).cpu()
    h = x.double() @ w1.double() + b1.double()
    gate = h[:, inner:]
    mid = h[:, :inner] * (0.5 * gate * (1.0 + torch.erf(gate / 2.0 ** 0.5)))
    exp = mid @ w2.double() + b2.double()
    ref = oc.cascade_matmul_ref(oc.gated_projection_ref(x, w1, b1), w2) + b2
    ek, eo = oc.error_metrics(y, exp), oc.error_metrics(ref, exp)
    print("chain", prepared, ek["rel_fro"], eo["rel_fro"], ek["max_abs"], eo["max_abs"], flush=True)
    assert ek["rel_fro"] <= 1.25 * eo["rel_fro"] and ek["max_abs"] <= 1.25 * eo["max_abs"]
    # the intermediate result: what the slots hold is the oracle's gated projection to the accuracy of its two terms
    mid_ref = oc.gated_projection_ref(x, w1, b1)
    em, er = oc.error_metrics(slots.to_dense().cpu(), mid), oc.error_metrics(mid_ref, mid)
    assert em["rel_fro"] <= 1.25 * er["rel_fro"] + 2.0 ** -16


@pytest.mark.gpu
@pytest.mark.parametrize("prepared", [False, True])
def test_chained_feed_forward_module_and_its_fallback(gpu_device, prepared):
    from basedxl_amd import BasedXLChainedFeedForward
    torch.manual_seed(13)
    proj, out = torch.nn.Linear(640, 2 * 2560), torch.nn.Linear(2560, 640)
    ff = BasedXLChainedFeedForward(proj, out, prepared=prepared).to(DEV)
    ff.geglu.weight, ff.geglu.bias = ff.geglu.weight.to(DEV), ff.geglu.bias.to(DEV)
    ff.linear.weight, ff.linear.bias = ff.linear.weight.to(DEV), ff.linear.bias.to(DEV)
    x = torch.randn(2, 2048, 640, device=DEV)
    y = ff(x)
    assert ff.chained_calls == 1 and y.shape == (2, 2048, 640)
    want = ff.linear(ff.geglu(x))                        # the same layers one by one
    torch.testing.assert_close(y, want, rtol=0, atol=2e-4)
    xr = x.cpu().reshape(-1, 640)
    ref = oc.cascade_matmul_ref(oc.gated_projection_ref(xr, ff.geglu.weight.cpu(), ff.geglu.bias.cpu()), ff.linear.weight.cpu()) + ff.linear.bias.cpu()
    h = xr.double() @ ff.geglu.weight.cpu().double() + ff.geglu.bias.cpu().double()
    gate = h[:, 2560:]
    exp = (h[:, :2560] * (0.5 * gate * (1.0 + torch.erf(gate / 2.0 ** 0.5)))) @ ff.linear.weight.cpu().double() + ff.linear.bias.cpu().double()
    ek, eo = oc.error_metrics(y.cpu().reshape(-1, 640), exp), oc.error_metrics(ref, exp)
    assert ek["rel_fro"] <= 1.25 * eo["rel_fro"] and ek["max_abs"] <= 1.25 * eo["max_abs"]
    # rows that are no multiple of 256: layer by layer
    y2 = ff(x[:, :100])
    assert ff.chained_calls == 1
    torch.testing.assert_close(y2, want[:, :100], rtol=0, atol=2e-4)
    # 1024 rows make 64 large tiles for 256 CUs: the cost estimates prefer a smaller tile and a gate pass, so
    # the block runs layer by layer although the chain would take the shape
    y3 = ff(x[:, :512])
    assert ff.chained_calls == 1
    torch.testing.assert_close(y3, want[:, :512], rtol=0, atol=2e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("form", ["raw x raw", "raw x slots", "raw x slots, 64 x 80 tile", "slots x slots"])
def test_non_finite_operands_poison_their_row_or_column_only_on_the_k_over_waves_kernels(gpu_device, form):
    """As for the other kernels: a NaN or an infinity in A spoils exactly its row, one in B exactly its
    column.  K = 96 leaves the fourth wave of a workgroup without a stage of its own: it multiplies the
    problem's first columns of A (where the infinity sits) by zeros, which must not reach any other row."""
    from basedxl_amd import ChainedWeight, LeftSlots, PreparedWeight, cascaded_lowp_matmul, cascaded_lowp_matmul_chained
    names = _lib.variant_names()
    g = torch.Generator().manual_seed(23)
    a = torch.randn(100, 96, generator=g)
    b = torch.randn(96, 84, generator=g) * 0.02

    def run(a_, b_):
        ad, bd = a_.to(DEV), b_.to(DEV)
        if form == "raw x raw":
            return cascaded_lowp_matmul(ad, bd, variant=names.index("k64x160x16_wk4_bf16x2_tri")).cpu()
        if form == "raw x slots":
            return cascaded_lowp_matmul(ad, PreparedWeight(bd, lowp="bf16", terms=2), variant=names.index("k64x160x16_wk4_bf16x2_tri_bpre")).cpu()
        if form == "raw x slots, 64 x 80 tile":     # (K = 96: three 32-k stages, again none for the fourth wave)
            return cascaded_lowp_matmul(ad, PreparedWeight(bd, lowp="bf16", terms=2), variant=names.index("k64x80x32_wk4_bf16x2_tri_bpre")).cpu()
        return cascaded_lowp_matmul_chained(LeftSlots.from_tensor(ad), ChainedWeight(bd)).cpu()

    clean = run(a, b)
    a2, b2 = a.clone(), b.clone()
    a2[5, 40] = float("nan")
    a2[70, 3] = float("inf")
    b2[77, 9] = -float("inf")
    got = run(a2, b2)
    want = oc.cascade_matmul_ref(a2, b2, "bf16", 2, "tri")
    bad = torch.zeros(100, 84, dtype=torch.bool)
    bad[5, :] = bad[70, :] = True
    bad[:, 9] = True
    assert torch.isnan(got[bad]).all() and torch.isnan(want[bad]).all()
    assert torch.equal(got[~bad], clean[~bad])
    # what lies between the rows of a strided left operand is never multiplied, not even by zeros
    padded = torch.full((100, 104), float("nan"))
    padded[:, :96] = a
    pd = padded.to(DEV)[:, :96]
    bd = b.to(DEV)
    if form == "raw x raw":
        again = cascaded_lowp_matmul(pd, bd, variant=names.index("k64x160x16_wk4_bf16x2_tri"))
    elif form.startswith("raw x slots"):
        name = "k64x80x32_wk4_bf16x2_tri_bpre" if "64 x 80" in form else "k64x160x16_wk4_bf16x2_tri_bpre"
        again = cascaded_lowp_matmul(pd, PreparedWeight(bd, lowp="bf16", terms=2), variant=names.index(name))
    else:
        again = cascaded_lowp_matmul_chained(LeftSlots.from_tensor(pd), ChainedWeight(bd))
    assert torch.equal(again.cpu(), clean)


@pytest.mark.gpu
def test_chain_replays_from_a_captured_graph(gpu_device):
    from basedxl_amd import ChainedWeight, LeftSlots, cascaded_lowp_matmul_chained, cascaded_lowp_matmul_glu_chained
    g = torch.Generator(device=DEV).manual_seed(17)
    x = torch.randn(512, 320, device=DEV, generator=g)
    w1 = torch.randn(320, 2560, device=DEV, generator=g) * 0.05
    w2 = ChainedWeight(torch.randn(1280, 320, device=DEV, generator=g) * 0.05)
    slots = LeftSlots.empty((512,), 1280, DEV)
    out = torch.empty(512, 320, device=DEV)

    def run():
        cascaded_lowp_matmul_glu_chained(x, w1, out=slots)
        return cascaded_lowp_matmul_chained(slots, w2, out=out)

    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for rep in range(3):
        x.copy_(torch.randn(512, 320, device=DEV, generator=g) * (1.0 + rep))
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = run().clone()
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


@pytest.mark.gpu
@pytest.mark.parametrize("M,K,N", [(8192, 2560, 640), (2048, 1280, 1280)])
def test_k_over_waves_kernels_repeat_bit_for_bit_when_the_launch_has_several_rounds(gpu_device, M, K, N):
    """The three forms of the kernel (both operands raw, right operand prepared, both as slots) read the
    left operand's fragments from LDS that loads fill asynchronously; the waits that cover those loads are
    written by hand.  A launch of two rounds of workgroups with a long K keeps the memory system busy
    enough for a missing wait to show as results that change from launch to launch: forty launches must
    give the bits of the first, and the first must meet the error bound."""
    from basedxl_amd import (ChainedWeight, LeftSlots, PreparedWeight, cascaded_lowp_matmul, cascaded_lowp_matmul_chained)
    names = _lib.variant_names()
    g = torch.Generator(device=DEV).manual_seed(M + N)
    a = torch.randn(M, K, device=DEV, generator=g)
    b = torch.randn(K, N, device=DEV, generator=g) * 0.02
    ref = a.double() @ b.double()
    pw, sl, cw = PreparedWeight(b), LeftSlots.from_tensor(a), ChainedWeight(b)
    p8 = PreparedWeight(b, lowp="fp8", terms=3)
    forms = {"raw": lambda: cascaded_lowp_matmul(a, b, variant=names.index("k64x160x16_wk4_bf16x2_tri")),
             "prepared": lambda: cascaded_lowp_matmul(a, pw, variant=names.index("k64x160x16_wk4_bf16x2_tri_bpre")),
             "prepared, 64 x 80 tile": lambda: cascaded_lowp_matmul(a, pw, variant=names.index("k64x80x32_wk4_bf16x2_tri_bpre")),
             "slots": lambda: cascaded_lowp_matmul_chained(sl, cw),
             # the fp8-rate kernel of the same design (all loads into registers: the compiler's own waits)
             "fp8 slots": lambda: cascaded_lowp_matmul(a, p8, variant=names.index("k64x160x64_f8k64wk4_fp8x3_tri_bpre"))}
    for label, fn in forms.items():
        print("repeat", M, K, N, label, flush=True)
        first = fn()
        rel = float((first.double() - ref).norm() / ref.norm())
        assert rel < (4.5e-5 if label.startswith("fp8") else 6e-6), (label, rel)   # the cascades' 3.5e-5 / 4.4e-6, not a wrong tile's 1e-3
        for rep in range(40):
            assert torch.equal(fn(), first), (label, rep)
