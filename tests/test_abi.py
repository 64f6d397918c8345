"""CPU-only checks of the C ABI: the library loads, exports everything the header declares,
and its argument validation (which runs before any GPU work) returns the documented codes."""
import ctypes
import os
import re

import pytest

from basedxl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "cascmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cascmm_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared()
    assert "cascmm_gemm" in names and len(names) >= 8
    handle = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(handle, n), f"{n} declared in include/cascmm.h but not exported"
    assert sorted(_lib.SIGNATURES) == names


def test_version_and_strerror():
    l = _lib.lib()
    assert l.cascmm_version() == 100
    assert l.cascmm_strerror(0) == b"ok"
    for code in range(-9, 0):
        assert l.cascmm_strerror(code) not in (None, b"unknown status")
    assert l.cascmm_strerror(-99) == b"unknown status"


def test_variant_table():
    names = _lib.variant_names()
    assert len(names) == len(set(names)) > 10
    assert any("bf16x2_tri" in n for n in names)
    assert _lib.lib().cascmm_variant_name(-1) is None
    assert _lib.lib().cascmm_variant_name(len(names)) is None


def test_every_variant_names_its_kernel_and_the_kernel_has_a_listing():
    """`cascmm_variant_kernel` gives the device function's symbol without a GPU; the listing that
    `dump_ptx=True` writes (the counterpart of the reference's PTX dump,
    basedxl/triton/cascaded_lowp_matmul.py:170-171) is that function's gfx950 assembly."""
    from basedxl_amd.cascaded_lowp_matmul import kernel_listing
    l = _lib.lib()
    names = _lib.variant_names()
    kinds = {"_w512_": "cascmm_w512_kernel", "_wavek_": "cascmm_wavek_kernel", "_f8k64_": "cascmm_f8k64_kernel"}
    for i, n in enumerate(names):
        sym = l.cascmm_variant_kernel(i)
        assert sym and sym.decode().startswith("_ZN6cascmm"), n
        for tag, fn in kinds.items():
            assert (tag in n) == (fn in sym.decode()), (n, sym)
    assert l.cascmm_variant_kernel(-1) is None and l.cascmm_variant_kernel(len(names)) is None
    if not os.path.exists(os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")):
        pytest.skip("the listing needs hipcc")
    v = names.index("t256x320x32_w512_bf16x2_tri")
    text = kernel_listing(v)
    assert text.startswith("// gfx950 kernel variant: t256x320x32_w512_bf16x2_tri\n// kernel: _ZN6cascmm18cascmm_w512_kernelILi0E")
    assert "no listing" not in text and "s_endpgm" in text
    assert text.count("v_mfma_f32_32x32x16_bf16") == 120          # 20 blocks x 3 products x 2 k halves of a stage
    vgprs = int(re.search(r"\.amdhsa_next_free_vgpr (\d+)", text).group(1))
    assert 448 < vgprs <= 512                                        # (nearly) the whole register file of a SIMD: one wave on it
    assert ".amdhsa_private_segment_fixed_size 0\n" in text          # and nothing spilled to scratch memory


def _gemm(M, N, K, lda=None, ldb=None, ldc=None, dtype=0, fmt=0, terms=2, products=0, A=8, B=8, C=8):
    l = _lib.lib()
    return l.cascmm_gemm(A, B, C, None, M, N, K, lda if lda is not None else K, ldb if ldb is not None else N,
                         ldc if ldc is not None else N, dtype, fmt, terms, products, None, None, 0, None)


def test_argument_validation_codes():
    # all of these return before touching the device
    assert _gemm(-1, 4, 4) == -2
    assert _gemm(4, 4, 4, lda=3) == -2
    assert _gemm(4, 4, 4, ldb=3) == -2
    assert _gemm(4, 4, 4, ldc=3) == -2
    assert _gemm(4, 4, 4, dtype=7) == -3
    assert _gemm(4, 4, 4, fmt=9) == -4
    assert _gemm(4, 4, 4, terms=0) == -4
    assert _gemm(4, 4, 4, terms=4) == -4
    assert _gemm(4, 4, 4, products=2) == -4
    assert _gemm(2 ** 31, 4, 4) == -9
    assert _gemm(4, 4, 4, C=None) == -1
    assert _gemm(4, 4, 4, A=None) == -1
    assert _gemm(4, 4, 4, A=6) == -6
    # empty problems are fine and launch nothing
    assert _gemm(0, 4, 4, A=None, B=None, C=None) == 0
    assert _gemm(4, 0, 4, A=None, B=None, C=None) == 0


def test_select_variant_prefers_sensible_tiles():
    l = _lib.lib()
    names = _lib.variant_names()
    v = l.cascmm_select_variant(4096, 640, 640, 640, 640, 640, 0, 0, 2, 0)
    assert v >= 0 and "bf16x2_tri" in names[v]
    # K not a multiple of 8 must take a bounds-checked kernel
    v = l.cascmm_select_variant(10, 30, 20, 20, 30, 30, 0, 0, 2, 0)
    assert v >= 0 and "generic" in names[v]
    v = l.cascmm_select_variant(128, 128, 128, 128, 128, 128, 0, 1, 3, 0)
    assert v >= 0 and "fp16x3_tri" in names[v]
    assert l.cascmm_select_variant(4, 4, 4, 4, 4, 4, 0, 5, 2, 0) == -4


def test_baseline_shapes_get_the_kernels_the_measurements_name():
    """The kernels behind the committed profiles and the bench's traffic figures: if the cost model
    drifts to another tile for these shapes, those figures describe the wrong kernel."""
    l = _lib.lib()
    names = _lib.variant_names()
    pick = lambda M, K, N: names[l.cascmm_select_variant(M, N, K, K, N, N, 0, 0, 2, 0) & 0xFFFF]
    assert pick(2048, 1280, 10240) == "t256x320x32_w512_bf16x2_tri"               # cfg3, first GEMM
    assert pick(154, 2048, 1280) == "t32x32x32_wavek_bf16x2_tri" and pick(154, 2048, 640) == "t32x32x32_wavek_bf16x2_tri"   # cfg4
    assert pick(16, 2816, 1280).startswith("skinny")   # few tiles, deep K: split over workgroups
    grouped = names[l.cascmm_select_variant_grouped(3, 4096, 640, 640, 640, 640, 640, 0, 0, 2, 0) & 0xFFFF]
    assert grouped == "t256x128x32_w4x1x1_d2_bf16x2_tri"                           # cfg2, to_q / to_k / to_v
    assert pick(4096, 640, 640) == "t64x160x64_w2x1x2_d2_p8_bf16x2_tri"            # cfg2, to_out
    assert pick(8192, 640, 5120) == "t256x320x32_w512_bf16x2_tri"                  # cfg5: the 640-stage feed-forward, whole large tiles
    # one 64 x 160 tile per CU and K split over the waves: cfg3's second GEMM and the 1280-channel projections
    assert pick(2048, 5120, 1280) == "k64x160x16_wk4_bf16x2_tri" and pick(2048, 1280, 1280) == "k64x160x16_wk4_bf16x2_tri"
    # weights kept split, 1024 rows (one GPU's half-latent share): 64 x 160 tiles would occupy half the chip; the 64 x 80
    # tile of the same design
    pickp = lambda M, K, N: names[l.cascmm_select_variant_prepared(1, M, N, K, K, N, 0, 0, 2, 0) & 0xFFFF]
    assert pickp(1024, 1280, 1280) == "k64x80x32_wk4_bf16x2_tri_bpre" and pickp(2048, 1280, 1280) == "k64x160x16_wk4_bf16x2_tri_bpre"
    # three fp8 terms, weights kept split: the tile of the fp8-rate kernel that a sweep over the UNet's
    # shapes measured faster (256 rows where the tiles fill the chip, 128 rows where they would not)
    pick8 = lambda M, K, N: names[l.cascmm_select_variant_prepared(1, M, N, K, K, N, 0, 2, 3, 0) & 0xFFFF]
    for M, K, N in [(2048, 1280, 10240), (8192, 640, 5120), (8192, 640, 1280), (4096, 640, 5120), (1024, 1280, 10240)]:
        assert pick8(M, K, N) == "t256x160x64_f8k64_fp8x3_tri_bpre", (M, K, N)
    for M, K, N in [(2048, 1280, 2560), (8192, 640, 640), (8192, 2560, 640), (1024, 5120, 1280), (154, 2048, 2560)]:
        assert pick8(M, K, N) == "t128x160x64_f8k64_fp8x3_tri_bpre", (M, K, N)
    # ... and where 64 x 160 tiles make about one per CU, the kernel that splits K over the waves of a workgroup
    for M, K, N in [(2048, 1280, 1280), (2048, 5120, 1280), (4096, 640, 640), (4096, 2560, 640)]:
        assert pick8(M, K, N) == "k64x160x64_f8k64wk4_fp8x3_tri_bpre", (M, K, N)
    # three fp16 terms (cfg3 names them): both operands split into pre-scaled slots first; the 256 x 160 tile where
    # the tiles fill the chip several times over, K over the waves of a workgroup where there is about one tile per CU
    pick16 = lambda M, K, N: names[l.cascmm_select_variant(M, N, K, K, N, N, 0, 1, 3, 0) & 0xFFFF]
    assert pick16(2048, 1280, 10240) == "t256x160x32_f16k_fp16x3_tri"
    assert pick16(2048, 5120, 1280) == "k64x160x32_f16wk4_fp16x3_tri" and pick16(2048, 1280, 1280) == "k64x160x32_f16wk4_fp16x3_tri"
    assert "f16" not in pick16(128, 128, 128).split("_")[1]   # a small problem is not worth the passes
    pickp = lambda M, K, N: names[l.cascmm_select_variant_prepared(1, M, N, K, K, N, 0, 0, 2, 0) & 0xFFFF]
    assert pickp(2048, 1280, 10240) == "t256x320x32_w512_bf16x2_tri_bpre"
    assert pickp(2048, 5120, 1280) == "k64x160x16_wk4_bf16x2_tri_bpre" and pickp(2048, 1280, 1280) == "k64x160x16_wk4_bf16x2_tri_bpre"


def test_counter_traffic_table_names_real_kernels_and_summaries():
    """The table behind the bench's `roofline.traffic`: every row parses, names a kernel of the variant
    table and a summary file that exists, and the rows of the pinned shapes name the kernels the
    selection above pins for them (otherwise the bench would report null for them)."""
    import os
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    sys.path.insert(0, root)
    try:
        import bench
    finally:
        sys.path.remove(root)
    rows = bench.counter_traffic()
    names = set(_lib.variant_names())
    assert {("ffn", "ff.net.0.proj (W1)"), ("ffn", "ff.net.2 (W2)"), ("attn", "to_q/to_k/to_v grouped"), ("kv", "N=1280"), ("kv", "N=640")} <= set(rows)
    for key, row in rows.items():
        assert row["kernel"] in names, key
        assert os.path.isfile(os.path.join(root, row["profile"])), key
        assert row["bytes"] > 0 and len(row["commit"]) >= 7
    assert rows[("ffn", "ff.net.0.proj (W1)")]["kernel"] == "t256x320x32_w512_bf16x2_tri"
    assert rows[("ffn", "ff.net.2 (W2)")]["kernel"] == "k64x160x16_wk4_bf16x2_tri"
    assert rows[("kv", "N=1280")]["kernel"] == "t32x32x32_wavek_bf16x2_tri"
    got, why = bench.traffic_for("ffn", "ff.net.0.proj (W1)", "some_other_kernel")
    assert got is None and "not of the one that ran" in why


def test_scale_search_argument_validation():
    l = _lib.lib()
    ok = 16   # any non-NULL value: these calls return before touching the device
    assert l.cascmm_tensor_exps(ok, 4, 4, 4, 7, None, ok, ok, None) == -3          # dtype
    assert l.cascmm_tensor_exps(ok, 4, 4, 3, 0, None, ok, ok, None) == -2          # ld < cols
    assert l.cascmm_tensor_exps(ok, -1, 4, 4, 0, None, ok, ok, None) == -2
    assert l.cascmm_tensor_exps(None, 4, 4, 4, 0, None, ok, ok, None) == -1
    assert l.cascmm_tensor_exps(ok, 4, 4, 4, 0, None, None, ok, None) == -1
    assert l.cascmm_tensor_exps(ok, 4, 4, 4, 0, None, ok, None, None) == -1         # the scratch is not optional
    assert l.cascmm_tensor_exps(ok, 2 ** 31, 4, 4, 0, None, ok, ok, None) == -9


def test_cpu_tensors_are_rejected_without_fallback():
    import torch
    from basedxl_amd import cascaded_lowp_matmul

    with pytest.raises(RuntimeError, match="no CPU fallback"):
        cascaded_lowp_matmul(torch.randn(4, 4), torch.randn(4, 4))
    with pytest.raises(AssertionError, match="Incompatible dimensions"):
        cascaded_lowp_matmul(torch.randn(4, 4), torch.randn(5, 4))
    with pytest.raises(AssertionError, match="Matrix B must be contiguous"):
        cascaded_lowp_matmul(torch.randn(4, 4), torch.randn(4, 4).t())


def test_unet_shape_table_matches_the_architecture():
    """The SDXL Linear workload: 70 transformer blocks, about 8.6 TFLOP of Linear work per step
    at batch 2 and a 128x128 latent; the half-latent share halves the image-token GEMMs only."""
    from basedxl_amd.unet_shapes import sdxl_linear_shapes, total_flops

    full = sdxl_linear_shapes()
    assert sum(s.count for s in full if s.name.startswith("attn1.to_out")) == 70
    assert 8.0e12 < total_flops(full) < 9.5e12
    half = sdxl_linear_shapes(half_latent=True)
    kv = [s for s in half if s.name.startswith("attn2.to_kv")]
    assert len(kv) == 2
    assert all(s.M == 154 and s.K == 2048 for s in kv)
    assert [s.M for s in half if s.name.startswith("attn1.to_out")] == [4096, 1024]
    assert 0.5 * total_flops(full) < total_flops(half) < 0.52 * total_flops(full) + total_flops(kv)
    convs = sdxl_linear_shapes(convs=True)
    assert sum(s.count for s in convs if not s.routed_by_reference) == 11


def test_fast_kernels_are_not_chosen_when_offsets_would_overflow():
    """The fast kernels address B with 32-bit byte offsets from the top of a column block: a B of
    2 GiB or more must go to the bounds-checked kernels (64-bit addressing)."""
    l = _lib.lib()
    names = _lib.variant_names()
    ok = l.cascmm_select_variant(4096, 16384, 16384, 16384, 16384, 16384, 0, 0, 2, 0)
    big = l.cascmm_select_variant(4096, 32768, 32768, 32768, 32768, 32768, 0, 0, 2, 0)
    assert ok >= 0 and "generic" not in names[ok]
    assert big >= 0 and "generic" in names[big]


def test_slot_kernels_of_the_three_term_fp16_cascade_are_sized_and_bounded():
    """The fp16 kernels that split both operands into operand slots first: the workspace the library asks for holds
    both operands' slots (6 bytes per element); they are offered only where a slot buffer stays below 2 GiB (32-bit
    offsets), K is a multiple of their 32-k stage, and -- the LDS-tiled one -- K is at most 1536."""
    l = _lib.lib()
    names = _lib.variant_names()
    pick16 = lambda M, K, N: names[l.cascmm_select_variant(M, N, K, K, N, N, 0, 1, 3, 0) & 0xFFFF]
    M, K, N = 2048, 1280, 10240
    assert l.cascmm_workspace_bytes(M, N, K, _lib.DT_F32, _lib.FMT_FP16, 3, _lib.PROD_TRI) >= 6 * (M * K + K * N)
    assert pick16(4096, 2560, 5120) == "k64x160x32_f16wk4_fp16x3_tri"       # deep K: never the LDS-tiled kernel
    assert "_f16" not in pick16(2048, 1296, 1280)                            # K % 32 != 0
    assert "_f16" not in pick16(65536, 8192, 1280)                           # the slots of A would pass 2 GiB


def test_library_tables_are_consistent():
    """Every entry of the measured-cost table names exactly one compiled variant (a renamed kernel
    would otherwise fall back to the analytic estimate without a word), and no variant name repeats."""
    assert _lib.lib().cascmm_selftest() == 0
    names = _lib.variant_names()
    assert len(names) == len(set(names))


def test_product_package_never_touches_the_oracle_or_the_reference_tree():
    """The oracle is test infrastructure: nothing under basedxl_amd/ (Python or HIP sources) imports,
    names or opens it, and nothing there reads the reference's tree; importing the package must not
    pull the oracle in either."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    pkg = os.path.join(root, "basedxl_amd")
    for dirpath, _dirs, files in os.walk(pkg):
        if os.path.basename(dirpath) in ("build", "__pycache__"):
            continue
        for f in files:
            if not f.endswith((".py", ".h", ".hip")):
                continue
            text = open(os.path.join(dirpath, f), encoding="utf-8").read()
            assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), f
            assert "oracle/" not in text and "/root/reference" not in text, f
    code = "import sys, basedxl_amd, basedxl_amd.modules, basedxl_amd.unet, basedxl_amd.unet_skeleton; " \
           "sys.exit(1 if any(m == 'oracle' or m.startswith('oracle.') for m in sys.modules) else 0)"
    assert subprocess.run([sys.executable, "-c", code], cwd=root).returncode == 0
