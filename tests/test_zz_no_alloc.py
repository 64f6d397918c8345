"""The allocation-free entry point, cascmm_gemm_noalloc, called through the C ABI: its results
must equal cascmm_gemm's (given a workspace) bit for bit, call after call on the shared built-in
scratch, and problems beyond the scratch limit must be refused."""
import ctypes

import pytest
import torch

from basedxl_amd import _lib
from oracle import cascade as oc

pytestmark = pytest.mark.gpu

SCRATCH_BYTES = 8 << 20


def _call(l, fn, a, b, out, bias, extra):
    M, K = a.shape
    N = b.shape[1]
    stream = torch.cuda.current_stream().cuda_stream
    return fn(a.data_ptr(), b.data_ptr(), out.data_ptr(), bias.data_ptr() if bias is not None else None, M, N, K, K, N, N,
              _lib.DT_F32, _lib.FMT_BF16, 2, _lib.PROD_TRI, None, *extra(stream))


def test_noalloc_entry_equals_the_workspace_entry_on_consecutive_calls(gpu_device):
    l = _lib.lib()
    # two calls in a row on the shared scratch, the second with a smaller problem; both shapes take
    # the K-split path (few row tiles), i.e. they do use the scratch
    for (M, K, N), seed in (((154, 2048, 1280), 0), ((77, 1024, 640), 1)):
        print("noalloc case", M, K, N, flush=True)
        a_cpu, b_cpu = oc.make_operands(M, K, N, seed=seed, w_std=0.02)
        a, b = a_cpu.to(gpu_device), b_cpu.to(gpu_device)
        bias = torch.randn(N, device=gpu_device)
        need = l.cascmm_workspace_bytes(M, N, K, _lib.DT_F32, _lib.FMT_BF16, 2, _lib.PROD_TRI)
        assert 0 < need <= SCRATCH_BYTES
        ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
        want = torch.full((M, N), float("nan"), device=gpu_device)
        got = torch.full((M, N), float("nan"), device=gpu_device)
        st = _call(l, l.cascmm_gemm, a, b, want, bias, lambda s: (ws.data_ptr(), ws.numel(), s))
        assert st == 0, l.cascmm_strerror(st)
        torch.cuda.synchronize()
        # the driver's own count of free device memory sees any allocation, the library's included
        # (torch's counters only see torch's); the look-up of the buffer's address comes first, as a
        # caller that records its first call into a graph would do it
        assert l.cascmm_init() == 0
        before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
        st = _call(l, l.cascmm_gemm_noalloc, a, b, got, bias, lambda s: (s,))
        assert st == 0, l.cascmm_strerror(st)
        torch.cuda.synchronize()
        assert (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == before
        assert torch.equal(got, want)
        exp = oc.fp64_matmul(a_cpu, b_cpu) + bias.cpu().double()
        ek = oc.error_metrics(got.cpu(), exp)
        eo = oc.error_metrics(oc.cascade_matmul_ref(a_cpu, b_cpu) + bias.cpu(), exp)
        assert ek["rel_fro"] <= 1.25 * eo["rel_fro"] and ek["max_abs"] <= 1.25 * eo["max_abs"]


def test_noalloc_entry_records_into_a_graph_and_replays(gpu_device):
    """What the entry point is for: a call under stream capture.  The capture records the library's
    kernels (that the call itself allocates nothing is checked on the eager calls above: the graph
    object and its memory pool are the caller's and do take device memory), and
    every replay, with fresh operand values and eager work in between, equals the eager cascmm_gemm."""
    l = _lib.lib()
    M, K, N = 154, 2048, 640
    g = torch.Generator(device="cuda:0").manual_seed(4)
    a = torch.randn(M, K, device=gpu_device, generator=g)
    b = torch.randn(K, N, device=gpu_device, generator=g) * 0.02
    got = torch.empty(M, N, device=gpu_device)
    want = torch.empty(M, N, device=gpu_device)
    need = l.cascmm_workspace_bytes(M, N, K, _lib.DT_F32, _lib.FMT_BF16, 2, _lib.PROD_TRI)
    assert 0 < need <= SCRATCH_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device=gpu_device)
    assert l.cascmm_init() == 0                      # the address look-up stays outside the capture
    assert _call(l, l.cascmm_gemm_noalloc, a, b, got, None, lambda s: (s,)) == 0     # eager warm-up
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        st = _call(l, l.cascmm_gemm_noalloc, a, b, got, None, lambda s: (s,))
    assert st == 0, l.cascmm_strerror(st)
    for rep in range(3):
        a.copy_(torch.randn(M, K, device=gpu_device, generator=g) * (1.0 + rep))
        got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert _call(l, l.cascmm_gemm, a, b, want, None, lambda s: (ws.data_ptr(), ws.numel(), s)) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), rep


def test_noalloc_entry_refuses_what_exceeds_its_scratch_and_runs_what_needs_none(gpu_device):
    l = _lib.lib()
    # 1024 x 5120 x 1280 would split K with 4 x 1024 x 1280 x 4 bytes of partial results
    M, K, N = 1024, 5120, 1280
    assert 2 * M * N * 4 > SCRATCH_BYTES
    a = torch.randn(M, K, device=gpu_device)
    b = torch.randn(K, N, device=gpu_device)
    out = torch.zeros(M, N, device=gpu_device)
    st = _call(l, l.cascmm_gemm_noalloc, a, b, out, None, lambda s: (s,))
    assert st == -10 and b"scratch" in l.cascmm_strerror(st)
    torch.cuda.synchronize()
    assert not out.any()                       # nothing was launched
    # a problem whose kernel needs no scratch at all runs as cascmm_gemm does
    M, K, N = 4096, 640, 640
    a, b = torch.randn(M, K, device=gpu_device), torch.randn(K, N, device=gpu_device)
    want, got = torch.empty(M, N, device=gpu_device), torch.empty(M, N, device=gpu_device)
    assert _call(l, l.cascmm_gemm, a, b, want, None, lambda s: (None, 0, s)) == 0
    assert _call(l, l.cascmm_gemm_noalloc, a, b, got, None, lambda s: (s,)) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # the three-term cascades' slot kernels are a choice, not a need: where their operand slots would not fit the
    # scratch (here 26 MB for fp16 x 3), the call runs on a kernel that splits inside the GEMM, as cascmm_gemm
    # does when it is given no workspace
    M, K, N = 2048, 1280, 1280
    a, b = torch.randn(M, K, device=gpu_device), torch.randn(K, N, device=gpu_device) * 0.02
    want, got = torch.empty(M, N, device=gpu_device), torch.empty(M, N, device=gpu_device)
    for fmt in (_lib.FMT_FP16, _lib.FMT_FP8):
        stream = torch.cuda.current_stream().cuda_stream
        args = (a.data_ptr(), b.data_ptr(), None, None, M, N, K, K, N, N, _lib.DT_F32, fmt, 3, _lib.PROD_TRI, None)
        assert l.cascmm_workspace_bytes(M, N, K, _lib.DT_F32, fmt, 3, _lib.PROD_TRI) > SCRATCH_BYTES
        assert l.cascmm_gemm(*args[:2], want.data_ptr(), *args[3:], None, 0, stream) == 0
        assert l.cascmm_gemm_noalloc(*args[:2], got.data_ptr(), *args[3:], stream) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), fmt
