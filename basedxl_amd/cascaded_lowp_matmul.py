"""cascaded_lowp_matmul for MI355X: same call surface as the reference operator
(basedxl/triton/cascaded_lowp_matmul.py:139-173), arithmetic done by hand-written gfx950
kernels behind the C ABI of include/cascmm.h.

The operands are split on the fly into ``terms`` low-precision terms (``lowp``), the kept
partial products run on MFMA with fp32 accumulation and are summed in registers.

Differences from the reference wrapper, all behind keyword-only arguments with defaults:
  * ``lowp`` / ``terms`` / ``products`` choose the cascade (default for fp32 tensors: two bf16
    terms, the three products hi.hi + hi.lo + lo.hi; fp16 / bf16 tensors, which the reference
    runs its UNet in, default to one term of their own format: exact operands, fp32 accumulation);
  * ``bias`` fuses the ``x + bias`` that basedxl/modules/lowp_linear.py:17-19 does separately;
  * there is no torch.matmul fallback for small shapes (:155-156): every shape, including
    M = 154 text tokens, runs the HIP kernels, and a batched ``b`` loops over its batch.
"""
from __future__ import annotations

from typing import Dict, Optional, Tuple

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.DT_F32, torch.float16: _lib.DT_F16, torch.bfloat16: _lib.DT_BF16}

#: persistent split-K / re-lay workspaces (contents need no initialisation), one per (device index,
#: stream handle) for eager launches and one per device (key "capture") for launches recorded into a
#: device graph
_workspaces: Dict[Tuple[int, object], torch.Tensor] = {}
_MIN_WORKSPACE = 1 << 20


#: capture buffers that a larger one has replaced.  A device graph recorded earlier has the old
#: buffer's address baked into its launches and writes its partial results there on every replay, so
#: the memory must stay this package's for as long as the process lives (buffers double in size, which
#: bounds what is kept to the size of the current one).
_retired_capture_buffers: list = []


def _grow_capture_workspace(index: int, dev: torch.device, nbytes: int) -> torch.Tensor:
    key = (index, "capture")
    old = _workspaces.get(key)
    if old is not None:
        _retired_capture_buffers.append(old)
        nbytes = max(nbytes, 2 * old.numel())
    ws = _workspaces[key] = torch.empty(max(nbytes, _MIN_WORKSPACE), dtype=torch.uint8, device=dev)
    return ws


def reserve_workspace(nbytes: int, device=None) -> None:
    """Make sure the workspace that launches recorded into a device graph use holds ``nbytes``, so
    that a capture allocates nothing.  Every eager launch does this for its own need, so a capture
    that follows the usual eager warm-up of the same calls finds its workspace already there.  A
    buffer that has to grow is replaced, never freed: graphs recorded against it keep replaying into
    memory that nothing else can own."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    ws = _workspaces.get((index, "capture"))
    if ws is None or ws.numel() < nbytes:
        _grow_capture_workspace(index, dev, nbytes)


def _workspace(device: torch.device, stream: int, nbytes: int) -> Optional[torch.Tensor]:
    """Launches on one stream are ordered, so they can share one buffer; launches replayed from
    graphs share the per-device capture buffer (graphs that use it must not replay concurrently)."""
    if nbytes == 0:
        return None
    index = device.index if device.index is not None else torch.cuda.current_device()
    if torch.cuda.is_current_stream_capturing():
        ws = _workspaces.get((index, "capture"))
        if ws is None or ws.numel() < nbytes:
            # no eager warm-up came first: the buffer comes from the graph's own pool (an
            # allocation inside the capture, but no fill: nothing is recorded for it)
            ws = _grow_capture_workspace(index, device, nbytes)
        return ws
    reserve_workspace(nbytes, device)
    key = (index, stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, _MIN_WORKSPACE), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


_ws_need: Dict[tuple, int] = {}


def _workspace_bytes(M: int, N: int, K: int, dt: int, fmt: int, terms: int, products: int) -> int:
    """cascmm_workspace_bytes, remembered per problem (it walks the whole variant table)."""
    key = (M, N, K, dt, fmt, terms, products)
    need = _ws_need.get(key)
    if need is None:
        need = _ws_need[key] = _lib.lib().cascmm_workspace_bytes(M, N, K, dt, fmt, terms, products)
    return need


def _check_bias(bias: Optional[torch.Tensor], like: torch.Tensor, n: int) -> Optional[torch.Tensor]:
    """A bias the kernels can read: on the device of ``like``, its dtype, 1-D, ``n`` long, contiguous.
    Checked before any launch: the C side sees only a pointer."""
    if bias is None:
        return None
    _check_device_tensor(bias, "bias")
    if bias.device != like.device:
        raise ValueError(f"bias is on {bias.device} but the operands are on {like.device}")
    if bias.dtype != like.dtype or bias.dim() != 1 or bias.shape[0] != n:
        raise ValueError(f"bias must be a 1-D tensor of length N = {n} with the dtype of a ({like.dtype}), "
                         f"got shape {tuple(bias.shape)} {bias.dtype}")
    return bias.contiguous()


_exp_scratch: Dict[Tuple[int, int], torch.Tensor] = {}


def _scale_scratch(dev: torch.device, stream: int) -> torch.Tensor:
    """The two zeroed device int32 the one-launch scale search needs (it leaves them zeroed): one per
    (device, stream) for eager launches, one per device for launches recorded into a device graph."""
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    capturing = torch.cuda.is_current_stream_capturing()
    key = (index, "capture" if capturing else stream)
    if not capturing and (index, "capture") not in _exp_scratch:
        _exp_scratch[(index, "capture")] = torch.zeros(2, dtype=torch.int32, device=dev)
    scratch = _exp_scratch.get(key)
    if scratch is None:
        scratch = _exp_scratch[key] = torch.zeros(2, dtype=torch.int32, device=dev)
    return scratch


def _activation_exps(a2: torch.Tensor, lda: int, second: Optional[torch.Tensor], out_ptr: int, stream: int) -> None:
    """{e_A, e_B} at ``out_ptr`` (device int32[2]) in one launch: the fp8 scale exponent of ``a2`` found
    on the device, next to the kept exponent ``second`` of the other operand (skipped when None)."""
    scratch = _scale_scratch(a2.device, stream)
    _lib.check(_lib.lib().cascmm_tensor_exps(a2.data_ptr(), a2.shape[0], a2.shape[1], lda, _DTYPES[a2.dtype],
                                             second.data_ptr() if second is not None else None, out_ptr,
                                             scratch.data_ptr(), stream), "cascmm_tensor_exps")


def _gemm_fp8_autoscale(a2: torch.Tensor, b_ptr: int, b_prepared: bool, out2: torch.Tensor, bias: Optional[torch.Tensor],
                        M: int, N: int, K: int, lda: int, ldb: int, ldc: int, terms: int, products: int,
                        b_exp: torch.Tensor) -> None:
    """One fp8 GEMM on fp32 tensors whose activation scale is found inside the call (the weight's is
    kept): cascmm_gemm_fp8_autoscale, which folds the search into the operand split of the fp8-rate
    kernel and otherwise runs the one-launch search followed by the GEMM."""
    dev = a2.device
    stream = torch.cuda.current_stream(dev).cuda_stream
    ws = _workspace(dev, stream, _workspace_bytes(M, N, K, _lib.DT_F32, _lib.FMT_FP8, terms, products))
    exps = torch.empty(2, dtype=torch.int32, device=dev)
    scratch = _scale_scratch(dev, stream)
    st = _lib.lib().cascmm_gemm_fp8_autoscale(
        a2.data_ptr(), b_ptr, 1 if b_prepared else 0, out2.data_ptr(), bias.data_ptr() if bias is not None else None,
        M, N, K, lda, ldb, ldc, terms, products, b_exp.data_ptr(), exps.data_ptr(), scratch.data_ptr(),
        ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0, stream)
    _lib.check(st, "cascmm_gemm_fp8_autoscale")


def _check_device_tensor(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"cascaded_lowp_matmul: {name} is on {t.device}; the operator only runs on an AMD GPU "
            "(there is no CPU fallback)")


def tensor_scale_exp(x: torch.Tensor) -> torch.Tensor:
    """Device int32[1]: the fp8 tensor-scale exponent e of ``x`` (max|x| * 2**e in (224, 448]),
    computed on the GPU.  Callers with a constant operand (a layer's weight) compute it once and
    pass it as ``b_exp``."""
    _check_device_tensor(x, "x")
    x2 = _rows(x.reshape(-1, x.shape[-1]))
    e = torch.empty(1, dtype=torch.int32, device=x.device)
    stream = torch.cuda.current_stream(x.device).cuda_stream
    _lib.check(_lib.lib().cascmm_tensor_exp(x2.data_ptr(), x2.shape[0], x2.shape[1],
                                            x2.stride(0) if x2.shape[0] > 1 else max(x2.shape[1], 1),
                                            _DTYPES[x.dtype], e.data_ptr(), stream), "cascmm_tensor_exp")
    return e


def default_cascade(dtype: torch.dtype) -> Tuple[str, int]:
    """The cascade used when the caller names none: two bf16 terms for fp32 tensors; fp16 / bf16
    tensors are multiplied as one term of their own format (exact operands, fp32 accumulation)."""
    if dtype == torch.float16:
        return "fp16", 1
    if dtype == torch.bfloat16:
        return "bf16", 1
    return "bf16", 2


class PreparedWeight:
    """A constant right operand ``w`` ([K, N]: the ``[in, out]`` weight of
    basedxl/modules/lowp_linear.py:12) split once on the GPU into the terms of a cascade and
    kept as MFMA operand slots; ``cascaded_lowp_matmul(a, prepared)`` then splits only ``a``.
    The arithmetic is the same as with the raw weight (same split, same products).  Kernels for
    prepared weights exist for bf16 x 2, bf16 x 3, fp16 x 3 and fp8 x 3 with the 'tri' product set and
    for fp16 / bf16 tensors as one term of their own format, K a multiple of 64 and N of 4; the
    product with any other combination fails with CascmmError (use the raw weight there).

    ``glu=True``: ``w`` is the ``[in, 2 * inner]`` weight of a gated projection (diffusers' GEGLU:
    ``h = x @ w + b; y = h[:, :inner] * gelu(h[:, inner:])``); its columns are stored so that a
    kernel holds a value column and its gate column together, and the product with it returns
    ``y`` ([..., inner]) directly, the gate applied in the GEMM's store (inner % 32 == 0)."""

    def __init__(self, w: torch.Tensor, *, lowp: Optional[str] = None, terms: Optional[int] = None, glu: bool = False):
        _check_device_tensor(w, "w")
        if w.dim() != 2 or w.dtype not in _DTYPES:
            raise ValueError("PreparedWeight needs a 2-D fp32 / fp16 / bf16 tensor")
        d_lowp, d_terms = default_cascade(w.dtype)
        lowp = d_lowp if lowp is None else lowp
        terms = d_terms if terms is None else terms
        if lowp not in _lib.FMT_BY_NAME:
            raise ValueError(f"lowp must be one of {sorted(_lib.FMT_BY_NAME)}, got {lowp!r}")
        self.K, self.N = int(w.shape[0]), int(w.shape[1])
        self.shape = (self.K, self.N)
        self.lowp, self.terms, self.fmt = lowp, int(terms), _lib.FMT_BY_NAME[lowp]
        self.dtype, self.device = w.dtype, w.device
        self.glu = bool(glu)
        if self.glu and self.N % 64 != 0:
            raise ValueError("glu=True needs a weight whose width is a multiple of 64")
        self.out_features = self.N // 2 if self.glu else self.N
        w2 = _rows(w)
        l = _lib.lib()
        stream = torch.cuda.current_stream(w.device).cuda_stream
        self.exp = tensor_scale_exp(w2) if self.fmt == _lib.FMT_FP8 else None
        nbytes = l.cascmm_prepared_bytes(self.K, self.N, self.fmt, self.terms)
        self.slots = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=w.device)
        prepare = l.cascmm_prepare_weight_glu if self.glu else l.cascmm_prepare_weight
        _lib.check(prepare(w2.data_ptr(), self.K, self.N, w2.stride(0) if self.K > 1 else max(self.N, 1),
                           _DTYPES[w.dtype], self.fmt, self.terms, self.exp.data_ptr() if self.exp is not None else None,
                           self.slots.data_ptr(), self.slots.numel(), stream), "cascmm_prepare_weight")

    @classmethod
    def from_slots(cls, slots: torch.Tensor, K: int, N: int, dtype: torch.dtype, lowp: str, terms: int, glu: bool = False,
                   exp: Optional[torch.Tensor] = None) -> "PreparedWeight":
        """The object around operand slots that already exist (``prepared.slots`` of an earlier
        preparation with the same K, N, dtype and cascade); nothing is computed."""
        if lowp not in _lib.FMT_BY_NAME:
            raise ValueError(f"lowp must be one of {sorted(_lib.FMT_BY_NAME)}, got {lowp!r}")
        if lowp == "fp8" and (exp is None or exp.dtype != torch.int32 or exp.numel() != 1 or exp.device != slots.device):
            raise ValueError("fp8 operand slots need the tensor-scale exponent they were prepared with "
                             "(exp: int32[1] on the device of the slots)")
        self = cls.__new__(cls)
        self.K, self.N, self.shape = int(K), int(N), (int(K), int(N))
        self.lowp, self.terms, self.fmt = lowp, int(terms), _lib.FMT_BY_NAME[lowp]
        self.dtype, self.device = dtype, slots.device
        self.glu = bool(glu)
        self.out_features = self.N // 2 if self.glu else self.N
        self.exp, self.slots = exp, slots
        return self

    def usable_with(self, a2: torch.Tensor, products: str = "tri") -> bool:
        """Whether the prepared kernels take this left operand: fp32 (or fp16 / bf16 tensors with a
        weight of the same dtype kept as one term of that format), K a multiple of 64, rows 16-byte
        aligned (anything else goes through the raw weight)."""
        if self.K % 64 != 0 or self.N % 4 != 0 or a2.data_ptr() % 16 != 0:
            return False
        if not self.has_kernel(a2.dtype, products):
            return False
        if a2.dtype == torch.float32:
            return a2.shape[0] <= 1 or a2.stride(0) % 4 == 0
        return (a2.dtype == self.dtype and self.terms == 1 and default_cascade(a2.dtype)[0] == self.lowp
                and (a2.shape[0] <= 1 or a2.stride(0) % 8 == 0))

    def has_kernel(self, dtype: torch.dtype, products: str = "tri") -> bool:
        """Whether the library has a prepared-operand kernel for this weight's cascade with left
        operands of ``dtype`` (a host-side table lookup, remembered)."""
        key = (dtype, products)
        hit = self._kernel_known.get(key) if hasattr(self, "_kernel_known") else None
        if hit is None:
            if not hasattr(self, "_kernel_known"):
                self._kernel_known = {}
            st = -1
            if dtype in _DTYPES and products in _lib.PROD_BY_NAME:
                st = _lib.lib().cascmm_select_variant_prepared(1, 256, self.N, self.K, self.K, self.N, _DTYPES[dtype],
                                                               self.fmt, self.terms, _lib.PROD_BY_NAME[products])
            hit = self._kernel_known[key] = st >= 0
        return hit


def cascaded_lowp_matmul_prepared(a_list, w_list, *, outs=None, biases=None, products: str = "tri", variant: int = -1):
    """``a_list[i]`` ([..., K] fp32) times the prepared weight ``w_list[i]`` in ONE launch (1..8
    problems of one shape and one cascade); returns the list of results."""
    import ctypes

    n = len(a_list)
    if n == 0 or n != len(w_list) or n > 8:
        raise ValueError("need 1..8 problems, one prepared weight per a")
    w0 = w_list[0]
    if products not in _lib.PROD_BY_NAME:
        raise ValueError(f"products must be 'tri' or 'full', got {products!r}")
    a2s = []
    for a, w in zip(a_list, w_list):
        if not isinstance(w, PreparedWeight):
            raise TypeError("w_list must hold PreparedWeight objects")
        assert a.shape[-1] == w.K, "Incompatible dimensions"
        _check_device_tensor(a, "a")
        if (w.K, w.N, w.fmt, w.terms, w.glu) != (w0.K, w0.N, w0.fmt, w0.terms, w0.glu) or a.dtype != a_list[0].dtype:
            raise ValueError("grouped problems must share one shape, cascade and activation dtype")
        if a.dtype not in _DTYPES:
            raise TypeError(f"unsupported dtype {a.dtype}")
        a2 = _rows(a.reshape(-1, w.K))
        # the prepared kernels load 16 bytes of a row at a time: rows that do not start on such a
        # boundary are copied, as basedxl/triton/cascaded_lowp_matmul.py:158 copies every `a`
        per16 = 16 // a2.element_size()
        if a2.data_ptr() % 16 != 0 or (a2.shape[0] > 1 and a2.stride(0) % per16 != 0):
            a2 = a2.contiguous()
        a2s.append(a2)
    M, K, N = a2s[0].shape[0], w0.K, w0.N
    NO = w0.out_features                       # columns of the result (N / 2 for a gated weight)
    lda = a2s[0].stride(0) if M > 1 else max(K, 1)
    for a2 in a2s:
        if a2.shape[0] != M or (M > 1 and a2.stride(0) != lda):
            raise ValueError("grouped problems must share M and the row stride of a")
    dev = a_list[0].device
    adt = a_list[0].dtype
    if outs is None:
        outs = [torch.empty((M, NO), device=dev, dtype=adt) for _ in range(n)]
    for o in outs:
        _check_device_tensor(o, "out")
        if o.numel() != M * NO or not o.is_contiguous() or o.dtype != adt:
            raise ValueError("every out must be a contiguous [M, N] tensor of the dtype of a")
    if biases is not None:
        if len(biases) != n:
            raise ValueError("one bias (or None) per problem")
        biases = [_check_bias(bb, a2s[0], N) for bb in biases]   # (a gated weight takes all N = 2 * inner entries)
    if w0.fmt == _lib.FMT_FP8 and any(w.exp is None for w in w_list):
        raise ValueError("an fp8 PreparedWeight needs its tensor-scale exponent (exp)")
    arr = ctypes.c_void_p * n
    pa = arr(*[t.data_ptr() for t in a2s])
    pb = arr(*[w.slots.data_ptr() for w in w_list])
    pc = arr(*[t.data_ptr() for t in outs])
    pbias = arr(*[(None if bb is None else bb.data_ptr()) for bb in biases]) if biases is not None else None
    stream = torch.cuda.current_stream(dev).cuda_stream
    if w0.fmt == _lib.FMT_FP8 and n == 1 and not w0.glu and adt == torch.float32 and variant < 0:
        _gemm_fp8_autoscale(a2s[0], w0.slots.data_ptr(), True, outs[0], None if biases is None else biases[0], M, N, K,
                            lda, N, max(NO, 1), w0.terms, _lib.PROD_BY_NAME[products], w0.exp)
        return [outs[0].reshape(*a_list[0].shape[:-1], NO)]
    exps = None
    if w0.fmt == _lib.FMT_FP8:
        exps = torch.empty(2 * n, dtype=torch.int32, device=dev)
        first = {}                                   # one pass per distinct left operand (q / k / v share theirs)
        for i in range(n):
            j = first.setdefault(a2s[i].data_ptr(), i)
            if j == i:
                _activation_exps(a2s[i], lda, w_list[i].exp, exps.data_ptr() + 8 * i, stream)
            else:
                exps[2 * i:2 * i + 1].copy_(exps[2 * j:2 * j + 1])
                exps[2 * i + 1:2 * i + 2].copy_(w_list[i].exp.reshape(1))
    common = (n, pa, pb, pc, pbias, M, N, K, lda, max(NO, 1), _DTYPES[adt], w0.fmt, w0.terms,
              _lib.PROD_BY_NAME[products], exps.data_ptr() if exps is not None else None)
    if w0.glu:
        st = _lib.lib().cascmm_gemm_prepared_glu(*common, stream, variant)
    else:
        # room for the partial results of a K split (single fp32 problems with few tiles) or for the
        # operand slots of the activations (three fp8 terms)
        ws = None
        if adt == torch.float32 and (n == 1 or w0.fmt == _lib.FMT_FP8):
            need = _workspace_bytes(M, N, K, _DTYPES[adt], w0.fmt, w0.terms, _lib.PROD_BY_NAME[products])
            ws = _workspace(dev, stream, need)
        st = _lib.lib().cascmm_gemm_prepared(*common, ws.data_ptr() if ws is not None else None,
                                             ws.numel() if ws is not None else 0, stream, variant)
    _lib.check(st, "cascmm_gemm_prepared")
    return [o.reshape(*a.shape[:-1], NO) for o, a in zip(outs, a_list)]


def _gemm_2d(a2: torch.Tensor, b2: torch.Tensor, out2: torch.Tensor, bias: Optional[torch.Tensor],
             fmt: int, terms: int, products: int, variant: int, b_exp: Optional[torch.Tensor] = None,
             tensor_exps: Optional[torch.Tensor] = None) -> None:
    M, K = a2.shape
    N = b2.shape[1]
    dt = _DTYPES[a2.dtype]
    l = _lib.lib()
    stream = torch.cuda.current_stream(a2.device).cuda_stream
    ws_bytes = _workspace_bytes(M, N, K, dt, fmt, terms, products)
    ws = _workspace(a2.device, stream, ws_bytes)
    exps = None
    if fmt == _lib.FMT_FP8 and tensor_exps is not None:
        # static scales: {e_A, e_B} chosen by the caller (calibrated once), no pass over the operands
        if tensor_exps.dtype != torch.int32 or tensor_exps.numel() != 2 or not tensor_exps.is_cuda:
            raise ValueError("tensor_exps must be a device int32 tensor {e_A, e_B}")
        exps = tensor_exps.contiguous()
    elif fmt == _lib.FMT_FP8 and b_exp is not None and variant < 0 and a2.dtype == torch.float32:
        _gemm_fp8_autoscale(a2, b2.data_ptr(), False, out2, bias, M, N, K, a2.stride(0) if M > 1 else max(K, 1),
                            b2.stride(0) if K > 1 else max(N, 1), out2.stride(0) if M > 1 else max(N, 1), terms, products, b_exp)
        return
    elif fmt == _lib.FMT_FP8:
        exps = torch.empty(2, dtype=torch.int32, device=a2.device)
        _activation_exps(a2, a2.stride(0) if M > 1 else max(K, 1), b_exp, exps.data_ptr(), stream)
        if b_exp is None:
            _activation_exps(b2, b2.stride(0) if K > 1 else max(N, 1), None, exps.data_ptr() + 4, stream)
    st = l.cascmm_gemm_variant(
        a2.data_ptr(), b2.data_ptr(), out2.data_ptr(), bias.data_ptr() if bias is not None else None,
        M, N, K, a2.stride(0) if M > 1 else max(K, 1), b2.stride(0) if K > 1 else max(N, 1),
        out2.stride(0) if M > 1 else max(N, 1),
        dt, fmt, terms, products,
        exps.data_ptr() if exps is not None else None,
        ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
        stream, variant)
    _lib.check(st, "cascmm_gemm")


def cascaded_lowp_matmul_grouped(a_list, b_list, *, outs=None, biases=None, lowp: Optional[str] = None,
                                 terms: Optional[int] = None,
                                 products: str = "tri", variant: int = -1, b_exps=None):
    """Several independent cascade GEMMs of one shape in ONE kernel launch.

    ``a_list[i]`` ([..., K], the same tensor may appear several times) times ``b_list[i]``
    ([K, N], contiguous) -> ``outs[i]``.  This is what the reference gets for to_k / to_v by
    concatenating the two weights into one Linear (basedxl/modules/attn.py:23-39); here the
    weights stay separate and up to 8 problems share one persistent launch, which removes
    the launch gap and the cold start of every GEMM after the first.  ``b_exps`` (fp8): the tensor
    scale exponents of the right operands (``tensor_scale_exp(b)``, device int32[1] each) when the
    caller keeps them, as a layer does for its constant weight; otherwise they are found in every call.
    """
    import ctypes

    n = len(a_list)
    if n == 0 or n != len(b_list) or n > 8:
        raise ValueError("need 1..8 problems, one b per a")
    d_lowp, d_terms = default_cascade(a_list[0].dtype)
    lowp = d_lowp if lowp is None else lowp
    terms = d_terms if terms is None else terms
    if lowp not in _lib.FMT_BY_NAME or products not in _lib.PROD_BY_NAME:
        raise ValueError("bad lowp / products")
    fmt, prod = _lib.FMT_BY_NAME[lowp], _lib.PROD_BY_NAME[products]
    K, N = b_list[0].shape[-2], b_list[0].shape[-1]
    a2s, res = [], []
    for i, (a, b) in enumerate(zip(a_list, b_list)):
        assert a.shape[-1] == b.shape[-2], "Incompatible dimensions"
        assert b.is_contiguous(), "Matrix B must be contiguous"
        _check_device_tensor(a, "a")
        _check_device_tensor(b, "b")
        if b.dim() != 2 or tuple(b.shape) != (K, N) or a.dtype != a_list[0].dtype or b.dtype != a.dtype:
            raise ValueError("grouped problems must share one shape and dtype")
        a2s.append(_rows(a.reshape(-1, K)))
    M = a2s[0].shape[0]
    lda = a2s[0].stride(0) if M > 1 else max(K, 1)
    for a2 in a2s:
        if a2.shape[0] != M or (M > 1 and a2.stride(0) != lda):
            raise ValueError("grouped problems must share M and the row stride of a")
    if a_list[0].dtype not in _DTYPES:
        raise TypeError(f"unsupported dtype {a_list[0].dtype}")
    dev = a_list[0].device
    if outs is None:
        outs = [torch.empty((M, N), device=dev, dtype=a_list[0].dtype) for _ in range(n)]
    for o in outs:
        _check_device_tensor(o, "out")
        if o.numel() != M * N or not o.is_contiguous() or o.dtype != a_list[0].dtype:
            raise ValueError("every out must be a contiguous [M, N] tensor of the dtype of a")
    if biases is not None:
        if len(biases) != n:
            raise ValueError("one bias (or None) per problem")
        biases = [_check_bias(bb, a2s[0], N) for bb in biases]
    arr = ctypes.c_void_p * n
    pa = arr(*[t.data_ptr() for t in a2s])
    pb = arr(*[t.data_ptr() for t in b_list])
    pc = arr(*[t.data_ptr() for t in outs])
    pbias = arr(*[(None if bb is None else bb.data_ptr()) for bb in biases]) if biases is not None else None
    stream = torch.cuda.current_stream(dev).cuda_stream
    exps = None
    if fmt == _lib.FMT_FP8:
        # tensor scale exponents {e_A, e_B} of every problem, computed on the device
        exps = torch.empty(2 * n, dtype=torch.int32, device=dev)
        dt = _DTYPES[a_list[0].dtype]
        first = {}                                   # one pass per distinct left operand (q / k / v share theirs)
        for i in range(n):
            j = first.setdefault(a2s[i].data_ptr(), i)
            kept = b_exps[i] if b_exps is not None else None
            if j == i:
                _activation_exps(a2s[i], lda, kept, exps.data_ptr() + 8 * i, stream)
            else:
                exps[2 * i:2 * i + 1].copy_(exps[2 * j:2 * j + 1])
                if kept is not None:
                    exps[2 * i + 1:2 * i + 2].copy_(kept.reshape(1))
            if kept is None:
                _activation_exps(b_list[i], max(N, 1), None, exps.data_ptr() + 8 * i + 4, stream)
    # 16-bit tensors as one term of their own format: room for every right operand re-laid as operand slots
    ws = None
    if a_list[0].dtype != torch.float32:
        need = _workspace_bytes(M, N, K, _DTYPES[a_list[0].dtype], fmt, terms, prod)
        ws = _workspace(dev, stream, n * need) if need else None
    st = _lib.lib().cascmm_gemm_grouped(n, pa, pb, pc, pbias, M, N, K, lda, max(N, 1), max(N, 1),
                                        _DTYPES[a_list[0].dtype], fmt, terms, prod,
                                        exps.data_ptr() if exps is not None else None,
                                        ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
                                        stream, variant)
    _lib.check(st, "cascmm_gemm_grouped")
    return [o.reshape(*a.shape[:-1], N) for o, a in zip(outs, a_list)]


def _rows(t: torch.Tensor) -> torch.Tensor:
    """2-D view whose rows are contiguous (row stride free); copies only when it must."""
    if t.stride(-1) != 1 and t.shape[-1] > 1:
        return t.contiguous()
    if t.shape[0] > 1 and t.stride(0) < t.shape[1]:
        return t.contiguous()
    return t


def gated_variant(a: torch.Tensor, b: torch.Tensor, *, lowp: Optional[str] = None, terms: Optional[int] = None,
                  products: str = "tri") -> int:
    """Index of the kernel that computes ``value * gelu(gate)`` of ``a @ b`` from the RAW ``[K, 2 * inner]``
    weight in its store, or a negative status when there is none for these tensors (then the caller runs
    the plain product and applies the gate)."""
    if not (a.is_cuda and b.is_cuda and a.dtype == b.dtype == torch.float32 and b.dim() == 2 and b.is_contiguous()):
        return _lib.ERR_BAD_FORMAT
    d_lowp, d_terms = default_cascade(a.dtype)
    lowp, terms = d_lowp if lowp is None else lowp, d_terms if terms is None else terms
    K, N = b.shape
    M = a.numel() // K if K else 0
    if a.shape[-1] != K or M == 0 or N % 2 != 0:
        return _lib.ERR_BAD_FORMAT
    a2 = a.reshape(M, K)
    if a2.stride(1) != 1 or a2.data_ptr() % 16 != 0 or b.data_ptr() % 16 != 0:
        return _lib.ERR_BAD_FORMAT
    return _lib.lib().cascmm_select_variant_glu(M, N, K, a2.stride(0), N, N // 2, _DTYPES[a.dtype], _lib.FMT_BY_NAME[lowp],
                                                terms, _lib.PROD_BY_NAME[products])


def cascaded_lowp_matmul_glu(a: torch.Tensor, b: torch.Tensor, *, bias: Optional[torch.Tensor] = None,
                             out: Optional[torch.Tensor] = None, lowp: Optional[str] = None, terms: Optional[int] = None,
                             products: str = "tri", variant: int = -1) -> torch.Tensor:
    """``h = a @ b + bias; value, gate = h.chunk(2, -1); return value * gelu(gate)`` (diffusers' GEGLU around
    one of the nn.Linear layers the reference routes, basedxl/unet.py:81-87) in ONE kernel on the raw
    weight ``b`` ``[K, 2 * inner]``: ``h`` never reaches memory.  Only where :func:`gated_variant` finds a
    kernel (fp32 tensors, two bf16 terms, rows % 256 == 0, inner % 160 == 0, K % 32 == 0); raises otherwise."""
    assert a.shape[-1] == b.shape[-2], "Incompatible dimensions"
    assert b.is_contiguous(), "Matrix B must be contiguous"
    _check_device_tensor(a, "a")
    _check_device_tensor(b, "b")
    d_lowp, d_terms = default_cascade(a.dtype)
    lowp, terms = d_lowp if lowp is None else lowp, d_terms if terms is None else terms
    K, N = b.shape
    if N % 2 != 0:
        raise ValueError("a gated projection has an even number of columns")
    bias = _check_bias(bias, a, N)
    batch_dims = a.shape[:-1]
    M = batch_dims.numel()
    a2 = _rows(a.reshape(M, K))
    inner = N // 2
    if out is None:
        out = torch.empty((M, inner), device=a.device, dtype=a.dtype)
    else:
        _check_device_tensor(out, "out")
        if out.dtype != a.dtype or out.numel() != M * inner:
            raise ValueError(f"out must hold {M * inner} elements of {a.dtype}")
    out2 = out if out.dim() == 2 and out.shape == (M, inner) else out.view(M, inner)
    if inner > 1 and out2.stride(1) != 1:
        raise ValueError("out must have unit stride along its columns")
    stream = torch.cuda.current_stream(a.device).cuda_stream
    st = _lib.lib().cascmm_gemm_glu(a2.data_ptr(), b.data_ptr(), out2.data_ptr(), None if bias is None else bias.data_ptr(),
                                    M, N, K, a2.stride(0) if M > 1 else max(K, 1), N, out2.stride(0) if M > 1 else max(inner, 1),
                                    _DTYPES[a.dtype], _lib.FMT_BY_NAME[lowp], terms, _lib.PROD_BY_NAME[products], stream, variant)
    _lib.check(st, "cascmm_gemm_glu")
    return out.reshape(*batch_dims, inner)


class LeftSlots:
    """A left operand ``a`` ([..., K] fp32) already split into the two bf16 terms of the default cascade
    and kept as MFMA operand slots, ``[2 terms][K / 8][M] x 16 bytes``: what the gated store of a
    feed-forward block's first GEMM writes for the second one (:func:`cascaded_lowp_matmul_glu_chained`),
    or what :meth:`from_tensor` makes of any fp32 tensor in a pass of its own."""

    def __init__(self, slots: torch.Tensor, batch_shape, K: int):
        self.slots, self.batch_shape, self.K = slots, tuple(batch_shape), int(K)
        self.M = 1
        for d in self.batch_shape:
            self.M *= int(d)
        self.device = slots.device

    @classmethod
    def empty(cls, batch_shape, K: int, device) -> "LeftSlots":
        M = 1
        for d in batch_shape:
            M *= int(d)
        nbytes = _lib.lib().cascmm_left_slots_bytes(M, K)
        if nbytes == 0:
            raise ValueError(f"left operand slots need K % 16 == 0 and M, K > 0 (got M = {M}, K = {K})")
        return cls(torch.empty(nbytes, dtype=torch.uint8, device=device), batch_shape, K)

    @classmethod
    def from_tensor(cls, a: torch.Tensor) -> "LeftSlots":
        _check_device_tensor(a, "a")
        if a.dtype != torch.float32:
            raise TypeError("left operand slots are made from fp32 tensors")
        K = a.shape[-1]
        a2 = a.reshape(-1, K)
        if a2.stride(-1) != 1 or a2.data_ptr() % 16 != 0 or (a2.shape[0] > 1 and a2.stride(0) % 4 != 0):
            a2 = a2.contiguous()
        out = cls.empty(a.shape[:-1], K, a.device)
        stream = torch.cuda.current_stream(a.device).cuda_stream
        _lib.check(_lib.lib().cascmm_prepare_left(a2.data_ptr(), a2.shape[0], K, a2.stride(0) if a2.shape[0] > 1 else K,
                                                  out.slots.data_ptr(), out.slots.numel(), stream), "cascmm_prepare_left")
        return out

    def terms(self) -> torch.Tensor:
        """The two terms as fp32 ``[2, ..., K]`` in the natural order of k (torch arithmetic: for tests
        and inspection, not a fast path)."""
        M, K = self.M, self.K
        t = self.slots.view(torch.bfloat16).view(2, K // 8, M, 8).float()
        kg = torch.arange(K // 8, device=self.device).view(-1, 1)
        pos = torch.arange(8, device=self.device).view(1, -1)
        k = (16 * (kg >> 1) + 8 * (pos >> 2) + 4 * (kg & 1) + (pos & 3)).flatten()
        out = torch.empty(2, M, K, device=self.device)
        out[:, :, k] = t.permute(0, 2, 1, 3).reshape(2, M, K)
        return out.reshape(2, *self.batch_shape, K)

    def to_dense(self) -> torch.Tensor:
        """hi + lo as fp32 ``[..., K]`` (the fp32 value rounded to 16 significant bits)."""
        t = self.terms()
        return t[0] + t[1]


class ChainedWeight:
    """The ``[K, N]`` fp32 weight of a feed-forward block's second Linear, split once into two bf16 terms
    in the order of k in which :class:`LeftSlots` holds its operand (counterpart of the one-time
    transpose at basedxl/modules/lowp_linear.py:12)."""

    def __init__(self, w: torch.Tensor):
        _check_device_tensor(w, "w")
        if w.dim() != 2 or w.dtype != torch.float32:
            raise ValueError("ChainedWeight needs a 2-D fp32 tensor")
        self.K, self.N = int(w.shape[0]), int(w.shape[1])
        if self.K % 16 != 0:
            raise ValueError("ChainedWeight needs K % 16 == 0")
        self.device = w.device
        w2 = _rows(w)
        l = _lib.lib()
        self.slots = torch.empty(max(l.cascmm_prepared_bytes(self.K, self.N, _lib.FMT_BF16, 2), 16), dtype=torch.uint8, device=w.device)
        stream = torch.cuda.current_stream(w.device).cuda_stream
        _lib.check(l.cascmm_prepare_weight_chained(w2.data_ptr(), self.K, self.N, w2.stride(0) if self.K > 1 else max(self.N, 1),
                                                   self.slots.data_ptr(), self.slots.numel(), stream), "cascmm_prepare_weight_chained")


def chained_supported(M: int, N: int, K: int) -> bool:
    """Whether :func:`cascaded_lowp_matmul_chained` takes the shape (``[M, K]`` slots times ``[K, N]``)."""
    return bool(_lib.lib().cascmm_chained_supported(M, N, K))


def cascaded_lowp_matmul_chained(a: LeftSlots, w: ChainedWeight, *, bias: Optional[torch.Tensor] = None,
                                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``a @ w (+ bias)`` with BOTH operands already split (two bf16 terms, products hi.hi + hi.lo + lo.hi,
    fp32 accumulation): the second GEMM of a feed-forward block, one launch, no workspace."""
    if not isinstance(a, LeftSlots) or not isinstance(w, ChainedWeight):
        raise TypeError("cascaded_lowp_matmul_chained takes LeftSlots and a ChainedWeight")
    assert a.K == w.K, "Incompatible dimensions"
    if a.device != w.device:
        raise ValueError("operands are on different devices")
    M, K, N = a.M, a.K, w.N
    if out is None:
        out = torch.empty((M, N), device=a.device, dtype=torch.float32)
    else:
        _check_device_tensor(out, "out")
        if out.dtype != torch.float32 or out.numel() != M * N:
            raise ValueError(f"out must hold {M * N} fp32 elements")
    out2 = out if out.dim() == 2 and out.shape == (M, N) else out.view(M, N)
    if N > 1 and out2.stride(1) != 1:
        raise ValueError("out must have unit stride along N")
    if bias is not None:
        bias = _check_bias(bias, out2, N)
    stream = torch.cuda.current_stream(a.device).cuda_stream
    _lib.check(_lib.lib().cascmm_gemm_chained(a.slots.data_ptr(), w.slots.data_ptr(), out2.data_ptr(),
                                              None if bias is None else bias.data_ptr(), M, N, K,
                                              out2.stride(0) if M > 1 else max(N, 1), stream), "cascmm_gemm_chained")
    return out.reshape(*a.batch_shape, N)


def glu_chained_supported(a: torch.Tensor, N: int) -> bool:
    """Whether :func:`cascaded_lowp_matmul_glu_chained` takes ``a`` ([..., K]) times a ``[K, N]`` gated
    weight: the large-tile kernel's shapes (rows % 256, N % 320, K % 32 all zero), fp32 on the GPU."""
    K = a.shape[-1]
    M = a.numel() // K if K else 0
    return bool(a.is_cuda and a.dtype == torch.float32 and M > 0 and M % 256 == 0 and N % 320 == 0 and K % 32 == 0
                and K >= 32 and chained_supported(M, 32, N // 2) and 4 * M * (N // 2) < 2 ** 31)


def glu_chained_worthwhile(a: torch.Tensor, N: int) -> bool:
    """Whether the library's cost estimates put the large-tile kernel with the gate in its store -- the
    only kernel that can write operand slots -- ahead of the best plain kernel plus a gate pass for ``a``
    times a ``[K, N]`` gated weight.  With few tiles on many CUs (1024 rows) they do not, and a
    feed-forward block is faster layer by layer."""
    K = a.shape[-1]
    M = a.numel() // K if K else 0
    return glu_chained_supported(a, N) and _lib.lib().cascmm_select_variant_glu(
        M, N, K, K, N, N // 2, _lib.DT_F32, _lib.FMT_BF16, 2, _lib.PROD_TRI) >= 0


def cascaded_lowp_matmul_glu_chained(a: torch.Tensor, w, *, bias: Optional[torch.Tensor] = None,
                                     out: Optional[LeftSlots] = None) -> LeftSlots:
    """``h = a @ w + bias; value, gate = h.chunk(2, -1); value * gelu(gate)`` like
    :func:`cascaded_lowp_matmul_glu`, with the result written as the :class:`LeftSlots` of the next GEMM
    instead of fp32: ``h`` and the fp32 result never reach memory, and the next GEMM has nothing to split.
    ``w``: the raw ``[K, 2 * inner]`` fp32 weight or a ``PreparedWeight(..., glu=True)`` of it (two bf16
    terms).  Raises CascmmError where :func:`glu_chained_supported` is false."""
    _check_device_tensor(a, "a")
    prepared = isinstance(w, PreparedWeight)
    if prepared:
        if not w.glu or (w.lowp, w.terms) != ("bf16", 2):
            raise ValueError("the prepared weight must be a gated one of two bf16 terms")
        K, N, wptr = w.K, w.N, w.slots.data_ptr()
    else:
        _check_device_tensor(w, "w")
        assert w.is_contiguous(), "Matrix B must be contiguous"
        K, N, wptr = w.shape[-2], w.shape[-1], w.data_ptr()
    assert a.shape[-1] == K, "Incompatible dimensions"
    if a.dtype != torch.float32:
        raise TypeError("the chained gated product takes fp32 tensors")
    bias = _check_bias(bias, a, N)
    batch_dims = a.shape[:-1]
    M = batch_dims.numel()
    a2 = _rows(a.reshape(M, K))
    if a2.data_ptr() % 16 != 0 or (M > 1 and a2.stride(0) % 4 != 0):
        a2 = a2.contiguous()
    if out is None:
        out = LeftSlots.empty(batch_dims, N // 2, a.device)
    elif out.M != M or out.K != N // 2:
        raise ValueError("out holds slots of another shape")
    stream = torch.cuda.current_stream(a.device).cuda_stream
    _lib.check(_lib.lib().cascmm_gemm_glu_chained(a2.data_ptr(), wptr, 1 if prepared else 0, out.slots.data_ptr(), out.slots.numel(),
                                                  None if bias is None else bias.data_ptr(), M, N, K,
                                                  a2.stride(0) if M > 1 else max(K, 1), N, stream), "cascmm_gemm_glu_chained")
    return out


def kernel_listing(variant: int) -> str:
    """What `dump_ptx=True` writes: the variant's name, its kernel's symbol and the kernel's gfx950
    assembly (compiled from the library's sources on first use; without a compiler the two header
    lines and the reason)."""
    l = _lib.lib()
    name, sym = l.cascmm_variant_name(variant), l.cascmm_variant_kernel(variant)
    head = f"// gfx950 kernel variant: {name.decode() if name else variant}\n// kernel: {sym.decode() if sym else '?'}\n"
    if not sym:
        return head
    from . import build
    try:
        return head + build.kernel_isa(sym.decode())
    except (OSError, RuntimeError, KeyError) as e:
        return head + f"// no listing: {e}\n"


def cascaded_lowp_matmul(
    a: torch.Tensor,
    b: torch.Tensor,
    *,
    out: Optional[torch.Tensor] = None,
    dump_ptx: bool = False,
    lowp: Optional[str] = None,
    terms: Optional[int] = None,
    products: str = "tri",
    bias: Optional[torch.Tensor] = None,
    variant: int = -1,
    b_exp: Optional[torch.Tensor] = None,
    tensor_exps: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    if lowp is None or terms is None:
        d_lowp, d_terms = default_cascade(a.dtype)
        lowp = d_lowp if lowp is None else lowp
        terms = d_terms if terms is None else terms
    if isinstance(b, PreparedWeight):
        res = out.view(-1, b.out_features) if out is not None else None
        return cascaded_lowp_matmul_prepared([a], [b], outs=None if res is None else [res],
                                             biases=None if bias is None else [bias], products=products,
                                             variant=variant)[0]
    assert a.shape[-1] == b.shape[-2], "Incompatible dimensions"
    # assert a.is_contiguous(), "Matrix A must be contiguous"
    assert b.is_contiguous(), "Matrix B must be contiguous"
    _check_device_tensor(a, "a")
    _check_device_tensor(b, "b")
    if a.dtype not in _DTYPES:
        raise TypeError(f"cascaded_lowp_matmul: unsupported dtype {a.dtype}")
    if b.dtype != a.dtype:
        raise TypeError(f"cascaded_lowp_matmul: a is {a.dtype} but b is {b.dtype}")
    if lowp not in _lib.FMT_BY_NAME:
        raise ValueError(f"lowp must be one of {sorted(_lib.FMT_BY_NAME)}, got {lowp!r}")
    if products not in _lib.PROD_BY_NAME:
        raise ValueError(f"products must be 'tri' or 'full', got {products!r}")
    fmt, prod = _lib.FMT_BY_NAME[lowp], _lib.PROD_BY_NAME[products]
    bias = _check_bias(bias, a, b.shape[-1])

    K, N = b.shape[-2], b.shape[-1]

    if b.dim() > 2:
        # batched right operand: torch.matmul broadcasting, one GEMM per batch entry
        if a.dim() < 2:
            raise ValueError("a must have at least 2 dims when b is batched")
        batch = torch.broadcast_shapes(a.shape[:-2], b.shape[:-2])
        rows = a.shape[-2]
        a_b = a.expand(*batch, rows, K).reshape(-1, rows, K)
        b_b = b.expand(*batch, K, N).reshape(-1, K, N)
        res = out if out is not None else torch.empty((*batch, rows, N), device=a.device, dtype=a.dtype)
        if tuple(res.shape) != (*batch, rows, N) or not res.is_contiguous():
            raise ValueError("out must be a contiguous tensor of the broadcast result shape")
        res_b = res.view(-1, rows, N)
        for i in range(a_b.shape[0]):
            _gemm_2d(_rows(a_b[i]), b_b[i].contiguous(), res_b[i], bias, fmt, terms, prod, variant)
        return res

    batch_dims = a.shape[:-1]
    M = batch_dims.numel()
    a2 = _rows(a.reshape(M, K))

    if out is None:
        out = torch.empty((M, N), device=a.device, dtype=a.dtype)
    else:
        _check_device_tensor(out, "out")
        if out.dtype != a.dtype:
            raise TypeError("out must have the dtype of a")
        if out.numel() != M * N:
            raise ValueError(f"out has {out.numel()} elements, expected {M * N}")
    out2 = out if out.dim() == 2 and out.shape == (M, N) else out.view(M, N)
    if N > 1 and out2.stride(1) != 1:
        raise ValueError("out must have unit stride along N")

    _gemm_2d(a2, b, out2, bias, fmt, terms, prod, variant, b_exp, tensor_exps)

    if dump_ptx:
        # the reference writes the PTX of the kernel it launched (cascaded_lowp_matmul.py:170-171);
        # here the file holds the gfx950 assembly of the GEMM kernel that ran
        l = _lib.lib()
        v = variant if variant >= 0 else l.cascmm_select_variant(
            M, N, K, a2.stride(0), b.stride(0), out2.stride(0), _DTYPES[a.dtype], fmt, terms, prod)
        with open("dump.ptx", "w") as f:
            f.write(kernel_listing(v & 0xFFFF))

    return out.reshape(*batch_dims, N)
