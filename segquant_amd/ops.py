"""torch-facing wrappers over the C ABI of libsegq.

torch is plumbing here: it owns device memory and the current stream.  Every
function takes CUDA (ROCm) tensors, allocates outputs with torch, hands raw
pointers to the library and raises ``RuntimeError`` on a non-zero status, which
is what the reference's pybind functions do (segquant/src/real_quant/seg_utils.h).

Two layers:

* :func:`quantize` and :func:`gemm` expose the library's own, richer interface
  (column segments, ranges, merged DualScale codes, fused bias).
* :func:`real_quantized_gemm_scaled`, :func:`real_quantized_gemm_dual_scaled`,
  :func:`real_quantized_quantize_weights` and :func:`fake_e4m3fy` keep the
  reference's tensor contract (segquant/src/real_quant/real_gemm.cu:643-894,
  :538-638; segquant/src/fake_quant/quantizer_fp8.cpp:25-39).
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import _lib as L

FMT_INT8 = "int8"
FMT_INT4 = "int4"
FMT_E4M3 = "fpe4m3"

_CODE = {FMT_INT8: L.CODE_I8, FMT_E4M3: L.CODE_E4M3, FMT_INT4: L.CODE_I4}
_DTYPE = {torch.float32: L.F32, torch.float16: L.F16, torch.bfloat16: L.BF16}


def _dt(t: torch.dtype) -> int:
    try:
        return _DTYPE[t]
    except KeyError:
        raise RuntimeError(f"unsupported float dtype {t}") from None


def _need_cuda(*ts):
    for t in ts:
        if t is not None and not t.is_cuda:
            raise RuntimeError("libsegq needs tensors on the GPU")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device=None) -> int:
    """The current torch stream of ``device`` (default: the current device) as a hipStream_t."""
    if device is None or device.index is None:
        idx = torch.cuda.current_device()
    else:
        idx = device.index
    if _raw_stream is not None:  # the short way: no Stream object is built
        return _raw_stream(idx)
    return torch.cuda.current_stream(idx).cuda_stream


# When set to a list, every quantise / GEMM launch is bracketed by events on the
# launching stream and (kind, start, end, info) is appended; see record_launches.
_launch_log = None


class record_launches:
    """Context manager: collect (kind, start_event, end_event, info) for each
    kernel launch made through this module.  Read ``elapsed_time`` after a
    device synchronisation."""

    def __init__(self):
        self.log = []

    def __enter__(self):
        global _launch_log
        self._prev = _launch_log
        _launch_log = self.log
        return self.log

    def __exit__(self, *exc):
        global _launch_log
        _launch_log = self._prev
        return False


def recording_launches() -> bool:
    """Whether a ``record_launches`` block is active (kernels are then launched one per call
    so that each can be bracketed by its own events)."""
    return _launch_log is not None


def _launch(kind, info, fn):
    if _launch_log is None:
        return fn()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    rc = fn()
    e1.record()
    _launch_log.append((kind, e0, e1, info))
    return rc


# enum segq_pre_op
PRE_OPS = {"gelu_tanh": 1, "gelu": 2, "silu": 3}


def code_dtype(fmt: str) -> torch.dtype:
    """Storage dtype of codes: int8 as int8, e4m3 and packed int4 as uint8
    (segquant/src/real_quant/seg_utils.h:25-45)."""
    return torch.int8 if fmt == FMT_INT8 else torch.uint8


# ---------------------------------------------------------------------------
# quantise
# ---------------------------------------------------------------------------
def quantize(x: torch.Tensor, fmt: str, scale: torch.Tensor, scale_neg: Optional[torch.Tensor] = None, **kw):
    """Quantise a 2-D float matrix ``x`` (rows, cols) to codes: :func:`quantize_desc` + one
    ``segq_quantize`` launch.  Returns the code tensor, or ``(Xp, Xn)`` when ``two_tensors``."""
    d, result, info, _keep = quantize_desc(x, fmt, scale, scale_neg, **kw)
    L.check(_launch("quantize", info, lambda: L.lib().segq_quantize(C.byref(d), _stream())))
    return result


def quantize_launch(q):
    """Enqueue the quantise launch described by ``q`` (the tuple :func:`quantize_desc` returns);
    returns its code tensor(s)."""
    d, result, info, _keep = q
    L.check(_launch("quantize", info, lambda: L.lib().segq_quantize(C.byref(d), _stream())))
    return result


def quantize_many(qs):
    """Enqueue several quantise launches (tuples from :func:`quantize_desc`) through one
    ``segq_quantize_many`` call: neighbours that the same kernel instance serves share a launch.
    Returns the code tensor(s) of each."""
    if not qs:
        return []
    arr = (L.QuantDesc * len(qs))(*[q[0] for q in qs])  # (copies of the descriptors; the tensors stay alive in qs)
    info = dict(many=[q[2] for q in qs])
    L.check(_launch("quantize", info, lambda: L.lib().segq_quantize_many(arr, len(qs), _stream())))
    return [q[1] for q in qs]


def quantize_desc(x: torch.Tensor, fmt: str, scale: torch.Tensor, scale_neg: Optional[torch.Tensor] = None, *,
             seg_rows: int = 0, seg_stride: int = 0, row_stride: int = 0,
             kseg_bounds: Optional[Sequence[int]] = None, kseg_stride: int = 0,
             dual: bool = False, dual_kseg_mask: int = 0xFFFFFFFF, dynamic: bool = False,
             two_tensors: bool = False, out: Optional[torch.Tensor] = None,
             out_neg: Optional[torch.Tensor] = None, pre_op: Optional[str] = None,
             gate: Optional[torch.Tensor] = None, col_div: Optional[torch.Tensor] = None):
    """The ``segq_quant_desc`` of a quantise launch, its output tensor(s), the launch's
    description for ``record_launches`` and the tensors the descriptor points into
    (keep them alive until the launch is enqueued).

    See ``segq_quantize`` in include/segq.h for the scale indexing.  The result is the
    code tensor, or ``(Xp, Xn)`` when ``two_tensors`` (DualScale in the
    reference's two-tensor layout).  With ``dynamic`` the scale tensors are
    written by the kernel.  ``pre_op`` ("gelu_tanh", "gelu", "silu") fuses the
    activation function in front of the linear: op(x) is quantised, or
    x * op(gate) when ``gate`` (same shape and dtype as ``x``) is given.
    ``col_div``: one divisor per column (SmoothQuant's ``s``, any float dtype; it is
    used rounded to ``x.dtype`` as the reference's ``x.div_(s.to(x.dtype))`` does),
    applied after the ``pre_op``.
    """
    _need_cuda(x, scale, scale_neg, gate)
    if x.dim() != 2 or x.stride(1) != 1:
        raise RuntimeError("quantize expects a 2-D tensor with a contiguous last dimension")
    rows, cols = x.shape
    ccols = cols // 2 if fmt == FMT_INT4 else cols
    if out is None:
        out = torch.empty((rows, ccols), dtype=code_dtype(fmt), device=x.device)
    if two_tensors and out_neg is None:
        out_neg = torch.empty_like(out)
    d = L.QuantDesc()
    d.x = x.data_ptr(); d.x_dtype = _dt(x.dtype); d.code_fmt = _CODE[fmt]
    d.rows = rows; d.cols = cols; d.ldx = x.stride(0) if rows > 1 else cols
    d.codes = out.data_ptr(); d.codes_neg = out_neg.data_ptr() if two_tensors else None
    d.ld_codes = out.stride(0) if rows > 1 else ccols
    if scale.dtype != torch.float32 or (scale_neg is not None and scale_neg.dtype != torch.float32):
        raise RuntimeError("scales must be float32")
    d.scale = scale.data_ptr(); d.scale_neg = scale_neg.data_ptr() if scale_neg is not None else None
    d.seg_rows = seg_rows; d.seg_stride = seg_stride; d.row_stride = row_stride; d.kseg_stride = kseg_stride
    if kseg_bounds is None:
        d.n_kseg = 1
    else:
        d.n_kseg = len(kseg_bounds) - 1
        if d.n_kseg > L.SEGQ_MAX_KSEG:
            raise RuntimeError(f"at most {L.SEGQ_MAX_KSEG} column segments")
        for i, b in enumerate(kseg_bounds):
            d.kseg_bounds[i] = int(b)
    d.dual = 1 if dual else 0; d.dual_kseg_mask = dual_kseg_mask & 0xFFFFFFFF; d.dynamic = 1 if dynamic else 0
    if pre_op is not None:
        if pre_op not in PRE_OPS:
            raise RuntimeError(f"pre_op must be one of {sorted(PRE_OPS)}")
        d.pre_op = PRE_OPS[pre_op]
    if col_div is not None:
        _need_cuda(col_div)
        if col_div.numel() != cols:
            raise RuntimeError("col_div needs one entry per column")
        col_div = col_div.reshape(-1).to(x.dtype).to(torch.float32).contiguous()
        d.col_div = col_div.data_ptr()
    if gate is not None:
        if pre_op is None or gate.shape != x.shape or gate.dtype != x.dtype or gate.stride(1) != 1:
            raise RuntimeError("gate needs a pre_op and the shape, dtype and contiguous rows of x")
        d.gate = gate.data_ptr(); d.ld_gate = gate.stride(0) if rows > 1 else cols
    info = dict(rows=rows, cols=cols, x_bytes=x.element_size() * (2 if gate is not None else 1),
                code_bytes=0.5 if fmt == FMT_INT4 else 1.0, tensors=2 if two_tensors else 1, dynamic=bool(dynamic))
    return d, ((out, out_neg) if two_tensors else out), info, (x, scale, scale_neg, gate, col_div, out, out_neg)


# ---------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------
@dataclass
class Range:
    """A run of contraction columns sharing one (sx, sw) pair; see segq_krange."""
    k_begin: int
    k_len: int
    sx: Optional[torch.Tensor]
    sw: Optional[torch.Tensor]
    a_sel: int = 0
    sx_row_stride: int = 0
    sw_col_stride: int = 0


_int4_ws = {}
_retired_ws = []  # outgrown buffers stay allocated: a captured HIP graph may still hold their address


def int4_workspace(device, nbytes: int) -> torch.Tensor:
    """A scratch tensor of at least ``nbytes`` for ``gemm``'s ``workspace`` (expanded int4
    weights, parked partial sums of int8 ranges, split-K partial results), one per device
    and stream: launches on one stream run in order and the contents only live for the
    duration of one GEMM launch, so every layer on that stream can share it.  Grown on
    demand; a buffer that was handed out is never freed."""
    dev = torch.device(device)
    if dev.index is None:
        dev = torch.device(dev.type, torch.cuda.current_device())
    key = (dev, _stream(dev))
    ws = _int4_ws.get(key)
    if ws is None or ws.numel() < nbytes:
        if ws is not None:
            _retired_ws.append(ws)
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        _int4_ws[key] = ws
    return ws


def gemm_workspace_bytes(g) -> int:
    """Workspace the launch described by ``g`` (the tuple :func:`gemm_desc` returns) would use if it
    were lent as much as the library can make use of; 0 if it has no use for one
    (``segq_gemm_workspace_bytes``)."""
    n = C.c_int64(0)
    L.check(L.lib().segq_gemm_workspace_bytes(C.byref(g[0]), C.byref(n)))
    return n.value


# tile ids of the 8-wave kernels (segq_gemm_desc.tile) -> rows x columns of the output tile
TILE_SHAPES = {1: "256x256", 2: "256x128", 3: "128x128", 4: "64x128", 5: "128x256", 6: "256x256", 7: "256x256", 8: "256x128",
               11: "256x256", 12: "256x128", 13: "128x256", 14: "128x128", 15: "192x288", 16: "288x192", 17: "256x192", 18: "192x256", 19: "128x128", 20: "384x192", 21: "128x96"}


def gemm_plan(g, workspace: Optional[torch.Tensor] = None) -> dict:
    """What the library would launch for ``g`` (lent ``workspace``, if given): its tile id and
    shape, the number of workgroups sharing a tile's K steps, whether ranges are parked
    (``segq_gemm_plan``)."""
    d = g[0]
    if workspace is not None:
        d.workspace = workspace.data_ptr(); d.workspace_bytes = workspace.numel() * workspace.element_size()
    tile, splits, parked = C.c_int32(0), C.c_int32(0), C.c_int32(0)
    L.check(L.lib().segq_gemm_plan(C.byref(d), C.byref(tile), C.byref(splits), C.byref(parked)))
    family = "gemm_pipe_kernel" if tile.value >= 11 else "gemm_kernel"
    return dict(tile=tile.value, shape=TILE_SHAPES.get(tile.value, "?"), splits=splits.value, parked=bool(parked.value),
                kernel=f"segq::{family}<{TILE_SHAPES.get(tile.value, '?').replace('x', ',')}>")


def gemm_launch(g, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Enqueue the GEMM described by ``g``, lending it ``workspace`` (a byte tensor) if given."""
    d, out, info, _keep = g
    if workspace is not None:
        _need_cuda(workspace)
        d.workspace = workspace.data_ptr(); d.workspace_bytes = workspace.numel() * workspace.element_size()
    L.check(_launch("gemm", info, lambda: L.lib().segq_gemm(C.byref(d), _stream())))
    return out


def park_bytes(m: int, n: int) -> int:
    """Workspace that lets int8 codes with several ranges run on every tile size
    (one fp32 tile per workgroup; the largest tile is 288 wide)."""
    return 4 * (m + 288) * (n + 288)


def split_bytes(m: int, n: int, splits: int = 16, park: bool = False) -> int:
    """Workspace for a GEMM whose K steps are shared by up to ``splits`` workgroups per
    tile: the fp32 partial results and, for int8 with several ranges (``park``), the
    parking room of all those workgroups.  (Two shares are kept as whole tiles, with one
    arrival counter per tile behind them; ``gemm_workspace_bytes`` gives the exact figure.)"""
    counters = 4 * -(-m // 128) * -(-n // 128) + 512
    return splits * park_bytes(m, n) * (2 if park else 1) + counters



def gemm(a: torch.Tensor, b: torch.Tensor, ranges: Sequence[Range], **kw) -> torch.Tensor:
    """Segmented GEMM with fused de-quantisation and bias: :func:`gemm_desc` + one ``segq_gemm`` call."""
    d, out, info, _keep = gemm_desc(a, b, ranges, **kw)
    L.check(_launch("gemm", info, lambda: L.lib().segq_gemm(C.byref(d), _stream())))
    return out


def linear(q, g, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``segq_linear``: the quantise launch described by ``q`` and the GEMM described by ``g`` (the
    tuples :func:`quantize_desc` and :func:`gemm_desc` return) in one call of the library, the
    GEMM lent ``workspace`` if given.  The GEMM must read the code tensor(s) the quantise step
    writes, and with dynamic scales the scale tensors it fills."""
    qd, _codes, qinfo, _k1 = q
    gd, out, ginfo, _k2 = g
    if workspace is not None:
        _need_cuda(workspace)
        gd.workspace = workspace.data_ptr(); gd.workspace_bytes = workspace.numel() * workspace.element_size()
    L.check(_launch("linear", dict(q=qinfo, g=ginfo), lambda: L.lib().segq_linear(C.byref(qd), C.byref(gd), _stream())))
    return out


def gemm_desc(a: torch.Tensor, b: torch.Tensor, ranges: Sequence[Range], *, m: int, n: int, a_fmt: str, b_fmt: str,
         out_dtype, lda: int, ldb: int, a_neg: Optional[torch.Tensor] = None,
         bias: Optional[torch.Tensor] = None, batch: int = 1, batch_stride_a: int = 0, batch_stride_b: int = 0,
         batch_stride_sx: int = 0, batch_stride_sw: int = 0, out: Optional[torch.Tensor] = None,
         tile: int = 0, workspace: Optional[torch.Tensor] = None,
         group_dequant: Optional[torch.Tensor] = None, split_k: int = 0,
         addend: Optional[torch.Tensor] = None, lowrank=None, out_codes: Optional[dict] = None):
    """The ``segq_gemm_desc`` of a segmented GEMM with fused de-quantisation and bias, its output
    tensor, the launch's description and the tensors the descriptor points into.

    ``out_codes``: ``dict(fmt=, scale=, scale_neg=None, pre_op=None)``: the launch writes the CODES
    the next linear's quantise step would make of the output (rounded to ``out_dtype``, ``pre_op``
    applied, static per-tensor ``scale``; with ``scale_neg`` the two DualScale tensors) instead of
    the floats; the returned "output" is then the code tensor, or the pair (Xp, Xn).  See
    ``segq_gemm_desc.out_codes``.

    ``lowrank``: a pair ``(T, L2T)`` of 16-bit matrices in the output's dtype, (m, r) and (n, r)
    with r a multiple of 32: ``T @ L2T.T`` is added to the result inside the epilogue (the SVD
    optimiser's branch x L1 L2 with T = x L1; see ``segq_gemm_desc.lowrank_t``).

    ``out_dtype`` is a torch float dtype, or the string ``"acc"`` for the raw
    accumulators (int32 for integer codes, float32 for e4m3).  ``workspace``: a
    byte tensor the library may expand int4 weights into, or park the sums of
    finished int8 ranges in (see ``int4_workspace``, ``park_bytes``).
    """
    _need_cuda(a, b, a_neg, bias)
    raw = out_dtype == "acc"
    if raw:
        tdt = torch.float32 if a_fmt == FMT_E4M3 else torch.int32
    else:
        tdt = out_dtype
    oc = oc_neg = None
    if out_codes is not None:
        if raw or batch != 1 or out is not None:
            raise RuntimeError("out_codes needs a float out_dtype, one problem and no out tensor")
        oc = torch.empty((m, n), dtype=code_dtype(out_codes["fmt"]), device=a.device)
        if out_codes.get("scale_neg") is not None:
            oc_neg = torch.empty_like(oc)
    elif out is None:
        out = torch.empty((batch, m, n) if batch > 1 else (m, n), dtype=tdt, device=a.device)
    d = L.GemmDesc()
    d.a_fmt = _CODE[a_fmt]; d.b_fmt = _CODE[b_fmt]
    d.out_dtype = L.ACC if raw else _dt(tdt)
    d.m = m; d.n = n
    d.a = a.data_ptr(); d.a_neg = a_neg.data_ptr() if a_neg is not None else None; d.lda = lda
    d.b = b.data_ptr(); d.ldb = ldb
    d.ldo = n
    if oc is not None:
        sc, scn = out_codes["scale"], out_codes.get("scale_neg")
        _need_cuda(sc, scn)
        if sc.dtype != torch.float32 or sc.numel() != 1 or (scn is not None and (scn.dtype != torch.float32 or scn.numel() != 1)):
            raise RuntimeError("out_codes takes one float32 scale (and one for the negative side)")
        d.out_codes = oc.data_ptr(); d.ld_out_codes = n
        d.out_codes_neg = oc_neg.data_ptr() if oc_neg is not None else None
        d.out_scale = sc.data_ptr(); d.out_scale_neg = scn.data_ptr() if scn is not None else None
        d.out_code_fmt = _CODE[out_codes["fmt"]]
        pre = out_codes.get("pre_op")
        if pre is not None and pre not in PRE_OPS:
            raise RuntimeError(f"pre_op must be one of {sorted(PRE_OPS)}")
        d.out_pre_op = PRE_OPS[pre] if pre is not None else 0
    else:
        d.out = out.data_ptr()
    if oc is None and batch == 1 and out.dim() == 2:  # a view of a wider buffer (a column slice, padded rows) is written in place
        if out.shape != (m, n) or out.dtype != tdt or (n > 1 and out.stride(1) != 1) or (m > 1 and out.stride(0) < n):
            raise RuntimeError("out must be an (m, n) tensor of the output dtype with contiguous rows")
        if m > 1:
            d.ldo = out.stride(0)
    if bias is not None:
        if bias.numel() != n or not bias.is_contiguous():
            raise RuntimeError("bias must be a contiguous vector with one entry per output column")
        d.bias = bias.data_ptr(); d.bias_dtype = _dt(bias.dtype)
    d.batch = batch; d.batch_stride_a = batch_stride_a; d.batch_stride_b = batch_stride_b
    d.batch_stride_out = m * n; d.batch_stride_sx = batch_stride_sx; d.batch_stride_sw = batch_stride_sw
    if not 1 <= len(ranges) <= L.SEGQ_MAX_RANGES:
        raise RuntimeError(f"1..{L.SEGQ_MAX_RANGES} ranges")
    d.n_ranges = len(ranges); d.tile = tile; d.split_k = split_k
    if workspace is not None:
        _need_cuda(workspace)
        d.workspace = workspace.data_ptr(); d.workspace_bytes = workspace.numel() * workspace.element_size()
    if addend is not None:
        _need_cuda(addend)
        if raw or addend.dtype != tdt or addend.shape != out.shape or not addend.is_contiguous():
            raise RuntimeError("addend must be a contiguous tensor of the output's shape and dtype")
        d.addend = addend.data_ptr(); d.ld_addend = n
    if lowrank is not None:
        t_lr, l2t = lowrank
        _need_cuda(t_lr, l2t)
        if raw or t_lr.dtype != tdt or l2t.dtype != tdt or t_lr.dim() != 2 or l2t.dim() != 2 or t_lr.shape[0] != m or \
                l2t.shape[0] != n or t_lr.shape[1] != l2t.shape[1] or t_lr.stride(1) != 1 or l2t.stride(1) != 1:
            raise RuntimeError("lowrank is (T (m, r), L2T (n, r)) in the output's dtype with contiguous rows")
        d.lowrank_t = t_lr.data_ptr(); d.ld_lowrank_t = t_lr.stride(0)
        d.lowrank_l2t = l2t.data_ptr(); d.ld_lowrank_l2t = l2t.stride(0)
        d.lowrank_rank = t_lr.shape[1]
    if group_dequant is not None:
        _need_cuda(group_dequant)
        if group_dequant.dtype != torch.float32 or group_dequant.dim() != 2 or group_dequant.stride(1) != 1:
            raise RuntimeError("group_dequant is a float32 matrix (groups, n) with contiguous rows")
        d.group_dequant = group_dequant.data_ptr(); d.group_dequant_stride = group_dequant.stride(0)
    for i, r in enumerate(ranges):
        kr = d.ranges[i]
        kr.k_begin = r.k_begin; kr.k_len = r.k_len; kr.a_sel = r.a_sel
        kr.sx_row_stride = r.sx_row_stride; kr.sw_col_stride = r.sw_col_stride
        _need_cuda(r.sx, r.sw)
        for s in (r.sx, r.sw):
            if s is not None and s.dtype != torch.float32:
                raise RuntimeError("scales must be float32")
        kr.sx = r.sx.data_ptr() if r.sx is not None else None
        kr.sw = r.sw.data_ptr() if r.sw is not None else None
    info = dict(m=m, n=n, batch=batch, k_alg=sum(r.k_len for r in ranges if r.a_sel in (0, 2)),
                k_exec=sum(r.k_len for r in ranges), a_fmt=a_fmt, b_fmt=b_fmt)
    if oc is not None:
        out = (oc, oc_neg) if oc_neg is not None else oc
        info["codes_out"] = True
    return d, out, info, (a, b, a_neg, bias, workspace, group_dequant, addend, lowrank, out, out_codes, list(ranges))


# ---------------------------------------------------------------------------
# the reference's tensor contract
# ---------------------------------------------------------------------------
def _shapes(inputs: torch.Tensor, weights: torch.Tensor, fmt_w: str):
    S = inputs.shape[0]
    K = inputs.shape[-1]
    M = 1
    for d in inputs.shape[1:-1]:
        M *= d
    if weights.shape[0] != S:
        raise RuntimeError("inputs and weights must have the same number of segments")
    if fmt_w == FMT_INT4:
        N = weights.shape[1] * 2 // K  # segquant/src/real_quant/real_gemm.cu:670
        if weights.dim() != 2 or N * K != weights.shape[1] * 2:
            raise RuntimeError("int4 weights must be (segments, N*K/2) bytes")
    else:
        if weights.dim() != 3 or weights.shape[2] != K:
            raise RuntimeError("weights must be (segments, N, K)")
        N = weights.shape[1]
    return S, M, N, K


def _check_contract(inputs, weights, fmt_w, *scales):
    _need_cuda(inputs, weights, *scales)
    if not inputs.is_contiguous() or not weights.is_contiguous():
        raise RuntimeError("tensor must be contiguous")
    if weights.dtype != code_dtype(fmt_w):
        raise RuntimeError("tensor dtype failed")
    for s in scales:
        if s.dtype != torch.float32 or not s.is_contiguous():
            raise RuntimeError("scales must be contiguous float32")


def real_quantized_gemm_scaled(fmt_a: str, fmt_w: str, inputs: torch.Tensor, weights: torch.Tensor,
                               scale_x: torch.Tensor, scale_w: torch.Tensor) -> torch.Tensor:
    """``<prefix>_real_quantized_gemm_scaled`` (segquant/src/real_quant/real_gemm.cu:643-750).

    inputs (S, ..., M, K) float; weights (S, N, K) codes or (S, N*K/2) bytes for
    int4; scale_x has S or S*M entries, scale_w S or S*N; returns a new
    (S, ..., M, N) tensor in ``inputs.dtype``.  One quantise launch over all S
    segments and one batched GEMM launch; no temporaries beyond the codes.
    """
    _check_contract(inputs, weights, fmt_w, scale_x, scale_w)
    S, M, N, K = _shapes(inputs, weights, fmt_w)
    per_seg_x = scale_x.numel() == S
    per_seg_w = scale_w.numel() == S
    if not per_seg_x and scale_x.numel() != S * M:
        raise RuntimeError(f"scale_x has {scale_x.numel()} entries, expected {S} or {S * M}")
    if not per_seg_w and scale_w.numel() != S * N:
        raise RuntimeError(f"scale_w has {scale_w.numel()} entries, expected {S} or {S * N}")
    codes = quantize(inputs.view(S * M, K), fmt_a, scale_x, seg_rows=M,
                     seg_stride=1 if per_seg_x else M, row_stride=0 if per_seg_x else 1)
    out = torch.empty((*inputs.shape[:-1], N), dtype=inputs.dtype, device=inputs.device)
    kb = K // 2 if fmt_w == FMT_INT4 else K
    ka = K // 2 if fmt_a == FMT_INT4 else K
    gemm(codes, weights, [Range(0, K, scale_x, scale_w, 0, 0 if per_seg_x else 1, 0 if per_seg_w else 1)],
         m=M, n=N, a_fmt=fmt_a, b_fmt=fmt_w, out_dtype=inputs.dtype, lda=ka, ldb=kb,
         batch=S, batch_stride_a=M * ka, batch_stride_b=N * kb,
         batch_stride_sx=1 if per_seg_x else M, batch_stride_sw=1 if per_seg_w else N, out=out)
    return out


def real_quantized_gemm_dual_scaled(fmt_a: str, fmt_w: str, inputs: torch.Tensor, weights: torch.Tensor,
                                    pos_scale_x: torch.Tensor, neg_scale_x: torch.Tensor,
                                    scale_w: torch.Tensor) -> torch.Tensor:
    """``<prefix>_real_quantized_gemm_dual_scaled`` (segquant/src/real_quant/real_gemm.cu:752-894).

    The activations are stored once, as the code of the branch each element
    took; the GEMM reads them as two ranges (non-negative codes with the
    positive scale, negative codes with the negative scale).
    """
    _check_contract(inputs, weights, fmt_w, pos_scale_x, neg_scale_x, scale_w)
    S, M, N, K = _shapes(inputs, weights, fmt_w)
    per_seg_x = pos_scale_x.numel() == S
    per_seg_w = scale_w.numel() == S
    if pos_scale_x.numel() != neg_scale_x.numel() or (not per_seg_x and pos_scale_x.numel() != S * M):
        raise RuntimeError("pos/neg scale_x must both have S or S*M entries")
    if not per_seg_w and scale_w.numel() != S * N:
        raise RuntimeError(f"scale_w has {scale_w.numel()} entries, expected {S} or {S * N}")
    codes = quantize(inputs.view(S * M, K), fmt_a, pos_scale_x, neg_scale_x, seg_rows=M,
                     seg_stride=1 if per_seg_x else M, row_stride=0 if per_seg_x else 1, dual=True)
    out = torch.empty((*inputs.shape[:-1], N), dtype=inputs.dtype, device=inputs.device)
    kb = K // 2 if fmt_w == FMT_INT4 else K
    rs, cs = (0 if per_seg_x else 1), (0 if per_seg_w else 1)
    gemm(codes, weights,
         [Range(0, K, pos_scale_x, scale_w, 2, rs, cs), Range(0, K, neg_scale_x, scale_w, 3, rs, cs)],
         m=M, n=N, a_fmt=fmt_a, b_fmt=fmt_w, out_dtype=inputs.dtype, lda=K, ldb=kb,
         batch=S, batch_stride_a=M * K, batch_stride_b=N * kb,
         batch_stride_sx=1 if per_seg_x else M, batch_stride_sw=1 if per_seg_w else N, out=out)
    return out


def real_quantized_quantize_weights(fmt: str, weights: torch.Tensor, outputs: torch.Tensor, scale_w) -> None:
    """``real_quantized_quantize_weights`` (segquant/src/real_quant/seg_utils.h:82-119):
    a python float selects the one-scale overload, a tensor the per-row one."""
    _need_cuda(weights, outputs)
    if weights.dim() != 2 or not weights.is_contiguous() or not outputs.is_contiguous():
        raise RuntimeError("tensor must be contiguous")
    if outputs.dtype != code_dtype(fmt):
        raise RuntimeError("tensor dtype failed")
    n, k = weights.shape
    need = n * k // 2 if fmt == FMT_INT4 else n * k
    if fmt == FMT_INT4 and (n * k) % 2:
        raise RuntimeError("Quantization to int4 requires the number of elements to be even")
    if outputs.numel() != need:
        raise RuntimeError("output numel must match the weight" + (" (half of it for int4)" if fmt == FMT_INT4 else ""))
    lib = L.lib()
    if isinstance(scale_w, torch.Tensor):
        _need_cuda(scale_w)
        if scale_w.dtype != torch.float32 or scale_w.numel() != n or not scale_w.is_contiguous():
            raise RuntimeError("scale_w must be a contiguous float32 vector with one entry per row")
        rc = lib.segq_quantize_weights_rows(weights.data_ptr(), _dt(weights.dtype), n, k, outputs.data_ptr(),
                                            _CODE[fmt], scale_w.data_ptr(), _stream())
    elif isinstance(scale_w, float):
        rc = lib.segq_quantize_weights_scalar(weights.data_ptr(), _dt(weights.dtype), n, k, outputs.data_ptr(),
                                              _CODE[fmt], C.c_float(scale_w), _stream())
    else:  # the float overload is noconvert (seg_utils.h:99)
        raise TypeError("scale_w must be a python float or a float32 tensor")
    L.check(rc)


def quantize_weights_groups(fmt: str, weights: torch.Tensor, scales: torch.Tensor, group: int = 128) -> torch.Tensor:
    """Weight codes with one scale per (row, group of ``group`` contraction columns).

    ``weights`` is (n, k) float, ``scales`` a contiguous float32 (k / group, n) matrix of
    multiplicative scales (``code = round(w * scale)``), the layout whose reciprocal
    ``segq_gemm`` takes as ``group_dequant``.  Returns (n, k) codes, or (n, k / 2) bytes
    for int4.  The reference has no group-wise scales
    (segquant/src/real_quant/real_gemm.cu:538-638 takes a scalar or one scale per row);
    a group is quantised exactly like a K segment with static per-row scales.  One launch
    (``segq_quantize_weights_groups``) for any number of groups.
    """
    _need_cuda(weights, scales)
    if weights.dim() != 2 or not weights.is_contiguous():
        raise RuntimeError("tensor must be contiguous")
    n, k = weights.shape
    if group % 32 or k % group:
        raise RuntimeError("the group size must be a multiple of 32 that divides k")
    ng = k // group
    if scales.dtype != torch.float32 or tuple(scales.shape) != (ng, n) or not scales.is_contiguous():
        raise RuntimeError(f"scales must be a contiguous float32 ({ng}, {n}) matrix")
    out = torch.empty((n, k // 2 if fmt == FMT_INT4 else k), dtype=code_dtype(fmt), device=weights.device)
    L.check(L.lib().segq_quantize_weights_groups(weights.data_ptr(), _dt(weights.dtype), n, k, out.data_ptr(), _CODE[fmt],
                                                 scales.data_ptr(), group, _stream()))
    return out


def repack_int4_cols_to_rows(colpacked: torch.Tensor, out_features: int, cols: int) -> torch.Tensor:
    """int4 codes packed down the columns, as the reference's GPTQ loop leaves them (a flat uint8
    tensor read as (cols, out / 2): two output rows per byte), to the row-packed layout every
    int4 consumer reads: a flat uint8 tensor of ``out * cols / 2`` bytes, (out, cols / 2), two
    input channels per byte.  Device counterpart of ``GPTQCalibrator.colpacked1d_to_rowpacked1d``
    (segquant/calibrator/calibrator.py:202-223)."""
    _need_cuda(colpacked)
    if out_features % 2 or cols % 2:
        raise AssertionError("Output and columns must be even for int4 quantization.")
    if colpacked.dtype != torch.uint8 or colpacked.numel() != out_features * cols // 2 or not colpacked.is_contiguous():
        raise RuntimeError("colpacked must be a contiguous uint8 tensor of out * cols / 2 bytes")
    res = torch.empty(out_features * cols // 2, dtype=torch.uint8, device=colpacked.device)
    L.check(L.lib().segq_repack_int4_cols_to_rows(colpacked.data_ptr(), res.data_ptr(), out_features, cols, _stream()))
    return res


def fake_e4m3fy(inputs: torch.Tensor) -> torch.Tensor:
    """``fake_e4m3fy`` on the GPU (segquant/src/fake_quant/quantizer_fp8.cu:43-51)."""
    _need_cuda(inputs)
    x = inputs.contiguous()
    out = torch.empty_like(x)
    L.check(L.lib().segq_fake_e4m3(x.data_ptr(), out.data_ptr(), _dt(x.dtype), x.numel(), _stream()))
    return out
