"""CPU oracle for the real-quantized segmented linear.  TEST INFRASTRUCTURE ONLY.

This file is a from-scratch numpy restatement of the arithmetic that the
reference implements in CUDA/CUTLASS and in its torch "fake quant" path.  It
is the checker for the HIP kernels: only tests, the smoke check and the bench's
``cpu_baseline`` leg may import it.  Nothing in the shipped package does.

Every public function names the reference file:line it restates.  Conventions
taken from the reference:

* a *scale* is multiplicative: ``code = round(x * scale)``, ``scale = qmax/amax``;
  dequantisation divides by ``scale_x * scale_w``
  (segquant/src/real_quant/quantizer.cuh:65, dequantizer.cuh:48).
* activations are ``(S, ..., M, K)``, weights ``(S, N, K)`` (8-bit codes) or
  ``(S, N*K/2)`` bytes (int4, low nibble = even element); a scale tensor with
  ``numel == S`` is per segment, otherwise it is read flat as ``(S, M)`` /
  ``(S, N)`` (segquant/src/real_quant/real_gemm.cu:644-670, :703, :743).

How each function is pinned (none of it by importing the reference):

=====================  =====================================================
int8 / int4 codes      closed form + brute force over ties, limits, NaN, inf
int4 pack / unpack     exhaustive over all nibble pairs, round trip
e4m3 encode / decode   torch's ``float8_e4m3fn`` cast on clamped input, the
                       exhaustive 256-entry decode table, every midpoint
                       between neighbouring representable values
int32 accumulators     brute-force triple loop on tiny shapes; fp64 BLAS is
                       exact for these magnitudes
dequant, bias          closed form
segment semantics      concatenation / summation invariants
scale formulas         closed forms incl. the 2^-24 epsilon and 127-vs-128
fake-quant path        identities against the code path (dequantised codes)
smooth / svd split     limits of the formula (alpha 0 and 1, epsilon, clamp); the split
                       reassembles the weight and its residual has the energy of
                       the discarded singular values (Eckart-Young); x W^T is
                       unchanged by smoothing
int4 column repack     element-by-element definition (row r, channel c lives in
                       nibble r & 1 of byte c * out/2 + r/2) and round trip through
                       unpack_int4
=====================  =====================================================

The reference's own tests hold no golden vectors for this path, so the pins
above are all there is.  Parity status of the pieces that exist only in this
build and not in the reference (dynamic per-token scales, unequal K segments,
group-wise int4 scales): closed form only.
"""
from __future__ import annotations

import numpy as np

EPS = 1.0 / (1 << 24)  # segquant/quantizers/quantizer.py:167, :404

FMT_INT8 = "int8"
FMT_INT4 = "int4"
FMT_E4M3 = "fpe4m3"


# ---------------------------------------------------------------------------
# float helpers
# ---------------------------------------------------------------------------
def _f32(x) -> np.ndarray:
    return np.asarray(x, dtype=np.float32)


def round_to_bf16(x) -> np.ndarray:
    """fp32 -> nearest bf16 (ties to even), returned as fp32 values."""
    x = np.ascontiguousarray(_f32(x))
    u = x.view(np.uint32).astype(np.uint64)
    nan = np.isnan(x)
    lsb = (u >> 16) & 1
    u = (u + 0x7FFF + lsb) & 0xFFFF0000
    out = u.astype(np.uint32).view(np.float32).copy()
    out[nan] = np.nan
    return out.reshape(x.shape)


def round_to_dtype(x, dtype: str) -> np.ndarray:
    """Round fp32 values to the grid of ``dtype`` ("fp32" | "fp16" | "bf16")."""
    if dtype == "fp32":
        return _f32(x).copy()
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return _f32(x).astype(np.float16).astype(np.float32)
    if dtype == "bf16":
        return round_to_bf16(x)
    raise ValueError(dtype)


# ---------------------------------------------------------------------------
# e4m3 (OCP "e4m3fn": bias 7, max 448, no inf, NaN = S.1111.111)
# ---------------------------------------------------------------------------
def e4m3_decode_table() -> np.ndarray:
    """All 256 code values as fp32.  Codes 0x7F / 0xFF are NaN."""
    t = np.zeros(256, dtype=np.float64)
    for c in range(256):
        s = -1.0 if c & 0x80 else 1.0
        e = (c >> 3) & 0xF
        m = c & 7
        if e == 0xF and m == 7:
            t[c] = np.nan
        elif e == 0:
            t[c] = s * m * 2.0 ** -9
        else:
            t[c] = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    return t.astype(np.float32)


_E4M3_TABLE = e4m3_decode_table()


def e4m3_decode(codes) -> np.ndarray:
    return _E4M3_TABLE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(v) -> np.ndarray:
    """fp32 -> e4m3 code: round to nearest even, saturate to +-448, NaN -> 0x7F.

    Restates the hardware cast the reference relies on,
    ``static_cast<__nv_fp8_e4m3>(float)`` (segquant/src/real_quant/quantizer.cuh:21-29,
    segquant/src/fake_quant/quantizer_fp8.cpp:35-36).  The sign of a NaN is
    dropped (0x7F): what CUDA's conversion is documented to return for a NaN input (no run of
    it was possible here, so this case is not pinned by a reference output).
    """
    v = _f32(v)
    shape = v.shape
    v = v.reshape(-1)
    nan = np.isnan(v)
    sign = np.signbit(v).astype(np.uint8) << 7
    a = np.abs(v.astype(np.float64))
    a = np.where(nan, 0.0, np.minimum(a, 448.0))
    code = np.zeros(a.shape, dtype=np.int64)
    sub = a < 2.0 ** -6
    # subnormals: multiples of 2^-9; 8 * 2^-9 is the first normal and has code 8
    code[sub] = np.rint(a[sub] * 2.0 ** 9).astype(np.int64)
    nrm = ~sub
    if nrm.any():
        mant, ex = np.frexp(a[nrm])  # a = mant * 2^ex, mant in [0.5, 1)
        e = ex.astype(np.int64) - 1
        q = np.rint((mant * 2.0 - 1.0) * 8.0).astype(np.int64)
        carry = q == 8
        e = e + carry
        q = np.where(carry, 0, q)
        code[nrm] = ((e + 7) << 3) | q
    out = code.astype(np.uint8) | sign
    out[nan] = 0x7F
    return out.reshape(shape)


def e4m3_roundtrip(v) -> np.ndarray:
    """``float(e4m3(v))`` -- the reference's fake_e4m3fy
    (segquant/src/fake_quant/quantizer_fp8.cpp:25-39, quantizer_fp8.cu:34-41)."""
    return e4m3_decode(e4m3_encode(v))


# ---------------------------------------------------------------------------
# integer codes (segquant/src/real_quant/quantizer.cuh:31-50)
# ---------------------------------------------------------------------------
def int8_codes(v) -> np.ndarray:
    """``int8(rintf(fminf(fmaxf(v, -128), 127)))``; clamp first, then round half
    to even.  fmaxf drops a NaN operand, so NaN becomes -128."""
    v = _f32(v)
    c = np.clip(np.where(np.isnan(v), np.float32(-128.0), v), -128.0, 127.0)
    return np.rint(c).astype(np.int8)


def int4_codes(v) -> np.ndarray:
    """Signed 4-bit value in [-8, 7] (as int8), before packing."""
    v = _f32(v)
    c = np.clip(np.where(np.isnan(v), np.float32(-8.0), v), -8.0, 7.0)
    return np.rint(c).astype(np.int8)


def pack_int4(q) -> np.ndarray:
    """Flat element i -> byte i/2; even i in the low nibble, odd i in the high
    nibble, two's complement (segquant/src/real_quant/quantizer.cuh:37-50)."""
    q = np.asarray(q, dtype=np.int8).reshape(-1)
    if q.size % 2:
        q = np.concatenate([q, np.zeros(1, np.int8)])
    u = q.astype(np.uint8) & 0xF
    return (u[0::2] | (u[1::2] << 4)).astype(np.uint8)


def unpack_int4(b, n=None) -> np.ndarray:
    """Inverse of :func:`pack_int4`; returns sign-extended int8 values."""
    b = np.asarray(b, dtype=np.uint8).reshape(-1)
    lo = (b & 0xF).astype(np.int8)
    hi = (b >> 4).astype(np.int8)
    lo = np.where(lo > 7, lo - 16, lo).astype(np.int8)
    hi = np.where(hi > 7, hi - 16, hi).astype(np.int8)
    out = np.empty(b.size * 2, dtype=np.int8)
    out[0::2] = lo
    out[1::2] = hi
    return out if n is None else out[:n]


def codes_of(v, fmt: str) -> np.ndarray:
    """Scaled fp32 value -> storage code (int8, signed int4 value, or e4m3 byte)."""
    if fmt == FMT_INT8:
        return int8_codes(v)
    if fmt == FMT_INT4:
        return int4_codes(v)
    if fmt == FMT_E4M3:
        return e4m3_encode(v)
    raise ValueError(fmt)


def code_values(codes, fmt: str) -> np.ndarray:
    """Numeric value of storage codes as fp64 (exact)."""
    if fmt in (FMT_INT8, FMT_INT4):
        return np.asarray(codes).astype(np.float64)
    if fmt == FMT_E4M3:
        return e4m3_decode(codes).astype(np.float64)
    raise ValueError(fmt)


# ---------------------------------------------------------------------------
# scale indexing (quantizer.cuh:148-157, dequantizer.cuh:8-33)
# ---------------------------------------------------------------------------
def _expand_scale_x(scale_x, S: int, M: int) -> np.ndarray:
    """-> (S, M, 1).  numel == S: one scale per segment, else flat (S, M)."""
    s = _f32(scale_x).reshape(-1)
    if s.size == S:
        return np.broadcast_to(s.reshape(S, 1, 1), (S, M, 1))
    if s.size != S * M:
        raise ValueError(f"scale_x has {s.size} elements, expected {S} or {S * M}")
    return s.reshape(S, M, 1)


def _expand_scale_w(scale_w, S: int, N: int) -> np.ndarray:
    """-> (S, 1, N).  numel == S: one scale per segment, else flat (S, N)."""
    s = _f32(scale_w).reshape(-1)
    if s.size == S:
        return np.broadcast_to(s.reshape(S, 1, 1), (S, 1, N))
    if s.size != S * N:
        raise ValueError(f"scale_w has {s.size} elements, expected {S} or {S * N}")
    return s.reshape(S, 1, N)


# ---------------------------------------------------------------------------
# activation / weight quantisation
# ---------------------------------------------------------------------------
def quantize_act(x, scale_x, fmt: str) -> np.ndarray:
    """Activation codes, kernel K6 (segquant/src/real_quant/quantizer.cuh:159-176).

    ``x`` is (S, ..., M, K) in any float dtype (converted to fp32 exactly);
    returns codes of shape (S, M, K) (unpacked, also for int4).
    """
    x = np.asarray(x)
    S, K = x.shape[0], x.shape[-1]
    xf = x.astype(np.float32).reshape(S, -1, K)
    M = xf.shape[1]
    v = xf * _expand_scale_x(scale_x, S, M)  # fp32 * fp32 -> fp32
    return codes_of(v, fmt)


def quantize_act_dual(x, pos_scale_x, neg_scale_x, fmt: str):
    """DualScale codes, kernel K7 (segquant/src/real_quant/quantizer.cuh:178-206).

    ``x >= 0`` (which includes -0.0) takes the positive scale and leaves
    code(0) in Xn; everything else (negatives and NaN) takes the negative scale
    and leaves code(0) in Xp.  Returns (Xp, Xn), each (S, M, K).
    """
    x = np.asarray(x)
    S, K = x.shape[0], x.shape[-1]
    xf = x.astype(np.float32).reshape(S, -1, K)
    M = xf.shape[1]
    pos = xf >= 0
    zero = codes_of(np.zeros((), np.float32), fmt)
    cp = codes_of(xf * _expand_scale_x(pos_scale_x, S, M), fmt)
    cn = codes_of(xf * _expand_scale_x(neg_scale_x, S, M), fmt)
    xp = np.where(pos, cp, zero).astype(cp.dtype)
    xn = np.where(pos, zero, cn).astype(cn.dtype)
    return xp, xn


def merge_dual_codes(xp, xn, x) -> np.ndarray:
    """Single-tensor form of (Xp, Xn): the code of whichever branch was taken.

    This layout exists only in this build (the reference stores both tensors);
    it loses nothing because the untaken branch always holds code(0).
    """
    pos = np.asarray(x).astype(np.float32).reshape(xp.shape) >= 0
    return np.where(pos, xp, xn).astype(xp.dtype)


def quantize_weights(w, scale_w, fmt: str) -> np.ndarray:
    """Weight codes, kernels K2/K4 (segquant/src/real_quant/quantizer.cuh:55-68,
    :103-118; host side real_gemm.cu:538-638).  ``scale_w`` is a python float
    (per tensor) or a vector with one entry per row of ``w`` (N, K).
    Returns (N, K) codes (unpacked for int4)."""
    w = np.asarray(w).astype(np.float32)
    if np.ndim(scale_w) == 0:
        v = w * np.float32(scale_w)
    else:
        s = _f32(scale_w).reshape(-1)
        if s.size != w.shape[0]:
            raise ValueError("per-row weight scale needs one entry per row")
        v = w * s.reshape(-1, 1)
    return codes_of(v, fmt)


def activation(x, op: str, gate=None, dtype: str = "fp32") -> np.ndarray:
    """The activation function in front of a linear, as torch evaluates it for a
    tensor of ``dtype``: in fp32, each operator's result rounded to ``dtype``
    (backend/torch/layers/activations.py:52-57 GELU, :77-80 SwiGLU, :110-121
    GEGLU; backend/torch/modules/transformer_flux.py:91 GELU(tanh)).  ``op`` is
    "gelu_tanh", "gelu" or "silu"; with ``gate`` the result is x * op(gate).
    The arithmetic around the transcendental function is done in fp32 step by
    step, as torch and the kernel do it (so 1 + tanh(.) cancels to exactly 0 in
    the far negative tail, as it does there); tanh / erf / exp themselves are
    taken in fp64 and rounded to fp32, i.e. correctly rounded, where a device's
    tanhf / erff / expf may be an ulp off.  Pinned against torch's CPU operators
    (library routine) in the tests."""
    from scipy.special import erf
    f32 = np.float32

    def f(t):
        t = _f32(t)
        if op == "gelu_tanh":
            inner = f32(0.7978845608028654) * (t + f32(0.044715) * (t * t * t))
            r = f32(0.5) * t * (f32(1.0) + np.tanh(inner.astype(np.float64)).astype(f32))
        elif op == "gelu":
            r = t * f32(0.5) * (f32(1.0) + erf((t * f32(0.7071067811865476)).astype(np.float64)).astype(f32))
        elif op == "silu":
            with np.errstate(over="ignore"):
                r = t / (f32(1.0) + np.exp(-t.astype(np.float64)).astype(f32))
        else:
            raise ValueError(f"unknown activation {op}")
        return round_to_dtype(r.astype(f32), dtype)

    if gate is None:
        return f(x)
    return round_to_dtype((_f32(x) * f(gate)).astype(np.float32), dtype)


def smooth_divide(x, s, dtype: str = "fp32") -> np.ndarray:
    """SmoothQuant's activation step ``x.div_(s.to(x.dtype))``
    (segquant/optimum/optimizer.py:467-470): an fp32 division by the divisor rounded
    to the tensor's dtype, the quotient rounded to that dtype; ``s`` has one entry per
    column.  IEEE division is correctly rounded everywhere, so torch's CPU result pins
    this bit for bit."""
    sd = round_to_dtype(_f32(s).reshape(1, -1), dtype)
    return round_to_dtype((_f32(x) / sd).astype(np.float32), dtype)


def repack_int4_cols_to_rows(colpacked_1d, out: int, cols: int) -> np.ndarray:
    """The reference's ``GPTQCalibrator.colpacked1d_to_rowpacked1d``
    (segquant/calibrator/calibrator.py:202-223), step for step in numpy: the flat input is viewed
    as (cols, out / 2) and transposed, split into low and high nibbles (output rows 2j and 2j + 1),
    each (out / 2, cols) nibble plane packed two input channels per byte (even channel low), and the
    two planes interleaved row by row.  Returns the flat (out * cols / 2,) uint8 array."""
    assert out % 2 == 0 and cols % 2 == 0, "Output and columns must be even for int4 quantization."
    q = np.asarray(colpacked_1d, dtype=np.uint8).reshape(cols, out // 2).T
    low, high = q & 0x0F, (q >> 4) & 0x0F

    def pack(arr):
        return (arr[:, 0::2] | (arr[:, 1::2] << 4)).astype(np.uint8)

    lp, hp = pack(low), pack(high)
    res = np.empty((lp.shape[0] * 2, lp.shape[1]), dtype=np.uint8)
    res[0::2] = lp
    res[1::2] = hp
    return res.reshape(-1)


def smooth_factors(max_x, max_w, alpha: float) -> np.ndarray:
    """SmoothQuant's per-input-channel factor ``s = max_x^alpha / max_w^(1 - alpha)``; entries at or
    below 2^-31 become 1; the result is clamped to [1e-4, 1e4], fp32
    (segquant/optimum/optimizer.py:440-457)."""
    mx, mw = _f32(max_x), _f32(max_w)
    with np.errstate(divide="ignore", invalid="ignore"):
        s = (mx ** np.float32(alpha)) / (mw ** np.float32(1 - alpha))
    s = np.where(s <= 1.0 / (1 << 31), np.float32(1.0), s).astype(np.float32)
    return np.clip(s, np.float32(1e-4), np.float32(1e4)).astype(np.float32)


def svd_split(w_smooth, rank: int):
    """The SVD optimiser's split of a smoothed weight chunk (out, in), in fp64
    (segquant/optimum/optimizer.py:640-684): with ``W^T = U S V^T``, ``L1 = U_r S_r`` (in, r),
    ``L2 = V_r^T`` (r, out) and the residual ``W - (L1 L2)^T`` (out, in) that gets quantised."""
    t = np.asarray(w_smooth, dtype=np.float64).T
    u, sv, vt = np.linalg.svd(t, full_matrices=False)
    l1 = u[:, :rank] * sv[:rank]
    l2 = vt[:rank, :]
    return l1, l2, (t - l1 @ l2).T


def smooth_svd_linear(x, s, res_codes, scale_x, scale_w, fmt_a: str, fmt_w: str, l1=None, l2=None, bias=None) -> np.ndarray:
    """One chunk of a smoothed (and optionally low-rank-split) linear in fp64, as the reference's
    forward composes it (optimizer.py:514-517, :724-731): the quantised product of ``x / s`` with
    the residual's codes, de-quantised, plus ``(x / s) L1 L2``.  ``x`` (M, K) fp32 values already
    in the input's dtype grid, ``s`` (K,), per-tensor or per-row ``scale_x``, per-tensor or
    per-column ``scale_w``."""
    xs = _f32(x) / _f32(s)[None, :]
    sx = np.asarray(scale_x, dtype=np.float32).reshape(-1)
    codes = quantize_act(xs[None], sx, fmt_a)[0]
    sw = np.asarray(scale_w, dtype=np.float64).reshape(1, -1)
    out = gemm_acc(codes, res_codes, fmt_a, fmt_w) / (sx.astype(np.float64).reshape(-1, 1) * sw)
    if l1 is not None:
        out = out + (xs.astype(np.float64) @ np.asarray(l1, dtype=np.float64)) @ np.asarray(l2, dtype=np.float64)
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.float64).reshape(1, -1)
    return out


def group_amax(w, group: int) -> np.ndarray:
    """|w| maxima over runs of ``group`` input channels: (N, K) -> (N, K / group).
    Group-wise weight scales are not in the reference (its weight scales are per
    tensor or per row, segquant/src/real_quant/real_gemm.cu:538-638); a group is
    defined here as a K segment of the weight with its own per-row scale, so every
    formula below is the per-row one applied to a (N, group) slice.  Parity
    unpinned by the reference; pinned by that reduction (tests compare against the
    per-row functions slice by slice, and ``group == K`` against per-row whole)."""
    w = _f32(w)
    n, k = w.shape
    if k % group:
        raise ValueError("group must divide K")
    return np.abs(w).reshape(n, k // group, group).max(axis=-1)


def quantize_weights_groups(w, scale_w, group: int, fmt: str) -> np.ndarray:
    """Weight codes with one multiplicative scale per (row, group): the code rule of
    ``quantize_weights`` (quantizer.cuh:103-118) with ``scale_w`` of shape
    (N, K / group).  Returns (N, K) codes (unpacked for int4)."""
    w = _f32(w)
    n, k = w.shape
    s = _f32(scale_w).reshape(n, k // group)
    v = (w.reshape(n, k // group, group) * s[:, :, None]).astype(np.float32)
    return codes_of(v.reshape(n, k), fmt)


def linear_groups(a_codes, b_codes, scale_x, scale_w, group: int, bias=None) -> np.ndarray:
    """``out[m, n] = sum_g acc_g[m, n] / (sx[m] * sw[n, g]) + bias[n]`` in fp64, where
    ``acc_g`` is the exact integer product over group g: the de-quantisation rule of
    dequantizer.cuh:35-51 applied to every group's partial sum.  ``scale_x`` (M,) or
    scalar, ``scale_w`` (N, K / group)."""
    a = np.asarray(a_codes).astype(np.float64)
    b = np.asarray(b_codes).astype(np.float64)
    m, k = a.shape
    n = b.shape[0]
    sx = np.broadcast_to(np.asarray(scale_x, dtype=np.float64).reshape(-1, 1), (m, 1))
    sw = np.asarray(scale_w, dtype=np.float64).reshape(n, k // group)
    out = np.zeros((m, n))
    for g in range(k // group):
        acc = a[:, g * group:(g + 1) * group] @ b[:, g * group:(g + 1) * group].T
        out += acc / (sx * sw[None, :, g])
    if bias is not None:
        out = out + np.asarray(bias, dtype=np.float64).reshape(1, -1)
    return out


# ---------------------------------------------------------------------------
# contraction (segquant/src/real_quant/real_gemm.cu:208-305)
# ---------------------------------------------------------------------------
def gemm_acc(a_codes, b_codes, fmt_a: str, fmt_b: str) -> np.ndarray:
    """``acc[m, n] = sum_k A[m, k] * B[n, k]`` as fp64.

    Exact for integer codes: |acc| <= K * 128 * 128 < 2^53, and fp64 BLAS adds
    integers below 2^53 without rounding, so the result equals the int32
    accumulator bit for bit.  For e4m3 every product is exact in fp32 and the
    fp64 sum is the reference value that fp32 accumulation is compared against.
    """
    a = code_values(a_codes, fmt_a)
    b = code_values(b_codes, fmt_b)
    return a @ b.T


def gemm_acc_bruteforce(a_codes, b_codes) -> np.ndarray:
    """Triple loop in python ints; pins :func:`gemm_acc` on tiny shapes."""
    a = np.asarray(a_codes).astype(np.int64)
    b = np.asarray(b_codes).astype(np.int64)
    M, K = a.shape
    N = b.shape[0]
    out = np.zeros((M, N), dtype=np.int64)
    for m in range(M):
        for n in range(N):
            s = 0
            for k in range(K):
                s += int(a[m, k]) * int(b[n, k])
            out[m, n] = s
    return out


# ---------------------------------------------------------------------------
# dequantisation (segquant/src/real_quant/dequantizer.cuh:35-74)
# ---------------------------------------------------------------------------
def dequant(acc, scale_x, scale_w, out_dtype: str = "fp32") -> np.ndarray:
    """``T(float(acc) / (sx * sw))`` for acc of shape (S, M, N), kernel K8."""
    acc = np.asarray(acc)
    S, M, N = acc.shape
    yq = acc.astype(np.float32)
    s = _expand_scale_x(scale_x, S, M) * _expand_scale_w(scale_w, S, N)  # fp32 product
    return round_to_dtype(yq / s, out_dtype)


def dequant_dual(acc_p, acc_n, pos_scale_x, neg_scale_x, scale_w, out_dtype: str = "fp32") -> np.ndarray:
    """``T(Yp/(pos*sw) + Yn/(neg*sw))``, fp32 sum, one rounding; kernel K9."""
    acc_p = np.asarray(acc_p)
    S, M, N = acc_p.shape
    sw = _expand_scale_w(scale_w, S, N)
    yp = acc_p.astype(np.float32) / (_expand_scale_x(pos_scale_x, S, M) * sw)
    yn = np.asarray(acc_n).astype(np.float32) / (_expand_scale_x(neg_scale_x, S, M) * sw)
    return round_to_dtype(yp + yn, out_dtype)


# ---------------------------------------------------------------------------
# host pipelines H1 / H2 (segquant/src/real_quant/real_gemm.cu:643-894)
# ---------------------------------------------------------------------------
def _weight_values(weights, S: int, K: int, fmt_w: str) -> np.ndarray:
    w = np.asarray(weights)
    if fmt_w == FMT_INT4:
        wb = w.reshape(S, -1)
        N = wb.shape[1] * 2 // K  # real_gemm.cu:670
        return np.stack([unpack_int4(wb[s]).reshape(N, K) for s in range(S)])
    return w.reshape(S, -1, K)


def real_quantized_gemm_scaled(inputs, weights, scale_x, scale_w, fmt_a: str, fmt_w: str,
                               out_dtype: str = "fp32", return_acc: bool = False):
    """The reference's ``<prefix>_real_quantized_gemm_scaled`` end to end
    (segquant/src/real_quant/real_gemm.cu:643-750): quantise the activations,
    contract each segment with its weight codes, dequantise.  ``inputs`` is
    (S, ..., M, K); the result is (S, ..., M, N) holding values on the grid of
    ``out_dtype``.  The scalar fast path (:707-712) multiplies by a reciprocal
    instead of dividing; that differs from this formula by at most one fp32 ulp
    and is not modelled separately."""
    x = np.asarray(inputs)
    S, K = x.shape[0], x.shape[-1]
    xq = quantize_act(x, scale_x, fmt_a)
    wv = _weight_values(weights, S, K, fmt_w)
    acc = np.stack([gemm_acc(xq[s], wv[s], fmt_a, fmt_w) for s in range(S)])
    out = dequant(acc, scale_x, scale_w, out_dtype).reshape(*x.shape[:-1], wv.shape[1])
    return (out, acc) if return_acc else out


def real_quantized_gemm_dual_scaled(inputs, weights, pos_scale_x, neg_scale_x, scale_w,
                                    fmt_a: str, fmt_w: str, out_dtype: str = "fp32",
                                    return_acc: bool = False):
    """The reference's ``<prefix>_real_quantized_gemm_dual_scaled``
    (segquant/src/real_quant/real_gemm.cu:752-894)."""
    x = np.asarray(inputs)
    S, K = x.shape[0], x.shape[-1]
    xp, xn = quantize_act_dual(x, pos_scale_x, neg_scale_x, fmt_a)
    wv = _weight_values(weights, S, K, fmt_w)
    acc_p = np.stack([gemm_acc(xp[s], wv[s], fmt_a, fmt_w) for s in range(S)])
    acc_n = np.stack([gemm_acc(xn[s], wv[s], fmt_a, fmt_w) for s in range(S)])
    out = dequant_dual(acc_p, acc_n, pos_scale_x, neg_scale_x, scale_w, out_dtype)
    out = out.reshape(*x.shape[:-1], wv.shape[1])
    return (out, acc_p, acc_n) if return_acc else out


def recombine(out_chunks, seg_mode: str, bias=None, out_dtype: str = "fp32") -> np.ndarray:
    """Tail of ``SegmentLinear.forward`` (segquant/layers/SegmentLinear.py:228-241).

    weight-seg: (S, ..., n) -> (..., S*n).  input-seg: sum over S, done in the
    output dtype as the reference does.  Bias is added in the output dtype.
    """
    o = np.asarray(out_chunks, dtype=np.float32)
    if seg_mode == "weight":
        res = np.moveaxis(o, 0, -2).reshape(*o.shape[1:-1], -1)
    elif seg_mode == "input":
        res = o[0]
        for s in range(1, o.shape[0]):
            res = round_to_dtype(res + o[s], out_dtype)
    else:
        raise ValueError(seg_mode)
    if bias is not None:
        res = round_to_dtype(res + _f32(bias), out_dtype)
    return res


# ---------------------------------------------------------------------------
# scale formulas (segquant/quantizers/quantizer.py:161-248, :398-452)
# ---------------------------------------------------------------------------
def int_qrange(bits: int):
    return -(2 ** (bits - 1)), 2 ** (bits - 1) - 1  # quantizer.py:151-152


def _scalar_over_tensor(limit, amax) -> np.ndarray:
    """``limit / tensor`` as torch evaluates it for a python scalar on the left:
    ``tensor.reciprocal() * limit``, two fp32 roundings (torch/_tensor.py,
    ``__rtruediv__``).  This is what the reference's per-axis formulas compute."""
    clamped = np.maximum(_f32(amax), np.float32(EPS))
    return ((np.float32(1.0) / clamped) * np.float32(limit)).astype(np.float32)


def row_scale_div(amax, limit) -> np.ndarray:
    """``limit / max(amax, eps)`` as ONE correctly rounded fp32 division: the
    definition the quantise kernel uses for dynamic per-row scales (which the
    reference has no working counterpart of, optimum/optimizer.py:96-100)."""
    return (np.float32(limit) / np.maximum(_f32(amax), np.float32(EPS))).astype(np.float32)


def int_scale(amax, bits: int = 8):
    """Symmetric per-tensor: ``qmax/amax`` if amax > eps else 1.0 (python float
    arithmetic, quantizer.py:206-210).  Array input: ``qmax / clamp(amax, eps)``
    evaluated by torch in fp32 (quantizer.py:211-219)."""
    _, qmax = int_qrange(bits)
    if np.ndim(amax) == 0:
        amax = float(amax)
        return qmax / amax if amax > EPS else 1.0
    return _scalar_over_tensor(qmax, amax)


def int_dual_scales(pos_amax, neg_amax, bits: int = 8):
    """``pos = qmax/pos_amax``, ``neg = qmin/(-neg_amax)`` (quantizer.py:170-203)."""
    qmin, qmax = int_qrange(bits)
    if np.ndim(pos_amax) == 0:
        pos_amax, neg_amax = float(pos_amax), float(neg_amax)
        neg = qmin / (-neg_amax) if neg_amax > EPS else 1.0
        pos = qmax / pos_amax if pos_amax > EPS else 1.0
        return pos, neg
    # qmin / (-clamp(neg_amax)): the same reciprocal-times-scalar, signs cancel exactly
    return _scalar_over_tensor(qmax, pos_amax), _scalar_over_tensor(-qmin, neg_amax)


def fp8_scale(amax):
    """``448/amax`` with the same epsilon rules (quantizer.py:437-452)."""
    if np.ndim(amax) == 0:
        amax = float(amax)
        return 448.0 / amax if amax > EPS else 1.0
    return _scalar_over_tensor(448.0, amax)


def fp8_dual_scales(pos_amax, neg_amax):
    """448 on both sides (quantizer.py:406-436)."""
    return fp8_scale(pos_amax), fp8_scale(neg_amax)


def dual_amax(x, axis=None):
    """Strict masks ``x > 0`` / ``x < 0``; an empty side has amax 0
    (quantizer.py:172-189)."""
    x = _f32(x)
    pos = np.where(x > 0, np.abs(x), 0.0)
    neg = np.where(x < 0, np.abs(x), 0.0)
    if axis is None:
        return float(pos.max()), float(neg.max())
    return pos.max(axis=axis), neg.max(axis=axis)


# ---------------------------------------------------------------------------
# fake-quant reference path (segquant/quantizers/quantizer.py:250-281, :462-528)
# ---------------------------------------------------------------------------
def fake_quant_int(x, scale, bits: int = 8) -> np.ndarray:
    """``clamp(round(x*s), qmin, qmax) / s`` in fp32 (quantizer.py:277-281;
    symmetric, zero point 0)."""
    qmin, qmax = int_qrange(bits)
    x = _f32(x)
    s = _f32(scale)
    return (np.clip(np.rint(x * s), qmin, qmax) / s).astype(np.float32)


def fake_quant_int_dual(x, pos_scale, neg_scale, bits: int = 8) -> np.ndarray:
    """quantizer.py:259-265."""
    qmin, qmax = int_qrange(bits)
    x = _f32(x)
    ps, ns = _f32(pos_scale), _f32(neg_scale)
    q = np.where(x >= 0, np.clip(np.rint(x * ps), 0, qmax), np.clip(np.rint(x * ns), qmin, 0))
    return np.where(x >= 0, q / ps, q / ns).astype(np.float32)


def simulate_fp(x, fp_min: float, fp_max: float, mant_bits: int) -> np.ndarray:
    """The reference's pure-torch float simulation, which has no subnormals:
    anything below ``fp_min`` becomes zero (quantizer.py:462-482)."""
    x = _f32(x)
    a = np.minimum(np.abs(x), np.float32(fp_max))
    a = np.where(a < fp_min, np.float32(0), a)
    expo = np.floor(np.log2(np.maximum(a, np.float32(fp_min))))
    mant = a / np.exp2(expo)
    mant_r = np.rint((mant - 1) * 2 ** mant_bits) / 2 ** mant_bits
    return ((1 + mant_r) * np.exp2(expo) * np.sign(x)).astype(np.float32)


E4M3_FP_MIN = (2.0 ** -6) * (240 / 448.0)  # quantizer.py:384


def fake_quant_fp8(x, scale, simulate: str = "e4m3") -> np.ndarray:
    """``e4m3(x*s)/s`` with ``|x| < 2^-24 -> 0`` (quantizer.py:484-528).
    ``simulate="e4m3"`` is the branch taken when the fake_e4m3fy extension is
    present; ``"simulate_fp"`` is the pure-torch fallback."""
    x = _f32(x)
    s = _f32(scale)
    v = x * s
    if simulate == "e4m3":
        q = e4m3_roundtrip(v)
    else:
        q = simulate_fp(v, E4M3_FP_MIN, 448.0, 3)
    out = (q / s).astype(np.float32)
    return np.where(np.abs(x) < EPS, np.float32(0), out)


def fake_quant_fp8_dual(x, pos_scale, neg_scale) -> np.ndarray:
    """quantizer.py:487-507 (e4m3 branch)."""
    x = _f32(x)
    ps, ns = _f32(pos_scale), _f32(neg_scale)
    v = np.where(x >= 0, x * ps, x * ns)
    q = e4m3_roundtrip(v)
    out = np.where(x >= 0, q / ps, q / ns).astype(np.float32)
    return np.where(np.abs(x) < EPS, np.float32(0), out)


def segmented_matmul(a, b) -> np.ndarray:
    """``a @ b^T`` per segment with leading-dim broadcast
    (segquant/layers/segment_tensor_manager.py:83-94).  a (S, ..., K), b (S, N, K)."""
    a = _f32(a)
    b = _f32(b)
    bt = np.swapaxes(b, -1, -2)
    while bt.ndim < a.ndim:
        bt = np.expand_dims(bt, 1)
    return a @ bt


def segment_views(x, w, seg_mode: str, chunks: int):
    """Segment views of the input and the weight
    (segquant/layers/segment_tensor_manager.py:15-23, :45-51).
    Returns (x_seg (S, ..., k), w_seg (S, n, k))."""
    x = np.asarray(x)
    w = np.asarray(w)
    N, K = w.shape
    if seg_mode == "weight":
        xs = np.broadcast_to(x[None], (chunks, *x.shape))
        ws = w.reshape(chunks, N // chunks, K)
    elif seg_mode == "input":
        xs = np.moveaxis(x.reshape(*x.shape[:-1], chunks, K // chunks), -2, 0)
        ws = np.moveaxis(w.reshape(N, chunks, K // chunks), 1, 0)
    else:
        raise ValueError(seg_mode)
    return xs, ws
