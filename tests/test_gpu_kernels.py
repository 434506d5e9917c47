"""GPU parity tests of the HIP kernels against the CPU oracle, through the C ABI.

Integer codes, int4 packing and int32 accumulators must be bit-exact.  The fp8
MFMA sums each 128-long group of exact products with a limited-width aligned
adder, so fp8 accumulators are compared with the exact fp64 sum to within
FP8_ACC_TOL of sum |a||b| (measured on codes drawn uniformly from the whole
e4m3 range: 4e-5 typically, 2.6e-4 the largest over some 10^8 outputs of
randomly drawn shapes, tiles and ranges).  De-quantised outputs use the tolerances the path is
specified with: 1e-3 relative for int8, 1e-2 for fp8 against the fp32
fake-quant result.
"""
import numpy as np
import pytest
import torch

from oracle import segq_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FP8_ACC_TOL = 3e-4
FMTS = [O.FMT_INT8, O.FMT_E4M3, O.FMT_INT4]
TDT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from segquant_amd import ops as _ops
    _ops.L.lib()  # fail loudly if the library is not built
    return _ops


def _np(t):
    return t.detach().float().cpu().numpy() if t.dtype in (torch.bfloat16, torch.float16) else t.detach().cpu().numpy()


def _codes_np(t, fmt, cols=None):
    a = t.cpu().numpy()
    if fmt == O.FMT_INT4:
        return np.stack([O.unpack_int4(r) for r in a.reshape(a.shape[0], -1)])
    return a


def _special_matrix(rows, cols, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, cols, generator=g) * 3
    x[0, :18] = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 0.0, -0.0, 1e30, -1e30, float("inf"), float("-inf"),
                              float("nan"), 126.5, 127.5, -127.5, -128.5, 1e-30])
    return x.to(dtype)


# ------------------------------------------------------------------ quantise
@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dt", ["fp32", "bf16", "fp16"])
def test_quantize_per_tensor_and_per_row_bit_exact(ops, fmt, dt):
    rows, cols = 37, 208
    x = _special_matrix(rows, cols, 1, TDT[dt]).to(DEV)
    xn = _np(x)
    for per_row in (False, True):
        s = (torch.rand(rows if per_row else 1) * 20 + 0.5).to(DEV)
        c = ops.quantize(x, fmt, s, row_stride=1 if per_row else 0)
        want = O.quantize_act(xn[None], s.cpu().numpy(), fmt)[0]
        got = _codes_np(c, fmt)
        assert np.array_equal(got, want), (fmt, dt, per_row)


def test_e4m3_hardware_cast_on_every_midpoint(ops):
    tab = O.e4m3_decode_table()
    pos = np.sort(tab[:0x7F])
    mids = ((pos[:-1].astype(np.float64) + pos[1:]) / 2).astype(np.float32)
    pts = np.concatenate([pos, mids, np.nextafter(mids, np.float32(0)), np.nextafter(mids, np.float32(1e9)),
                          np.float32([449, 464, 465, 480, 1e9, np.inf])])
    pts = np.concatenate([pts, -pts, np.float32([np.nan])])
    pad = (-len(pts)) % 16
    pts = np.concatenate([pts, np.zeros(pad, np.float32)])
    x = torch.from_numpy(pts).view(1, -1).to(DEV)
    one = torch.ones(1, device=DEV)
    c = ops.quantize(x, O.FMT_E4M3, one).cpu().numpy()[0]
    assert np.array_equal(c, O.e4m3_encode(pts))
    rt = ops.fake_e4m3fy(x).cpu().numpy()[0]
    want = O.e4m3_roundtrip(pts)
    assert np.array_equal(np.isnan(rt), np.isnan(want))
    assert np.array_equal(rt[~np.isnan(rt)], want[~np.isnan(want)])


@pytest.mark.parametrize("fmt", FMTS)
def test_quantize_reference_segment_indexing(ops, fmt):
    S, B, M, K = 3, 2, 5, 64
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(S, B, M, K, generator=g) * 2).to(torch.bfloat16).to(DEV)
    rows = B * M
    for per_tok in (False, True):
        s = (torch.rand(S * rows if per_tok else S, generator=g) * 30 + 1).to(DEV)
        c = ops.quantize(x.view(S * rows, K), fmt, s, seg_rows=rows, seg_stride=rows if per_tok else 1,
                         row_stride=1 if per_tok else 0)
        want = O.quantize_act(_np(x), s.cpu().numpy(), fmt).reshape(S * rows, K)
        assert np.array_equal(_codes_np(c, fmt), want)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantize_dual_two_tensor_and_merged(ops, fmt):
    S, M, K = 2, 9, 96
    g = torch.Generator().manual_seed(3)
    x = torch.randn(S, M, K, generator=g)
    x[0, 0, :4] = torch.tensor([0.0, -0.0, float("nan"), -1e-20])
    x = x.to(DEV)
    pos = (torch.rand(S, generator=g) * 30 + 1).to(DEV)
    neg = (torch.rand(S, generator=g) * 60 + 1).to(DEV)
    xp, xn = ops.quantize(x.view(S * M, K), fmt, pos, neg, seg_rows=M, seg_stride=1, dual=True, two_tensors=True)
    wp, wn = O.quantize_act_dual(_np(x), pos.cpu().numpy(), neg.cpu().numpy(), fmt)
    assert np.array_equal(_codes_np(xp, fmt), wp.reshape(S * M, K))
    assert np.array_equal(_codes_np(xn, fmt), wn.reshape(S * M, K))
    merged = ops.quantize(x.view(S * M, K), fmt, pos, neg, seg_rows=M, seg_stride=1, dual=True)
    want = O.merge_dual_codes(wp, wn, _np(x)).reshape(S * M, K)
    assert np.array_equal(_codes_np(merged, fmt), want)


def test_quantize_column_segments_with_partial_dual(ops):
    M, K = 11, 160
    bounds = [0, 48, 160]
    g = torch.Generator().manual_seed(4)
    x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([10.0, 20.0], device=DEV)
    neg = torch.tensor([99.0, 40.0], device=DEV)
    c = ops.quantize(x, O.FMT_INT8, pos, neg, kseg_bounds=bounds, kseg_stride=1, dual=True, dual_kseg_mask=0b10)
    xn = _np(x)
    w0 = O.quantize_act(xn[None, :, :48], np.float32([10.0]), O.FMT_INT8)[0]
    wp, wn = O.quantize_act_dual(xn[None, :, 48:], np.float32([20.0]), np.float32([40.0]), O.FMT_INT8)
    w1 = O.merge_dual_codes(wp, wn, xn[None, :, 48:])[0]
    assert np.array_equal(c.cpu().numpy(), np.concatenate([w0, w1], axis=1))
    # two-tensor layout: the plain segment keeps its one code in the first tensor
    xn_t = torch.full((M, K), 77, dtype=torch.int8, device=DEV)
    xp_t, xn_t = ops.quantize(x, O.FMT_INT8, pos, neg, kseg_bounds=bounds, kseg_stride=1, dual=True,
                              dual_kseg_mask=0b10, two_tensors=True, out_neg=xn_t)
    assert np.array_equal(xp_t.cpu().numpy(), np.concatenate([w0, wp[0]], axis=1))
    assert np.array_equal(xn_t.cpu().numpy()[:, 48:], wn[0]) and (xn_t.cpu().numpy()[:, :48] == 77).all()


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dual", [False, True])
def test_quantize_dynamic_per_row(ops, fmt, dual):
    M, K = 13, 16 * 300  # longer than one cached pass of 256 threads
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g)
    x[1] = x[1].abs()  # no negatives in this row
    x[2] = 0
    x = x.to(torch.bfloat16).to(DEV)
    s = torch.empty(M, device=DEV)
    sn = torch.empty(M, device=DEV) if dual else None
    c = ops.quantize(x, fmt, s, sn, row_stride=1, dual=dual, dynamic=True)
    xn = _np(x)
    bits = 4 if fmt == O.FMT_INT4 else 8
    lim_p = {O.FMT_INT8: 127.0, O.FMT_INT4: 7.0, O.FMT_E4M3: 448.0}[fmt]
    lim_n = {O.FMT_INT8: 128.0, O.FMT_INT4: 8.0, O.FMT_E4M3: 448.0}[fmt]
    if dual:
        pa, na = O.dual_amax(xn, axis=-1)
        ws, wn = O.row_scale_div(pa, lim_p), O.row_scale_div(na, lim_n)
        assert np.array_equal(s.cpu().numpy(), ws) and np.array_equal(sn.cpu().numpy(), wn)
        wp, wq = O.quantize_act_dual(xn[None], ws, wn, fmt)
        want = O.merge_dual_codes(wp, wq, xn[None])[0]
    else:
        amax = np.abs(xn).max(axis=-1)
        ws = O.row_scale_div(amax, lim_p)
        assert np.array_equal(s.cpu().numpy(), ws)
        want = O.quantize_act(xn[None], ws, fmt)[0]
    assert np.array_equal(_codes_np(c, fmt), want)


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("dual", [False, True])
@pytest.mark.parametrize("K", [3072, 4800, 12288])   # one wave per row and workgroup / per row / one workgroup per row
@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_quantize_dynamic_rows_with_nan_inf_and_extremes(ops, fmt, dual, K, dt):
    """Per-row scales of rows that hold a NaN, an infinity, a value next to the largest finite
    one, or nothing above 1e-30.  A single scale is max|x| the way torch's amax takes it: a NaN
    in the row makes the scale NaN and every code of the row the NaN code; DualScale's strict
    masks leave a NaN on neither side (segquant/quantizers/quantizer.py:172-189, :212).  An
    infinite maximum gives scale 0.  Scales and codes bit-exact against the oracle."""
    g = torch.Generator().manual_seed(77)
    x = torch.randn(7, K, generator=g)
    x[1, 5] = float("nan"); x[2, 7] = float("inf"); x[3, 9] = float("-inf"); x[4, 11] = 3e38
    x[5] = 0; x[5, 3] = 1e-30
    x[6, K - 1] = float("nan")  # in the last lane's last run
    x = x.to(TDT[dt]).to(DEV)
    s = torch.empty(7, device=DEV)
    sn = torch.empty(7, device=DEV) if dual else None
    c = ops.quantize(x, fmt, s, sn, row_stride=1, dual=dual, dynamic=True)
    xn = _np(x)
    lim_p = {O.FMT_INT8: 127.0, O.FMT_E4M3: 448.0}[fmt]
    lim_n = {O.FMT_INT8: 128.0, O.FMT_E4M3: 448.0}[fmt]
    same = lambda a, b: np.array_equal(a, b, equal_nan=True)
    with np.errstate(all="ignore"):
        if dual:
            pa, na = O.dual_amax(xn, axis=-1)
            ws, wn = O.row_scale_div(pa, lim_p), O.row_scale_div(na, lim_n)
            assert same(sn.cpu().numpy(), wn)
            wp, wq = O.quantize_act_dual(xn[None], ws, wn, fmt)
            want = O.merge_dual_codes(wp, wq, xn[None])[0]
        else:
            ws = O.row_scale_div(np.abs(xn).max(axis=-1), lim_p)
            assert np.isnan(ws[1]) and np.isnan(ws[6]) and ws[2] == 0 and ws[3] == 0
            want = O.quantize_act(xn[None], ws, fmt)[0]
    assert same(s.cpu().numpy(), ws)
    assert np.array_equal(_codes_np(c, fmt), want)


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("dual", [False, True])
def test_quantize_many_shares_launches_and_matches_single_calls(ops, fmt, dual):
    """segq_quantize_many: tensors of the same kind (dynamic per-row scales, one column segment,
    the same row-length class) go through one launch, others through their own, in any mix and
    order; codes and scales are those of one segq_quantize call each, bit for bit.  Five batchable
    tensors in a row (more than one shared launch holds), a longer row class in between, an fp32
    input, a static one and an empty one."""
    g = torch.Generator().manual_seed(91)
    def dyn(M, K, dt=torch.bfloat16):
        x = (torch.randn(M, K, generator=g) * 3).to(dt).to(DEV)
        mk = lambda: (torch.empty(M, device=DEV), torch.empty(M, device=DEV) if dual else None)
        return x, mk
    cases = [dyn(37, 3072), dyn(5, 3056), dyn(64, 3072), dyn(129, 2960), dyn(3, 3072),   # one length class (CPL 3)
             dyn(20, 5120), dyn(7, 3072), dyn(9, 3072, torch.float32), dyn(0, 3072), dyn(11, 3072, torch.float16),
             dyn(4, 3072, torch.float16)]
    single, many, keep = [], [], []
    for x, mk in cases:
        s1, n1 = mk()
        single.append((ops.quantize(x, fmt, s1, n1, row_stride=1, dual=dual, dynamic=True) if x.shape[0] else None, s1, n1))
        s2, n2 = mk()
        many.append(ops.quantize_desc(x, fmt, s2, n2, row_stride=1, dual=dual, dynamic=True))
        keep.append((s2, n2))
    # a static per-tensor launch in the middle of the list
    xs = (torch.randn(33, 3072, generator=g)).to(torch.bfloat16).to(DEV)
    st = torch.full((1,), 17.5, device=DEV)
    want_static = ops.quantize(xs, fmt, st)
    many.insert(3, ops.quantize_desc(xs, fmt, st))
    with ops.record_launches() as log:
        res = ops.quantize_many(many)
        torch.cuda.synchronize()
    assert len(log) == 1  # one call into the library
    got_static = res.pop(3)
    assert torch.equal(got_static if not isinstance(got_static, tuple) else got_static[0],
                       want_static if not isinstance(want_static, tuple) else want_static[0])
    it = iter(res)
    for (x, _), (c1, s1, n1), (s2, n2) in zip(cases, single, keep):
        c2 = next(it)
        if not x.shape[0]:
            assert (c2[0] if isinstance(c2, tuple) else c2).shape[0] == 0
            continue
        assert torch.equal(s1, s2) and (n1 is None or torch.equal(n1, n2))
        a, b = (c1 if isinstance(c1, tuple) else (c1,)), (c2 if isinstance(c2, tuple) else (c2,))
        for u, v in zip(a, b):
            assert torch.equal(u, v)


@pytest.mark.parametrize("fmt", FMTS)
def test_quantize_weights_both_overloads(ops, fmt):
    N, K = 24, 64
    g = torch.Generator().manual_seed(6)
    w = (torch.randn(N, K, generator=g) * 0.02).to(DEV)
    out = torch.empty(N * K // 2 if fmt == O.FMT_INT4 else (N, K), dtype=ops.code_dtype(fmt), device=DEV)
    ops.real_quantized_quantize_weights(fmt, w, out, 311.5)
    want = O.quantize_weights(_np(w), 311.5, fmt)
    assert np.array_equal(_codes_np(out.view(N, -1), fmt), want)
    s = (torch.rand(N, generator=g) * 300 + 50).to(DEV)
    ops.real_quantized_quantize_weights(fmt, w, out, s)
    want = O.quantize_weights(_np(w), s.cpu().numpy(), fmt)
    assert np.array_equal(_codes_np(out.view(N, -1), fmt), want)
    with pytest.raises(TypeError):
        ops.real_quantized_quantize_weights(fmt, w, out, 3)


# ------------------------------------------------------------------ GEMM accumulators
def _rand_codes(shape, fmt, seed):
    g = np.random.default_rng(seed)
    if fmt == O.FMT_INT8:
        c = g.integers(-128, 128, size=shape).astype(np.int8)
        c.reshape(-1)[:7] = [-128, 127, -128, -128, 127, 0, -1]
        return c
    if fmt == O.FMT_INT4:
        return g.integers(-8, 8, size=shape).astype(np.int8)
    c = g.integers(0, 256, size=shape).astype(np.uint8)
    c[(c & 0x7F) == 0x7F] = 0x3A  # no NaN codes
    return c


def _to_dev_codes(c, fmt):
    if fmt == O.FMT_INT4:
        return torch.from_numpy(np.stack([O.pack_int4(r) for r in c])).to(DEV)
    return torch.from_numpy(c).to(DEV)


@pytest.mark.parametrize("tile", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("fa,fb", [(O.FMT_INT8, O.FMT_INT8), (O.FMT_E4M3, O.FMT_E4M3), (O.FMT_INT8, O.FMT_INT4)])
@pytest.mark.parametrize("M,N,K", [(256, 256, 256), (300, 200, 416), (3, 18, 64), (130, 515, 1056)])
def test_gemm_raw_accumulators(ops, tile, fa, fb, M, N, K):
    a = _rand_codes((M, K), fa, 10)
    b = _rand_codes((N, K), fb, 11)
    ad, bd = _to_dev_codes(a, fa), _to_dev_codes(b, fb)
    ldb = K // 2 if fb == O.FMT_INT4 else K
    out = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], m=M, n=N, a_fmt=fa, b_fmt=fb, out_dtype="acc",
                   lda=K, ldb=ldb, tile=tile)
    ref = O.gemm_acc(a, b, fa, fb)
    if fa == O.FMT_E4M3:
        got = out.cpu().numpy().astype(np.float64)
        mag = np.abs(O.code_values(a, fa)) @ np.abs(O.code_values(b, fb)).T
        assert (np.abs(got - ref) <= FP8_ACC_TOL * mag + 1e-30).all()
    else:
        assert np.array_equal(out.cpu().numpy().astype(np.int64), ref.astype(np.int64))


WIDE_TILES = [11, 12, 13, 14, 15, 16, 17, 18, 20]   # the 8-wave kernels; 15 to 18 and 20 (192x288, 288x192, 256x192, 192x256, 384x192) serve plain 8-bit codes only
# (19 and 21, the many-stage kernels for few tokens, int8 only: test_gemm_many_stage_tiles_for_few_tokens)


def _bf16_ulp(ref):
    return np.abs(ref) * 2.0 ** -7 + 1e-30


@pytest.mark.parametrize("tile", WIDE_TILES)
@pytest.mark.parametrize("fa,fb", [(O.FMT_INT8, O.FMT_INT8), (O.FMT_E4M3, O.FMT_E4M3), (O.FMT_INT8, O.FMT_INT4)])
@pytest.mark.parametrize("M,N,K", [(512, 576, 256), (300, 700, 384), (77, 130, 128)])
def test_gemm_eight_wave_tiles(ops, tile, fa, fb, M, N, K):
    """Raw accumulators (exact) and the fused bf16 epilogue (scales per row and per
    column, bias; at most one bf16 unit from the oracle's single rounding) on
    every 8-wave tile, on a shape of whole tiles and on ragged ones."""
    a = _rand_codes((M, K), fa, 40)
    b = _rand_codes((N, K), fb, 41)
    ad, bd = _to_dev_codes(a, fa), _to_dev_codes(b, fb)
    ldb = K // 2 if fb == O.FMT_INT4 else K
    kw = dict(m=M, n=N, a_fmt=fa, b_fmt=fb, lda=K, ldb=ldb, tile=tile)
    if tile >= 15 and fb == O.FMT_INT4:
        with pytest.raises(RuntimeError):
            ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", **kw)
        return
    ref = O.gemm_acc(a, b, fa, fb)
    out = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", **kw)
    if fa == O.FMT_E4M3:
        mag = np.abs(O.code_values(a, fa)) @ np.abs(O.code_values(b, fb)).T
        assert (np.abs(out.cpu().numpy().astype(np.float64) - ref) <= FP8_ACC_TOL * mag + 1e-30).all()
    else:
        assert np.array_equal(out.cpu().numpy().astype(np.int64), ref.astype(np.int64))
    g = torch.Generator().manual_seed(42)
    sx = torch.rand(M, generator=g) + 0.5
    sw = torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g)
    y = ops.gemm(ad, bd, [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)], out_dtype=torch.bfloat16,
                 bias=bias.to(DEV), **kw)
    want = ref / (sx.numpy().astype(np.float64)[:, None] * sw.numpy().astype(np.float64)[None, :]) + bias.numpy()
    got = y.float().cpu().numpy().astype(np.float64)
    slack = FP8_ACC_TOL * mag / (sx.numpy()[:, None] * sw.numpy()[None, :]) if fa == O.FMT_E4M3 else 0.0
    assert (np.abs(got - want) <= _bf16_ulp(want) + slack).all()
    # two K ranges with their own activation and weight scales: int32 accumulators are
    # folded into fp32 ones (not on the 192x288 / 288x192 tiles), fp32 accumulators
    # are rescaled in place at the boundary (every tile)
    K0 = 128
    if K <= K0:
        return
    sx2 = torch.rand(M, generator=g) + 0.5
    sw2 = torch.rand(N, generator=g) + 0.5
    rg = [ops.Range(0, K0, sx.to(DEV), sw.to(DEV), 0, 1, 1), ops.Range(K0, K - K0, sx2.to(DEV), sw2.to(DEV), 0, 1, 1)]
    if tile >= 15 and fa == O.FMT_INT8:
        with pytest.raises(RuntimeError):
            ops.gemm(ad, bd, rg, out_dtype=torch.float32, bias=bias.to(DEV), **kw)
        return
    y2 = ops.gemm(ad, bd, rg, out_dtype=torch.float32, bias=bias.to(DEV), **kw)
    f64 = lambda t: t.numpy().astype(np.float64)
    p0 = O.gemm_acc(a[:, :K0], b[:, :K0], fa, fb) / (f64(sx)[:, None] * f64(sw)[None, :])
    p1 = O.gemm_acc(a[:, K0:], b[:, K0:], fa, fb) / (f64(sx2)[:, None] * f64(sw2)[None, :])
    want2 = p0 + p1 + bias.numpy()
    got2 = y2.cpu().numpy().astype(np.float64)
    if fa == O.FMT_E4M3:
        av, bv = np.abs(O.code_values(a, fa)), np.abs(O.code_values(b, fb))
        slack2 = FP8_ACC_TOL * ((av[:, :K0] @ bv[:, :K0].T) / (f64(sx)[:, None] * f64(sw)[None, :])
                                + (av[:, K0:] @ bv[:, K0:].T) / (f64(sx2)[:, None] * f64(sw2)[None, :]))
    else:
        slack2 = 0.0
    assert (np.abs(got2 - want2) <= 4e-6 * (np.abs(p0) + np.abs(p1) + np.abs(bias.numpy())[None, :]) + slack2).all()


@pytest.mark.parametrize("tile", [19, 21])
@pytest.mark.parametrize("M,N,K", [(256, 2176, 1536), (200, 330, 128), (77, 130, 256), (130, 260, 384), (64, 1152, 768), (256, 9216, 1536)])
def test_gemm_many_stage_tiles_for_few_tokens(ops, tile, M, N, K):
    """Tiles 19 and 21: the int8 128 x 128 kernel with four LDS stages and the 128 x 96 one with five
    (the library's own choice when the tiles do not fill the CUs once; 128 x 96 where it tiles the
    columns exactly and still fits the CUs once, as on the 256 x 1536 -> 9216 adaLN shape).
    Contractions shorter than, equal to and longer than the number of stages, ragged M and N: raw
    accumulators exact, the fused fp32 and bf16 epilogues within their rounding of the closed form;
    what they do not serve is refused."""
    fmt = O.FMT_INT8
    a, b = _rand_codes((M, K), fmt, 81), _rand_codes((N, K), fmt, 82)
    ad, bd = _to_dev_codes(a, fmt), _to_dev_codes(b, fmt)
    kw = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K, tile=tile)
    ref = O.gemm_acc(a, b, fmt, fmt)
    out = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", **kw)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), ref.astype(np.int64))
    g = torch.Generator().manual_seed(83)
    sx, sw, bias = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
    want = ref / (sx.numpy().astype(np.float64)[:, None] * sw.numpy().astype(np.float64)[None, :]) + bias.numpy()
    rg = [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)]
    y32 = ops.gemm(ad, bd, rg, out_dtype=torch.float32, bias=bias.to(DEV), **kw)
    assert np.abs(_np(y32).astype(np.float64) - want).max() <= 2e-6 * np.abs(want).max()
    y16 = ops.gemm(ad, bd, rg, out_dtype=torch.bfloat16, bias=bias.to(DEV), **kw)
    assert (np.abs(y16.float().cpu().numpy().astype(np.float64) - want) <= _bf16_ulp(want)).all()
    own = 21 if N % 96 == 0 and -(-M // 128) * (N // 96) <= 256 else 19
    if -(-M // 128) * -(-N // 128) >= 32 and tile == own:  # the library's own choice for such a shape
        gd = ops.gemm_desc(ad, bd, rg, out_dtype=torch.bfloat16, bias=bias.to(DEV), **{**kw, "tile": 0})
        assert ops.gemm_plan(gd)["tile"] == own
        assert torch.equal(ops.gemm_launch(gd, None), y16)
    two = [ops.Range(0, 128, sx.to(DEV), sw.to(DEV), 0, 1, 1), ops.Range(128, K - 128, sx.to(DEV), sw.to(DEV), 0, 1, 1)]
    if K > 128:
        with pytest.raises(RuntimeError):  # one range only
            ops.gemm(ad, bd, two, out_dtype=torch.float32, **kw)
    e_a, e_b = _to_dev_codes(_rand_codes((M, K), O.FMT_E4M3, 84), O.FMT_E4M3), _to_dev_codes(_rand_codes((N, K), O.FMT_E4M3, 85), O.FMT_E4M3)
    with pytest.raises(RuntimeError):  # int8 only
        ops.gemm(e_a, e_b, [ops.Range(0, K, None, None)], out_dtype="acc", **{**kw, "a_fmt": O.FMT_E4M3, "b_fmt": O.FMT_E4M3})


@pytest.mark.parametrize("tile", [0, 11, 15, 16, 20])
def test_gemm_more_tiles_than_compute_units(ops, tile):
    """4608 x 4608 outputs are 288 to 384 tiles, more than the 256 CUs hold at once."""
    M, N, K = 4608, 4608, 256
    a = _rand_codes((M, K), O.FMT_INT8, 43)
    b = _rand_codes((N, K), O.FMT_INT8, 44)
    ad, bd = _to_dev_codes(a, O.FMT_INT8), _to_dev_codes(b, O.FMT_INT8)
    ref = O.gemm_acc(a, b, O.FMT_INT8, O.FMT_INT8)
    kw = dict(m=M, n=N, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT8, lda=K, ldb=K, tile=tile)
    out = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", **kw)
    assert np.array_equal(out.cpu().numpy().astype(np.int64), ref.astype(np.int64))
    g = torch.Generator().manual_seed(45)
    sx = torch.rand(M, generator=g) + 0.5
    sw = torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g)
    swn = sw.numpy().astype(np.float64)[None, :]
    y = ops.gemm(ad, bd, [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)], out_dtype=torch.bfloat16,
                 bias=bias.to(DEV), **kw)
    want = ref / (sx.numpy().astype(np.float64)[:, None] * swn) + bias.numpy()
    assert (np.abs(y.float().cpu().numpy().astype(np.float64) - want) <= _bf16_ulp(want)).all()
    # two K segments with their own activation scales: the fp32 fold between ranges
    sx2 = torch.rand(M, generator=g) + 0.5
    rg = [ops.Range(0, 128, sx.to(DEV), sw.to(DEV), 0, 1, 1), ops.Range(128, 128, sx2.to(DEV), sw.to(DEV), 0, 1, 1)]
    if tile >= 15:  # these tiles have no second accumulator set
        with pytest.raises(RuntimeError):
            ops.gemm(ad, bd, rg, out_dtype=torch.bfloat16, bias=bias.to(DEV), **kw)
        return
    y = ops.gemm(ad, bd, rg, out_dtype=torch.bfloat16, bias=bias.to(DEV), **kw)
    want = (O.gemm_acc(a[:, :128], b[:, :128], O.FMT_INT8, O.FMT_INT8) / (sx.numpy().astype(np.float64)[:, None] * swn)
            + O.gemm_acc(a[:, 128:], b[:, 128:], O.FMT_INT8, O.FMT_INT8) / (sx2.numpy().astype(np.float64)[:, None] * swn)
            + bias.numpy())
    got = y.float().cpu().numpy().astype(np.float64)
    assert (np.abs(got - want) <= _bf16_ulp(want) + 1e-5 * np.abs(want).max()).all()


def test_gemm_int4_weights_expanded_into_a_lent_workspace(ops):
    """With a workspace the int4 weights are expanded to int8 first: same accumulators
    bit for bit as unpacking inside the GEMM, ragged shapes, a batch, K segments with
    a sign-selected DualScale range, and a workspace that is too small (ignored)."""
    M, N, K, Z = 200, 300, 416, 2
    a = np.stack([_rand_codes((M, K), O.FMT_INT8, 70 + z) for z in range(Z)])
    b = np.stack([_rand_codes((N, K), O.FMT_INT4, 80 + z) for z in range(Z)])
    ad = torch.stack([_to_dev_codes(a[z], O.FMT_INT8) for z in range(Z)])
    bd = torch.stack([_to_dev_codes(b[z], O.FMT_INT4) for z in range(Z)])
    kw = dict(m=M, n=N, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT4, lda=K, ldb=K // 2, batch=Z, batch_stride_a=M * K,
              batch_stride_b=N * K // 2)
    ws = torch.empty(Z * N * K, dtype=torch.uint8, device=DEV)
    fused = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", **kw)
    lent = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", workspace=ws, **kw)
    small = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", workspace=ws[:100], **kw)
    assert torch.equal(fused, lent) and torch.equal(fused, small)
    for z in range(Z):
        assert np.array_equal(lent[z].cpu().numpy().astype(np.int64), O.gemm_acc(a[z], b[z], O.FMT_INT8, O.FMT_INT4).astype(np.int64))
    g = torch.Generator().manual_seed(90)
    sx, sx2, sw, bias = (torch.rand(M, generator=g) + 0.5).to(DEV), (torch.rand(M, generator=g) + 0.5).to(DEV), \
        (torch.rand(N, generator=g) + 0.5).to(DEV), torch.randn(N, generator=g).to(DEV)
    rg = [ops.Range(0, 128, sx, sw, 0, 1, 1), ops.Range(128, K - 128, sx2, sw, 2, 1, 1), ops.Range(128, K - 128, sx, sw, 3, 1, 1)]
    kw1 = dict(kw, batch=1, batch_stride_a=0, batch_stride_b=0)
    y0 = ops.gemm(ad[0], bd[0], rg, out_dtype=torch.float32, bias=bias, **kw1)
    y1 = ops.gemm(ad[0], bd[0], rg, out_dtype=torch.float32, bias=bias, workspace=ws, **kw1)
    assert (y0 - y1).abs().max().item() <= 2e-6 * y0.abs().max().item()


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("tile", [0, 11, 12, 14, 16, 17, 18])
def test_gemm_split_k(ops, fmt, tile):
    """The K steps of every tile shared by 2..7 workgroups, shares that begin and end inside
    ranges, one range and three (K segments + a two-tensor DualScale segment), ragged M and N,
    an N that allows no vector stores: equal to the unsplit launch up to fp32 summation order,
    and to the closed form; what cannot be split is refused."""
    M, N, K0, K1 = 210, 330, 384, 640
    K = K0 + K1
    a, a2, b = _rand_codes((M, K), fmt, 61), _rand_codes((M, K), fmt, 62), _rand_codes((N, K), fmt, 63)
    ad, a2d, bd = (_to_dev_codes(t, fmt) for t in (a, a2, b))
    g = torch.Generator().manual_seed(64)
    s0 = torch.rand(1, generator=g) + 0.5
    sx, sx2 = torch.rand(M, generator=g) + 0.5, torch.rand(M, generator=g) + 0.5
    sw, bias = torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
    one = [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)]
    three = [ops.Range(0, K0, s0.to(DEV), sw.to(DEV), 0, 0, 1), ops.Range(K0, K1, sx.to(DEV), sw.to(DEV), 0, 1, 1),
             ops.Range(K0, K1, sx2.to(DEV), sw.to(DEV), 1, 1, 1)]
    ws = torch.empty(ops.split_bytes(M, N, 8, park=True), dtype=torch.uint8, device=DEV)
    tol = 3e-6 if fmt == O.FMT_INT8 else 3e-4
    for n_cols in (N, N - 1):  # N - 1: rows of the fp32 partial results are not 16-byte multiples
        kw = dict(m=M, n=n_cols, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K, bias=bias[:n_cols].contiguous().to(DEV), a_neg=a2d, tile=tile)
        for rg in (one, three):
            rg = [ops.Range(r.k_begin, r.k_len, r.sx, r.sw[:n_cols].contiguous(), r.a_sel, r.sx_row_stride, r.sw_col_stride) for r in rg]
            ref = ops.gemm(ad, bd, rg, out_dtype=torch.float32, split_k=1, workspace=ws, **kw)
            for sk in (2, 3, 7):
                out = ops.gemm(ad, bd, rg, out_dtype=torch.float32, split_k=sk, workspace=ws, **kw)
                assert (out - ref).abs().max().item() <= tol * ref.abs().max().item(), (n_cols, len(rg), sk)
            o16 = ops.gemm(ad, bd, rg, out_dtype=torch.bfloat16, split_k=3, workspace=ws, **kw)
            r16 = ops.gemm(ad, bd, rg, out_dtype=torch.bfloat16, split_k=1, workspace=ws, **kw)
            assert (o16.float() - r16.float()).abs().max().item() <= 2.0 ** -7 * r16.float().abs().max().item()
    av, a2v, bv = (O.code_values(t, fmt) for t in (a, a2, b))
    swn = sw.numpy().astype(np.float64)[None, :]
    want = (av[:, :K0] @ bv[:, :K0].T / (float(s0) * swn) + av[:, K0:] @ bv[:, K0:].T / (sx.numpy().astype(np.float64)[:, None] * swn) +
            a2v[:, K0:] @ bv[:, K0:].T / (sx2.numpy().astype(np.float64)[:, None] * swn) + bias.numpy().astype(np.float64))
    out = ops.gemm(ad, bd, three, out_dtype=torch.float32, split_k=5, workspace=ws, m=M, n=N, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K,
                   bias=bias.to(DEV), a_neg=a2d, tile=tile)
    assert np.abs(_np(out).astype(np.float64) - want).max() <= (5e-6 if fmt == O.FMT_INT8 else 1e-3) * np.abs(want).max()
    with pytest.raises(RuntimeError):  # no workspace
        ops.gemm(ad, bd, one, out_dtype=torch.float32, split_k=2, m=M, n=N, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K)
    with pytest.raises(RuntimeError):  # the general kernels do not split
        ops.gemm(ad, bd, one, out_dtype=torch.float32, split_k=2, workspace=ws, tile=3, m=M, n=N, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K)


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("tile", [11, 12, 14, 17, 18])
def test_gemm_two_shares_finished_in_the_launch(ops, fmt, tile):
    """A tile split in two along K is finished by whichever of its two workgroups arrives second
    (no second kernel): equal to the unsplit launch up to fp32 summation order, the same bits on
    every run (a + b = b + a), with bias, addend and a bf16 output, over many tiles, a workspace
    that is reused dirty, and a workspace of exactly the size the library asks for."""
    M, N, K = 1024, 1152, 2048
    a, b = _rand_codes((M, K), fmt, 71), _rand_codes((N, K), fmt, 72)
    ad, bd = _to_dev_codes(a, fmt), _to_dev_codes(b, fmt)
    g = torch.Generator().manual_seed(73)
    sx, sw, bias = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
    add = torch.randn(M, N, generator=g).to(torch.bfloat16).to(DEV)
    rg = [ops.Range(0, 768, sx.to(DEV), sw.to(DEV), 0, 1, 1), ops.Range(768, K - 768, sx.to(DEV) * 1.5, sw.to(DEV), 0, 1, 1)]
    kw = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K, bias=bias.to(DEV), tile=tile, addend=add, out_dtype=torch.bfloat16)
    gd = ops.gemm_desc(ad, bd, rg, split_k=2, **kw)
    big = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    plan = ops.gemm_plan(gd, big)
    assert plan["splits"] == 2 and plan["tile"] == tile
    need = ops.gemm_workspace_bytes(gd)
    shape = ops.TILE_SHAPES[tile].split("x")
    tiles = -(-M // int(shape[0])) * -(-N // int(shape[1]))
    assert need >= tiles * 2 * int(shape[0]) * int(shape[1]) * 4 + tiles * 4
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device=DEV)  # dirty: the counters are cleared by the launch
    ref = ops.gemm(ad, bd, rg, split_k=1, workspace=big, **kw)
    outs = [ops.gemm(ad, bd, rg, split_k=2, workspace=ws, **kw).clone() for _ in range(4)]
    for o in outs:
        assert torch.equal(o, outs[0])
    assert (outs[0].float() - ref.float()).abs().max().item() <= 2.0 ** -7 * ref.float().abs().max().item()
    o32 = ops.gemm(ad, bd, rg, split_k=2, workspace=ws, **{**kw, "out_dtype": torch.float32, "addend": None})
    r32 = ops.gemm(ad, bd, rg, split_k=1, workspace=big, **{**kw, "out_dtype": torch.float32, "addend": None})
    assert (o32 - r32).abs().max().item() <= (3e-6 if fmt == O.FMT_INT8 else 3e-4) * r32.abs().max().item()


@pytest.mark.parametrize("tile", [0, 11, 12, 13, 14, 15, 16, 17, 18])
def test_gemm_int8_ranges_parked_in_a_lent_workspace(ops, tile):
    """int8 with K segments and a two-tensor DualScale segment on every 8-wave tile: the sums of
    finished ranges wait in the caller's workspace instead of a second register set.  Checked
    against the closed form (fp64) and the second-accumulator kernels, ragged M and N, per-tensor
    / per-token scales mixed, twice in a row on the same workspace; a workspace that is too small
    is not used (same result as without)."""
    M, N, K0, K1 = 333, 500, 256, 384
    K = K0 + K1
    a, a2 = _rand_codes((M, K), O.FMT_INT8, 51), _rand_codes((M, K), O.FMT_INT8, 52)
    b = _rand_codes((N, K), O.FMT_INT8, 53)
    ad, a2d, bd = (_to_dev_codes(t, O.FMT_INT8) for t in (a, a2, b))
    g = torch.Generator().manual_seed(54)
    s0 = torch.rand(1, generator=g) + 0.5
    sx, sx2 = torch.rand(M, generator=g) + 0.5, torch.rand(M, generator=g) + 0.5
    sw, bias = torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
    rg = [ops.Range(0, K0, s0.to(DEV), sw.to(DEV), 0, 0, 1), ops.Range(K0, K1, sx.to(DEV), sw.to(DEV), 0, 1, 1),
          ops.Range(K0, K1, sx2.to(DEV), sw.to(DEV), 1, 1, 1)]
    kw = dict(m=M, n=N, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT8, lda=K, ldb=K, bias=bias.to(DEV), a_neg=a2d)
    swn = sw.numpy().astype(np.float64)[None, :]
    want = (O.gemm_acc(a[:, :K0], b[:, :K0], O.FMT_INT8, O.FMT_INT8) / (float(s0) * swn) +
            O.gemm_acc(a[:, K0:], b[:, K0:], O.FMT_INT8, O.FMT_INT8) / (sx.numpy().astype(np.float64)[:, None] * swn) +
            O.gemm_acc(a2[:, K0:], b[:, K0:], O.FMT_INT8, O.FMT_INT8) / (sx2.numpy().astype(np.float64)[:, None] * swn) +
            bias.numpy().astype(np.float64))
    ws = torch.empty(ops.park_bytes(M, N), dtype=torch.uint8, device=DEV)
    out = ops.gemm(ad, bd, rg, out_dtype=torch.float32, workspace=ws, tile=tile, **kw)
    assert np.abs(_np(out).astype(np.float64) - want).max() <= 3e-6 * np.abs(want).max()
    again = ops.gemm(ad, bd, rg, out_dtype=torch.float32, workspace=ws, tile=tile, **kw)
    assert torch.equal(out, again)
    if tile in (0, 12, 13, 14):  # tiles the second-accumulator kernels exist for
        plain = ops.gemm(ad, bd, rg, out_dtype=torch.float32, tile=tile, **kw)
        assert (out - plain).abs().max().item() <= 2e-6 * plain.abs().max().item()
        small = ops.gemm(ad, bd, rg, out_dtype=torch.float32, workspace=ws[:4096], tile=tile, **kw)
        assert torch.equal(small, plain)
    o16 = ops.gemm(ad, bd, rg, out_dtype=torch.bfloat16, workspace=ws, tile=tile, **kw)
    assert (np.abs(_np(o16).astype(np.float64) - want) <= _bf16_ulp(want) + 1e-5 * np.abs(want).max()).all()


@pytest.mark.parametrize("op", ["gelu_tanh", "gelu", "silu"])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("dt", ["bf16", "fp32", "fp16"])
def test_quantize_with_fused_activation(ops, op, gated, dt):
    """op(x), or x * op(gate), evaluated inside the quantise kernel.  The kernel's tanhf /
    erff / expf may be an ulp off the oracle's correctly rounded ones, which moves a value
    across a rounding boundary now and then: codes may differ by one step on a small
    fraction of the elements, never by more.  Static per-tensor scale with DualScale into two
    tensors (wave-per-row and workgroup-per-row shapes do not matter here), then dynamic
    per-row scales on both dynamic kernels, checked with the scales the kernel reports."""
    import torch.nn.functional as F
    tdt = TDT[dt]
    for rows, cols in ((33, 1024), (9, 4608)):
        g = torch.Generator().manual_seed(41)
        x = (torch.randn(rows, cols, generator=g) * 2.5).to(tdt)
        gate = (torch.randn(rows, cols, generator=g) * 2).to(tdt) if gated else None
        xd, gd = x.to(DEV), (gate.to(DEV) if gated else None)
        want_act = O.activation(x.float().numpy(), op, gate=gate.float().numpy() if gated else None, dtype=dt)
        # the same thing from torch's own operators on the device: a second, independent check
        fn = {"gelu_tanh": lambda t: F.gelu(t, approximate="tanh"), "gelu": F.gelu, "silu": F.silu}[op]
        torch_act = fn(xd) if not gated else xd * fn(gd)
        pa, na = O.dual_amax(want_act)
        ps, ns = O.int_dual_scales(pa, na, 8)
        sp, sn = torch.tensor([ps], device=DEV), torch.tensor([ns], device=DEV)
        cp, cn = ops.quantize(xd, O.FMT_INT8, sp, sn, dual=True, two_tensors=True, pre_op=op, gate=gd)
        wp, wn = O.quantize_act_dual(want_act[None], np.float32([ps]), np.float32([ns]), O.FMT_INT8)
        tp, tn = ops.quantize(torch_act, O.FMT_INT8, sp, sn, dual=True, two_tensors=True)
        for got, want, tor in ((cp, wp[0], tp), (cn, wn[0], tn)):
            d = np.abs(got.cpu().numpy().astype(np.int32) - want.astype(np.int32))
            assert d.max() <= 1 and (d != 0).mean() <= 4e-3, (d.max(), (d != 0).mean())
            dt_ = (got.int() - tor.int()).abs()
            assert dt_.max().item() <= 1 and (dt_ != 0).float().mean().item() <= 4e-3
        # dynamic per-row scales, e4m3 codes
        scale = torch.empty(rows, device=DEV)
        c = ops.quantize(xd, O.FMT_E4M3, scale, row_stride=1, dynamic=True, pre_op=op, gate=gd)
        want_scale = O.row_scale_div(np.abs(want_act).max(axis=1), 448.0)
        got_scale = scale.cpu().numpy()
        assert (np.abs(got_scale - want_scale) <= 2.0 ** -6 * want_scale).all()  # an ulp of the row's largest value
        wc = O.quantize_act(want_act[None], got_scale, O.FMT_E4M3)[0]
        # (e4m3 keeps three mantissa bits however small the value, so the negative tail of the
        # gelus, where fp32 evaluations of 1 + tanh / 1 + erf carry cancellation noise, lands on
        # neighbouring codes far more often than with the integer codes above)
        same = c.cpu().numpy() == wc
        assert same.mean() >= 1 - 2e-2
        v_got, v_want = O.e4m3_decode(c.cpu().numpy()), O.e4m3_decode(wc)
        assert (np.abs(v_got - v_want) <= 0.126 * np.abs(v_want) + 2.0 ** -9).all()  # neighbouring e4m3 values


@pytest.mark.parametrize("dt", ["bf16", "fp32", "fp16"])
def test_quantize_with_column_divisors(ops, dt):
    """SmoothQuant's x / s inside the quantise kernel: bit-exact against the oracle (IEEE
    division, no transcendental function involved), static and dynamic, alone and after a
    fused activation (there to the fused activation's own bound)."""
    tdt = TDT[dt]
    rows, cols = 37, 1040
    g = torch.Generator().manual_seed(45)
    x = (torch.randn(rows, cols, generator=g) * 3).to(tdt)
    sdiv = torch.rand(cols, generator=g) * 4 + 0.05
    xd = x.to(DEV)
    want = O.smooth_divide(x.float().numpy(), sdiv.numpy(), dt)
    s = (torch.rand(rows, generator=g) * 20 + 0.5)
    for fmt in FMTS:
        c = ops.quantize(xd, fmt, s.to(DEV), row_stride=1, col_div=sdiv.to(DEV))
        assert np.array_equal(_codes_np(c, fmt), O.quantize_act(want[None], s.numpy(), fmt)[0])
    scale = torch.empty(rows, device=DEV)
    c = ops.quantize(xd, O.FMT_INT8, scale, row_stride=1, dynamic=True, col_div=sdiv.to(DEV))
    want_scale = O.row_scale_div(np.abs(want).max(axis=1), 127.0)
    assert np.array_equal(scale.cpu().numpy(), want_scale)
    assert np.array_equal(c.cpu().numpy(), O.quantize_act(want[None], want_scale, O.FMT_INT8)[0])
    act = O.smooth_divide(O.activation(x.float().numpy(), "silu", dtype=dt), sdiv.numpy(), dt)
    c = ops.quantize(xd, O.FMT_INT8, s.to(DEV), row_stride=1, col_div=sdiv.to(DEV), pre_op="silu")
    d = np.abs(c.cpu().numpy().astype(np.int32) - O.quantize_act(act[None], s.numpy(), O.FMT_INT8)[0].astype(np.int32))
    assert d.max() <= 1 and (d != 0).mean() <= 4e-3


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3, O.FMT_INT4])
@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_gemm_addend(ops, fmt, dt):
    """out = acc / (sx sw) + bias + addend, rounded once: every kernel family (general, 8-wave
    through LDS and direct, 32 x 32, split K), ragged shapes, a batch."""
    M, N, K, Z = 150, 264, 256, 2
    fa = O.FMT_INT8 if fmt == O.FMT_INT4 else fmt
    a = np.stack([_rand_codes((M, K), fa, 70 + z) for z in range(Z)])
    b = np.stack([_rand_codes((N, K), fmt, 80 + z) for z in range(Z)])
    ad = torch.stack([_to_dev_codes(a[z], fa) for z in range(Z)])
    bd = torch.stack([_to_dev_codes(b[z], fmt) for z in range(Z)])
    g = torch.Generator().manual_seed(91)
    sx, sw = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g)
    scale = 3000.0 if fmt != O.FMT_E4M3 else 50000.0
    add = (torch.randn(Z, M, N, generator=g) * scale).to(TDT[dt])
    kb = K // 2 if fmt == O.FMT_INT4 else K
    rg = [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)]
    want = np.stack([O.gemm_acc(a[z], b[z], fa, fmt) / (sx.numpy().astype(np.float64)[:, None] * sw.numpy().astype(np.float64)[None, :])
                     + bias.numpy().astype(np.float64) + add[z].float().numpy().astype(np.float64) for z in range(Z)])
    tol = (4e-6 if dt == "fp32" else 2.0 ** -8) + (3e-4 if fmt == O.FMT_E4M3 else 0.0)
    tiles = [0, 1, 3, 14] + ([11, 16] if fmt != O.FMT_INT4 else [])
    for tile in tiles:
        kw = dict(m=M, n=N, a_fmt=fa, b_fmt=fmt, out_dtype=TDT[dt], lda=K, ldb=kb, bias=bias.to(DEV), tile=tile)
        out = ops.gemm(ad, bd, rg, batch=Z, batch_stride_a=M * K, batch_stride_b=N * kb, addend=add.to(DEV), **kw)
        assert np.abs(_np(out).astype(np.float64) - want).max() <= tol * np.abs(want).max(), tile
    if fmt != O.FMT_INT4:
        ws = torch.empty(ops.split_bytes(M, N, 4), dtype=torch.uint8, device=DEV)
        out = ops.gemm(ad[0], bd[0], rg, m=M, n=N, a_fmt=fa, b_fmt=fmt, out_dtype=TDT[dt], lda=K, ldb=kb, bias=bias.to(DEV),
                       addend=add[0].contiguous().to(DEV), split_k=2, workspace=ws)
        assert np.abs(_np(out).astype(np.float64) - want[0]).max() <= tol * np.abs(want[0]).max()
    with pytest.raises(RuntimeError):
        ops.gemm(ad[0], bd[0], [ops.Range(0, K, None, None)], m=M, n=N, a_fmt=fa, b_fmt=fmt, out_dtype="acc", lda=K, ldb=kb,
                 addend=add[0].contiguous().to(DEV))


@pytest.mark.parametrize("fmt_w", [O.FMT_INT4, O.FMT_INT8])
@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_group_wise_weight_scales(ops, fmt_w, dt):
    """Weights with one scale per (row, group of 128 input channels): codes bit-exact against
    the oracle, and the GEMM with group factors against the closed form, on ragged M and N,
    on a single range with per-token scales, and on K segments with a two-tensor DualScale
    segment.  (No counterpart in the reference: the oracle's group functions are the per-row
    ones applied group by group.)"""
    M, N, K, G = 203, 330, 1280, 128
    g = torch.Generator().manual_seed(31)
    w = torch.randn(N, K, generator=g) * 0.02
    w[:, 5] *= 30  # one group per row with a far larger maximum than its neighbours
    bits = 4 if fmt_w == O.FMT_INT4 else 8
    sw = O.int_scale(O.group_amax(w.numpy(), G), bits)  # (N, K / G)
    sw_t = torch.from_numpy(np.ascontiguousarray(sw.T)).to(DEV)
    codes = ops.quantize_weights_groups(fmt_w, w.to(DEV), sw_t, G)
    want_codes = O.quantize_weights_groups(w.numpy(), sw, G, fmt_w)
    assert np.array_equal(_codes_np(codes, fmt_w), want_codes)
    a = _rand_codes((M, K), O.FMT_INT8, 32)
    a2 = _rand_codes((M, K), O.FMT_INT8, 33)
    ad, a2d = _to_dev_codes(a, O.FMT_INT8), _to_dev_codes(a2, O.FMT_INT8)
    sx = (torch.rand(M, generator=g) + 0.5)
    sx2 = (torch.rand(M, generator=g) + 0.5)
    bias = torch.randn(N, generator=g)
    one = torch.ones(1, device=DEV)
    factors = (1.0 / sw_t).contiguous()
    ws = torch.empty(N * K, dtype=torch.uint8, device=DEV)
    kw = dict(m=M, n=N, a_fmt=O.FMT_INT8, b_fmt=fmt_w, out_dtype=TDT[dt], lda=K, ldb=K // 2 if fmt_w == O.FMT_INT4 else K,
              bias=bias.to(DEV), workspace=ws, group_dequant=factors)
    tol = 4e-6 if dt == "fp32" else 2.0 ** -8
    # (a) one range, per-token scales, on each of the tiles the group kernel is built for
    want = O.linear_groups(a, want_codes, sx.numpy(), sw, G, bias.numpy())
    for tile in (0, 12, 13, 14):
        out = ops.gemm(ad, codes, [ops.Range(0, K, sx.to(DEV), one, 0, 1, 0)], tile=tile, **kw)
        assert np.abs(_np(out).astype(np.float64) - want).max() <= tol * np.abs(want).max(), tile
    # (b) K segments [0, 512) and [512, 1280); the second read twice, from two code tensors
    rg = [ops.Range(0, 512, sx.to(DEV), one, 0, 1, 0), ops.Range(512, K - 512, sx2.to(DEV), one, 0, 1, 0),
          ops.Range(512, K - 512, sx.to(DEV), one, 1, 1, 0)]
    outs = [ops.gemm(ad, codes, rg, a_neg=a2d, tile=tile, **kw) for tile in (12, 13, 14)]
    out = outs[2]
    nog = O.linear_groups  # per part: groups are indexed by absolute K, so slice the scales with the codes
    want = (nog(a[:, :512], want_codes[:, :512], sx.numpy(), sw[:, :4], G) +
            nog(a[:, 512:], want_codes[:, 512:], sx2.numpy(), sw[:, 4:], G) +
            nog(a2[:, 512:], want_codes[:, 512:], sx.numpy(), sw[:, 4:], G) + bias.numpy().astype(np.float64))
    for o in outs:
        assert np.abs(_np(o).astype(np.float64) - want).max() <= tol * np.abs(want).max()
    # what the group kernel does not serve is refused, not approximated
    with pytest.raises(RuntimeError):
        ops.gemm(ad, codes, [ops.Range(0, K, sx.to(DEV), one, 2, 1, 0)], **kw)
    if fmt_w == O.FMT_INT4:
        with pytest.raises(RuntimeError):
            ops.gemm(ad, codes, [ops.Range(0, K, sx.to(DEV), one, 0, 1, 0)], **dict(kw, workspace=None))


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_gemm_sign_selected_halves_of_merged_codes(ops, fmt):
    M, N, K = 70, 90, 320
    a = _rand_codes((M, K), fmt, 12)
    b = _rand_codes((N, K), fmt, 13)
    ad, bd = _to_dev_codes(a, fmt), _to_dev_codes(b, fmt)
    av = O.code_values(a, fmt)
    neg = (a.view(np.uint8) & 0x80) != 0 if fmt == O.FMT_E4M3 else a < 0
    for sel, keep in ((2, ~neg), (3, neg)):
        out = ops.gemm(ad, bd, [ops.Range(0, K, None, None, a_sel=sel)], m=M, n=N, a_fmt=fmt, b_fmt=fmt,
                       out_dtype="acc", lda=K, ldb=K)
        ref = np.where(keep, av, 0.0) @ O.code_values(b, fmt).T
        got = out.cpu().numpy().astype(np.float64)
        if fmt == O.FMT_INT8:
            assert np.array_equal(got, ref)
        else:
            assert (np.abs(got - ref) <= FP8_ACC_TOL * (np.abs(av) @ np.abs(O.code_values(b, fmt)).T) + 1e-30).all()


def test_gemm_batched_sub_range_and_second_tensor(ops):
    S, M, N, K = 3, 40, 50, 256
    a = _rand_codes((S, M, K), O.FMT_INT8, 14)
    a2 = _rand_codes((S, M, K), O.FMT_INT8, 15)
    b = _rand_codes((S, N, K), O.FMT_INT8, 16)
    ad, a2d, bd = (torch.from_numpy(t).to(DEV) for t in (a, a2, b))
    out = ops.gemm(ad, bd, [ops.Range(64, 96, None, None, a_sel=1)], m=M, n=N, a_fmt=O.FMT_INT8,
                   b_fmt=O.FMT_INT8, out_dtype="acc", lda=K, ldb=K, a_neg=a2d, batch=S,
                   batch_stride_a=M * K, batch_stride_b=N * K)
    for s in range(S):
        ref = O.gemm_acc(a2[s][:, 64:160], b[s][:, 64:160], O.FMT_INT8, O.FMT_INT8)
        assert np.array_equal(out[s].cpu().numpy().astype(np.int64), ref.astype(np.int64))


# ------------------------------------------------------------------ fused epilogue
@pytest.mark.parametrize("odt", ["fp32", "bf16", "fp16"])
@pytest.mark.parametrize("fa,fb", [(O.FMT_INT8, O.FMT_INT8), (O.FMT_E4M3, O.FMT_E4M3), (O.FMT_INT8, O.FMT_INT4)])
def test_gemm_dequant_bias_all_scale_shapes(ops, odt, fa, fb):
    M, N, K = 77, 133, 192
    a = _rand_codes((M, K), fa, 20)
    b = _rand_codes((N, K), fb, 21)
    if fa == O.FMT_E4M3:  # keep magnitudes finite in fp16
        a &= 0xBF
        b &= 0xBF
    ad, bd = _to_dev_codes(a, fa), _to_dev_codes(b, fb)
    g = torch.Generator().manual_seed(22)
    bias = torch.randn(N, generator=g).to(DEV)
    acc = O.gemm_acc(a, b, fa, fb)
    mag = np.abs(O.code_values(a, fa)) @ np.abs(O.code_values(b, fb)).T
    for per_row in (False, True):
        for per_col in (False, True):
            sx = (torch.rand(M if per_row else 1, generator=g) * 50 + 1).to(DEV)
            sw = (torch.rand(N if per_col else 1, generator=g) * 500 + 1).to(DEV)
            out = ops.gemm(ad, bd, [ops.Range(0, K, sx, sw, 0, int(per_row), int(per_col))], m=M, n=N,
                           a_fmt=fa, b_fmt=fb, out_dtype=TDT[odt], lda=K, ldb=K // 2 if fb == O.FMT_INT4 else K,
                           bias=bias)
            sxn = np.broadcast_to(sx.cpu().numpy().reshape(-1, 1), (M, 1))
            swn = np.broadcast_to(sw.cpu().numpy().reshape(1, -1), (1, N))
            exact = acc / (sxn.astype(np.float64) * swn) + bias.cpu().numpy()
            got = _np(out).astype(np.float64)
            if fa == O.FMT_E4M3:
                ulp = {"fp32": 0.0, "bf16": 2.0 ** -8, "fp16": 2.0 ** -11}[odt]
                tol = FP8_ACC_TOL * mag / (sxn.astype(np.float64) * swn) + ulp * np.abs(exact) + 1e-6
                assert (np.abs(got - exact) <= tol).all()
            elif odt == "fp32":
                assert np.abs(got - exact).max() <= 2e-6 * np.abs(exact).max()
            else:
                want = O.round_to_dtype(exact.astype(np.float32), odt).astype(np.float64)
                ulp = 2.0 ** (-7 if odt == "bf16" else -10)
                assert (np.abs(got - want) <= ulp * np.abs(want) + 1e-30).all()
                assert (got != want).mean() < 1e-3  # only ties flip


def test_gemm_fold_two_k_segments_plus_dual(ops):
    """K = [attn | mlp]: segment 0 single scale, segment 1 DualScale -> three ranges."""
    M, N, K0, K1 = 150, 200, 128, 320
    K = K0 + K1
    g = torch.Generator().manual_seed(30)
    x = torch.randn(M, K, generator=g)
    x[:, K0:] = torch.nn.functional.gelu(x[:, K0:] * 2, approximate="tanh")
    w = torch.randn(N, K, generator=g) * 0.02
    xn, wn = x.numpy(), w.numpy()
    s0 = np.float32(O.int_scale(float(np.abs(xn[:, :K0]).max())))
    pa, na = O.dual_amax(xn[:, K0:])
    ps, ns = (np.float32(t) for t in O.int_dual_scales(pa, na))
    sw = np.float32(O.int_scale(float(np.abs(wn).max())))
    wq = O.quantize_weights(wn, float(sw), O.FMT_INT8)
    xd = x.to(DEV)
    pos = torch.tensor([s0, ps], device=DEV)
    neg = torch.tensor([s0, ns], device=DEV)
    swd = torch.tensor([sw], device=DEV)
    codes = ops.quantize(xd, O.FMT_INT8, pos, neg, kseg_bounds=[0, K0, K], kseg_stride=1, dual=True,
                         dual_kseg_mask=0b10)
    bias = torch.randn(N, generator=g).to(DEV)
    ranges = [ops.Range(0, K0, pos[0:1], swd, 0), ops.Range(K0, K1, pos[1:2], swd, 2),
              ops.Range(K0, K1, neg[1:2], swd, 3)]
    for tile in (2, 3, 4, 5):
        out = ops.gemm(codes, torch.from_numpy(wq).to(DEV), ranges, m=M, n=N, a_fmt=O.FMT_INT8,
                       b_fmt=O.FMT_INT8, out_dtype=torch.float32, lda=K, ldb=K, bias=bias, tile=tile)
        # oracle: three exact partial sums, each divided by its scales
        c0 = O.quantize_act(xn[None, :, :K0], [s0], O.FMT_INT8)[0]
        cp, cn = O.quantize_act_dual(xn[None, :, K0:], [ps], [ns], O.FMT_INT8)
        y = (O.gemm_acc(c0, wq[:, :K0], O.FMT_INT8, O.FMT_INT8) / (np.float64(s0) * sw)
             + O.gemm_acc(cp[0], wq[:, K0:], O.FMT_INT8, O.FMT_INT8) / (np.float64(ps) * sw)
             + O.gemm_acc(cn[0], wq[:, K0:], O.FMT_INT8, O.FMT_INT8) / (np.float64(ns) * sw)
             + bias.cpu().numpy())
        got = out.cpu().numpy().astype(np.float64)
        assert np.abs(got - y).max() <= 1e-5 * np.abs(y).max(), tile
        # and within the path's tolerance of the fp32 fake-quant linear
        xf = np.concatenate([O.fake_quant_int(xn[:, :K0], s0), O.fake_quant_int_dual(xn[:, K0:], ps, ns)], axis=1)
        ref = xf @ O.fake_quant_int(wn, sw).T + bias.cpu().numpy()
        assert np.abs(got - ref).max() <= 1e-3 * np.abs(ref).max()


# ------------------------------------------------------------------ the reference's op contract
GRID = [(O.FMT_INT8, O.FMT_INT8, 1e-3), (O.FMT_E4M3, O.FMT_E4M3, 1e-2), (O.FMT_INT8, O.FMT_INT4, 1e-3)]


def _fake(x, fmt, s):
    return O.fake_quant_fp8(x, s) if fmt == O.FMT_E4M3 else O.fake_quant_int(x, s, 4 if fmt == O.FMT_INT4 else 8)


def _scale_of(amax, fmt):
    return O.fp8_scale(amax) if fmt == O.FMT_E4M3 else O.int_scale(amax, 4 if fmt == O.FMT_INT4 else 8)


@pytest.mark.parametrize("fa,fw,tol", GRID)
@pytest.mark.parametrize("axis", [False, True])
@pytest.mark.parametrize("seg", ["none", "weight", "input"])
@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_reference_contract_scaled(ops, fa, fw, tol, axis, seg, dt):
    """Same grid as the reference's test_mix_real (test/test_linear.py:901-913):
    types x per-tensor / per-token+per-channel x segmentation."""
    B, Mtok, K, N = 2, 3, 256, 192
    S = 1 if seg == "none" else 2
    g = torch.Generator().manual_seed(40)
    x = torch.randn(B, Mtok, K, generator=g).to(TDT[dt])
    w = torch.randn(N, K, generator=g) * 0.02
    xs, ws = O.segment_views(_np(x), w.numpy(), "weight" if seg == "none" else seg, S)
    xs = np.ascontiguousarray(xs)
    ws = np.ascontiguousarray(ws)
    M = B * Mtok
    if axis:
        sx = np.stack([_scale_of(np.abs(xs[s]).reshape(M, -1).max(-1), fa) for s in range(S)]).astype(np.float32)
        sw = np.stack([_scale_of(np.abs(ws[s]).max(-1), fw) for s in range(S)]).astype(np.float32)
    else:
        sx = np.float32([_scale_of(float(np.abs(xs[s]).max()), fa) for s in range(S)])
        sw = np.float32([_scale_of(float(np.abs(ws[s]).max()), fw) for s in range(S)])
    wq = np.stack([O.quantize_weights(ws[s], sw[s] if axis else float(sw[s]), fw) for s in range(S)])
    wq_dev = (torch.from_numpy(np.stack([O.pack_int4(wq[s]) for s in range(S)])) if fw == O.FMT_INT4
              else torch.from_numpy(wq)).to(DEV)
    xin = torch.from_numpy(xs).to(TDT[dt]).to(DEV)
    out = ops.real_quantized_gemm_scaled(fa, fw, xin, wq_dev, torch.from_numpy(sx).to(DEV),
                                         torch.from_numpy(sw).to(DEV))
    assert out.shape == (S, B, Mtok, ws.shape[1]) and out.dtype == TDT[dt]
    # oracle of the real pipeline (same codes): tight
    wq_or = wq_dev.cpu().numpy()
    want = O.real_quantized_gemm_scaled(xs, wq_or, sx, sw, fa, fw, out_dtype=dt)
    got = _np(out).astype(np.float64)
    ulp = {"fp32": 2e-6, "bf16": 2.0 ** -7}[dt]
    if fa == O.FMT_E4M3:
        ulp += 1e-3  # limited-width accumulation inside the fp8 MFMA
    scale = np.abs(want).max()
    assert np.abs(got - want).max() <= ulp * scale
    # fp32 fake-quant reference: the path's stated tolerance (fp32 output only;
    # a bf16 result carries its own 2^-9 rounding)
    if dt == "fp32":
        sxb = sx.reshape(S, M, 1) if axis else sx.reshape(S, 1, 1)
        swb = sw.reshape(S, -1, 1) if axis else sw.reshape(S, 1, 1)
        xf = np.stack([_fake(xs[s].reshape(M, -1), fa, sxb[s]) for s in range(S)])
        wf = np.stack([_fake(ws[s], fw, swb[s]) for s in range(S)])
        ref = O.segmented_matmul(xf, wf).reshape(got.shape)
        assert np.abs(got - ref).max() <= tol * np.abs(ref).max()


@pytest.mark.parametrize("fa,fw,tol", GRID)
@pytest.mark.parametrize("axis", [False, True])
def test_reference_contract_dual_scaled(ops, fa, fw, tol, axis):
    S, M, K, N = 2, 10, 128, 96
    g = torch.Generator().manual_seed(41)
    x = torch.nn.functional.silu(torch.randn(S, M, K, generator=g) * 3)
    w = torch.randn(S, N, K, generator=g) * 0.02
    xn, wn = x.numpy(), w.numpy()
    bits_a = 8
    if axis:
        pa, na = O.dual_amax(xn, axis=-1)
        ps, ns = O.fp8_dual_scales(pa, na) if fa == O.FMT_E4M3 else O.int_dual_scales(pa, na, bits_a)
        sw = np.stack([_scale_of(np.abs(wn[s]).max(-1), fw) for s in range(S)]).astype(np.float32)
    else:
        pn = [O.dual_amax(xn[s]) for s in range(S)]
        sc = [O.fp8_dual_scales(*t) if fa == O.FMT_E4M3 else O.int_dual_scales(*t, bits_a) for t in pn]
        ps, ns = np.float32([t[0] for t in sc]), np.float32([t[1] for t in sc])
        sw = np.float32([_scale_of(float(np.abs(wn[s]).max()), fw) for s in range(S)])
    wq = np.stack([O.quantize_weights(wn[s], sw[s] if axis else float(sw[s]), fw) for s in range(S)])
    wq_dev = (torch.from_numpy(np.stack([O.pack_int4(wq[s]) for s in range(S)])) if fw == O.FMT_INT4
              else torch.from_numpy(wq)).to(DEV)
    out = ops.real_quantized_gemm_dual_scaled(fa, fw, x.to(DEV), wq_dev, torch.from_numpy(np.float32(ps)).to(DEV),
                                              torch.from_numpy(np.float32(ns)).to(DEV), torch.from_numpy(sw).to(DEV))
    want = O.real_quantized_gemm_dual_scaled(xn, wq_dev.cpu().numpy(), ps, ns, sw, fa, fw)
    got = out.cpu().numpy().astype(np.float64)
    assert np.abs(got - want).max() <= (1e-3 if fa == O.FMT_E4M3 else 3e-6) * np.abs(want).max()
    psb = np.float32(ps).reshape(S, -1, 1)
    nsb = np.float32(ns).reshape(S, -1, 1)
    swb = sw.reshape(S, -1, 1)
    xf = np.stack([(O.fake_quant_fp8_dual(xn[s], psb[s], nsb[s]) if fa == O.FMT_E4M3
                    else O.fake_quant_int_dual(xn[s], psb[s], nsb[s])) for s in range(S)])
    wf = np.stack([_fake(wn[s], fw, swb[s]) for s in range(S)])
    ref = O.segmented_matmul(xf, wf)
    assert np.abs(got - ref).max() <= tol * np.abs(ref).max()


def test_errors_are_runtime_errors(ops):
    x = torch.randn(1, 4, 40, device=DEV)  # K = 40 is not a multiple of 16
    w = torch.zeros(1, 8, 40, dtype=torch.int8, device=DEV)
    s = torch.ones(1, device=DEV)
    with pytest.raises(RuntimeError):
        ops.real_quantized_gemm_scaled(O.FMT_INT8, O.FMT_INT8, x, w, s, s)
    with pytest.raises(RuntimeError):
        ops.real_quantized_gemm_scaled(O.FMT_INT8, O.FMT_INT8, x.cpu(), w, s, s)


# ------------------------------------------------------------------ quantise + GEMM in one call
@pytest.mark.parametrize("mode", ["static", "dynamic", "dual"])
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_segq_linear_one_call_against_the_oracle(ops, mode, fmt):
    """segq_linear through the C ABI: static per-tensor, dynamic per-token and DualScale (two code
    tensors) activations, checked against the oracle's codes, scales and closed-form output; and
    its refusal of descriptors whose GEMM does not read what the quantise step writes."""
    M, K, N = 200, 384, 320
    g = torch.Generator().manual_seed(40)
    x = torch.randn(M, K, generator=g)
    if mode == "dual":
        x = torch.nn.functional.gelu(x * 2, approximate="tanh")
    x = x.to(torch.bfloat16)
    xn = x.float().numpy()
    w = (torch.randn(N, K, generator=g) * 0.02).numpy()
    lim = 448.0 if fmt == O.FMT_E4M3 else 127.0
    sw = np.float32(O.fp8_scale(float(np.abs(w).max())) if fmt == O.FMT_E4M3 else O.int_scale(float(np.abs(w).max())))
    wq = O.quantize_weights(w, float(sw), fmt)
    bias = torch.randn(N, generator=g)
    xd, wd, swd, bd = x.to(DEV), torch.from_numpy(wq).to(DEV), torch.tensor([sw], device=DEV), bias.to(DEV)
    kw = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.float32, lda=K, ldb=K, bias=bd)
    if mode == "static":
        s = np.float32(lim / np.abs(xn).max())
        sd = torch.tensor([s], device=DEV)
        q = ops.quantize_desc(xd, fmt, sd)
        gd = ops.gemm_desc(q[1], wd, [ops.Range(0, K, sd, swd, 0, 0, 0)], **kw)
        codes = O.quantize_act(xn[None], [s], fmt)[0]
        want = O.gemm_acc(codes, wq, fmt, fmt) / (np.float64(s) * sw)
    elif mode == "dynamic":
        sd = torch.empty(M, device=DEV)
        q = ops.quantize_desc(xd, fmt, sd, row_stride=1, dynamic=True)
        gd = ops.gemm_desc(q[1], wd, [ops.Range(0, K, sd, swd, 0, 1, 0)], **kw)
        s = O.row_scale_div(np.abs(xn).max(axis=1), lim)
        codes = O.quantize_act(xn[None], s, fmt)[0]
        want = O.gemm_acc(codes, wq, fmt, fmt) / (s.astype(np.float64)[:, None] * sw)
    else:
        pa, na = O.dual_amax(xn)
        ps, ns = (np.float32(t) for t in (O.fp8_dual_scales(pa, na) if fmt == O.FMT_E4M3 else O.int_dual_scales(pa, na)))
        pd, nd = torch.tensor([ps], device=DEV), torch.tensor([ns], device=DEV)
        q = ops.quantize_desc(xd, fmt, pd, nd, dual=True, two_tensors=True)
        cp_t, cn_t = q[1]
        gd = ops.gemm_desc(cp_t, wd, [ops.Range(0, K, pd, swd, 0, 0, 0), ops.Range(0, K, nd, swd, 1, 0, 0)], a_neg=cn_t, **kw)
        cp, cn = O.quantize_act_dual(xn[None], [ps], [ns], fmt)
        codes = cp[0]
        want = (O.gemm_acc(cp[0], wq, fmt, fmt) / (np.float64(ps) * sw) + O.gemm_acc(cn[0], wq, fmt, fmt) / (np.float64(ns) * sw))
    out = ops.linear(q, gd)
    want = want + bias.numpy().astype(np.float64)
    got_codes = (q[1][0] if mode == "dual" else q[1]).cpu().numpy()
    assert np.array_equal(got_codes.view(np.uint8), codes.view(np.uint8))
    if mode == "dual":
        assert np.array_equal(q[1][1].cpu().numpy().view(np.uint8), cn[0].view(np.uint8))
    if mode == "dynamic":
        assert np.array_equal(sd.cpu().numpy(), s)
    got = out.cpu().numpy().astype(np.float64)
    tol = 1e-5 if fmt == O.FMT_INT8 else 1e-3
    assert np.abs(got - want).max() <= tol * np.abs(want).max()
    # the same result as the two calls made separately
    sep = ops.gemm(got_codes_t := (q[1][0] if mode == "dual" else q[1]), wd, gd[3][-1],
                   a_neg=q[1][1] if mode == "dual" else None, **kw)
    assert torch.equal(sep, out)
    # refusals: a GEMM that reads other codes, another row count, scales the dynamic step does not write
    other = torch.empty_like(got_codes_t)
    bad = ops.gemm_desc(other, wd, gd[3][-1], a_neg=q[1][1] if mode == "dual" else None, **kw)
    with pytest.raises(RuntimeError, match="must read the codes"):
        ops.linear(q, bad)
    bad = ops.gemm_desc(got_codes_t, wd, gd[3][-1], a_neg=q[1][1] if mode == "dual" else None, **{**kw, "m": M - 8})
    with pytest.raises(RuntimeError, match="do not match"):
        ops.linear(q, bad)
    if mode == "dual":
        bad = ops.gemm_desc(got_codes_t, wd, gd[3][-1], a_neg=other, **kw)
        with pytest.raises(RuntimeError, match="a_neg"):
            ops.linear(q, bad)
    if mode == "dynamic":
        elsewhere = torch.ones(M, device=DEV)
        bad = ops.gemm_desc(got_codes_t, wd, [ops.Range(0, K, elsewhere, swd, 0, 1, 0)], **kw)
        with pytest.raises(RuntimeError, match="does not write"):
            ops.linear(q, bad)


# ------------------------------------------------------------------ weight-side formats
@pytest.mark.parametrize("out,cols", [(2, 2), (6, 4), (130, 34), (128, 256), (1280, 5120), (3074, 1026)])
def test_int4_column_to_row_repack_bit_exact(ops, out, cols):
    """segq_repack_int4_cols_to_rows against the oracle's restatement of the reference's
    colpacked1d_to_rowpacked1d, over every byte value and on ragged patches."""
    g = np.random.default_rng(out * 7 + cols)
    src = g.integers(0, 256, size=cols * out // 2).astype(np.uint8)
    src[:256] = np.arange(256, dtype=np.uint8)[:src[:256].size]
    got = ops.repack_int4_cols_to_rows(torch.from_numpy(src).to(DEV), out, cols).cpu().numpy()
    assert np.array_equal(got, O.repack_int4_cols_to_rows(src, out, cols))
    with pytest.raises(AssertionError):
        ops.repack_int4_cols_to_rows(torch.zeros(3, dtype=torch.uint8, device=DEV), 3, 2)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dt", ["fp32", "bf16"])
def test_group_wise_weight_codes_one_launch_any_number_of_groups(ops, fmt, dt):
    """segq_quantize_weights_groups on 40 groups (more than the eight column segments one
    activation launch takes) and a group size other than 128, bit-exact against the oracle."""
    for N, K, G in [(48, 5120, 128), (33, 640, 32), (20, 2048, 256)]:
        g = torch.Generator().manual_seed(N + K)
        w = (torch.randn(N, K, generator=g) * 0.05).to(TDT[dt])
        wn = _np(w).astype(np.float32)
        lim = {O.FMT_INT8: 127.0, O.FMT_INT4: 7.0, O.FMT_E4M3: 448.0}[fmt]
        scale = (lim / np.maximum(O.group_amax(wn, G), 2.0 ** -24)).astype(np.float32)  # (N, K / G)
        sc = torch.from_numpy(np.ascontiguousarray(scale.T)).to(DEV)                     # (K / G, N)
        codes = ops.quantize_weights_groups(fmt, w.to(DEV), sc, G)
        want = O.quantize_weights_groups(wn, scale, G, fmt)
        assert np.array_equal(_codes_np(codes, fmt).view(np.uint8), want.view(np.uint8)), (N, K, G)


# ------------------------------------------------------------------ low-rank branch in the epilogue
def _e4m3_codes(g, shape):
    """Moderate e4m3 codes (|value| <= 16) without the NaN patterns."""
    c = g.integers(0, 256, size=shape).astype(np.uint8)
    c = (c & 0x80) | np.minimum(c & 0x7F, 0x58)
    return c.astype(np.uint8)


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("dt", ["bf16", "fp16"])
@pytest.mark.parametrize("ranges", [1, 3])
@pytest.mark.parametrize("lend", [False, True])
def test_gemm_low_rank_branch_in_the_epilogue(ops, fmt, dt, ranges, lend):
    """out = sum_r A_r B_r^T / (sx_r sw_r) + bias + T L2 with the low-rank product computed by the
    epilogue's MFMAs: against the fp64 closed form on every 8-wave tile, with one range and with
    three (a second accumulator set, parked ranges when a workspace is lent, fp32 sums rescaled in
    place for e4m3), ragged M and N, ranks 32 and 96."""
    M, N, K = 330, 424, 768
    g = np.random.default_rng(77)
    a = g.integers(-128, 128, size=(M, K)).astype(np.int8) if fmt == O.FMT_INT8 else _e4m3_codes(g, (M, K))
    a2 = g.integers(-128, 128, size=(M, K)).astype(np.int8) if fmt == O.FMT_INT8 else _e4m3_codes(g, (M, K))
    b = g.integers(-128, 128, size=(N, K)).astype(np.int8) if fmt == O.FMT_INT8 else _e4m3_codes(g, (N, K))
    av, a2v, bv = (O.code_values(t, fmt) for t in (a, a2, b))
    tg = torch.Generator().manual_seed(78)
    sx0 = torch.rand(1, generator=tg) * 50 + 20
    sx1, sx2 = torch.rand(M, generator=tg) * 50 + 20, torch.rand(M, generator=tg) * 50 + 20
    sw = torch.rand(N, generator=tg) * 50 + 20
    bias = torch.randn(N, generator=tg)
    ad, a2d, bd = (torch.from_numpy(t).to(DEV) for t in (a, a2, b))
    if ranges == 1:
        rg = [ops.Range(0, K, sx1.to(DEV), sw.to(DEV), 0, 1, 1)]
        base = (av @ bv.T) / (sx1.numpy().astype(np.float64)[:, None] * sw.numpy().astype(np.float64)[None, :])
    else:
        K0 = 256
        swd = sw.to(DEV)
        rg = [ops.Range(0, K0, sx0.to(DEV), swd, 0, 0, 1), ops.Range(K0, K - K0, sx1.to(DEV), swd, 0, 1, 1),
              ops.Range(K0, K - K0, sx2.to(DEV), swd, 1, 1, 1)]
        s0, s1, s2, swn = (t.numpy().astype(np.float64) for t in (sx0, sx1, sx2, sw))
        base = ((av[:, :K0] @ bv[:, :K0].T) / (s0[0] * swn[None, :]) + (av[:, K0:] @ bv[:, K0:].T) / (s1[:, None] * swn[None, :])
                + (a2v[:, K0:] @ bv[:, K0:].T) / (s2[:, None] * swn[None, :]))
    for rank in (32, 96):
        t_lr = (torch.randn(M, rank, generator=tg) * 0.5).to(TDT[dt])
        l2t = (torch.randn(N, rank, generator=tg) * 0.5).to(TDT[dt])
        want = base + bias.numpy().astype(np.float64) + t_lr.double().numpy() @ l2t.double().numpy().T
        ws = torch.empty(ops.park_bytes(M, N), dtype=torch.uint8, device=DEV) if lend else None
        for tile in (0, 11, 12, 13, 14, 15, 16, 17, 18):
            if ranges == 3 and fmt == O.FMT_INT8 and not lend and tile in (11, 15, 16, 17, 18):
                continue  # these tiles have no second accumulator set: they need the workspace
            if tile in (13, 15, 16):  # tiles that are not built with the finish in output units
                with pytest.raises(RuntimeError):
                    ops.gemm(ad, bd, rg, m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=TDT[dt], lda=K, ldb=K, bias=bias.to(DEV),
                             a_neg=a2d if ranges == 3 else None, tile=tile, workspace=ws, lowrank=(t_lr.to(DEV), l2t.to(DEV)))
                continue
            out = ops.gemm(ad, bd, rg, m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=TDT[dt], lda=K, ldb=K, bias=bias.to(DEV),
                           a_neg=a2d if ranges == 3 else None, tile=tile, workspace=ws, lowrank=(t_lr.to(DEV), l2t.to(DEV)))
            got = out.float().cpu().numpy().astype(np.float64)
            ulp = 2.0 ** -8 if dt == "bf16" else 2.0 ** -11
            tol = ulp * np.abs(want) + (3e-4 if fmt == O.FMT_E4M3 else 1e-5) * np.abs(want).max()
            assert (np.abs(got - want) <= tol).all(), (tile, rank, float((np.abs(got - want) / tol).max()))
    # what the branch does not serve is refused, not ignored
    t_lr, l2t = torch.zeros(M, 32, device=DEV), torch.zeros(N, 32, device=DEV)
    with pytest.raises(RuntimeError):
        ops.gemm(ad, bd, rg[:1], m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.float32, lda=K, ldb=K, lowrank=(t_lr, l2t))
    with pytest.raises(RuntimeError, match="low-rank"):
        ops.gemm(ad, bd, rg[:1], m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=TDT[dt], lda=K, ldb=K, tile=3,
                 lowrank=(t_lr.to(TDT[dt]), l2t.to(TDT[dt])))


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_empty_inputs_through_the_wrappers(ops, fmt):
    """No rows to quantise, no rows or no columns to multiply: the calls succeed, give tensors of
    the right empty shape and leave a poisoned neighbour untouched."""
    K, N = 256, 192
    x = torch.randn(0, K, dtype=torch.bfloat16, device=DEV)
    s = torch.full((1,), 3.0, device=DEV)
    codes = ops.quantize(x, fmt, s)
    assert codes.shape == (0, K)
    sd = torch.empty(0, device=DEV)
    codes = ops.quantize(x, fmt, sd, row_stride=1, dynamic=True)
    assert codes.shape == (0, K)
    b = _to_dev_codes(_rand_codes((N, K), fmt, 5), fmt)
    one = torch.ones(1, device=DEV)
    guard = torch.full((4, N), 7.0, dtype=torch.bfloat16, device=DEV)
    out = ops.gemm(codes, b, [ops.Range(0, K, one, one, 0, 0, 0)], m=0, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.bfloat16,
                   lda=K, ldb=K, out=guard[:0])
    assert out.shape == (0, N)
    a = _to_dev_codes(_rand_codes((8, K), fmt, 6), fmt)
    out = ops.gemm(a, b[:0], [ops.Range(0, K, one, one, 0, 0, 0)], m=8, n=0, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.bfloat16,
                   lda=K, ldb=K)
    assert out.shape == (8, 0)
    torch.cuda.synchronize()
    assert bool((guard == 7.0).all())


@pytest.mark.parametrize("pad,off", [(16, 8), (5, 3)])   # 16-byte aligned rows of the view, and not
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_gemm_writes_into_a_view_of_a_wider_buffer(ops, fmt, pad, off):
    """segq_gemm_desc.ldo larger than n: the output is a column slice of a wider row-major buffer
    (the way fused projections are laid side by side).  Every kind of launch writes the same
    values as into a contiguous tensor and nothing outside the slice: the general kernel, the
    8-wave tiles incl. 384x192, K shares finished in the launch and by the second kernel, parked
    ranges, group factors, raw accumulators and fp32 output."""
    one = torch.ones(1, device=DEV)
    g = torch.Generator().manual_seed(123)

    def run(M, N, K, ranges_of, odt, **kw):
        a, a2, b = _rand_codes((M, K), fmt, 50), _rand_codes((M, K), fmt, 51), _rand_codes((N, K), fmt, 52)
        ad, a2d, bd = _to_dev_codes(a, fmt), _to_dev_codes(a2, fmt), _to_dev_codes(b, fmt)
        sx = (torch.rand(M, generator=g) + 0.5).to(DEV)
        sw = (torch.rand(N, generator=g) + 0.5).to(DEV)
        rg = ranges_of(K, sx, sw)
        bias = None if odt == "acc" else torch.randn(N, generator=g).to(DEV)
        common = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=odt, lda=K, ldb=K, a_neg=a2d, bias=bias, **kw)
        want = ops.gemm(ad, bd, rg, **common)
        tdt = want.dtype
        poison = 77 if tdt == torch.int32 else 77.0
        buf = torch.full((M, N + pad), poison, dtype=tdt, device=DEV)
        got = ops.gemm(ad, bd, rg, out=buf[:, off:off + N], **common)
        torch.cuda.synchronize()
        assert got.data_ptr() == buf[:, off:].data_ptr()
        assert torch.equal(buf[:, off:off + N], want), (M, N, K, odt, kw)
        assert bool((buf[:, :off] == poison).all()) and bool((buf[:, off + N:] == poison).all()), (M, N, K, odt, kw)

    plain = lambda K, sx, sw: [ops.Range(0, K, sx, sw, 0, 1, 1)]
    dual = lambda K, sx, sw: [ops.Range(0, K // 2, sx, sw, 0, 1, 1), ops.Range(K // 2, K // 2, sx, one, 0, 1, 0),
                              ops.Range(K // 2, K // 2, sx, sw, 1, 1, 1)]
    ws = lambda: torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    run(70, 90, 320, plain, torch.bfloat16)                                   # general kernel
    run(70, 90, 320, plain, "acc")
    run(300, 700, 384, plain, torch.bfloat16, tile=11)
    run(300, 700, 384, plain, torch.float32, tile=15)
    run(400, 200, 256, plain, torch.bfloat16, tile=20)
    run(400, 200, 256, plain, "acc", tile=20)
    run(300, 200, 2048, plain, torch.bfloat16, tile=17, split_k=2, workspace=ws())   # finished in the launch
    run(300, 200, 2048, plain, torch.float16, tile=17, split_k=4, workspace=ws())    # summed by the second kernel
    run(300, 200, 1024, dual, torch.bfloat16, tile=16 if fmt == O.FMT_E4M3 else 11, workspace=ws())  # rescaled in place / parked
    run(300, 200, 1024, dual, torch.bfloat16)                                  # the library's choice without a workspace
    if fmt == O.FMT_INT8:
        fac = (torch.rand(1024 // 128, 200, generator=g) + 0.5).to(DEV)
        run(300, 200, 1024, lambda K, sx, sw: [ops.Range(0, K, sx, one, 0, 1, 0)], torch.bfloat16, group_dequant=fac)


@pytest.mark.parametrize("fa,fb", [(O.FMT_INT8, O.FMT_INT8), (O.FMT_E4M3, O.FMT_E4M3), (O.FMT_INT8, O.FMT_INT4)])
def test_gemm_reads_operands_from_views_of_wider_buffers(ops, fa, fb):
    """lda and ldb larger than K: both code matrices (and the second activation tensor) are column
    slices, at 16-byte offsets, of wider row-major buffers whose other columns hold other codes.
    Same result as from contiguous copies on the general kernel, the 8-wave tiles, K shares, parked /
    rescaled ranges and group factors."""
    one = torch.ones(1, device=DEV)
    g = torch.Generator().manual_seed(321)
    w4 = fb == O.FMT_INT4

    def run(M, N, K, ranges_of, odt, **kw):
        a, a2, b = _rand_codes((M, K), fa, 60), _rand_codes((M, K), fa, 61), _rand_codes((N, K), fb, 62)
        ad, a2d, bd = _to_dev_codes(a, fa), _to_dev_codes(a2, fa), _to_dev_codes(b, fb)   # bd: (N, K / 2) bytes when int4
        if bd.dim() == 1:
            bd = bd.view(N, -1)
        def widen(t, left, right, seed):
            wide = torch.from_numpy(np.random.default_rng(seed).integers(0, 120, size=(t.shape[0], left + t.shape[1] + right))
                                    .astype(np.uint8)).to(DEV).view(t.dtype)
            wide[:, left:left + t.shape[1]] = t
            return wide, wide[:, left:left + t.shape[1]]
        abuf, av = widen(ad, 32, 48, 1)
        a2buf, a2v = widen(a2d, 32, 48, 2)       # same stride as a: one lda serves both
        bbuf, bv = widen(bd, 16, 16, 3)
        sx = (torch.rand(M, generator=g) + 0.5).to(DEV)
        sw = (torch.rand(N, generator=g) + 0.5).to(DEV)
        rg = ranges_of(K, sx, sw)
        bias = None if odt == "acc" else torch.randn(N, generator=g).to(DEV)
        common = dict(m=M, n=N, a_fmt=fa, b_fmt=fb, out_dtype=odt, bias=bias, **kw)
        want = ops.gemm(ad, bd, rg, lda=K, ldb=bd.shape[1], a_neg=a2d, **common)
        got = ops.gemm(av, bv, rg, lda=abuf.stride(0), ldb=bbuf.stride(0), a_neg=a2v, **common)
        assert av.data_ptr() % 16 == 0 and bv.data_ptr() % 16 == 0
        assert torch.equal(got, want), (M, N, K, odt, kw)

    plain = lambda K, sx, sw: [ops.Range(0, K, sx, sw, 0, 1, 1)]
    dual = lambda K, sx, sw: [ops.Range(0, K // 2, sx, sw, 0, 1, 1), ops.Range(K // 2, K // 2, sx, one, 0, 1, 0),
                              ops.Range(K // 2, K // 2, sx, sw, 1, 1, 1)]
    ws = lambda: torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    run(70, 90, 320, plain, torch.bfloat16)
    run(70, 90, 320, plain, "acc")
    run(300, 700, 384, plain, torch.bfloat16, tile=11)
    run(300, 200, 1024, dual, torch.bfloat16)
    run(300, 200, 1024, dual, torch.bfloat16, workspace=ws())
    if not w4:
        run(400, 200, 256, plain, torch.bfloat16, tile=20)
        run(300, 700, 384, plain, torch.float32, tile=15)
        run(300, 200, 2048, plain, torch.bfloat16, tile=17, split_k=2, workspace=ws())
        run(300, 200, 2048, plain, torch.float16, tile=17, split_k=4, workspace=ws())
    if fa == O.FMT_INT8:
        fac = (torch.rand(1024 // 128, 200, generator=g) + 0.5).to(DEV)
        run(300, 200, 1024, lambda K, sx, sw: [ops.Range(0, K, sx, one, 0, 1, 0)], torch.bfloat16, group_dequant=fac, workspace=ws())


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("dt", ["bf16", "fp32"])
def test_quantize_reads_and_writes_views_of_wider_buffers(ops, fmt, dt):
    """ldx, ld_codes and ld_gate larger than cols: the input (a GEGLU projection's value half, the
    gate being the other half of the same buffer) and the codes (one K segment of a wider code
    matrix) are column slices.  Same codes and scales as from contiguous copies for static,
    dynamic and DualScale launches on each dynamic kernel, and nothing written outside the slice."""
    g = torch.Generator().manual_seed(55)
    for K in (256, 3072, 4800, 12288):      # flat / one wave per row and workgroup / one wave per row / one workgroup per row
        M = 9
        wide = (torch.randn(M, 2 * K + 32, generator=g) * 2).to(TDT[dt]).to(DEV)
        x, gate = wide[:, 16:16 + K], wide[:, 16 + K:16 + 2 * K]     # 32- or 64-byte offsets
        xc, gc = x.contiguous(), gate.contiguous()
        ccols = K // 2 if fmt == O.FMT_INT4 else K
        for kind in ("static", "dynamic", "dual", "gated"):
            poison = 0x55
            cbuf = torch.full((M, ccols + 48), poison, dtype=torch.uint8, device=DEV).view(ops.code_dtype(fmt))
            cview = cbuf[:, 16:16 + ccols]
            mk = lambda: torch.empty(M, device=DEV)
            if kind == "static":
                s = torch.full((1,), 11.0, device=DEV)
                want = ops.quantize(xc, fmt, s)
                got = ops.quantize(x, fmt, s, out=cview)
            else:
                kw = dict(row_stride=1, dynamic=True, dual=kind == "dual")
                if kind == "gated":
                    kw.update(pre_op="gelu_tanh")
                s1, n1, s2, n2 = mk(), (mk() if kind == "dual" else None), mk(), (mk() if kind == "dual" else None)
                want = ops.quantize(xc, fmt, s1, n1, gate=gc if kind == "gated" else None, **kw)
                got = ops.quantize(x, fmt, s2, n2, gate=gate if kind == "gated" else None, out=cview, **kw)
                assert torch.equal(s1, s2) and (n1 is None or torch.equal(n1, n2)), (K, kind)
            torch.cuda.synchronize()
            assert torch.equal(cview, want), (K, kind)
            raw = cbuf.view(torch.uint8)
            assert bool((raw[:, :16] == poison).all()) and bool((raw[:, 16 + ccols:] == poison).all()), (K, kind)


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_gemm_split_k_on_the_384x192_tile(ops, fmt):
    """Tile 20 by id with its K steps shared by 2, 3 and 5 workgroups (the second kernel sums the
    shares): one range in both formats, and in e4m3 three ranges rescaled in place, against the
    unsplit launch and the closed form; int8 with several ranges is refused there."""
    M, N, K0, K1 = 400, 210, 384, 640
    K = K0 + K1
    a, a2, b = _rand_codes((M, K), fmt, 71), _rand_codes((M, K), fmt, 72), _rand_codes((N, K), fmt, 73)
    ad, a2d, bd = (_to_dev_codes(t, fmt) for t in (a, a2, b))
    g = torch.Generator().manual_seed(74)
    sx, sx2 = torch.rand(M, generator=g) + 0.5, torch.rand(M, generator=g) + 0.5
    sw, bias = torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
    one = [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)]
    three = [ops.Range(0, K0, sx2.to(DEV), sw.to(DEV), 0, 1, 1), ops.Range(K0, K1, sx.to(DEV), sw.to(DEV), 0, 1, 1),
             ops.Range(K0, K1, sx2.to(DEV), sw.to(DEV), 1, 1, 1)]
    ws = torch.empty(ops.split_bytes(M, N, 8, park=True), dtype=torch.uint8, device=DEV)
    kw = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, lda=K, ldb=K, bias=bias.to(DEV), a_neg=a2d, tile=20, workspace=ws)
    av, a2v, bv = (O.code_values(t, fmt) for t in (a, a2, b))
    f64 = lambda t: t.numpy().astype(np.float64)
    want1 = av @ bv.T / (f64(sx)[:, None] * f64(sw)[None, :]) + f64(bias)
    want3 = (av[:, :K0] @ bv[:, :K0].T / (f64(sx2)[:, None] * f64(sw)[None, :]) + av[:, K0:] @ bv[:, K0:].T / (f64(sx)[:, None] * f64(sw)[None, :]) +
             a2v[:, K0:] @ bv[:, K0:].T / (f64(sx2)[:, None] * f64(sw)[None, :]) + f64(bias))
    tol = 5e-6 if fmt == O.FMT_INT8 else 1e-3
    for rg, want in ((one, want1), (three, want3)):
        if rg is three and fmt == O.FMT_INT8:
            with pytest.raises(RuntimeError):
                ops.gemm(ad, bd, rg, out_dtype=torch.float32, split_k=1, **kw)
            continue
        for sk in (1, 2, 3, 5):
            out = ops.gemm(ad, bd, rg, out_dtype=torch.float32, split_k=sk, **kw)
            assert np.abs(_np(out).astype(np.float64) - want).max() <= tol * np.abs(want).max(), (len(rg), sk)
            assert ops.gemm_plan(ops.gemm_desc(ad, bd, rg, out_dtype=torch.float32, split_k=sk, **kw), ws)["splits"] == sk


@pytest.mark.parametrize("fa,fb", [(O.FMT_INT8, O.FMT_INT8), (O.FMT_E4M3, O.FMT_E4M3), (O.FMT_INT8, O.FMT_INT4)])
def test_gemm_smallest_problems(ops, fa, fb):
    """One row, one column, the shortest contraction (16, or 32 with int4 weights), on the library's
    own choice and on the smallest general and 8-wave tiles: raw sums and the fused output."""
    kmin = 32 if fb == O.FMT_INT4 else 16
    g = torch.Generator().manual_seed(9)
    for M, N, K in ((1, 1, kmin), (1, 16, kmin), (17, 1, 2 * kmin), (1, 130, 128), (2, 3, 256)):
        a, b = _rand_codes((M, K), fa, 90), _rand_codes((N, K), fb, 91)
        ad, bd = _to_dev_codes(a, fa), _to_dev_codes(b, fb)
        ldb = K // 2 if fb == O.FMT_INT4 else K
        ref = O.gemm_acc(a, b, fa, fb).astype(np.float64)
        sx, sw, bias = torch.rand(M, generator=g) + 0.5, torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
        want = ref / (sx.numpy().astype(np.float64)[:, None] * sw.numpy().astype(np.float64)[None, :]) + bias.numpy()
        mag = np.abs(O.code_values(a, fa)) @ np.abs(O.code_values(b, fb)).T if fa == O.FMT_E4M3 else 0.0
        for tile in (0, 4, 14):
            if tile == 14 and K % 128:   # the 8-wave tiles take K in whole 128-byte steps
                continue
            kw = dict(m=M, n=N, a_fmt=fa, b_fmt=fb, lda=K, ldb=ldb, tile=tile)
            out = ops.gemm(ad, bd, [ops.Range(0, K, None, None)], out_dtype="acc", **kw)
            assert out.shape == (M, N)
            assert (np.abs(out.cpu().numpy().astype(np.float64) - ref) <= FP8_ACC_TOL * mag + 1e-30).all(), (M, N, K, tile)
            for odt, tol in ((torch.float32, 2e-6), (torch.bfloat16, 2.0 ** -8)):
                y = ops.gemm(ad, bd, [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)], out_dtype=odt, bias=bias.to(DEV), **kw)
                slack = FP8_ACC_TOL * mag / (sx.numpy()[:, None] * sw.numpy()[None, :]) if fa == O.FMT_E4M3 else 0.0
                assert (np.abs(_np(y).astype(np.float64) - want) <= tol * np.abs(want) + slack + 1e-30).all(), (M, N, K, tile, odt)


@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("op", [None, "gelu_tanh", "silu"])
@pytest.mark.parametrize("dual", [False, True])
@pytest.mark.parametrize("dt", ["bf16", "fp16"])
def test_gemm_epilogue_writes_the_next_linears_codes(ops, fmt, op, dual, dt):
    """segq_gemm with out_codes: the epilogue adds the bias, rounds to the layer dtype, applies the
    activation function, rounds again and encodes with a static scale (DualScale: two tensors)
    instead of writing floats.  (a) Bit for bit the codes of the two launches it replaces: the same
    GEMM writing the 16-bit tensor, then segq_quantize with pre_op on it.  (b) Against the oracle:
    activation + quantize_act(_dual) on the oracle's own output rounded to the dtype; the device's
    reciprocals (1 ulp in the de-quantisation) and exp2 move a value across a rounding boundary
    now and then, so codes may differ by one step on a small share of the elements, never by
    more.  Shapes: whole tiles of both tiles built with this epilogue (explicit ids and the
    library's choice), and ragged ones."""
    tdt = TDT[dt]
    cases = [(256, 384, 256, 0), (512, 512, 128, 11), (384, 1152, 256, 14), (130, 208, 384, 14), (77, 144, 128, 0)]
    for M, N, K, tile in cases:
        g = np.random.default_rng(1000 + M + N)
        if fmt == O.FMT_INT8:
            a = g.integers(-127, 128, size=(M, K)).astype(np.int8)
            b = g.integers(-127, 128, size=(N, K)).astype(np.int8)
        else:
            a = O.e4m3_encode(g.standard_normal((M, K)).astype(np.float32) * 40)
            b = O.e4m3_encode(g.standard_normal((N, K)).astype(np.float32) * 40)
        sx = (g.random(M).astype(np.float32) + 0.5) * (40.0 if fmt == O.FMT_INT8 else 20.0)
        sw = (g.random(N).astype(np.float32) + 0.5) * 30.0
        bias = g.standard_normal(N).astype(np.float32) * 0.5
        ad, bd = torch.from_numpy(a).to(DEV), torch.from_numpy(b).to(DEV)
        sxd, swd, biasd = (torch.from_numpy(t).to(DEV) for t in (sx, sw, bias))
        rg = [ops.Range(0, K, sxd, swd, 0, 1, 1)]
        kw = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=tdt, lda=K, ldb=K, bias=biasd)
        # the tensor the layer would have stored, from the same kernel (e4m3 sums depend, in their last
        # bits, on the order in which a kernel family feeds K to the matrix cores)
        y16 = ops.gemm(ad, bd, rg, tile=tile or 14, **kw)
        act = O.activation(_np(y16), op, dtype=dt) if op else _np(y16)
        lim = 127.0 if fmt == O.FMT_INT8 else 448.0
        if dual:
            pa, na = O.dual_amax(act)
            ps, ns = np.float32(lim / max(pa, 1e-6)), np.float32((128.0 if fmt == O.FMT_INT8 else 448.0) / max(na, 1e-6))
            sp, sn = torch.tensor([ps], device=DEV), torch.tensor([ns], device=DEV)
        else:
            ps = np.float32(lim / np.abs(act).max())
            sp, sn = torch.tensor([ps], device=DEV), None
        spec = dict(fmt=fmt, scale=sp, scale_neg=sn, pre_op=op)
        got = ops.gemm(ad, bd, rg, tile=tile, out_codes=spec, **kw)
        # (a) the two launches it replaces
        two = ops.quantize(y16, fmt, sp, sn, dual=dual, two_tensors=dual, pre_op=op)
        for gc, tc in zip(got if dual else (got,), two if dual else (two,)):
            assert gc.shape == (M, N) and torch.equal(gc, tc), (M, N, K, tile)
        # (b) the oracle: the stored tensor is the oracle's output to one rounding unit of the dtype (the
        # device multiplies by reciprocals where the oracle divides), and the codes are the oracle's
        # activation + quantize_act(_dual) of that stored tensor.  (Fed with its own output instead, the
        # oracle lands two e4m3 codes away now and then: one unit of bf16 at x = -5 moves gelu(x) by 10 %.)
        acc = O.gemm_acc(a, b, fmt, fmt)
        y = acc / (sx.astype(np.float64)[:, None] * sw.astype(np.float64)[None, :]) + bias[None, :]
        ulp = 2.0 ** -8 if dt == "bf16" else 2.0 ** -11
        assert (np.abs(_np(y16).astype(np.float64) - y) <= ulp * np.abs(y) + (2e-4 if fmt == O.FMT_E4M3 else 2e-6) * np.abs(y).max()).all()
        act_o = act
        if dual:
            wp, wn = O.quantize_act_dual(act_o[None], np.float32([ps]), np.float32([ns]), fmt)
            pairs = ((got[0], wp[0]), (got[1], wn[0]))
        else:
            pairs = ((got, O.quantize_act(act_o[None], np.float32([ps]), fmt)[0]),)
        for gc, want in pairs:
            gcn = gc.cpu().numpy()
            if fmt == O.FMT_INT8:
                d = np.abs(gcn.astype(np.int32) - want.astype(np.int32))
                assert d.max() <= 1 and (d != 0).mean() <= 4e-3, (M, N, d.max(), (d != 0).mean())
            else:
                # (e4m3 keeps three mantissa bits however small the value: the gelus' negative tail, which is
                # all the Xn tensor holds, lands on a neighbouring code far more often than integer codes do)
                assert (gcn == want).mean() >= 1 - (8e-2 if op else 0.0)
                vg, vw = O.e4m3_decode(gcn), O.e4m3_decode(want)
                assert (np.abs(vg - vw) <= 0.126 * np.abs(vw) + 2.0 ** -9).all()
    # what the epilogue does not serve is refused, not mis-computed
    with pytest.raises(RuntimeError, match="out_codes"):
        ops.gemm(ad, bd, [ops.Range(0, 64, sxd, swd, 0, 1, 1), ops.Range(64, 64, sxd, swd, 0, 1, 1)], out_codes=spec, **kw)
