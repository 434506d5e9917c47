"""GPU parity at the benchmark's full sizes, through checks whose cost does not grow
with the product M*N*K.

The oracle cannot multiply 4608 x 12288 x 3072 in seconds, so the full-size GEMMs are
verified with a randomised product check: for a random integer vector r,
C r == A (B^T r) must hold exactly in integer arithmetic (int8 and int4 weights), and
r^T C likewise from the other side.  A wrong tile, a dropped K step or a misplaced
row or column changes one of the two with probability 1 - 3^-k for k wrong entries.
e4m3 accumulators are compared the same way within the MFMA's summation tolerance.
The fused epilogue (scales, bias, one rounding to bf16) is checked on a band of rows
and columns against the oracle's closed form, and the activation quantiser on the
full tensors against the oracle's codes.
"""
import numpy as np
import pytest
import torch

from oracle import segq_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SHAPES = [  # (name, M, K, N): the three linears of benchmark configuration 3 and configuration 5 at M = 4608
    ("qkv", 4608, 3072, 9216),
    ("mlp_up", 4608, 3072, 12288),
    ("mlp_down", 4608, 12288, 3072),
    ("proj_out", 4608, 15360, 3072),
]


@pytest.fixture(scope="module")
def ops():
    from segquant_amd import ops as _ops
    _ops.L.lib()
    return _ops


def _codes(shape, fmt, seed):
    g = np.random.default_rng(seed)
    if fmt == O.FMT_INT8:
        return g.integers(-128, 128, size=shape).astype(np.int8)
    if fmt == O.FMT_INT4:
        return g.integers(-8, 8, size=shape).astype(np.int8)
    c = g.integers(0, 256, size=shape).astype(np.uint8)
    c[(c & 0x7F) == 0x7F] = 0x3A
    return c


def _dev(c, fmt):
    if fmt == O.FMT_INT4:
        lo = (c[:, 0::2].astype(np.uint8) & 0xF)
        hi = (c[:, 1::2].astype(np.uint8) & 0xF)
        return torch.from_numpy((lo | (hi << 4)).astype(np.uint8)).to(DEV)
    return torch.from_numpy(c).to(DEV)


@pytest.mark.parametrize("name,M,K,N", SHAPES)
@pytest.mark.parametrize("fb,lend", [(O.FMT_INT8, False), (O.FMT_INT4, False), (O.FMT_INT4, True)])
def test_full_size_integer_accumulators_product_check(ops, name, M, K, N, fb, lend):
    """lend: int4 weights expanded into a workspace the caller lends (the int8 kernels
    run); otherwise unpacked inside the GEMM."""
    a = _codes((M, K), O.FMT_INT8, 100)
    b = _codes((N, K), fb, 101)
    ldb = K // 2 if fb == O.FMT_INT4 else K
    ws = ops.int4_workspace(DEV, N * K) if lend else None
    out = ops.gemm(_dev(a, O.FMT_INT8), _dev(b, fb), [ops.Range(0, K, None, None)], m=M, n=N, a_fmt=O.FMT_INT8,
                   b_fmt=fb, out_dtype="acc", lda=K, ldb=ldb, workspace=ws)
    c = out.cpu().numpy().astype(np.int64)
    g = np.random.default_rng(102)
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    for _ in range(2):
        r = g.integers(-1, 2, size=N).astype(np.int64)
        assert np.array_equal(c @ r, a64 @ (b64.T @ r))
        l = g.integers(-1, 2, size=M).astype(np.int64)
        assert np.array_equal(l @ c, (l @ a64) @ b64.T)


@pytest.mark.parametrize("name,M,K,N", SHAPES[:3])
def test_full_size_e4m3_accumulators_product_check(ops, name, M, K, N):
    a = _codes((M, K), O.FMT_E4M3, 110)
    b = _codes((N, K), O.FMT_E4M3, 111)
    out = ops.gemm(_dev(a, O.FMT_E4M3), _dev(b, O.FMT_E4M3), [ops.Range(0, K, None, None)], m=M, n=N,
                   a_fmt=O.FMT_E4M3, b_fmt=O.FMT_E4M3, out_dtype="acc", lda=K, ldb=K)
    c = out.cpu().numpy().astype(np.float64)
    av, bv = O.code_values(a, O.FMT_E4M3), O.code_values(b, O.FMT_E4M3)
    g = np.random.default_rng(112)
    r = g.integers(-1, 2, size=N).astype(np.float64)
    want = av @ (bv.T @ r)
    # every entry of C is within 2e-4 of sum |a||b| of the exact sum; the check sums N of them with signs
    slack = 2e-4 * (np.abs(av) @ (np.abs(bv).T @ np.abs(r)))
    assert (np.abs(c @ r - want) <= slack + 1e-6).all()
    l = g.integers(-1, 2, size=M).astype(np.float64)
    want = (l @ av) @ bv.T
    slack = 2e-4 * ((np.abs(l) @ np.abs(av)) @ np.abs(bv).T)
    assert (np.abs(l @ c - want) <= slack + 1e-6).all()


@pytest.mark.parametrize("name,M,K,N", SHAPES[:3])
def test_full_size_fused_epilogue_on_bands(ops, name, M, K, N):
    """bf16 output with per-row and per-column scales and bias: rows and columns of a
    few bands (first, last, and tile borders of every tile size) against the closed form."""
    a = _codes((M, K), O.FMT_INT8, 120)
    b = _codes((N, K), O.FMT_INT8, 121)
    g = torch.Generator().manual_seed(122)
    sx = torch.rand(M, generator=g) + 0.5
    sw = torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g)
    y = ops.gemm(_dev(a, O.FMT_INT8), _dev(b, O.FMT_INT8), [ops.Range(0, K, sx.to(DEV), sw.to(DEV), 0, 1, 1)], m=M,
                 n=N, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT8, out_dtype=torch.bfloat16, lda=K, ldb=K, bias=bias.to(DEV))
    got = y.float().cpu().numpy().astype(np.float64)
    rows = sorted({0, 1, 15, 16, 95, 96, 127, 128, 191, 192, 255, 256, 287, 288, 383, 384, M // 2, M - 385, M - 289, M - 193, M - 2, M - 1})
    cols = sorted({0, 1, 3, 4, 127, 128, 191, 192, 255, 256, 287, 288, N // 2 + 5, N - 289, N - 193, N - 2, N - 1})
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    sxn, swn, bn = sx.numpy().astype(np.float64), sw.numpy().astype(np.float64), bias.numpy().astype(np.float64)
    want_rows = (a64[rows] @ b64.T) / (sxn[rows][:, None] * swn[None, :]) + bn[None, :]
    assert (np.abs(got[rows] - want_rows) <= np.abs(want_rows) * 2.0 ** -7 + 1e-30).all()
    want_cols = (a64 @ b64[cols].T) / (sxn[:, None] * swn[cols][None, :]) + bn[cols][None, :]
    assert (np.abs(got[:, cols] - want_cols) <= np.abs(want_cols) * 2.0 ** -7 + 1e-30).all()


@pytest.mark.parametrize("K", [3072, 12288])
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_full_size_dynamic_quantize_against_oracle(ops, K, fmt):
    """4608 tokens, bf16 in, per-token dynamic scales: scales and codes of the whole
    tensor against the oracle (elementwise work: the oracle does it in seconds)."""
    M = 4608
    g = torch.Generator().manual_seed(130 + K)
    x = (torch.randn(M, K, generator=g) * 2).to(torch.bfloat16)
    scale = torch.empty(M, device=DEV)
    codes = ops.quantize(x.to(DEV), fmt, scale, row_stride=1, dynamic=True)
    xn = x.float().numpy()
    amax = np.abs(xn).max(axis=1)
    want_s = O.row_scale_div(amax, 127.0 if fmt == O.FMT_INT8 else 448.0)
    assert np.array_equal(scale.cpu().numpy(), want_s)
    want = O.quantize_act(xn[None], want_s, fmt)[0]
    assert np.array_equal(codes.cpu().numpy().view(np.uint8), want.view(np.uint8))


@pytest.mark.parametrize("M,K,N", [(8192, 1280, 10240), (8192, 5120, 1280), (2048, 1280, 10240)])
def test_full_size_group_wise_scales_product_check(ops, M, K, N):
    """Configuration 4 at full size with one weight scale per 128 input channels, int4 weights
    expanded into the lent workspace: out r == sum_g A_g (W_g^T (r / sw_g)) / sx."""
    G = 128
    a, b = _codes((M, K), O.FMT_INT8, 120), _codes((N, K), O.FMT_INT4, 121)
    g = np.random.default_rng(122)
    sx = (g.random(M) + 0.5).astype(np.float32)
    swg = (g.random((K // G, N)) + 0.5).astype(np.float32)  # (groups, N)
    factors = torch.from_numpy((1.0 / swg.astype(np.float64)).astype(np.float32)).to(DEV)
    one = torch.ones(1, device=DEV)
    out = ops.gemm(_dev(a, O.FMT_INT8), _dev(b, O.FMT_INT4), [ops.Range(0, K, torch.from_numpy(sx).to(DEV), one, 0, 1, 0)],
                   m=M, n=N, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT4, out_dtype=torch.float32, lda=K, ldb=K // 2,
                   workspace=ops.int4_workspace(DEV, N * K), group_dequant=factors)
    f = factors.double().cpu().numpy()
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    r = g.integers(-1, 2, size=N).astype(np.float64)
    l = g.integers(-1, 2, size=M).astype(np.float64)
    right = np.zeros(M)
    left = np.zeros(N)
    la = l / sx.astype(np.float64)
    for j in range(K // G):
        sl = slice(j * G, (j + 1) * G)
        right += a64[:, sl] @ (b64[:, sl].T @ (r * f[j]))
        left += ((la @ a64[:, sl]) @ b64[:, sl].T) * f[j]
    right /= sx.astype(np.float64)
    # fp32 accumulation over K / 128 groups, then a sum of up to 10240 signed entries: an error of a
    # few 1e-7 per entry, measured against the entries' size
    c = out.double().cpu().numpy()
    assert np.abs(c @ r - right).max() <= 2e-6 * max(np.abs(right).max(), np.sqrt(N) * np.abs(c).max())
    assert np.abs(l @ c - left).max() <= 2e-6 * max(np.abs(left).max(), np.sqrt(M) * np.abs(c).max())


def _bands(M, N):
    """Rows and columns on the borders of every tile size the library picks (128, 192, 256, 288),
    the first and last ones, and a few in the middle."""
    rows = sorted({r for r in (0, 1, 15, 16, 127, 128, 191, 192, 255, 256, 287, 288, M // 2, M // 2 + 1, M - 289, M - 257,
                               M - 193, M - 129, M - 2, M - 1) if 0 <= r < M})
    cols = sorted({c for c in (0, 1, 3, 4, 127, 128, 191, 192, 255, 256, 287, 288, N // 2 + 5, N - 289, N - 257, N - 193,
                               N - 129, N - 2, N - 1) if 0 <= c < N})
    return rows, cols


@pytest.mark.parametrize("M", [1024, 4608, 9216])
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
@pytest.mark.parametrize("lend", [False, True])
def test_full_size_config5_three_ranges_against_closed_form(ops, M, fmt, lend):
    """Configuration 5 (K = 3072 | 12288, the second segment read from two code tensors, per-token
    scales on it) at every M of the sweep, the library choosing tile and split (tile = 0): with the
    workspace the layer lends (int8 parks its finished ranges, few tokens share the K steps of a
    tile between workgroups) and without (second accumulator set / fp32 sums rescaled in place).
    Row and column bands of the fp32 output against the fp64 closed form
    sum_r A_r B_r^T / (sx_r sw) + bias (segquant/src/real_quant/dequantizer.cuh:53-74 for the
    two halves of the DualScale segment, real_gemm.cu:752-894)."""
    K0, K1, N = 3072, 12288, 3072
    K = K0 + K1
    a, a2, b = _codes((M, K), fmt, 130), _codes((M, K), fmt, 131), _codes((N, K), fmt, 132)
    ad, a2d, bd = _dev(a, fmt), _dev(a2, fmt), _dev(b, fmt)
    g = torch.Generator().manual_seed(133)
    s0 = torch.rand(1, generator=g) + 0.5
    sx, sx2 = torch.rand(M, generator=g) + 0.5, torch.rand(M, generator=g) + 0.5
    sw, bias = torch.rand(N, generator=g) + 0.5, torch.randn(N, generator=g)
    s0d, sxd, sx2d, swd = (t.to(DEV) for t in (s0, sx, sx2, sw))
    rg = [ops.Range(0, K0, s0d, swd, 0, 0, 1), ops.Range(K0, K1, sxd, swd, 0, 1, 1), ops.Range(K0, K1, sx2d, swd, 1, 1, 1)]
    gd = ops.gemm_desc(ad, bd, rg, m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.float32, lda=K, ldb=K, bias=bias.to(DEV), a_neg=a2d)
    ws = None
    if lend:  # exactly what the library says it can use (parking room, K shares)
        ws = torch.empty(max(ops.gemm_workspace_bytes(gd), 16), dtype=torch.uint8, device=DEV)
    out = ops.gemm_launch(gd, ws)
    got = out.cpu().numpy().astype(np.float64)
    av, a2v, bv = O.code_values(a, fmt), O.code_values(a2, fmt), O.code_values(b, fmt)
    s0n, sxn, sx2n, swn, bn = (t.numpy().astype(np.float64) for t in (s0, sx, sx2, sw, bias))

    def check(ri, ci):
        A0, A1, A2 = av[ri][:, :K0], av[ri][:, K0:], a2v[ri][:, K0:]
        B0, B1 = bv[ci][:, :K0], bv[ci][:, K0:]
        d0 = s0n[0] * swn[ci][None, :]
        d1 = sxn[ri][:, None] * swn[ci][None, :]
        d2 = sx2n[ri][:, None] * swn[ci][None, :]
        t0, t1, t2 = (A0 @ B0.T) / d0, (A1 @ B1.T) / d1, (A2 @ B1.T) / d2
        want = t0 + t1 + t2 + bn[ci][None, :]
        terms = np.abs(t0) + np.abs(t1) + np.abs(t2) + np.abs(bn[ci])[None, :]
        err = np.abs(got[np.ix_(ri, ci)] - want)
        # element-wise.  Integer sums are exact, so what is left is fp32 rounding of each term (a
        # hardware reciprocal and two products) and of their sum: a few ulp of the terms' sizes.
        # e4m3: the MFMA adds each 128-long group with a limited-width adder, 2e-4 of sum |a||b|.
        bound = 2e-6 * terms
        if fmt == O.FMT_E4M3:
            bound = bound + 2e-4 * ((np.abs(A0) @ np.abs(B0).T) / d0 + (np.abs(A1) @ np.abs(B1).T) / d1 +
                                    (np.abs(A2) @ np.abs(B1).T) / d2)
        assert (err <= bound).all(), float((err / bound).max())

    rows, cols = _bands(M, N)
    check(np.asarray(rows), np.arange(N))
    check(np.arange(M), np.asarray(cols))


LAYER_CASES = [(1, None, torch.float32), (2, None, torch.bfloat16), (3, None, torch.bfloat16), (4, None, torch.bfloat16),
               (5, 9216, torch.bfloat16), (5, 1024, torch.bfloat16)]


@pytest.mark.parametrize("config,M,dtype", LAYER_CASES)
def test_full_size_layers_against_the_oracle(config, M, dtype):
    """SegmentLinear at the benchmark's own sizes with the library's own tile choice and the layer's
    own workspace lending: configuration 1 (256 tokens, whole output), configuration 2 (4096 tokens:
    fc1 on the two-workgroup 128 x 128 kernel, fc2 DualScale in two code tensors), configuration 3
    (4608 tokens, per-token dynamic scales, the three FLUX linears on their own tiles), configuration 4
    (8192 and 2048 tokens: the row quantiser at K = 1280 / 5120, int4 weights expanded into the lent
    workspace, one factor per group of 128 input channels) and configuration 5
    at 9216 and 1024 tokens (int8 parked, e4m3 rescaled in place, split K), on row and column bands
    against the closed form built by the oracle from the layer's codes and scales
    (element-wise: one rounding to the output dtype plus the accumulation's own error)."""
    from _layer_oracle import _np32, oracle_layer_output
    from segquant_amd import workloads as W
    for spec in W.config_linears(config, M=M):
        layer, x = W.build_layer(spec, device=DEV, real_quant=True)
        assert layer.optimizer.real_quant, spec.name
        xin = x.to(spec.x_dtype).to(DEV)
        out = layer(xin)
        assert out.shape == (spec.M, spec.N) and out.dtype == spec.x_dtype
        got = _np32(out).astype(np.float64)
        x_np = _np32(xin)
        del xin, out
        fp8 = spec.act == O.FMT_E4M3
        ulp = {torch.float32: 2.0 ** -22, torch.bfloat16: 2.0 ** -8}[spec.x_dtype]
        rows, cols = _bands(spec.M, spec.N)
        if spec.M * spec.N * spec.K <= 2 ** 33:
            bands = [(None, None)]
        else:
            bands = [(rows, None), (None, cols)]
        for ri, ci in bands:
            want = oracle_layer_output(layer, spec, x_np, rows=ri, cols=ci)
            sub = got if ri is None and ci is None else got[np.ix_(np.arange(spec.M) if ri is None else ri,
                                                                   np.arange(spec.N) if ci is None else ci)]
            scale = np.abs(want).max()
            # one rounding of the output, plus the accumulation error measured against the largest output
            # (sums of K-range terms that cancel): fp32 for integer codes, the MFMA's summation for e4m3
            bound = ulp * np.abs(want) + (1e-3 if fp8 else 2e-6) * scale
            err = np.abs(sub - want)
            assert (err <= bound).all(), (spec.name, float((err / bound).max()))
        del layer
        torch.cuda.empty_cache()


@pytest.mark.parametrize("rank", [32, 64])
def test_full_size_svd_layer_low_rank_in_the_epilogue(rank):
    """Configuration 3's mlp_up (4608 x 3072 -> 12288, int8, per-token dynamic activations,
    per-channel weights, bf16) as an svd layer: SmoothQuant division in the quantise kernel, the
    rank-r branch added by the GEMM's epilogue.  Row and column bands against the oracle's closed
    form built from the layer's own factors, codes and scales (optimizer.py:514-517, :724-731)."""
    from _layer_oracle import _np32, oracle_smooth_layer_output
    from test_gpu_layers import _smooth_layer
    M, K, N = 4608, 3072, 12288
    layer, xd, _ = _smooth_layer("svd", "int8", "weight", 1, M, K, N, torch.bfloat16, True, axis=True, rank=rank, seed=9)
    assert layer.optimizer.fused_available()
    out = layer(xd)
    plan = layer.optimizer._plan
    assert plan["lr_ok"][(M, torch.bfloat16)] is True  # the epilogue branch ran, not the materialised addend
    got = _np32(out).astype(np.float64)
    x_np = _np32(xd)
    rows, cols = _bands(M, N)
    for ri, ci in ((rows, None), (None, cols)):
        want = oracle_smooth_layer_output(layer, "int8", "int8", x_np, rows=ri, cols=ci)
        sub = got[np.ix_(np.arange(M) if ri is None else ri, np.arange(N) if ci is None else ci)]
        # T = x (L1 / s), L1 / s and L2 are rounded to bf16 for the matrix cores: 2^-9 each, against the
        # size of the low-rank term (here of the order of the output itself)
        assert np.abs(sub - want).max() <= 1.2e-2 * np.abs(want).max()
        assert np.sqrt(((sub - want) ** 2).mean()) <= 2.5e-3 * np.abs(want).max()
