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
    rows = sorted({0, 1, 15, 16, 127, 128, 191, 192, 255, 256, 287, 288, M // 2, M - 289, M - 193, M - 2, M - 1})
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


@pytest.mark.parametrize("M", [1024, 4608])
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3])
def test_full_size_config5_ranges_parked_or_split(ops, M, fmt):
    """Configuration 5 (K = 3072 | 12288, the second segment read from two code tensors) with the
    workspace the layer lends: int8 parks its finished ranges, 1024 tokens of e4m3 share the K
    steps of a tile between workgroups.  Same answer as the launch without a workspace (second
    accumulator set / in-place rescaling, one workgroup per tile), to fp32 summation order."""
    K0, K1, N = 3072, 12288, 3072
    K = K0 + K1
    a, a2, b = _codes((M, K), fmt, 130), _codes((M, K), fmt, 131), _codes((N, K), fmt, 132)
    ad, a2d, bd = _dev(a, fmt), _dev(a2, fmt), _dev(b, fmt)
    g = torch.Generator().manual_seed(133)
    s0 = (torch.rand(1, generator=g) + 0.5).to(DEV)
    sx, sx2 = (torch.rand(M, generator=g) + 0.5).to(DEV), (torch.rand(M, generator=g) + 0.5).to(DEV)
    sw, bias = (torch.rand(N, generator=g) + 0.5).to(DEV), torch.randn(N, generator=g).to(DEV)
    rg = [ops.Range(0, K0, s0, sw, 0, 0, 1), ops.Range(K0, K1, sx, sw, 0, 1, 1), ops.Range(K0, K1, sx2, sw, 1, 1, 1)]
    kw = dict(m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.float32, lda=K, ldb=K, bias=bias, a_neg=a2d)
    plain = ops.gemm(ad, bd, rg, split_k=1, **kw)
    nbytes = max(ops.park_bytes(M, N), ops.split_bytes(M, N, max(ops.auto_splits(M, N, (K0 + 2 * K1) // 128), 1)))
    lent = ops.gemm(ad, bd, rg, workspace=torch.empty(nbytes, dtype=torch.uint8, device=DEV), **kw)
    tol = 3e-6 if fmt == O.FMT_INT8 else 2e-4
    assert (lent - plain).abs().max().item() <= tol * plain.abs().max().item()
