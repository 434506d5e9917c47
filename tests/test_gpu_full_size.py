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
