"""The allocation-free GEMM entry point (segq_gemm_noalloc), through the C ABI.

It must give what segq_gemm gives when the caller lends a workspace of
segq_gemm_workspace_bytes(d) bytes: bit for bit, since the same kernels make the same
decisions.  Every case is called twice in a row, the second time on a smaller problem,
so that what the first call left in the library's scratch array is there when the second
one runs.  Collected last (file name), so a failure here hides no other test.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import segq_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from segquant_amd import ops as _ops
    _ops.L.lib()
    return _ops


def _codes(shape, fmt, seed):
    g = np.random.default_rng(seed)
    if fmt == O.FMT_INT8:
        return torch.from_numpy(g.integers(-128, 128, size=shape).astype(np.int8)).to(DEV)
    if fmt == O.FMT_INT4:
        return torch.from_numpy(g.integers(0, 256, size=(shape[0], shape[1] // 2)).astype(np.uint8)).to(DEV)
    c = g.integers(0, 256, size=shape).astype(np.uint8)
    c[(c & 0x7F) == 0x7F] = 0x3A
    return torch.from_numpy(c).to(DEV)


_LAST_A = [None]   # the activation codes of the case built last (tests that rewrite the input in place)
_TENSORS = []      # every tensor of the parking case built last


def _both(ops, make_desc):
    """(result of segq_gemm with a lent workspace, result of segq_gemm_noalloc, workspace bytes)"""
    L = ops.L
    g = make_desc()
    need = ops.gemm_workspace_bytes(g)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
    want = ops.gemm_launch(g, ws if need else None).clone()
    g2 = make_desc()
    g2[1].fill_(float("nan") if g2[1].dtype.is_floating_point else 0)
    before = torch.cuda.memory_allocated()
    rc = L.lib().segq_gemm_noalloc(C.byref(g2[0]), torch.cuda.current_stream().cuda_stream)
    L.check(rc)
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    return want, g2[1], need


def _split_case(ops, M, N, K, fmt, seed, split_k=0):
    a, b = _codes((M, K), fmt, seed), _codes((N, K), fmt, seed + 1)
    _LAST_A[0] = a
    g = torch.Generator().manual_seed(seed)
    sx = (torch.rand(M, generator=g) + 0.5).to(DEV)
    sw = (torch.rand(N, generator=g) + 0.5).to(DEV)
    bias = torch.randn(N, generator=g).to(DEV)
    return lambda: ops.gemm_desc(a, b, [ops.Range(0, K, sx, sw, 0, 1, 1)], m=M, n=N, a_fmt=fmt, b_fmt=fmt,
                                 out_dtype=torch.bfloat16, lda=K, ldb=K, bias=bias, split_k=split_k)


def _park_case(ops, M, N, K0, K1, seed):
    K = K0 + K1
    fmt = O.FMT_INT8
    a, a2, b = _codes((M, K), fmt, seed), _codes((M, K), fmt, seed + 1), _codes((N, K), fmt, seed + 2)
    g = torch.Generator().manual_seed(seed)
    s0 = (torch.rand(1, generator=g) + 0.5).to(DEV)
    sx, sx2 = (torch.rand(M, generator=g) + 0.5).to(DEV), (torch.rand(M, generator=g) + 0.5).to(DEV)
    sw, bias = (torch.rand(N, generator=g) + 0.5).to(DEV), torch.randn(N, generator=g).to(DEV)
    _LAST_A[0] = a
    _TENSORS[:] = [a, a2, b, s0, sx, sx2, sw, bias]
    rg = [ops.Range(0, K0, s0, sw, 0, 0, 1), ops.Range(K0, K1, sx, sw, 0, 1, 1), ops.Range(K0, K1, sx2, sw, 1, 1, 1)]
    return lambda: ops.gemm_desc(a, b, rg, m=M, n=N, a_fmt=fmt, b_fmt=fmt, out_dtype=torch.float32, lda=K, ldb=K,
                                 bias=bias, a_neg=a2)


def _int4_case(ops, M, N, K, seed):
    a, b = _codes((M, K), O.FMT_INT8, seed), _codes((N, K), O.FMT_INT4, seed + 1)
    _LAST_A[0] = a
    return lambda: ops.gemm_desc(a, b, [ops.Range(0, K, None, None)], m=M, n=N, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT4,
                                 out_dtype="acc", lda=K, ldb=K // 2)


def test_noalloc_matches_the_lent_workspace_twice_in_a_row(ops):
    L = ops.L
    assert L.lib().segq_init() == 0
    assert L.lib().segq_noalloc_scratch_bytes() == 64 << 20
    cases = [
        # few tiles, long K: the K steps of a tile are shared by several workgroups (fp32 partial results)
        # (the library's own choice of shares, then shares asked for: four, and two, which meet inside the launch)
        ("split e4m3", _split_case(ops, 512, 1024, 8192, O.FMT_E4M3, 1), _split_case(ops, 384, 512, 4096, O.FMT_E4M3, 5, 4)),
        ("split int8", _split_case(ops, 512, 768, 8192, O.FMT_INT8, 11), _split_case(ops, 200, 256, 4096, O.FMT_INT8, 15, 2)),
        # int8 with three ranges: finished ranges parked as fp32
        ("park", _park_case(ops, 1536, 1408, 256, 512, 21), _park_case(ops, 1300, 1200, 128, 256, 25)),
        # int4 weights expanded to int8
        ("int4", _int4_case(ops, 700, 1536, 1024, 31), _int4_case(ops, 130, 200, 256, 35)),
    ]
    for name, first, second in cases:
        for which, case in (("first", first), ("second, smaller", second)):
            want, got, need = _both(ops, case)
            assert need > 0, (name, which, "this case was meant to use a workspace")
            assert torch.equal(want, got), (name, which)


def test_noalloc_refuses_what_does_not_fit_and_runs_what_needs_nothing(ops):
    L = ops.L
    # 16 shares of 2048 x 3072 fp32 partial results are 403 MB: more than the array holds.  The launch
    # runs with the shares that fit, as segq_gemm does when it is lent a workspace of the array's size
    a, b = _codes((2048, 16384), O.FMT_E4M3, 41), _codes((3072, 16384), O.FMT_E4M3, 42)
    one = torch.ones(1, device=DEV)
    mk16 = lambda: ops.gemm_desc(a, b, [ops.Range(0, 16384, one, one, 0, 0, 0)], m=2048, n=3072, a_fmt=O.FMT_E4M3, b_fmt=O.FMT_E4M3,
                                 out_dtype=torch.bfloat16, lda=16384, ldb=16384, split_k=16)
    g = mk16()
    assert ops.gemm_workspace_bytes(g) > L.lib().segq_noalloc_scratch_bytes()
    want = ops.gemm_launch(g, torch.empty(64 << 20, dtype=torch.uint8, device=DEV)).clone()
    g2 = mk16()
    L.check(L.lib().segq_gemm_noalloc(C.byref(g2[0]), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert torch.equal(want, g2[1])
    # group factors with int4 weights cannot run without room for the expanded weights: 8448 x 8192 bytes
    # are more than the array holds, and the call is refused with the launch's own status and a message
    n, k = 8448, 8192
    a4, b4 = _codes((128, k), O.FMT_INT8, 45), _codes((n, k), O.FMT_INT4, 46)
    fac = torch.ones((k // 128, n), device=DEV)
    sx = torch.ones(128, device=DEV)
    g = ops.gemm_desc(a4, b4, [ops.Range(0, k, sx, one, 0, 1, 0)], m=128, n=n, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT4,
                      out_dtype=torch.bfloat16, lda=k, ldb=k // 2, group_dequant=fac)
    rc = L.lib().segq_gemm_noalloc(C.byref(g[0]), torch.cuda.current_stream().cuda_stream)
    assert rc == 2 and b"scratch" in L.lib().segq_last_error()
    # a plain single-range launch has no use for a workspace and is the same launch as segq_gemm
    a, b = _codes((300, 512), O.FMT_INT8, 43), _codes((260, 512), O.FMT_INT8, 44)
    mk = lambda: ops.gemm_desc(a, b, [ops.Range(0, 512, None, None)], m=300, n=260, a_fmt=O.FMT_INT8, b_fmt=O.FMT_INT8,
                               out_dtype="acc", lda=512, ldb=512)
    want, got, need = _both(ops, mk)
    assert need == 0 and torch.equal(want, got)


def test_noalloc_runs_with_what_fits_when_the_launch_could_use_more(ops):
    """int8 with three ranges on 4608 x 4096 outputs would park 75 MB of fp32 sums: more than the
    scratch array.  The entry point then launches what segq_gemm launches when it is lent a workspace
    of the array's size (a second register set on smaller tiles), bit for bit."""
    L = ops.L
    mk = _park_case(ops, 4608, 4096, 128, 256, 51)
    g = mk()
    assert ops.gemm_workspace_bytes(g) > L.lib().segq_noalloc_scratch_bytes()
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    want = ops.gemm_launch(g, ws).clone()
    g2 = mk()
    g2[1].fill_(float("nan"))
    before = torch.cuda.memory_allocated()
    L.check(L.lib().segq_gemm_noalloc(C.byref(g2[0]), torch.cuda.current_stream().cuda_stream))
    assert torch.cuda.memory_allocated() == before
    torch.cuda.synchronize()
    assert torch.equal(want, g2[1])
    # and against the closed form on a band of rows (the smaller tiles sum the ranges in registers)
    rows = [0, 255, 256, 4607]
    a, a2, b = (t.cpu().numpy().astype(np.float64) for t in (_TENSORS[0], _TENSORS[1], _TENSORS[2]))
    s0, sx, sx2, sw, bias = (t.cpu().numpy().astype(np.float64) for t in _TENSORS[3:])
    ref = (a[rows, :128] @ b[:, :128].T) / (s0 * sw[None, :]) + (a[rows, 128:] @ b[:, 128:].T) / (sx[rows, None] * sw[None, :]) \
        + (a2[rows, 128:] @ b[:, 128:].T) / (sx2[rows, None] * sw[None, :]) + bias[None, :]
    got = g2[1][rows].double().cpu().numpy()
    assert np.abs(got - ref).max() <= 2e-6 * np.abs(ref).max()


def test_noalloc_under_stream_capture_replays(ops):
    """segq_gemm_noalloc recorded into a HIP graph after segq_init() (the callers it exists for) and
    replayed three times with the input rewritten and the program's own eager launches and
    synchronisations between the replays: two K shares meeting inside the launch (its stamp word is
    cleared by the second arrival, so a replay finds it clean), parked int8 ranges, expanded int4
    weights.  Every replay equals the eager segq_gemm on the codes then in the buffer, bit for bit."""
    L = ops.L
    assert L.lib().segq_init() == 0
    cases = [("two shares", _split_case(ops, 512, 768, 4096, O.FMT_INT8, 61, 2)),
             ("park", _park_case(ops, 1536, 1408, 256, 512, 65)),
             ("int4", _int4_case(ops, 300, 512, 512, 71))]
    for name, mk in cases:
        g = mk()
        need = ops.gemm_workspace_bytes(g)
        assert need > 0, name
        ws = torch.empty(need, dtype=torch.uint8, device=DEV)
        a_buf = _LAST_A[0]
        variants = [a_buf.clone(), torch.roll(a_buf, 1, 0).contiguous(), torch.flip(a_buf, [0]).contiguous()]
        eager = []
        for v in variants:
            a_buf.copy_(v)
            eager.append(ops.gemm_launch(mk(), ws).clone())
        gd = mk()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # kernel attributes are set outside the capture
            L.check(L.lib().segq_gemm_noalloc(C.byref(gd[0]), side.cuda_stream))
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            L.check(L.lib().segq_gemm_noalloc(C.byref(gd[0]), torch.cuda.current_stream().cuda_stream))
        for i in (1, 2, 0, 2):
            a_buf.copy_(variants[i])
            gd[1].fill_(0)
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(gd[1], eager[i]), (name, i)
            a_buf.copy_(variants[(i + 1) % 3])   # eager work of the program's own between replays
            again = ops.gemm_launch(mk(), ws)
            torch.cuda.synchronize()
            assert torch.equal(again, eager[(i + 1) % 3]), (name, i)
        del graph
