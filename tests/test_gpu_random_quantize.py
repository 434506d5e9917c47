"""Randomly drawn segq_quantize descriptors against the oracle, bit for bit.

Every seed draws the input type, the code format, a shape (rows of one to three column segments,
short enough for the wave-per-row kernels or long enough for the workgroup-per-row one), static
scales (per segment or per token) or dynamic per-token ones, DualScale on a subset of the column
segments into one merged or two code tensors, SmoothQuant's column divisors, and whether the input
is a column slice of a wider buffer.  No activation function (its bound is statistical and has a
test of its own): everything here is IEEE arithmetic and must match exactly, scales included.
"""
import numpy as np
import pytest
import torch

from oracle import segq_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TDT = {"fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
LIM_P = {O.FMT_INT8: 127.0, O.FMT_INT4: 7.0, O.FMT_E4M3: 448.0}
LIM_N = {O.FMT_INT8: 128.0, O.FMT_INT4: 8.0, O.FMT_E4M3: 448.0}
SEEDS_PER_TEST = 60


def _unpacked(t, fmt):
    a = t.cpu().numpy()
    if fmt == O.FMT_INT4:
        return np.stack([O.unpack_int4(r) for r in a.reshape(a.shape[0], -1)])
    return a


def _run(ops, case):
    g = np.random.default_rng(5000 + case)
    dt = ["fp32", "bf16", "fp16"][g.integers(0, 3)]
    fmt = [O.FMT_INT8, O.FMT_E4M3, O.FMT_INT4][g.integers(0, 3)]
    rows = int(g.choice([1, 5, 33, 130, 257]))
    nk = int(g.integers(1, 4))
    total = int(g.choice([64, 1040, 3072, 4096, 4800, 8192, 12288]))
    cuts = sorted(set(int(c) * 32 for c in g.integers(1, total // 32, size=nk - 1))) if nk > 1 and total >= 64 else []
    bounds = [0] + cuts + [total]
    nk = len(bounds) - 1
    dynamic = g.random() < 0.5
    per_tok = dynamic or g.random() < 0.5
    dual = g.random() < 0.5
    mask = int(g.integers(1, 1 << nk)) if dual else 0
    two = dual and g.random() < 0.5
    use_div = g.random() < 0.3
    sliced = g.random() < 0.3
    what = f"seed {case}: {dt} -> {fmt}, {rows} x {bounds}, dynamic={dynamic} per_tok={per_tok} dual mask={mask:b} two={two} div={use_div} sliced={sliced}"

    tg = torch.Generator().manual_seed(5000 + case)
    pad = 24 if sliced else 0
    full = (torch.randn(rows, total + pad, generator=tg) * 3).to(TDT[dt])
    full[0, :6] = torch.tensor([0.0, -0.0, 0.5, -0.5, 1.5, -2.5]).to(TDT[dt])
    if rows > 2:
        full[2] = full[2].abs()   # a row with nothing negative
    xd = full.to(DEV)[:, :total]
    v = full[:, :total].float().numpy()
    sdiv = None
    if use_div:
        sdiv = (torch.rand(total, generator=tg) * 4 + 0.05).to(TDT[dt]).float()
        v = O.smooth_divide(v, sdiv.numpy(), dt)

    shape = (nk, rows) if per_tok else (nk, 1)
    if dynamic:
        pos = torch.empty(shape, dtype=torch.float32, device=DEV)
        neg = torch.empty(shape, dtype=torch.float32, device=DEV) if dual else None
    else:
        pos = (torch.rand(shape, generator=tg) * 20 + 0.5).to(DEV)
        neg = (torch.rand(shape, generator=tg) * 20 + 0.5).to(DEV) if dual else None
    res = ops.quantize(xd, fmt, pos, neg, row_stride=1 if per_tok else 0, kseg_bounds=bounds if nk > 1 else None,
                       kseg_stride=rows if per_tok else 1, dual=dual, dual_kseg_mask=mask if dual else 0xFFFFFFFF,
                       dynamic=dynamic, two_tensors=two, col_div=sdiv.to(DEV) if use_div else None)
    torch.cuda.synchronize()
    got_p, got_n = (res if two else (res, None))
    got_p = _unpacked(got_p, fmt)
    got_n = _unpacked(got_n, fmt) if two else None
    sp, sn = pos.cpu().numpy(), (neg.cpu().numpy() if dual else None)
    for j in range(nk):
        seg = v[:, bounds[j]:bounds[j + 1]]
        cols = slice(bounds[j], bounds[j + 1])
        seg_dual = dual and (mask >> j) & 1
        if dynamic:
            if seg_dual:
                pa, na = O.dual_amax(seg, axis=-1)
                assert np.array_equal(sp[j], O.row_scale_div(pa, LIM_P[fmt])), what
                assert np.array_equal(sn[j], O.row_scale_div(na, LIM_N[fmt])), what
            else:
                assert np.array_equal(sp[j], O.row_scale_div(np.abs(seg).max(axis=-1), LIM_P[fmt])), what
        if seg_dual:
            wp, wn = O.quantize_act_dual(seg[None], sp[j], sn[j], fmt)
            if two:
                assert np.array_equal(got_p[:, cols], wp[0]), what
                assert np.array_equal(got_n[:, cols], wn[0]), what
            else:
                assert np.array_equal(got_p[:, cols], O.merge_dual_codes(wp, wn, seg[None])[0]), what
        else:
            assert np.array_equal(got_p[:, cols], O.quantize_act(seg[None], sp[j], fmt)[0]), what


@pytest.fixture(scope="module")
def ops():
    from segquant_amd import ops as _ops
    _ops.L.lib()  # fail loudly if the library is not built
    return _ops


@pytest.mark.parametrize("first", [0, 60, 120, 180])
def test_randomly_drawn_quantise_descriptors_are_bit_exact(ops, first):
    for case in range(first, first + SEEDS_PER_TEST):
        _run(ops, case)
