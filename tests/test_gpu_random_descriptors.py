"""Randomly drawn segq_gemm descriptors against the oracle's closed form.

Every seed draws code formats, a shape (ragged and whole-tile ones), a tile id (or the library's
choice), one to three ranges (consecutive K runs, DualScale pairs over one run through the sign
selections, runs read from the second code tensor), per-row / per-tensor and per-column /
per-tensor scales, the output type, a K split and whether a workspace is lent.  A draw the library
refuses (an explicit tile that is not built for the combination, a split that needs a workspace) is
skipped; a draw it accepts must match

    sum over ranges ( A_r[:, k0:k1] . B[:, k0:k1]^T ) / (sx_r sw_r) + bias

with the products summed exactly in fp64: int8 / int4 within 4e-6 of sum |term| (the fp32
arithmetic of the epilogue), e4m3 additionally within FP8_ACC_TOL of sum |a||b| (the matrix cores'
limited-width adder), 16-bit outputs one rounding further.
"""
import numpy as np
import pytest
import torch

from oracle import segq_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FP8_ACC_TOL = 3e-4
SEEDS_PER_TEST = 100


def _rand_codes(shape, fmt, g):
    if fmt == O.FMT_INT8:
        return g.integers(-128, 128, size=shape).astype(np.int8)
    if fmt == O.FMT_INT4:
        return g.integers(-8, 8, size=shape).astype(np.int8)
    c = g.integers(0, 256, size=shape).astype(np.uint8)
    c[(c & 0x7F) == 0x7F] = 0x3A  # no NaN codes
    return c


def _to_dev(c, fmt):
    if fmt == O.FMT_INT4:
        return torch.from_numpy(np.stack([O.pack_int4(r) for r in c])).to(DEV)
    return torch.from_numpy(c).to(DEV)


def _draw(case):
    g = np.random.default_rng(1000 + case)
    fa, fb = [(O.FMT_INT8, O.FMT_INT8), (O.FMT_E4M3, O.FMT_E4M3), (O.FMT_INT8, O.FMT_INT4)][g.integers(0, 3) if g.random() < 0.6 else 0]
    gran = 128 if g.random() < 0.6 else (32 if fb == O.FMT_INT4 else 16)
    nr = int(g.integers(1, 4))
    lens = [gran * int(g.integers(1, 1 + (1024 // gran) // nr + 1)) for _ in range(nr)]
    use_neg = nr > 1 and g.random() < 0.3
    M = int(g.choice([1, 3, 17, 64, 77, 128, 130, 200, 256, 300, 384, 500, 576, 777, 1024, 1152, 1400]))
    N = int(g.choice([16, 18, 96, 128, 130, 192, 200, 256, 288, 330, 384, 515, 576, 768, 1000, 1152, 1536]))
    tile = int(g.choice([0, 0, 0, 1, 2, 3, 4, 5, 11, 12, 13, 14, 15, 16, 17, 18, 19, 20, 21]))
    odt = [torch.float32, torch.bfloat16, torch.float16][g.integers(0, 3)]
    split = int(g.choice([0, 0, 0, 0, 0, 1, 2, 3]))
    lend = g.random() < 0.6
    has_bias = g.random() < 0.7
    specs, k = [], 0   # (k_begin, k_len, a_sel, per-row sx, per-column sw)
    for r in range(nr):
        a_sel = 0
        if r > 0 and specs[-1][2] == 0 and g.random() < 0.35:
            k0, ln = specs[-1][0], specs[-1][1]   # a DualScale pair over the previous run
            specs[-1] = (k0, ln, 2, specs[-1][3], specs[-1][4])
            a_sel = 3
        else:
            k0, ln = k, lens[r]
            k += ln
            if use_neg and g.random() < 0.5:
                a_sel = 1
        specs.append((k0, ln, a_sel, g.random() < 0.5, g.random() < 0.5))
    return g, fa, fb, M, N, k, tile, odt, split, lend, has_bias, specs


def _run(ops, case):
    g, fa, fb, M, N, K, tile, odt, split, lend, has_bias, specs = _draw(case)
    a, b = _rand_codes((M, K), fa, g), _rand_codes((N, K), fb, g)
    a2 = _rand_codes((M, K), fa, g) if any(s[2] == 1 for s in specs) else None
    av, bv = O.code_values(a, fa), O.code_values(b, fb)
    a2v = O.code_values(a2, fa) if a2 is not None else None
    want, mag, ranges, keep = np.zeros((M, N)), np.zeros((M, N)), [], []
    for k0, ln, a_sel, row_sx, col_sw in specs:
        sx = (g.random(M if row_sx else 1) * 30 + 10).astype(np.float32)
        sw = (g.random(N if col_sw else 1) * 30 + 10).astype(np.float32)
        blk = (a2v if a_sel == 1 else av)[:, k0:k0 + ln]
        if a_sel in (2, 3):   # the codes whose sign bit is clear / set, the rest read as zero
            neg = (a[:, k0:k0 + ln].view(np.uint8) & 0x80) != 0
            blk = np.where(neg, 0.0, blk) if a_sel == 2 else np.where(neg, blk, 0.0)
        den = sx.astype(np.float64)[:, None] * sw.astype(np.float64)[None, :]
        want += (blk @ bv[:, k0:k0 + ln].T) / den
        mag += (np.abs(blk) @ np.abs(bv[:, k0:k0 + ln]).T) / den
        sxd, swd = torch.from_numpy(sx).to(DEV), torch.from_numpy(sw).to(DEV)
        keep += [sxd, swd]
        ranges.append(ops.Range(k0, ln, sxd, swd, a_sel, 1 if row_sx else 0, 1 if col_sw else 0))
    bias = g.standard_normal(N).astype(np.float32) if has_bias else None
    if bias is not None:
        want += bias[None, :]
    what = (f"seed {case}: {fa}/{fb} M={M} N={N} K={K} tile={tile} ranges={[s[:3] for s in specs]} "
            f"out={odt} split={split} lend={lend} bias={has_bias}")
    try:
        gd = ops.gemm_desc(_to_dev(a, fa), _to_dev(b, fb), ranges, m=M, n=N, a_fmt=fa, b_fmt=fb, out_dtype=odt, lda=K,
                           ldb=K // 2 if fb == O.FMT_INT4 else K, a_neg=_to_dev(a2, fa) if a2 is not None else None,
                           bias=torch.from_numpy(bias).to(DEV) if bias is not None else None, tile=tile, split_k=split)
        ws = None
        if lend:
            nb = ops.gemm_workspace_bytes(gd)
            if nb:
                ws = torch.empty(nb, dtype=torch.uint8, device=DEV)
        out = ops.gemm_launch(gd, ws)
        torch.cuda.synchronize()
    except RuntimeError:
        return False   # refused before anything was launched
    got = out.float().cpu().numpy().astype(np.float64)
    tol = 4e-6 * (mag + (np.abs(bias)[None, :] if bias is not None else 0.0)) + 1e-30
    if fa == O.FMT_E4M3:
        tol = tol + FP8_ACC_TOL * mag
    if odt == torch.bfloat16:
        tol = tol + np.abs(want) * 2.0 ** -7
    if odt == torch.float16:
        tol = tol + np.abs(want) * 2.0 ** -10 + 2.0 ** -24
    assert np.isfinite(got).all(), what
    err = np.abs(got - want)
    assert (err <= tol).all(), f"{what}: {int((err > tol).sum())} elements off, worst {float((err - tol).max())}"
    return True


@pytest.fixture(scope="module")
def ops():
    from segquant_amd import ops as _ops
    _ops.L.lib()  # fail loudly if the library is not built
    return _ops


@pytest.mark.parametrize("first", [0, 100, 200, 300])
def test_randomly_drawn_descriptors_match_the_closed_form(ops, first):
    ran = sum(_run(ops, case) for case in range(first, first + SEEDS_PER_TEST))
    assert ran >= SEEDS_PER_TEST // 3   # most draws must be launches, not refusals
