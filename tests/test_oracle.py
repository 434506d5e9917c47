"""Pins for the CPU oracle: closed forms, library routines, brute force.

None of these tests retypes the oracle's own formula; each compares it with an
independent source (torch's float8 cast, python integer arithmetic, an
exhaustive table, an algebraic invariant).
"""
import math

import numpy as np
import pytest
import torch

from oracle import segq_oracle as O


# ------------------------------------------------------------------ e4m3
def test_e4m3_table_matches_torch_decode():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float().numpy()
    tab = O.e4m3_decode_table()
    assert np.array_equal(np.isnan(ref), np.isnan(tab))
    ok = ~np.isnan(ref)
    assert np.array_equal(ref[ok], tab[ok])
    assert tab[0x7E] == 448.0 and tab[0x08] == 2.0 ** -6 and tab[0x01] == 2.0 ** -9


def test_e4m3_encode_is_identity_on_representable_values():
    tab = O.e4m3_decode_table()
    codes = np.arange(256, dtype=np.uint8)
    ok = ~np.isnan(tab)
    enc = O.e4m3_encode(tab[ok])
    # -0.0 keeps its sign bit (0x80)
    assert np.array_equal(enc, codes[ok])


def test_e4m3_midpoints_round_to_even_mantissa():
    tab = O.e4m3_decode_table()
    pos = np.sort(tab[:0x7F])  # 0 .. 448, ascending, codes 0..0x7E
    for c in range(0x7E):
        lo, hi = float(pos[c]), float(pos[c + 1])
        mid = np.float32((lo + hi) / 2)  # exact in fp32
        want = c if c % 2 == 0 else c + 1
        assert O.e4m3_encode(mid) == want, (c, mid)
        assert O.e4m3_encode(-mid) == (want | 0x80)
        below = np.nextafter(mid, np.float32(0))
        above = np.nextafter(mid, np.float32(1e9))
        assert O.e4m3_encode(below) == c
        assert O.e4m3_encode(above) == c + 1


def test_e4m3_encode_matches_torch_cast_on_clamped_input():
    g = torch.Generator().manual_seed(7)
    x = torch.randn(200000, generator=g) * torch.exp(torch.randn(200000, generator=g) * 4)
    x = torch.cat([x, torch.tensor([0.0, -0.0, 448.0, 449.0, 464.0, 465.0, 1e9, -1e9,
                                    2.0 ** -10, 2.0 ** -9, 3 * 2.0 ** -10, 2.0 ** -6, 17., 19., 21., 23.])])
    ref = torch.clamp(x, -448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = O.e4m3_encode(x.numpy())
    assert np.array_equal(ref, got)


def test_e4m3_special_values():
    assert O.e4m3_encode(np.float32("nan")) == 0x7F
    assert O.e4m3_encode(np.float32("inf")) == 0x7E
    assert O.e4m3_encode(np.float32("-inf")) == 0xFE
    assert O.e4m3_encode(np.float32(1e30)) == 0x7E
    assert O.e4m3_encode(np.float32(2.0 ** -10)) == 0  # tie to even (0)
    assert O.e4m3_encode(np.float32(3 * 2.0 ** -10)) == 2  # tie between 1 and 2 -> 2


def test_simulate_fp_agrees_with_e4m3_for_normals_only():
    g = np.random.default_rng(3)
    x = (g.standard_normal(50000) * 50).astype(np.float32)
    x = x[np.abs(x) >= 2.0 ** -6]
    a = O.simulate_fp(x, O.E4M3_FP_MIN, 448.0, 3)
    b = O.e4m3_roundtrip(x)
    # rint in simulate_fp is also half-to-even, so they agree on normals
    assert np.array_equal(a, b)
    # subnormal range: e4m3 keeps multiples of 2^-9, simulate_fp flushes below fp_min
    tiny = np.float32(2.0 ** -8)
    assert O.e4m3_roundtrip(tiny) == tiny
    assert O.simulate_fp(tiny, O.E4M3_FP_MIN, 448.0, 3) == 0


# ------------------------------------------------------------------ int codes
def test_int8_codes_ties_limits_specials():
    v = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 127.49, -127.5, -128.5, 1e9, -1e9,
                  np.inf, -np.inf, np.nan, 0.0, -0.0], dtype=np.float32)
    want = [0, 2, 2, 0, -2, -2, 126, 127, 127, -128, -128, 127, -128, 127, -128, -128, 0, 0]
    assert O.int8_codes(v).tolist() == want


def test_int8_codes_equal_python_round_on_dense_sweep():
    v = np.linspace(-140, 140, 56001, dtype=np.float32)
    want = [int(max(-128, min(127, round(float(t))))) for t in v]  # python round is half-even
    assert O.int8_codes(v).tolist() == want


def test_int8_clamp_then_round_equals_round_then_clamp():
    # the fake path rounds first and clamps after (quantizer.py:277-278); the
    # kernel clamps first.  Integer bounds make them equal.
    g = np.random.default_rng(0)
    v = (g.standard_normal(100000) * 100).astype(np.float32)
    assert np.array_equal(O.int8_codes(v), np.clip(np.rint(v), -128, 127).astype(np.int8))


def test_int4_codes_and_pack_exhaustive():
    v = np.array([-9, -8.5, -8, -7.5, -0.5, 0.5, 6.5, 7, 7.5, 8, np.nan], dtype=np.float32)
    assert O.int4_codes(v).tolist() == [-8, -8, -8, -8, 0, 0, 6, 7, 7, 7, -8]
    for lo in range(-8, 8):
        for hi in range(-8, 8):
            b = O.pack_int4(np.array([lo, hi], dtype=np.int8))
            assert b.shape == (1,)
            assert int(b[0]) == ((lo & 0xF) | ((hi & 0xF) << 4))
            assert O.unpack_int4(b).tolist() == [lo, hi]
    q = np.random.default_rng(1).integers(-8, 8, size=4096).astype(np.int8)
    assert np.array_equal(O.unpack_int4(O.pack_int4(q)), q)


# ------------------------------------------------------------------ contraction
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_INT4])
def test_gemm_acc_matches_bruteforce(fmt):
    g = np.random.default_rng(5)
    lo, hi = (-128, 128) if fmt == O.FMT_INT8 else (-8, 8)
    a = g.integers(-128, 128, size=(5, 48)).astype(np.int8)
    b = g.integers(lo, hi, size=(7, 48)).astype(np.int8)
    a[0, :] = -128
    b[0, :] = lo
    acc = O.gemm_acc(a, b, O.FMT_INT8, fmt)
    assert np.array_equal(acc.astype(np.int64), O.gemm_acc_bruteforce(a, b))


def test_gemm_acc_extreme_magnitude_is_exact():
    K = 15360
    a = np.full((2, K), -128, dtype=np.int8)
    b = np.full((3, K), -128, dtype=np.int8)
    acc = O.gemm_acc(a, b, O.FMT_INT8, O.FMT_INT8)
    assert (acc == K * 128 * 128).all() and K * 128 * 128 < 2 ** 31


def test_gemm_acc_equals_torch_int32_matmul():
    g = torch.Generator().manual_seed(11)
    a = torch.randint(-128, 128, (33, 256), generator=g, dtype=torch.int32)
    b = torch.randint(-128, 128, (17, 256), generator=g, dtype=torch.int32)
    ref = (a @ b.T).numpy()
    acc = O.gemm_acc(a.numpy().astype(np.int8), b.numpy().astype(np.int8), O.FMT_INT8, O.FMT_INT8)
    assert np.array_equal(acc.astype(np.int32), ref)


def test_fp8_products_are_exact_in_fp32():
    t = O.e4m3_decode_table()
    t = t[~np.isnan(t)].astype(np.float64)
    p = np.outer(t, t)
    assert np.array_equal(p.astype(np.float32).astype(np.float64), p)


# ------------------------------------------------------------------ scale indexing
def test_scale_broadcast_rule_and_flat_indices():
    S, B, M, K, N = 3, 2, 4, 16, 5
    g = np.random.default_rng(2)
    x = g.standard_normal((S, B, M, K)).astype(np.float32)
    per_seg = np.array([1.0, 2.0, 4.0], dtype=np.float32)
    per_tok = (np.arange(S * B * M) + 1).astype(np.float32)
    c1 = O.quantize_act(x, per_seg, O.FMT_INT8)
    c2 = O.quantize_act(x, per_tok, O.FMT_INT8)
    xf = x.reshape(S, B * M, K)
    for s in range(S):
        for t in range(B * M):
            assert np.array_equal(c1[s, t], O.int8_codes(xf[s, t] * per_seg[s]))
            assert np.array_equal(c2[s, t], O.int8_codes(xf[s, t] * per_tok[s * B * M + t]))
    acc = g.integers(-1000, 1000, size=(S, B * M, N))
    sw = (np.arange(S * N) + 1).astype(np.float32)
    y = O.dequant(acc, per_tok, sw)
    for s in range(S):
        for t in range(B * M):
            for n in range(N):
                want = np.float32(acc[s, t, n]) / (per_tok[s * B * M + t] * sw[s * N + n])
                assert y[s, t, n] == np.float32(want)


# ------------------------------------------------------------------ dual scale
@pytest.mark.parametrize("fmt", [O.FMT_INT8, O.FMT_E4M3, O.FMT_INT4])
def test_dual_split_invariants(fmt):
    g = np.random.default_rng(9)
    x = g.standard_normal((1, 6, 32)).astype(np.float32)
    x[0, 0, :4] = [0.0, -0.0, 1e-30, -1e-30]
    xp, xn = O.quantize_act_dual(x, np.float32([30.0]), np.float32([50.0]), fmt)
    vp, vn = O.code_values(xp, fmt), O.code_values(xn, fmt)
    assert (vp * vn == 0).all() and (vp >= 0).all() and (vn <= 0).all()
    # x == 0 (either sign) goes to the positive branch: Xn holds code(0)
    assert (vn[0, 0, :2] == 0).all()
    merged = O.merge_dual_codes(xp, xn, x)
    assert np.array_equal(O.code_values(merged, fmt), vp + vn)


def test_dual_with_equal_scales_reduces_to_single_scale_accumulator():
    g = np.random.default_rng(4)
    x = g.standard_normal((1, 9, 64)).astype(np.float32)
    w = g.integers(-128, 128, size=(1, 11, 64)).astype(np.int8)
    s = np.float32([40.0])
    _, acc = O.real_quantized_gemm_scaled(x, w, s, np.float32([1.0]), O.FMT_INT8, O.FMT_INT8, return_acc=True)
    _, ap, an = O.real_quantized_gemm_dual_scaled(x, w, s, s, np.float32([1.0]), O.FMT_INT8, O.FMT_INT8,
                                                  return_acc=True)
    assert np.array_equal(ap + an, acc)


# ------------------------------------------------------------------ segments
def test_weight_seg_is_concat_and_input_seg_is_sum():
    g = np.random.default_rng(6)
    M, K, N, S = 7, 64, 12, 2
    x = g.standard_normal((M, K)).astype(np.float32)
    wq = g.integers(-128, 128, size=(N, K)).astype(np.int8)
    sx = np.float32([25.0])
    # unsegmented accumulators
    _, acc = O.real_quantized_gemm_scaled(x[None], wq[None], sx, np.float32([1.0]), O.FMT_INT8, O.FMT_INT8,
                                          return_acc=True)
    xs, ws = O.segment_views(x, wq, "weight", S)
    _, acc_w = O.real_quantized_gemm_scaled(xs, ws, np.repeat(sx, S), np.ones(S, np.float32), O.FMT_INT8,
                                            O.FMT_INT8, return_acc=True)
    assert np.array_equal(np.concatenate(list(acc_w), axis=-1), acc[0])
    xs, ws = O.segment_views(x, wq, "input", S)
    _, acc_i = O.real_quantized_gemm_scaled(xs, ws, np.repeat(sx, S), np.ones(S, np.float32), O.FMT_INT8,
                                            O.FMT_INT8, return_acc=True)
    assert np.array_equal(acc_i.sum(0), acc[0])
    out = np.arange(S * M * 3, dtype=np.float32).reshape(S, M, 3)
    assert np.array_equal(O.recombine(out, "weight"), np.concatenate([out[0], out[1]], axis=-1))
    assert np.array_equal(O.recombine(out, "input", bias=np.ones(3, np.float32)), out[0] + out[1] + 1)


# ------------------------------------------------------------------ scales
def test_scale_closed_forms():
    assert O.int_scale(2.0) == 63.5 and O.int_scale(0.0) == 1.0 and O.int_scale(2.0 ** -25) == 1.0
    assert O.int_scale(3.5, bits=4) == 2.0
    pos, neg = O.int_dual_scales(2.0, 4.0)
    assert pos == 63.5 and neg == 32.0  # 127 on the positive side, 128 on the negative
    pos, neg = O.int_dual_scales(0.0, 0.0)
    assert pos == 1.0 and neg == 1.0
    assert O.fp8_scale(7.0) == 64.0 and O.fp8_dual_scales(7.0, 14.0) == (64.0, 32.0)
    v = O.int_scale(np.float32([0.0, 1.0]))
    assert v[0] == np.float32(127.0) / np.float32(2.0 ** -24) and v[1] == 127.0
    # per-axis scales follow torch's scalar / tensor = reciprocal * scalar
    a = torch.rand(1000, generator=torch.Generator().manual_seed(3)) * 10 + 0.01
    assert np.array_equal(O.int_scale(a.numpy()), (127 / a.clamp(min=O.EPS)).numpy())
    assert np.array_equal(O.fp8_scale(a.numpy()), (448.0 / a.clamp(min=O.EPS)).numpy())
    p_, n_ = O.int_dual_scales(a.numpy(), a.numpy())
    assert np.array_equal(n_, (-128 / (-a.clamp(min=O.EPS))).numpy()) and np.array_equal(p_, O.int_scale(a.numpy()))
    assert np.array_equal(O.row_scale_div(a.numpy(), 127.0), (torch.full_like(a, 127.0) / a).numpy())
    p, n = O.dual_amax(np.float32([[-3, 0, 2], [0, 0, 0]]), axis=-1)
    assert p.tolist() == [2, 0] and n.tolist() == [3, 0]
    assert O.dual_amax(np.float32([1, 2])) == (2.0, 0.0)


# ------------------------------------------------------------------ fake quant vs code path
def test_fake_int_equals_dequantised_codes():
    g = np.random.default_rng(8)
    x = (g.standard_normal((64, 96)) * 3).astype(np.float32)
    s = np.float32(O.int_scale(float(np.abs(x).max())))
    codes = O.int8_codes(x * s)
    assert np.array_equal(O.fake_quant_int(x, s), codes.astype(np.float32) / s)
    pa, na = O.dual_amax(x)
    ps, ns = (np.float32(t) for t in O.int_dual_scales(pa, na))
    xp, xn = O.quantize_act_dual(x[None], [ps], [ns], O.FMT_INT8)
    want = np.where(x >= 0, xp[0].astype(np.float32) / ps, xn[0].astype(np.float32) / ns)
    assert np.array_equal(O.fake_quant_int_dual(x, ps, ns), want)


def test_fake_fp8_equals_dequantised_codes_and_zero_mask():
    g = np.random.default_rng(10)
    x = g.standard_normal((32, 64)).astype(np.float32)
    x[0, 0] = 2.0 ** -26
    s = np.float32(O.fp8_scale(float(np.abs(x).max())))
    fq = O.fake_quant_fp8(x, s)
    assert fq[0, 0] == 0
    want = O.e4m3_decode(O.e4m3_encode(x * s)) / s
    want[0, 0] = 0
    assert np.array_equal(fq, want)


def test_real_pipeline_matches_fake_path_within_tolerance():
    g = np.random.default_rng(12)
    M, K, N = 16, 128, 24
    x = g.standard_normal((M, K)).astype(np.float32)
    w = (g.standard_normal((N, K)) * 0.02).astype(np.float32)
    sx = np.float32(O.int_scale(float(np.abs(x).max())))
    sw = np.float32(O.int_scale(float(np.abs(w).max())))
    wq = O.quantize_weights(w, float(sw), O.FMT_INT8)
    y = O.real_quantized_gemm_scaled(x[None], wq[None], [sx], [sw], O.FMT_INT8, O.FMT_INT8)[0]
    ref = O.segmented_matmul(O.fake_quant_int(x, sx)[None], O.fake_quant_int(w, sw)[None])[0]
    assert np.abs(y - ref).max() <= 1e-3 * np.abs(ref).max()


def test_round_to_bf16_matches_torch():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(100000, generator=g) * 100
    assert np.array_equal(O.round_to_bf16(x.numpy()), x.to(torch.bfloat16).float().numpy())


# ---- group-wise weight scales (exist in this build only) ----------------------
def test_group_functions_reduce_to_the_per_row_ones():
    """A group is a K slice of the weight with per-row scales: slice by slice the
    group functions must equal the per-row functions, and one group spanning all
    of K must equal the per-row result on the whole matrix."""
    rng = np.random.default_rng(11)
    n, k, g = 12, 96, 32
    w = (rng.standard_normal((n, k)) * 0.05).astype(np.float32)
    amax = O.group_amax(w, g)
    assert amax.shape == (n, k // g)
    for j in range(k // g):
        np.testing.assert_array_equal(amax[:, j], np.abs(w[:, j * g:(j + 1) * g]).max(axis=1))
    scale = O.int_scale(amax, bits=4)
    codes = O.quantize_weights_groups(w, scale, g, O.FMT_INT4)
    for j in range(k // g):
        np.testing.assert_array_equal(codes[:, j * g:(j + 1) * g],
                                      O.quantize_weights(w[:, j * g:(j + 1) * g], scale[:, j], O.FMT_INT4))
    whole = O.int_scale(O.group_amax(w, k), bits=4)
    np.testing.assert_array_equal(O.quantize_weights_groups(w, whole, k, O.FMT_INT4),
                                  O.quantize_weights(w, whole.reshape(-1), O.FMT_INT4))
    # every group reaches the end of the code range at its own maximum
    assert (np.abs(codes).reshape(n, k // g, g).max(axis=-1) == 7).all()


def test_linear_groups_against_bruteforce_and_per_row():
    rng = np.random.default_rng(12)
    m, n, k, g = 5, 7, 64, 16
    a = rng.integers(-127, 128, (m, k)).astype(np.int8)
    b = rng.integers(-8, 8, (n, k)).astype(np.int8)
    sx = (rng.random(m) + 0.5).astype(np.float32)
    sw = (rng.random((n, k // g)) + 0.5).astype(np.float32)
    bias = rng.standard_normal(n).astype(np.float32)
    got = O.linear_groups(a, b, sx, sw, g, bias)
    want = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            t = 0.0
            for kk in range(k):
                t += int(a[i, kk]) * int(b[j, kk]) / (float(sx[i]) * float(sw[j, kk // g]))
            want[i, j] = t + float(bias[j])
    np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-9)
    # equal scales in all groups of a row: the per-row de-quantisation of the whole sum
    sw_same = np.repeat(sw[:, :1], k // g, axis=1)
    acc = O.gemm_acc(a, b, O.FMT_INT8, O.FMT_INT4)
    np.testing.assert_allclose(O.linear_groups(a, b, sx, sw_same, g),
                               acc / (sx.astype(np.float64)[:, None] * sw_same[:, 0].astype(np.float64)[None, :]),
                               rtol=1e-12)


# ---- activation functions fused into the quantise kernel ----------------------
@pytest.mark.parametrize("op", ["gelu_tanh", "gelu", "silu"])
@pytest.mark.parametrize("dt", ["fp32", "bf16", "fp16"])
def test_activation_matches_torch_cpu_operators(op, dt):
    """Library routine as the pin: torch's own operators on the CPU.  torch evaluates
    in fp32 with its vectorised tanh / erf / exp, the oracle in fp64: they may differ
    by an ulp of the tensor's dtype at rounding boundaries, nowhere by more."""
    import torch.nn.functional as F
    tdt = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[dt]
    g = torch.Generator().manual_seed(5)
    x = (torch.randn(64, 256, generator=g) * 3).to(tdt)
    x[0, :6] = torch.tensor([0.0, -0.0, 20.0, -20.0, 1e-3, -1e-3]).to(tdt)
    gate = (torch.randn(64, 256, generator=g) * 2).to(tdt)
    fn = {"gelu_tanh": lambda t: F.gelu(t, approximate="tanh"), "gelu": F.gelu, "silu": F.silu}[op]
    ulp = {"fp32": 2.0 ** -21, "bf16": 2.0 ** -6, "fp16": 2.0 ** -9}[dt]  # two ulps at the bottom of a binade
    xf, gf = x.float().numpy(), gate.float().numpy()
    # where 1 + tanh(.) or 1 + erf(.) cancels, an error of a few ulps in the function (torch's
    # vectorised erf is that far off) is an absolute error of ~1e-6 |argument|
    for want, got, slack in ((fn(x), O.activation(xf, op, dtype=dt), 1e-6 * np.abs(xf)),
                             (x * fn(gate), O.activation(xf, op, gate=gf, dtype=dt), 1e-6 * np.abs(gf) * np.abs(xf))):
        want = want.float().numpy()
        diff = np.abs(got - want)
        assert (diff <= ulp * np.abs(want) + slack + 1e-30).all()
    # closed-form anchors: gelu(0) = silu(0) = 0, large |x| -> x or 0, odd/even structure
    z = O.activation(np.array([0.0, 30.0, -30.0], dtype=np.float32), op)
    assert z[0] == 0.0 and z[1] == 30.0 and abs(z[2]) < 1e-6


@pytest.mark.parametrize("dt", ["fp32", "bf16", "fp16"])
def test_smooth_divide_is_torchs_in_place_division(dt):
    tdt = {"fp32": torch.float32, "bf16": torch.bfloat16, "fp16": torch.float16}[dt]
    g = torch.Generator().manual_seed(9)
    x = (torch.randn(40, 96, generator=g) * 4).to(tdt)
    s = torch.rand(96, generator=g) * 3 + 0.01
    want = x.clone().div_(s.to(tdt)).float().numpy()
    assert np.array_equal(O.smooth_divide(x.float().numpy(), s.numpy(), dt), want)


def test_dequant_dual_against_fp64_closed_form_and_reductions():
    """dequant_dual (segquant/src/real_quant/dequantizer.cuh:53-74) pinned without reference to its
    own formula's code: (a) the fp64 value Yp/(pos sw) + Yn/(neg sw) written out with explicit
    per-token / per-channel indices, to fp32 rounding; (b) with power-of-two scales every fp32
    operation is exact, so the result must equal the fp64 value bit for bit; (c) Yn = 0 reduces it
    to the single-scale dequant, and pos == neg to the dequant of Yp + Yn."""
    g = np.random.default_rng(11)
    S, M, N = 2, 5, 7  # all different: a transposed or mis-broadcast scale changes the result
    yp = g.integers(0, 3_000_000, size=(S, M, N)).astype(np.int32)
    yn = -g.integers(0, 3_000_000, size=(S, M, N)).astype(np.int32)
    for per_tok in (False, True):
        for per_ch in (False, True):
            pos = (g.random(S * M if per_tok else S) * 30 + 1).astype(np.float32)
            neg = (g.random(S * M if per_tok else S) * 60 + 1).astype(np.float32)
            sw = (g.random(S * N if per_ch else S) * 50 + 1).astype(np.float32)
            got = O.dequant_dual(yp, yn, pos, neg, sw)
            want = np.empty((S, M, N))
            for s in range(S):
                for m in range(M):
                    for n in range(N):
                        p = np.float64(pos[s * M + m] if per_tok else pos[s])
                        q = np.float64(neg[s * M + m] if per_tok else neg[s])
                        w = np.float64(sw[s * N + n] if per_ch else sw[s])
                        want[s, m, n] = yp[s, m, n] / (p * w) + yn[s, m, n] / (q * w)
            size = np.abs(yp / 1.0) + np.abs(yn / 1.0)
            assert got.dtype == np.float32
            assert (np.abs(got - want) <= 4 * 2.0 ** -24 * np.maximum(np.abs(want), size / 31.0)).all()
    # (b) exact arithmetic
    pos = np.float32([2.0, 8.0]); neg = np.float32([4.0, 0.5]); sw = np.float32([16.0, 2.0])
    yp2 = (yp >> 8).astype(np.int32); yn2 = -((-yn) >> 8).astype(np.int32)  # below 2^24: exact as fp32
    got = O.dequant_dual(yp2, yn2, pos, neg, sw)
    want = yp2 / (pos.astype(np.float64) * sw)[:, None, None] + yn2 / (neg.astype(np.float64) * sw)[:, None, None]
    assert np.array_equal(got.astype(np.float64), want.astype(np.float32).astype(np.float64))
    # bf16 output: one rounding of that sum
    got_bf = O.dequant_dual(yp2, yn2, pos, neg, sw, "bf16")
    assert np.array_equal(got_bf, O.round_to_bf16(want.astype(np.float32)))
    # (c) reductions
    assert np.array_equal(O.dequant_dual(yp2, np.zeros_like(yp2), pos, neg, sw), O.dequant(yp2, pos, sw))
    assert np.array_equal(O.dequant_dual(yp2, yn2, pos, pos, sw), O.dequant(yp2 + yn2, pos, sw))


def test_int4_column_to_row_repack_against_its_elementwise_definition():
    """repack_int4_cols_to_rows (segquant/calibrator/calibrator.py:202-223) pinned by the layouts'
    definitions, element by element: the source holds value (row r, channel c) in nibble r & 1 of
    byte c * out/2 + r/2; the result must hold it in nibble c & 1 of byte r * cols/2 + c/2, which
    is what unpack_int4 reads.  Shapes where out != cols so a transposed view cannot pass."""
    g = np.random.default_rng(5)
    for out, cols in [(2, 2), (4, 6), (6, 4), (16, 2), (2, 16), (34, 130), (130, 34)]:
        vals = g.integers(0, 16, size=(out, cols)).astype(np.uint8)  # nibble of (row, channel)
        src = np.zeros(cols * out // 2, dtype=np.uint8)
        for r in range(out):
            for c in range(cols):
                src[c * (out // 2) + r // 2] |= vals[r, c] << (4 * (r & 1))
        got = O.repack_int4_cols_to_rows(src, out, cols)
        want = np.zeros(out * cols // 2, dtype=np.uint8)
        for r in range(out):
            for c in range(cols):
                want[r * (cols // 2) + c // 2] |= vals[r, c] << (4 * (c & 1))
        assert np.array_equal(got, want), (out, cols)
        signed = ((vals.astype(np.int16) ^ 8) - 8).astype(np.int8)  # two's complement nibbles
        assert np.array_equal(np.stack([O.unpack_int4(row) for row in got.reshape(out, cols // 2)]), signed)
    with pytest.raises(AssertionError):
        O.repack_int4_cols_to_rows(np.zeros(3, dtype=np.uint8), 3, 2)


def test_smooth_factors_and_svd_split_against_what_the_mathematics_fixes():
    """smooth_factors (optimizer.py:440-457): alpha = 1 gives max_x, alpha = 0 gives 1 / max_w, dead
    channels give 1, the clamp holds.  svd_split (:640-684): L1 L2 plus the residual reassemble
    the weight, the residual's Frobenius norm is the energy of the discarded singular values
    (Eckart-Young), L2 has orthonormal rows, and a weight of rank r leaves no residual.  Smoothing
    does not change the product: (x / s)(W s)^T == x W^T."""
    g = np.random.default_rng(21)
    mx = np.abs(g.standard_normal(40)).astype(np.float32) * 10 + 0.1
    mw = np.abs(g.standard_normal(40)).astype(np.float32) + 0.05
    assert np.allclose(O.smooth_factors(mx, mw, 1.0), np.clip(mx, 1e-4, 1e4), rtol=1e-6)
    assert np.allclose(O.smooth_factors(mx, mw, 0.0), np.clip(1 / mw, 1e-4, 1e4), rtol=1e-6)
    assert np.allclose(O.smooth_factors(mx, mw, 0.5), np.sqrt(mx.astype(np.float64) / mw), rtol=1e-5)
    dead = O.smooth_factors(np.float32([0.0, 1e-30, 5.0]), np.float32([1.0, 1.0, 1e-12]), 0.5)
    assert dead[0] == 1.0 and dead[1] == 1.0 and dead[2] == np.float32(1e4)
    assert O.smooth_factors(np.float32([1e-9]), np.float32([1e3]), 0.5)[0] == np.float32(1e-4)
    w = g.standard_normal((24, 40))
    l1, l2, res = O.svd_split(w, 5)
    assert l1.shape == (40, 5) and l2.shape == (5, 24) and res.shape == (24, 40)
    assert np.allclose(res + (l1 @ l2).T, w, atol=1e-12)
    sv = np.linalg.svd(w, compute_uv=False)
    assert np.isclose(np.linalg.norm(res), np.sqrt((sv[5:] ** 2).sum()), rtol=1e-10)
    assert np.allclose(l2 @ l2.T, np.eye(5), atol=1e-12)
    low = g.standard_normal((24, 3)) @ g.standard_normal((3, 40))
    assert np.abs(O.svd_split(low, 3)[2]).max() < 1e-10
    x = g.standard_normal((7, 40))
    s = O.smooth_factors(mx, mw, 0.5).astype(np.float64)
    assert np.allclose((x / s) @ (w * s).T, x @ w.T, rtol=1e-12, atol=1e-12)
    # smooth_svd_linear with a weight that the codes represent exactly and unit scales is x W^T
    wi = g.integers(-100, 100, size=(24, 40)).astype(np.int8)
    xi = g.integers(-100, 100, size=(7, 40)).astype(np.float32)
    ones = np.ones(40, dtype=np.float32)
    got = O.smooth_svd_linear(xi, ones, wi, [1.0], [1.0], O.FMT_INT8, O.FMT_INT8, l1=l1, l2=l2, bias=np.arange(24))
    assert np.allclose(got, xi.astype(np.float64) @ wi.T.astype(np.float64) + (xi.astype(np.float64) @ l1) @ l2 + np.arange(24))
