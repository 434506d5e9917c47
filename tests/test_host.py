"""CPU tests: the C-ABI library loads and exports what include/segq.h declares,
and the host-side mirror (quantisers, calibrators, optimiser, SegmentLinear,
quantize()) computes the reference's fake-quant arithmetic, checked against the
numpy oracle.  No GPU compute happens here."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from oracle import fake_path_torch as F
from oracle import segq_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ------------------------------------------------------------------ the C ABI
def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "segq.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(segq_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from segquant_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    lib = ctypes.CDLL(_lib.LIB_PATH)
    declared = _declared_symbols()
    assert set(declared) == set(_lib.EXPORTS), (declared, _lib.EXPORTS)
    for name in declared:
        assert hasattr(lib, name), name
    lib.segq_version.restype = ctypes.c_int
    assert lib.segq_version() >= 100
    lib.segq_gemm_tile_count.restype = ctypes.c_int
    assert lib.segq_gemm_tile_count() >= 5


def test_struct_layouts_match_the_header():
    """ctypes mirrors must have the size the C compiler gives the header's structs."""
    import subprocess
    import tempfile
    from segquant_amd import _lib
    src = ('#include "segq.h"\n#include <stdio.h>\nint main(){printf("%zu %zu %zu\\n",'
           'sizeof(segq_quant_desc),sizeof(segq_krange),sizeof(segq_gemm_desc));return 0;}\n')
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "s.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "s")
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe], check=True)
        sizes = [int(t) for t in subprocess.run([exe], capture_output=True, text=True, check=True).stdout.split()]
    assert sizes == [ctypes.sizeof(_lib.QuantDesc), ctypes.sizeof(_lib.KRange), ctypes.sizeof(_lib.GemmDesc)]


def test_argument_errors_are_reported_without_a_gpu():
    from segquant_amd import _lib
    lib = _lib.lib()
    d = _lib.GemmDesc()
    d.m, d.n, d.batch = 4, 4, 1
    assert lib.segq_gemm(ctypes.byref(d), None) == 1  # SEGQ_ERR_ARG: null pointers
    assert b"null" in lib.segq_last_error()
    q = _lib.QuantDesc()
    q.rows, q.cols = 2, 24  # cols not a multiple of 16
    q.x = q.codes = q.scale = 16
    assert lib.segq_quantize(ctypes.byref(q), None) == 1
    assert b"multiple of 16" in lib.segq_last_error()
    with pytest.raises(RuntimeError):
        _lib.check(1)


def test_empty_problems_succeed_before_any_device_work():
    """No rows, no columns, no tensors in a list: nothing to launch, so the entry points return
    SEGQ_OK without looking at pointers or the device; negative sizes are argument errors."""
    from segquant_amd import _lib
    lib = _lib.lib()
    for m, n in ((0, 64), (64, 0), (0, 0)):
        d = _lib.GemmDesc()
        d.m, d.n, d.batch = m, n, 1
        assert lib.segq_gemm(ctypes.byref(d), None) == 0
    d = _lib.GemmDesc()
    d.m, d.n, d.batch = -1, 4, 1
    assert lib.segq_gemm(ctypes.byref(d), None) == 1
    for rows, cols in ((0, 3072), (7, 0)):
        q = _lib.QuantDesc()
        q.rows, q.cols = rows, cols
        assert lib.segq_quantize(ctypes.byref(q), None) == 0
    q = _lib.QuantDesc()
    q.rows, q.cols = -3, 16
    assert lib.segq_quantize(ctypes.byref(q), None) == 1
    assert lib.segq_quantize_many(None, 0, None) == 0
    q, d = _lib.QuantDesc(), _lib.GemmDesc()
    q.cols, q.dynamic, d.n, d.batch, d.n_ranges = 3072, 1, 64, 1, 1
    assert lib.segq_linear(ctypes.byref(q), ctypes.byref(d), None) == 0
    two = (_lib.QuantDesc * 2)()
    two[0].rows, two[0].cols, two[1].rows, two[1].cols = 0, 3072, 5, 0
    assert lib.segq_quantize_many(two, 2, None) == 0


# ------------------------------------------------------------------ registry / loaders
def test_ext_dict_has_the_reference_shape():
    from segquant_amd.layers import ext_dict
    from segquant_amd.utils import extension as E
    assert set(ext_dict) == set(E.supported_type)
    for entry in ext_dict.values():
        assert set(entry) == {"gemm_scaled_fn", "gemm_dual_scaled_fn"}
    if not torch.cuda.is_available():
        assert all(v is None for e in ext_dict.values() for v in e.values())
        ext, prefixes = E.load_real_quant_int8_ext(required=False)
        assert ext is None and prefixes == ("Wint8Aint8",)
        with pytest.raises(RuntimeError):
            E.load_real_quant_int8_ext(required=True)


def test_real_quant_without_gpu_raises_instead_of_falling_back():
    if torch.cuda.is_available():
        pytest.skip("needs a machine without a GPU")
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    with pytest.raises(RuntimeError):
        SegmentLinear(32, 16, input_quant_type="int8", weight_quant_type="int8",
                      input_quant_args={"real_quant": True}, weight_quant_args={"real_quant": True}, device="cpu")


def test_fake_e4m3fy_cpu_matches_oracle():
    from segquant_amd.utils.extension import load_fake_quant_fp8_ext
    x = torch.randn(5000) * 100
    x[:4] = torch.tensor([0.0, 1e9, -1e9, 2.0 ** -10])
    got = load_fake_quant_fp8_ext().fake_e4m3fy(x).numpy()
    assert np.array_equal(got, O.e4m3_roundtrip(x.numpy()))


# ------------------------------------------------------------------ quantisers
@pytest.mark.parametrize("bits", [8, 4])
def test_int_quantizer_scales_and_fake_quant(bits):
    from segquant_amd.quantizers.quantizer import IntQuantizer
    g = torch.Generator().manual_seed(0)
    x = torch.randn(6, 32, generator=g) * 3
    q = IntQuantizer(num_bits=bits)
    q.calibrate(x)
    q.calibrate(x * 0.5)  # running maximum keeps the larger one
    assert q.scale == O.int_scale(float(x.abs().max()), bits)
    assert np.array_equal(q.fake_quantize(x).numpy(), O.fake_quant_int(x.numpy(), np.float32(q.scale), bits))
    qa = IntQuantizer(num_bits=bits, axis=-1)
    qa.calibrate(x)
    assert np.array_equal(qa.scale.numpy(), O.int_scale(x.abs().amax(-1).numpy(), bits))
    qd = IntQuantizer(num_bits=bits, dual_scale=True)
    qd.calibrate(x)
    pos, neg = O.int_dual_scales(*O.dual_amax(x.numpy()), bits)
    assert (qd.pos_scale, qd.neg_scale) == (pos, neg)
    assert np.array_equal(qd.fake_quantize(x).numpy(),
                          O.fake_quant_int_dual(x.numpy(), np.float32(pos), np.float32(neg), bits))
    qz = IntQuantizer(num_bits=bits, dual_scale=True)
    qz.calibrate(torch.zeros(4, 4))
    assert (qz.pos_scale, qz.neg_scale) == (1.0, 1.0)


def test_int_quantizer_group_scales_and_fake_quant():
    """group_size: one weight scale per (row, run of input channels); the oracle's group
    functions are the checker."""
    from segquant_amd.quantizers.quantizer import FloatQuantizer, IntQuantizer
    g = torch.Generator().manual_seed(3)
    w = torch.randn(10, 96, generator=g) * 0.05
    q = IntQuantizer(num_bits=4, axis=1, group_size=32)
    q.calibrate(w)
    want = O.int_scale(O.group_amax(w.numpy(), 32), 4)
    assert tuple(q.scale.shape) == (10, 3) and np.array_equal(q.scale.numpy(), want)
    codes = O.quantize_weights_groups(w.numpy(), want, 32, O.FMT_INT4).astype(np.float32)
    deq = (codes.reshape(10, 3, 32) / want[:, :, None]).reshape(10, 96)
    assert np.array_equal(q.fake_quantize(w).numpy(), deq)
    for bad in (dict(axis=None), dict(axis=1, dual_scale=True), dict(axis=1, dynamic=True), dict(axis=1, symmetric=False)):
        with pytest.raises(AssertionError):
            IntQuantizer(num_bits=4, group_size=32, **bad)
    with pytest.raises(AssertionError):
        FloatQuantizer(axis=1, group_size=32)
    with pytest.raises(ValueError):
        IntQuantizer(num_bits=4, axis=1, group_size=40).calibrate(w)


def test_float_quantizer_scales_and_fake_quant():
    from segquant_amd.quantizers.quantizer import FloatQuantizer, QuantizerRegistry
    g = torch.Generator().manual_seed(1)
    x = torch.randn(8, 48, generator=g)
    x[0, 0] = 2.0 ** -26
    q = QuantizerRegistry.create("fpe4m3")
    assert isinstance(q, FloatQuantizer)
    q.calibrate(x)
    assert q.scale == O.fp8_scale(float(x.abs().max()))
    assert np.array_equal(q.fake_quantize(x).numpy(), O.fake_quant_fp8(x.numpy(), np.float32(q.scale)))
    qd = FloatQuantizer(dual_scale=True, axis=-1)
    qd.calibrate(x)
    pa, na = O.dual_amax(x.numpy(), axis=-1)
    ps, ns = O.fp8_dual_scales(pa, na)
    assert np.array_equal(qd.pos_scale.numpy(), ps) and np.array_equal(qd.neg_scale.numpy(), ns)
    want = O.fake_quant_fp8_dual(x.numpy(), ps[:, None], ns[:, None])
    assert np.array_equal(qd.fake_quantize(x).numpy(), want)
    a = FloatQuantizer._simulate_fp(x * 10, q.fp_min, q.fp_max, 3).numpy()
    assert np.array_equal(a, O.simulate_fp((x * 10).numpy(), O.E4M3_FP_MIN, 448.0, 3))


def test_registry_names_follow_dtype_values():
    from segquant_amd.config import DType
    from segquant_amd.quantizers.quantizer import QuantizerRegistry
    for d in DType:
        assert QuantizerRegistry.get(d.value) is not None, d
    assert QuantizerRegistry.create("int4").qmax == 7
    with pytest.raises(ValueError):
        QuantizerRegistry.create("nope")


# ------------------------------------------------------------------ SegmentLinear, fake path
def _make_layer(K, N, seg_mode, chunks, chunksizes=None, atype="int8", wtype="int8", axis=False, dual=False, seed=0):
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(N, K, generator=g) * 0.05
    b = torch.randn(N, generator=g) * 0.01
    layer = SegmentLinear(K, N, bias=True, seg_mode=seg_mode, chunks=chunks, chunksizes=chunksizes,
                          custom_weight_tensor=w, custom_bias_tensor=b, input_quant_type=atype,
                          weight_quant_type=wtype,
                          input_quant_args={"real_quant": False, "dual_scale": dual, "axis": -1 if axis else None},
                          weight_quant_args={"real_quant": False, "axis": 1 if axis else None}, device="cpu")
    return layer, w, b


@pytest.mark.parametrize("seg_mode,chunks", [("weight", 1), ("weight", 3), ("input", 2)])
@pytest.mark.parametrize("axis", [False, True])
@pytest.mark.parametrize("atype", ["int8", "fpe4m3"])
def test_segment_linear_fake_path_equals_oracle(seg_mode, chunks, axis, atype):
    M, K, N = 7, 64, 48
    layer, w, b = _make_layer(K, N, seg_mode, chunks, atype=atype, wtype=atype, axis=axis)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(M, K, generator=g)
    x_before = x.clone()
    layer.calibrate(x)
    layer.finish_calibrate()
    y = layer(x).numpy()
    assert torch.equal(x, x_before), "the fake path must not write into the caller's input"
    # oracle: same segment views, per-segment scales by the closed forms
    xs, ws = O.segment_views(x.numpy(), w.numpy(), seg_mode, chunks)
    sc = (lambda a: O.fp8_scale(a)) if atype == "fpe4m3" else (lambda a: O.int_scale(a, 8))
    fq = (lambda t, s: O.fake_quant_fp8(t, s)) if atype == "fpe4m3" else (lambda t, s: O.fake_quant_int(t, s, 8))
    outs = []
    for s in range(chunks):
        xi = np.ascontiguousarray(xs[s])
        wi = np.ascontiguousarray(ws[s]) if seg_mode == "weight" else w.numpy()
        if axis:
            sx = sc(np.abs(xi).max(-1))[:, None]
            sw_full = sc(np.abs(wi).max(-1))[:, None]
        else:
            sx = np.float32(sc(float(np.abs(xi).max())))
            sw_full = np.float32(sc(float(np.abs(wi).max())))
        wq = fq(wi, sw_full)
        if seg_mode == "input":
            wq = wq[:, s * (K // chunks):(s + 1) * (K // chunks)]
        outs.append(fq(xi, sx) @ wq.T)
    want = O.recombine(np.stack(outs), seg_mode, bias=b.numpy())
    assert np.abs(y - want).max() <= 2e-6 * np.abs(want).max()
    # chunked output has the reference's (S, ..., n) layout
    ch = layer(x, chunked=True)
    assert ch.shape == (chunks, M, N // chunks if seg_mode == "weight" else N)


def test_unequal_and_mixed_dual_segments_on_the_fake_path():
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    K, N, M = 96, 40, 9
    g = torch.Generator().manual_seed(2)
    w = torch.randn(N, K, generator=g) * 0.05
    x = torch.randn(M, K, generator=g)
    x[:, 32:] = torch.nn.functional.gelu(x[:, 32:])
    layer = SegmentLinear(K, N, bias=False, seg_mode="input", chunks=2, chunksizes=[32, 64], custom_weight_tensor=w,
                          input_quant_type="int8", weight_quant_type="int8",
                          input_quant_args={"real_quant": False, "dual_scale": [False, True], "axis": None},
                          weight_quant_args={"real_quant": False, "axis": None}, device="cpu")
    assert layer.optimizer.dual_segments == [False, True] and layer.optimizer.dual_scale
    layer.calibrate(x)
    layer.finish_calibrate()
    y = layer(x).numpy()
    xn, wn = x.numpy(), w.numpy()
    s0 = np.float32(O.int_scale(float(np.abs(xn[:, :32]).max())))
    ps, ns = (np.float32(t) for t in O.int_dual_scales(*O.dual_amax(xn[:, 32:])))
    sw = np.float32(O.int_scale(float(np.abs(wn).max())))
    xf = np.concatenate([O.fake_quant_int(xn[:, :32], s0), O.fake_quant_int_dual(xn[:, 32:], ps, ns)], axis=1)
    want = xf @ O.fake_quant_int(wn, sw).T
    assert np.abs(y - want).max() <= 2e-6 * np.abs(want).max()
    with pytest.raises(NotImplementedError):
        layer(x, chunked=True)  # stacked per-segment outputs need equal sizes, as in the reference


def test_constructor_checks_mirror_the_reference():
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    with pytest.raises(ValueError):
        SegmentLinear(8, 8, seg_mode="rows", input_quant_type="int8", weight_quant_type="int8", device="cpu")
    with pytest.raises(AssertionError):
        SegmentLinear(8, 8, custom_weight_tensor=torch.zeros(4, 8), input_quant_type="int8",
                      weight_quant_type="int8", device="cpu")
    with pytest.raises(ValueError):
        SegmentLinear(8, 8, input_quant_type="int8", weight_quant_type="int8",
                      weight_quant_args={"dual_scale": True}, device="cpu")
    with pytest.raises(ValueError):
        SegmentLinear(8, 8, input_quant_type="int8", weight_quant_type="int8", opt_type="gptq-search", device="cpu")
    assert type(SegmentLinear(8, 8, input_quant_type="int8", weight_quant_type="int8", opt_type="smooth",
                              device="cpu").optimizer).__name__ == "SmoothOptimizer"


def test_quantize_replaces_linears_and_keeps_outputs_close():
    from segquant_amd.config import Calibrate, DType, Optimum
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    from segquant_amd.torch.quantization import quantize

    class Net(torch.nn.Module):
        def __init__(self):
            super().__init__()
            self.a = torch.nn.Linear(32, 32)
            self.blocks = torch.nn.ModuleList([torch.nn.Linear(64, 48), torch.nn.Linear(48, 16)])
            self.skip = torch.nn.Linear(16, 16)

        def forward(self, x, e):
            h = torch.cat([self.a(x), e], dim=1)
            return self.skip(self.blocks[1](torch.nn.functional.silu(self.blocks[0](h))))

    torch.manual_seed(0)
    net = Net()
    g = torch.Generator().manual_seed(42)
    loader = [((torch.rand(3, 32, generator=g), torch.rand(3, 32, generator=g)),) for _ in range(5)]
    cfg = {"default": {"enable": True, "seglinear": True, "search_patterns": [], "real_quant": False,
                       "opt": {"type": Optimum.DEFAULT}, "calib": {"type": Calibrate.AMAX},
                       "input_quant": {"type": DType.INT8, "axis": None},
                       "weight_quant": {"type": DType.INT8, "axis": None}},
           "skip": {"enable": False}}
    x, e = torch.rand(3, 32, generator=g), torch.rand(3, 32, generator=g)
    ref = net(x, e)
    import copy
    qnet = quantize(copy.deepcopy(net), loader, cfg, seg_configs={"blocks.0": {"seg_mode": "input", "chunks": 2}},
                    dual_scale_linears={"blocks.1"})
    assert isinstance(qnet.a, SegmentLinear) and isinstance(qnet.blocks[0], SegmentLinear)
    assert isinstance(qnet.skip, torch.nn.Linear)  # disabled by pattern
    assert qnet.blocks[0].seg_mode == "input" and qnet.blocks[0].chunks == 2
    assert qnet.blocks[1].optimizer.dual_scale and not qnet.a.optimizer.dual_scale
    out = qnet(x, e)
    assert ((out - ref).norm() / ref.norm()).item() < 0.05
    off = copy.deepcopy(cfg)
    off["default"]["enable"] = False
    same = quantize(copy.deepcopy(net), loader, off)
    assert isinstance(same.a, torch.nn.Linear)


# ------------------------------------------------------------------ workloads and the CPU baseline
def test_workloads_are_deterministic_and_shaped_like_the_configs():
    from segquant_amd import workloads as W
    shapes = {1: [(256, 1536, 9216)], 2: [(4096, 1536, 6144), (4096, 6144, 1536)],
              3: [(4608, 3072, 9216), (4608, 3072, 12288), (4608, 12288, 3072)],
              4: [(8192, 1280, 10240), (8192, 5120, 1280), (2048, 1280, 10240)]}
    for c, want in shapes.items():
        assert [(s.M, s.K, s.N) for s in W.config_linears(c)] == want
    c5 = W.config_linears(5)
    assert sorted({s.M for s in c5}) == [1024, 4608, 9216] and all(s.chunksizes == [3072, 12288] for s in c5)
    sp = W.config_linears(3, M=8)[0]
    a, b = W.make_input(sp), W.make_input(sp)
    assert torch.equal(a, b) and a.shape == (8, 3072)
    assert not torch.equal(W.make_weight(sp), W.make_weight(W.config_linears(3, M=8)[1])[:9216])


def test_torch_fake_path_equals_numpy_oracle():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(12, 96, generator=g)
    x[:, 32:] = torch.nn.functional.gelu(x[:, 32:])
    w = torch.randn(20, 96, generator=g) * 0.05
    for fmt in ("int8", "fpe4m3"):
        sw = F.scale_of(w.abs().amax(), fmt)
        w_hat = F.fake_quant(w, fmt, sw)
        y = F.fake_linear(x, w_hat, None, fmt, [0, 32, 96], [False, True], per_token=True).numpy()
        xn = x.numpy()
        sc, dsc = (O.fp8_scale, O.fp8_dual_scales) if fmt == "fpe4m3" else (O.int_scale, O.int_dual_scales)
        s0 = sc(np.abs(xn[:, :32]).max(-1))[:, None]
        pa, na = O.dual_amax(xn[:, 32:], axis=-1)
        ps, ns = dsc(pa, na)
        if fmt == "fpe4m3":
            xf = np.concatenate([O.fake_quant_fp8(xn[:, :32], s0), O.fake_quant_fp8_dual(xn[:, 32:], ps[:, None], ns[:, None])], 1)
            wf = O.fake_quant_fp8(w.numpy(), np.float32(sw))
        else:
            xf = np.concatenate([O.fake_quant_int(xn[:, :32], s0), O.fake_quant_int_dual(xn[:, 32:], ps[:, None], ns[:, None])], 1)
            wf = O.fake_quant_int(w.numpy(), np.float32(sw))
        want = xf @ wf.T
        assert np.abs(y - want).max() <= 2e-6 * np.abs(want).max()


# ------------------------------------------------------------------ traceable operators
def test_custom_operators_have_shape_only_kernels_for_tracing():
    """The reference-named operators are torch.library custom ops: on meta / fake tensors they
    return the contract's output shape and dtype without touching a GPU, and a symbolic trace
    keeps them as single nodes."""
    from torch.fx.experimental.proxy_tensor import make_fx
    from torch._subclasses.fake_tensor import FakeTensorMode
    from segquant_amd import torch_ops  # noqa: F401  (registers the operators)
    x = torch.empty(3, 2, 5, 64, device="meta", dtype=torch.bfloat16)
    w8 = torch.empty(3, 48, 64, device="meta", dtype=torch.int8)
    w4 = torch.empty(3, 48 * 64 // 2, device="meta", dtype=torch.uint8)
    s = torch.empty(3, device="meta")
    o = torch.ops.segquant_amd.real_quantized_gemm_scaled(x, w8, s, s, "int8", "int8")
    assert o.shape == (3, 2, 5, 48) and o.dtype == torch.bfloat16 and o.device.type == "meta"
    o = torch.ops.segquant_amd.real_quantized_gemm_dual_scaled(x, w4, s, s, s, "int8", "int4")
    assert o.shape == (3, 2, 5, 48) and o.dtype == torch.bfloat16

    def f(x, w, sx, sw):
        return torch.ops.segquant_amd.real_quantized_gemm_scaled(x * 2, w, sx, sw, "fpe4m3", "fpe4m3").sum(0)

    with FakeTensorMode() as mode:
        args = [mode.from_tensor(t) for t in (torch.zeros(3, 5, 64), torch.zeros(3, 48, 64, dtype=torch.uint8),
                                              torch.ones(3), torch.ones(3))]
        g = make_fx(f)(*args)
    targets = [n.target for n in g.graph.nodes if n.op == "call_function"]
    assert torch.ops.segquant_amd.real_quantized_gemm_scaled.default in targets
    # real CPU tensors have no kernel: the call fails loudly
    with pytest.raises(RuntimeError):
        torch.ops.segquant_amd.real_quantized_gemm_scaled(torch.zeros(1, 2, 16), torch.zeros(1, 4, 16, dtype=torch.int8),
                                                          torch.ones(1), torch.ones(1), "int8", "int8")


def test_forward_parts_on_the_fake_path_is_the_concatenated_forward():
    """forward_parts([a, b], pre_ops) on a CPU (fake-quant) layer: the parts are activated and
    concatenated with torch operators and take the ordinary forward."""
    import torch
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    g = torch.Generator().manual_seed(3)
    lin = torch.nn.Linear(96, 40)
    layer = SegmentLinear(96, 40, bias=True, seg_mode="input", chunks=2, chunksizes=[32, 64],
                          custom_weight_tensor=lin.weight.data, custom_bias_tensor=lin.bias.data,
                          input_quant_type="int8", weight_quant_type="int8",
                          input_quant_args={"dual_scale": [False, True]}, weight_quant_args={}, device="cpu")
    a, b = torch.randn(7, 32, generator=g), torch.randn(7, 64, generator=g)
    x = torch.cat([a, torch.nn.functional.silu(b)], dim=1)
    layer.calibrate(x)
    layer.finish_calibrate()
    assert torch.equal(layer.forward_parts([a, b], pre_ops=[None, "silu"]), layer(x))
    with pytest.raises(Exception):
        SegmentLinear(96, 40, seg_mode="weight", chunks=2, input_quant_type="int8", weight_quant_type="int8",
                      device="cpu").optimizer.forward_parts([a, b])


@pytest.mark.parametrize("opt_type", ["smooth", "svd"])
@pytest.mark.parametrize("seg_mode,chunks", [("weight", 1), ("weight", 3), ("input", 2)])
def test_smooth_and_svd_layers_on_the_fake_path_equal_the_oracle(opt_type, seg_mode, chunks):
    """trace -> smooth -> calibrate -> forward of the smoothing optimisers (fake quantisation, CPU)
    against the closed form the oracle builds chunk by chunk: s from the traced maxima, the weight
    chunk times s split into L1 L2 and a residual, fake-quantised x / s times the fake-quantised
    residual plus (x / s) L1 L2 (segquant/optimum/optimizer.py:440-517, :640-731)."""
    import torch
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    K, N, M, r, alpha = 48, 36, 10, 4, 0.5
    g = torch.Generator().manual_seed(11)
    lin = torch.nn.Linear(K, N)
    x = torch.randn(M, K, generator=g) * (torch.rand(K, generator=g) * 4 + 0.2)
    layer = SegmentLinear(K, N, bias=True, seg_mode=seg_mode, chunks=chunks, custom_weight_tensor=lin.weight.data,
                          custom_bias_tensor=lin.bias.data, input_quant_type="int8", weight_quant_type="int8",
                          input_quant_args={}, weight_quant_args={}, opt_type=opt_type,
                          opt_kwargs={"alpha": alpha, **({"low_rank": r} if opt_type == "svd" else {})}, device="cpu")
    layer.trace(x)
    layer.smooth()
    layer.calibrate(x)
    layer.finish_calibrate()
    got = layer(x).double().numpy()
    xn, wn = x.numpy(), lin.weight.data.numpy()
    want = np.zeros((M, N))
    ksz, nsz = K // chunks, N // chunks
    for i in range(chunks):
        ks = slice(i * ksz, (i + 1) * ksz) if seg_mode == "input" else slice(0, K)
        ns = slice(0, N) if seg_mode == "input" else slice(i * nsz, (i + 1) * nsz)
        xc, wc = xn[:, ks], wn[ns, ks]
        s = O.smooth_factors(np.abs(xc).max(axis=0), np.abs(wc).max(axis=0), alpha)
        ws = (wc * s).astype(np.float32)
        xs = (xc / s).astype(np.float32)
        low = 0.0
        if opt_type == "svd":
            l1, l2, res = O.svd_split(ws, r)
            ws = res.astype(np.float32)
            low = (xs.astype(np.float64) @ l1.astype(np.float32)) @ l2.astype(np.float32)
        sx, sw = O.int_scale(float(np.abs(xs).max())), O.int_scale(float(np.abs(ws).max()))
        want[:, ns] += O.fake_quant_int(xs, sx).astype(np.float64) @ O.fake_quant_int(ws, sw).astype(np.float64).T + low
    want += lin.bias.data.double().numpy()
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max()
    ref = lin(x).double().detach().numpy()
    assert np.linalg.norm(got - ref) / np.linalg.norm(ref) < 0.05
    assert layer.optimizer.fused_available() is False  # no kernels on the CPU
    with pytest.raises(NotImplementedError):
        SegmentLinear(K, N, input_quant_type="int8", weight_quant_type="int8", opt_type=opt_type,
                      opt_kwargs={"search_alpha_config": {"enable": True, "min": 0.1, "max": 0.9, "step": 0.1}}, device="cpu")


def _plan(lib, m, n, ranges, fmt, out_dtype=2, lend=True, split_k=0, tile=0, lowrank=0):
    """segq_gemm_plan / segq_gemm_workspace_bytes on a descriptor of made-up (aligned, never
    dereferenced) device addresses: the library's decisions are host arithmetic and launch nothing.
    ranges: (k_begin, k_len, a_sel).  Returns (tile id, K shares, parked, workspace bytes)."""
    import ctypes as C
    from segquant_amd import _lib as L
    d = L.GemmDesc()
    d.a_fmt = d.b_fmt = fmt
    d.out_dtype = d.bias_dtype = out_dtype  # 2: bf16
    k = max(b + l for b, l, _ in ranges)
    d.m, d.n, d.lda, d.ldb, d.ldo, d.batch = m, n, k, k, n, 1
    d.a, d.a_neg, d.b, d.out, d.bias = 0x10000000, 0x20000000, 0x30000000, 0x40000000, 0x50000000
    d.n_ranges, d.tile, d.split_k = len(ranges), tile, split_k
    for i, (b, l, sel) in enumerate(ranges):
        d.ranges[i].k_begin, d.ranges[i].k_len, d.ranges[i].a_sel = b, l, sel
        d.ranges[i].sx_row_stride, d.ranges[i].sw_col_stride = 1, 1
        d.ranges[i].sx, d.ranges[i].sw = 0x60000000, 0x70000000
    if lowrank:
        d.lowrank_t, d.lowrank_l2t, d.lowrank_rank, d.ld_lowrank_t, d.ld_lowrank_l2t = 0x80000000, 0x90000000, lowrank, lowrank, lowrank
    need = C.c_int64(-1)
    assert lib.segq_gemm_workspace_bytes(C.byref(d), C.byref(need)) == 0, lib.segq_last_error()
    if lend:
        d.workspace, d.workspace_bytes = 0xA0000000, max(need.value, 16)
    t, s, p = C.c_int32(0), C.c_int32(0), C.c_int32(0)
    assert lib.segq_gemm_plan(C.byref(d), C.byref(t), C.byref(s), C.byref(p)) == 0, lib.segq_last_error()
    return t.value, s.value, p.value, need.value


def test_tile_and_share_choice_for_the_benchmark_shapes():
    """What the library picks (tile id, K shares, parking) for the shapes of the five benchmark
    configurations and for a few-token shape, with a workspace of the size it asks for and without
    one.  Pure host arithmetic: no GPU, nothing launched.  (256 CUs are assumed when there is no
    device to ask.)"""
    import ctypes as C
    from segquant_amd import _lib as L
    lib = L.lib()
    lib.segq_last_error.restype = C.c_char_p
    I8, F8 = 0, 1
    one = lambda k: [(0, k, 0)]
    c5 = [(0, 3072, 0), (3072, 12288, 0), (3072, 12288, 1)]   # attn | MLP positive codes | MLP negative codes
    fc2 = [(0, 6144, 0), (0, 6144, 1)]
    # configuration 3: whole rounds of 256 CUs with 192x288 / 384x192 / 288x192 tiles, nothing split
    assert _plan(lib, 4608, 9216, one(3072), I8)[:3] == (15, 1, 0)
    assert _plan(lib, 4608, 12288, one(3072), I8)[:3] == (20, 1, 0)     # three rounds, where 288x192 needs four
    assert _plan(lib, 4608, 12288, one(3072), F8)[:3] == (20, 1, 0)
    assert _plan(lib, 4608, 3072, one(12288), I8)[:3] == (16, 1, 0)
    assert _plan(lib, 8192, 8192, one(8192), I8)[:3] == (11, 1, 0)      # 384 does not divide 8192
    assert _plan(lib, 4608, 12288, [(0, 1536, 0), (1536, 1536, 0)], I8)[0] != 20   # int8 with two ranges: not on 384x192
    # configuration 1: 144 tiles of 128x128 do not fill the CUs: 192 tiles of 128x96 with five stages; fp32 output (0)
    assert _plan(lib, 256, 9216, one(1536), I8, out_dtype=0)[:3] == (21, 1, 0)
    assert _plan(lib, 256, 9216 + 128, one(1536), I8, out_dtype=0)[:3] == (19, 1, 0)   # 96 does not divide the columns: 128x128, four stages
    # configuration 2: fc1 in two whole rounds of 256x192; fc2 (DualScale: two ranges) as 128 tiles in two K shares
    assert _plan(lib, 4096, 6144, one(1536), F8)[:3] == (17, 1, 0)
    t, s, p, need = _plan(lib, 4096, 1536, fc2, F8)
    assert (t, s, p) == (17, 2, 0) and need == 128 * 2 * 256 * 192 * 4 + 128 * 4 + (-(128 * 4) % 256)
    assert _plan(lib, 4096, 1536, fc2, F8, lend=False)[1] == 1          # no workspace: no shares
    assert _plan(lib, 4096, 1536, fc2, F8, split_k=1)[1] == 1           # forbidden by the caller
    # configuration 5: 1024 tokens in 64 tiles x 4 shares (int8: parked ranges too), 4608 and 9216 whole
    assert _plan(lib, 1024, 3072, c5, F8)[:3] == (17, 4, 0)
    assert _plan(lib, 1024, 3072, c5, I8)[:3] == (17, 4, 1)
    assert _plan(lib, 4608, 3072, c5, I8)[:3] == (16, 1, 1)
    assert _plan(lib, 9216, 3072, c5, F8)[:3] == (16, 1, 0)
    t, s, p, need = _plan(lib, 4608, 3072, c5, I8, lend=False)          # int8, several ranges, nothing lent:
    assert p == 0 and need == 256 * 288 * 192 * 4 and t in (12, 13, 14)  # a second register set, smaller tiles
    # few tokens: K shares of the 128x128 tile
    t, s, p, _ = _plan(lib, 64, 9216, one(3072), I8)
    assert t == 14 and s in (2, 3)
    # the low-rank branch moves to a tile that is built with it
    assert _plan(lib, 4608, 12288, one(3072), I8, lowrank=32)[:2] == (11, 1)


def test_plan_refuses_what_the_launch_would_refuse():
    """segq_gemm_plan walks the launch's own dispatch down to the kernel instance: a descriptor whose
    launch has no kernel (an explicit tile that is not built for parked ranges or for the low-rank
    branch, a retired tile id) is refused by the plan with the same status, so callers that probe
    with the plan (the SVD optimiser does) never meet the refusal at launch time."""
    import ctypes as C
    from segquant_amd import _lib as L
    lib = L.lib()
    lib.segq_last_error.restype = C.c_char_p
    I8, F8 = 0, 1
    c5 = [(0, 3072, 0), (3072, 12288, 0), (3072, 12288, 1)]

    def status(m, n, ranges, fmt, tile, lowrank=0, lend=True):
        d = L.GemmDesc()
        d.a_fmt = d.b_fmt = fmt
        d.out_dtype = d.bias_dtype = 2
        k = max(b + l for b, l, _ in ranges)
        d.m, d.n, d.lda, d.ldb, d.ldo, d.batch = m, n, k, k, n, 1
        d.a, d.a_neg, d.b, d.out = 0x10000000, 0x20000000, 0x30000000, 0x40000000
        d.n_ranges, d.tile = len(ranges), tile
        for i, (b, l, sel) in enumerate(ranges):
            d.ranges[i].k_begin, d.ranges[i].k_len, d.ranges[i].a_sel = b, l, sel
            d.ranges[i].sx, d.ranges[i].sw = 0x60000000, 0x70000000
        if lowrank:
            d.lowrank_t, d.lowrank_l2t, d.lowrank_rank, d.ld_lowrank_t, d.ld_lowrank_l2t = 0x80000000, 0x90000000, lowrank, lowrank, lowrank
        if lend:
            d.workspace, d.workspace_bytes = 0xA0000000, 1 << 34
        t = C.c_int32(0)
        return lib.segq_gemm_plan(C.byref(d), C.byref(t), None, None)

    assert status(4608, 3072, c5, I8, 16) == 0                 # 288 x 192 parks
    assert status(4608, 3072, c5, I8, 20) == 2                 # 384 x 192 is built for one int8 range only
    assert status(4608, 3072, c5, I8, 19) == 2                 # and so is the four-stage 128 x 128 kernel
    assert status(4608, 3072, c5, F8, 20) == 0                 # e4m3 rescales in place on every tile
    assert status(4608, 3072, [(0, 3072, 0)], I8, 9) == 2      # retired ids
    assert status(4608, 3072, [(0, 3072, 0)], I8, 10) == 2
    assert status(4608, 9216, [(0, 3072, 0)], I8, 15, lowrank=32) == 2   # 192 x 288 has no low-rank finish
    assert status(4608, 9216, [(0, 3072, 0)], I8, 11, lowrank=32) == 0
    assert status(4608, 9216, [(0, 3072, 0)], I8, 0, lowrank=32) == 0    # the library's own choice always has a kernel
