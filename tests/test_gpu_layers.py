"""GPU tests of the host-side mirror (SegmentLinear, optimiser, quantize())
running on the HIP kernels, checked against the CPU oracle.

Every benchmark configuration is run at its real K and N and a reduced M so the
oracle finishes in seconds; the checks are (a) the exact closed form built from
the layer's own codes and scales, (b) the path's stated tolerance against the
fp32 fake-quant linear: 1e-3 relative for integer codes, 1e-2 for e4m3.
"""
import numpy as np
import pytest
import torch

from oracle import segq_oracle as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


from _layer_oracle import _np32, oracle_layer_output  # noqa: E402


CASES = [(1, 96), (2, 160), (3, 130), (4, 144), (5, 100)]


@pytest.mark.parametrize("config,M", CASES)
def test_benchmark_configs_fused_forward(config, M):
    from segquant_amd import workloads as W
    seen = set()
    for spec in W.config_linears(config, M=M):
        if (spec.name.split("_m")[0], spec.K, spec.N) in seen:
            continue
        seen.add((spec.name.split("_m")[0], spec.K, spec.N))
        layer, x = W.build_layer(spec, device=DEV, real_quant=True)
        assert layer.optimizer.real_quant, spec.name
        xin = x.to(spec.x_dtype).to(DEV)
        out = layer(xin)
        assert out.shape == (M, spec.N) and out.dtype == spec.x_dtype
        got = _np32(out).astype(np.float64)
        x_np = _np32(xin)
        want = oracle_layer_output(layer, spec, x_np, spec.x_dtype)
        scale = np.abs(want).max()
        fp8 = spec.act == O.FMT_E4M3
        tol = {torch.float32: 3e-6, torch.bfloat16: 2.0 ** -8}[spec.x_dtype] + (1e-3 if fp8 else 0.0)
        assert np.abs(got - want).max() <= tol * scale, (spec.name, np.abs(got - want).max() / scale)
        # (b) fp32 input through the same layer vs the fp32 fake-quant linear
        layer_f, _ = W.build_layer(spec, device=DEV, real_quant=False, x=x)
        ref = _np32(layer_f(x.to(DEV))).astype(np.float64)
        real32 = _np32(layer(x.to(DEV))).astype(np.float64)
        rel = np.abs(real32 - ref).max() / np.abs(ref).max()
        assert rel <= (1e-2 if fp8 else 1e-3), (spec.name, rel)


@pytest.mark.parametrize("kernel", ["Wint8Aint8", "Wfpe4m3Afpe4m3", "Wint4Aint8"])
@pytest.mark.parametrize("seg_mode", ["weight", "input"])
@pytest.mark.parametrize("axis", [False, True])
@pytest.mark.parametrize("dual", [False, True])
def test_chunked_route_matches_fused_route(kernel, seg_mode, axis, dual):
    """forward(chunked=True) goes through the reference-convention operator
    registered in ext_dict; recombining its output must give the fused result."""
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    w_t, a_t = kernel[1:].split("A")
    M, K, N, S = 24, 256, 192, 2
    g = torch.Generator().manual_seed(7)
    x = torch.randn(M, K, generator=g)
    if dual:
        x = torch.nn.functional.silu(x * 2)
    lin = torch.nn.Linear(K, N)
    layer = SegmentLinear(K, N, bias=True, seg_mode=seg_mode, chunks=S, custom_weight_tensor=lin.weight.data,
                          custom_bias_tensor=lin.bias.data, input_quant_type=a_t, weight_quant_type=w_t,
                          input_quant_args={"real_quant": True, "dual_scale": dual, "axis": -1 if axis else None},
                          weight_quant_args={"real_quant": True, "axis": 1 if axis else None}, device=DEV)
    xd = x.to(DEV)
    layer.calibrate(xd)
    layer.finish_calibrate()
    fused = layer(xd)
    chunks = layer(xd, chunked=True)
    assert chunks.shape[0] == S
    if seg_mode == "weight":
        rec = chunks.movedim(0, -2).reshape(M, -1)
    else:
        rec = chunks.sum(0)
    rec = rec + layer.bias_data
    tol = 2e-3 if a_t == "fpe4m3" else 1e-5
    assert (rec - fused).abs().max().item() <= tol * fused.abs().max().item()
    ref = lin.to(DEV)(xd)
    assert ((fused - ref).norm() / ref.norm()).item() < (0.2 if w_t == "int4" else 0.05)


class _ChunkModel(torch.nn.Module):
    """SiLU -> Linear(D, 6D) -> chunk(6): the adaLN pattern of the reference's
    TestModel (test/test_linear.py:69-92)."""

    def __init__(self, d):
        super().__init__()
        self.silu = torch.nn.SiLU()
        self.linear = torch.nn.Linear(d, 6 * d)
        self.norm = torch.nn.LayerNorm(d, elementwise_affine=False, eps=1e-6)

    def forward(self, x, emb):
        shift, scale, gate, *_ = self.linear(self.silu(emb)).chunk(6, dim=1)
        return self.norm(x) * (1 + scale) + shift, gate


class _ConcatModel(torch.nn.Module):
    """two linears -> cat -> Linear(2D, 3D): the reference's TestInputModel (:94-108)."""

    def __init__(self, d):
        super().__init__()
        self.linear_1 = torch.nn.Linear(d, d)
        self.linear_2 = torch.nn.Linear(d, d)
        self.linear = torch.nn.Linear(2 * d, 3 * d)

    def forward(self, x, emb):
        return self.linear(torch.cat([self.linear_1(x), self.linear_2(emb)], dim=1))


@pytest.mark.parametrize("atype,wtype", [("INT8", "INT8"), ("FP8E4M3", "FP8E4M3"), ("INT8", "INT4")])
@pytest.mark.parametrize("axis", [False, True])
@pytest.mark.parametrize("model_kind", ["chunk", "concat"])
def test_quantize_real_vs_fake_like_the_reference_grid(atype, wtype, axis, model_kind):
    """The reference's test_mix_real grid (test/test_linear.py:821-913) with its
    data recipe (5 calibration batches of rand(3, D), seeds 42 / 1234); it only
    prints the norms, here fake and real must agree."""
    import copy
    from segquant_amd.config import Calibrate, DType, Optimum
    from segquant_amd.torch.quantization import quantize
    D = 256
    torch.manual_seed(0)
    model = (_ChunkModel(D) if model_kind == "chunk" else _ConcatModel(D)).to(DEV)
    g = torch.Generator().manual_seed(42)
    loader = [((torch.rand(3, D, generator=g), torch.rand(3, D, generator=g)),) for _ in range(5)]
    cfg = {"default": {"enable": True, "seglinear": True, "search_patterns": [], "real_quant": False,
                       "opt": {"type": Optimum.DEFAULT}, "calib": {"type": Calibrate.AMAX},
                       "input_quant": {"type": DType[atype], "axis": -1 if axis else None},
                       "weight_quant": {"type": DType[wtype], "axis": 1 if axis else None}}}
    segs = ({"linear": {"seg_mode": "weight", "chunks": 6}} if model_kind == "chunk"
            else {"linear": {"seg_mode": "input", "chunks": 2}})
    dual = {"linear"} if model_kind == "chunk" else set()
    fake = quantize(copy.deepcopy(model), loader, copy.deepcopy(cfg), seg_configs=segs, dual_scale_linears=dual)
    cfg["default"]["real_quant"] = True
    real = quantize(copy.deepcopy(model), loader, copy.deepcopy(cfg), seg_configs=segs, dual_scale_linears=dual)
    assert real.linear.optimizer.real_quant and not fake.linear.optimizer.real_quant
    g = torch.Generator().manual_seed(1234)
    x, emb = torch.rand(3, D, generator=g).to(DEV), torch.rand(3, D, generator=g).to(DEV)
    with torch.no_grad():
        a = model(x, emb)
        b = fake(x, emb)
        c = real(x, emb)
    a, b, c = (t[0] if isinstance(t, tuple) else t for t in (a, b, c))
    tol = 1e-2 if atype == "FP8E4M3" else 1e-3
    assert (b - c).abs().max().item() <= tol * b.abs().max().item()
    assert ((a - c).norm() / a.norm()).item() < (0.25 if wtype == "INT4" else 0.08)


@pytest.mark.parametrize("op,gated", [("gelu_tanh", False), ("gelu", True), ("silu", True)])
def test_layer_with_the_activation_function_fused_into_its_quantise_kernel(op, gated):
    """forward(x, pre_op=...) == forward(op(x)) with torch's operator, to the rounding of the
    output dtype (a code may move by one step where the two tanh / erf / exp differ by an ulp),
    on the DualScale e4m3 MLP of config 2 and on the fake path of the same layer."""
    from segquant_amd import workloads as W
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    spec = [s for s in W.config_linears(2, M=192) if s.name == "fc2"][0]
    g = torch.Generator().manual_seed(7)
    pre = (torch.randn(192, spec.K, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
    gate = (torch.randn(192, spec.K, generator=g) * 1.5).to(torch.bfloat16).to(DEV) if gated else None
    act = SegmentLinear._activated(pre, op, gate)
    layer, _ = W.build_layer(spec, device=DEV, real_quant=True, x=act.float().cpu())
    want = layer(act).float()
    got = layer(pre, pre_op=op, gate=gate).float()
    assert (got - want).abs().max().item() <= 2e-2 * want.abs().max().item()
    assert ((got - want).abs() > 2.0 ** -7 * want.abs().max()).float().mean().item() <= 1e-2
    fake, _ = W.build_layer(spec, device=DEV, real_quant=False, x=act.float().cpu())
    pre32, gate32 = pre.float(), (gate.float() if gated else None)  # the fake path multiplies in the weight's fp32
    assert torch.equal(fake(pre32, pre_op=op, gate=gate32), fake(SegmentLinear._activated(pre32, op, gate32)))


def test_layer_hooks_for_smooth_division_and_low_rank_addend():
    """forward(x, col_div=s, addend=r) == forward(x / s) + r through the fused kernels (the
    division is exact, the addend joins before the one rounding), and the same on the fake path."""
    from segquant_amd import workloads as W
    spec = [s for s in W.config_linears(3, M=160) if s.name == "mlp_up"][0]
    g = torch.Generator().manual_seed(17)
    x = (torch.randn(160, spec.K, generator=g)).to(torch.bfloat16).to(DEV)
    sdiv = (torch.rand(spec.K, generator=g) * 2 + 0.25).to(DEV)
    add = (torch.randn(160, spec.N, generator=g) * 0.5).to(torch.bfloat16).to(DEV)
    xs = x / sdiv.to(torch.bfloat16)
    layer, _ = W.build_layer(spec, device=DEV, real_quant=True, x=xs.float().cpu())
    want = layer(xs).float() + add.float()
    got = layer(x, col_div=sdiv, addend=add).float()
    assert (got - want).abs().max().item() <= 2.0 ** -7 * want.abs().max().item()
    fake, _ = W.build_layer(spec, device=DEV, real_quant=False, x=xs.float().cpu())
    x32 = x.float()
    assert torch.allclose(fake(x32, col_div=sdiv, addend=add.float()), fake(x32 / sdiv) + add.float())


def test_reference_named_operators_trace_and_compile():
    """The chunked route calls the reference-named operator through torch.library: opcheck's
    schema / fake-tensor / dispatch checks pass, and a compiled function that calls it gives
    the eager result without a graph break."""
    from segquant_amd import torch_ops  # noqa: F401
    g = torch.Generator().manual_seed(3)
    S, M, N, K = 2, 48, 64, 128
    x = torch.randn(S, M, K, generator=g).to(torch.bfloat16).to(DEV)
    w = torch.randint(-127, 128, (S, N, K), generator=g, dtype=torch.int8).to(DEV)
    sx = (torch.rand(S * M, generator=g) * 20 + 5).to(DEV)
    sw = (torch.rand(S, generator=g) * 50 + 5).to(DEV)
    op = torch.ops.segquant_amd.real_quantized_gemm_scaled
    torch.library.opcheck(op, (x, w, sx, sw, "int8", "int8"),
                          test_utils=("test_schema", "test_faketensor", "test_autograd_registration"))
    torch.library.opcheck(torch.ops.segquant_amd.real_quantized_gemm_dual_scaled, (x, w, sx, sx * 2, sw, "int8", "int8"),
                          test_utils=("test_schema", "test_faketensor"))

    def f(x, w, sx, sw):
        return op(x, w, sx, sw, "int8", "int8").float().sum(0) * 0.5

    want = f(x, w, sx, sw)
    got = torch.compile(f, backend="aot_eager", fullgraph=True)(x, w, sx, sw)
    assert torch.equal(got, want)


def test_unsupported_kernel_type_warns_and_uses_fake_path(capsys):
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    lin = torch.nn.Linear(64, 32)
    layer = SegmentLinear(64, 32, custom_weight_tensor=lin.weight.data, custom_bias_tensor=lin.bias.data,
                          input_quant_type="int4", weight_quant_type="int4",
                          input_quant_args={"real_quant": True}, weight_quant_args={"real_quant": True}, device=DEV)
    assert "Wint4Aint4" in capsys.readouterr().out
    assert layer.optimizer.real_quant is False


@pytest.mark.parametrize("config,M", [(1, 64), (2, 96), (3, 80), (4, 3200), (5, 2100)])
def test_repeated_forwards_reuse_descriptors_and_buffers(config, M):
    """The layer keeps its launch descriptors per token count and, on one stream, its code and
    scale tensors: a third call must give what the first gave, a call on other data what a
    layer that never saw anything else gives, and outputs handed out earlier must stay intact."""
    from segquant_amd import workloads as W
    for spec in W.config_linears(config, M=M)[:2]:
        layer, x = W.build_layer(spec, device=DEV, real_quant=True)
        twin, _ = W.build_layer(spec, device=DEV, real_quant=True, x=x)
        g = torch.Generator().manual_seed(5)
        xa = x.to(spec.x_dtype).to(DEV)
        xb = (x * (torch.rand(x.shape[1], generator=g) + 0.5)).to(spec.x_dtype).to(DEV)
        first = layer(xa)            # builds the descriptors
        first_copy = first.clone()
        second = layer(xb)           # cached descriptors, first cached buffers
        third = layer(xa)            # everything reused
        other_stream = torch.cuda.Stream()
        other_stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(other_stream):
            fourth = layer(xb)       # another stream gets buffers of its own
        torch.cuda.current_stream().wait_stream(other_stream)
        assert torch.equal(first, first_copy) and torch.equal(third, first), spec.name
        assert torch.equal(second, twin(xb)) and torch.equal(fourth, second), spec.name
        q1, g1, _ = layer.optimizer.fused_launches(xa, layer.bias_data, fresh=True)
        q2, g2, _ = layer.optimizer.fused_launches(xb, layer.bias_data, fresh=True)
        assert q1[0] is not q2[0] and g1[1].data_ptr() != g2[1].data_ptr()
        codes1 = q1[1][0] if isinstance(q1[1], tuple) else q1[1]
        codes2 = q2[1][0] if isinstance(q2[1], tuple) else q2[1]
        assert codes1.data_ptr() != codes2.data_ptr()


@pytest.mark.parametrize("config,M", [(1, None), (2, None), (4, 2048), (5, 1024)])
def test_layer_forward_replays_from_a_captured_graph(config, M):
    """The layer's forward recorded into a HIP graph (the quantise and GEMM launches, the expansion
    of int4 weights, the sum of K shares; config 2's fc2 is two K shares that meet inside the launch,
    config 5 at 1024 tokens four shares and parked ranges) and replayed four times, with the input
    rewritten, other eager launches and synchronisations between the replays: every replay must
    equal the eager forward on the data then in the input buffer, bit for bit."""
    from segquant_amd import workloads as W
    for spec in W.config_linears(config, M=M):
        layer, x = W.build_layer(spec, device=DEV, real_quant=True)
        gen = torch.Generator().manual_seed(17)
        variants = [x.to(spec.x_dtype).to(DEV)] + [
            (x * (torch.rand(x.shape[1], generator=gen) + 0.5)).to(spec.x_dtype).to(DEV) for _ in range(3)]
        eager = [layer(v).clone() for v in variants]
        static_in = variants[0].clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # buffers, workspaces and kernel attributes of this stream exist before the capture
            for _ in range(2):
                layer(static_in)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            static_out = layer(static_in)
        for i in (0, 1, 2, 3, 1):
            static_in.copy_(variants[i])
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(static_out, eager[i]), (spec.name, i)
            again = layer(variants[(i + 1) % 4])  # the program's own eager work between replays
            torch.cuda.synchronize()
            assert torch.equal(again, eager[(i + 1) % 4]), (spec.name, i)
        del graph, layer
        torch.cuda.empty_cache()


@pytest.mark.parametrize("fmt", ["int8", "fpe4m3"])
def test_forward_parts_writes_the_concatenation_as_codes(fmt):
    """Config 5's proj_out fed by its two producers (attention output, MLP output before its
    GELU): without activation functions the result is bit for bit what the concatenated tensor
    gives; with the MLP's GELU(tanh) evaluated in the quantise kernel it agrees to the rounding of
    the codes (hardware exp2 / reciprocal against torch's tanhf move a code by one step on a few
    elements)."""
    from segquant_amd import workloads as W
    spec = [s for s in W.config_linears(5, M=192) if s.act == fmt][0]
    layer, x = W.build_layer(spec, device=DEV, real_quant=True)
    k0 = spec.chunksizes[0]
    pre = W.make_input(spec, activated=False).to(spec.x_dtype).to(DEV)
    attn, mlp_pre = pre[:, :k0].contiguous(), pre[:, k0:].contiguous()
    mlp_act = torch.nn.functional.gelu(mlp_pre, approximate="tanh")
    want = layer(torch.cat([attn, mlp_act], dim=1))
    same = layer.forward_parts([attn, mlp_act])
    assert torch.equal(same, want)
    # ... and that is the oracle's closed form of the layer on the concatenated input (codes of each
    # part with its own scales, three ranges, one rounding to bf16), not only the library's own answer
    from _layer_oracle import oracle_layer_output
    ref = oracle_layer_output(layer, spec, _np32(torch.cat([attn, mlp_act], dim=1)))
    got = _np32(same).astype(np.float64)
    bound = 2.0 ** -8 * np.abs(ref) + (1e-3 if fmt == "fpe4m3" else 2e-6) * np.abs(ref).max()
    assert (np.abs(got - ref) <= bound).all()
    fused = layer.forward_parts([attn, mlp_pre], pre_ops=[None, "gelu_tanh"])
    assert fused.shape == want.shape and fused.dtype == want.dtype
    w32, f32 = want.float(), fused.float()
    assert (f32 - w32).abs().max().item() <= 2e-2 * w32.abs().max().item()
    assert ((f32 - w32).abs() > 2.0 ** -7 * w32.abs().max()).float().mean().item() <= 1e-2
    # the fake path takes the same call
    fake, _ = W.build_layer(spec, device=DEV, real_quant=False, x=x)
    a32, m32 = attn.float(), mlp_pre.float()
    assert torch.equal(fake.forward_parts([a32, m32], pre_ops=[None, "gelu_tanh"]),
                       fake(torch.cat([a32, torch.nn.functional.gelu(m32, approximate="tanh")], dim=1)))


def _smooth_layer(opt_type, fmt, seg_mode, chunks, M, K, N, dtype, dynamic, axis, rank=32, seed=3):
    from segquant_amd.layers.SegmentLinear import SegmentLinear
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(N, K, generator=g) * 0.02
    b = torch.randn(N, generator=g) * 0.01
    x = torch.randn(M, K, generator=g) * (torch.rand(K, generator=g) * 3 + 0.3)
    x[:, torch.randperm(K, generator=g)[:max(1, K // 100)]] *= 20.0
    layer = SegmentLinear(K, N, bias=True, seg_mode=seg_mode, chunks=chunks, custom_weight_tensor=w, custom_bias_tensor=b,
                          input_quant_type=fmt, weight_quant_type=fmt,
                          input_quant_args={"real_quant": True, "axis": -1 if (dynamic or axis) else None, "dynamic": dynamic},
                          weight_quant_args={"real_quant": True, "axis": 1 if axis else None}, opt_type=opt_type,
                          opt_kwargs={"alpha": 0.5, **({"low_rank": rank, "precision": "float32"} if opt_type == "svd" else {})},
                          device=DEV)
    xd = x.to(dtype).to(DEV)
    layer.trace(xd)
    layer.smooth()
    layer.calibrate(xd)
    layer.finish_calibrate()
    layer._oracle_dtype = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}[dtype]
    return layer, xd, (w, b, x)


@pytest.mark.parametrize("opt_type", ["smooth", "svd"])
@pytest.mark.parametrize("fmt", ["int8", "fpe4m3"])
@pytest.mark.parametrize("seg_mode,chunks", [("weight", 1), ("input", 2)])
@pytest.mark.parametrize("dtype,dynamic", [(torch.bfloat16, True), (torch.float16, False), (torch.float32, False)])
def test_smooth_and_svd_layers_fused_route_against_the_oracle(opt_type, fmt, seg_mode, chunks, dtype, dynamic):
    """Smoothed (and low-rank-split) layers through the fused route: the division by s in the
    quantise kernel, one range per K segment with its own activation and weight scales, and the
    low-rank product added by the GEMM's epilogue (16-bit inputs) or as an addend (fp32).
    Against the oracle's closed form from the layer's own factors; and the reference's route
    (chunked operator + two batched products) must agree with the fused one."""
    from _layer_oracle import oracle_smooth_layer_output
    M, K, N = 200, 512, 384
    layer, xd, (w, b, x) = _smooth_layer(opt_type, fmt, seg_mode, chunks, M, K, N, dtype, dynamic, axis=True)
    assert layer.optimizer.fused_available()
    out = layer(xd)
    assert out.shape == (M, N) and out.dtype == dtype
    got = _np32(out).astype(np.float64)
    want = oracle_smooth_layer_output(layer, fmt, fmt, _np32(xd))
    scale = np.abs(want).max()
    # bf16 / fp16: T = x (L1 / s) and L2 are rounded to the input's dtype for the matrix cores
    tol = {torch.float32: 2e-5, torch.bfloat16: 1.2e-2, torch.float16: 2e-3}[dtype] + (1e-3 if fmt == "fpe4m3" else 0.0)
    assert np.abs(got - want).max() <= tol * scale, float(np.abs(got - want).max() / scale)
    chunked = layer(xd, chunked=True)
    rec = (chunked.sum(0) if seg_mode == "input" else chunked.movedim(0, -2).reshape(M, -1)) + layer.bias_data
    # (the reference's route computes dynamic scales with torch in the input's dtype, so its codes
    # differ from the fused route's by a step here and there: compare the two as a whole)
    assert ((rec.float() - out.float()).norm() / out.float().norm()).item() <= (3e-2 if fmt == "fpe4m3" else 1e-2)
    # the smoothed, split layer is still the linear it replaces (quantisation error only)
    ref = torch.nn.functional.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    assert ((out.float() - ref).norm() / ref.norm()).item() < 0.05


@pytest.mark.parametrize("opt_type", ["smooth", "svd"])
def test_smooth_and_svd_layers_with_a_fused_activation_function(opt_type):
    """pre_op on a smoothed layer is evaluated inside the quantise kernel (in front of the division by
    s); on an svd layer the low-rank branch multiplies the ACTIVATED input, so the layer evaluates
    the activation first.  Either way the result is the layer's forward on op(x) (svd: bit for bit;
    smooth: to the rounding of the codes, the kernel's exp2 / reciprocal against torch's tanhf), an
    external col_div is refused, and forward_parts falls back to the concatenated forward."""
    M, K, N = 200, 512, 384
    layer, xd, (w, b, x) = _smooth_layer(opt_type, "int8", "input", 2, M, K, N, torch.bfloat16, True, axis=True)
    pre = (torch.randn(M, K, generator=torch.Generator().manual_seed(5)) * 2).to(torch.bfloat16).to(DEV)
    act = torch.nn.functional.gelu(pre, approximate="tanh")
    want = layer(act)
    got = layer(pre, pre_op="gelu_tanh")
    if opt_type == "svd":
        assert torch.equal(got, want)
    else:
        w32, g32 = want.float(), got.float()
        assert (g32 - w32).abs().max().item() <= 2e-2 * w32.abs().max().item()
    with pytest.raises(RuntimeError, match="col_div"):
        layer(act, col_div=torch.ones(K, device=DEV))
    if opt_type == "svd":
        with pytest.raises(RuntimeError, match="low-rank"):
            layer.optimizer.fused_launches(pre, layer.bias_data, pre_op="gelu_tanh")
    parts = [act[:, :K // 2].contiguous(), act[:, K // 2:].contiguous()]
    assert torch.equal(layer.forward_parts(parts), want)


def test_smooth_layer_with_output_segments_takes_the_reference_route():
    """With output segmentation every segment smooths the whole input with its own s, so the layer
    runs the reference's route: S smoothed, quantised copies of the input through the batched
    operator.  Checked against the float linear."""
    M, K, N = 96, 256, 384
    layer, xd, (w, b, x) = _smooth_layer("svd", "int8", "weight", 3, M, K, N, torch.float32, False, axis=True, rank=16)
    assert not layer.optimizer.fused_available() and layer.optimizer.real_quant
    out = layer(xd)
    ref = torch.nn.functional.linear(x.to(DEV), w.to(DEV), b.to(DEV))
    assert out.shape == (M, N) and ((out - ref).norm() / ref.norm()).item() < 0.05


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_zero_tokens_give_an_empty_output(config):
    """An input with no token rows: the layers return (0, N) in the input's dtype on both
    routes without launching anything that reads memory; the next call with rows is unaffected."""
    from segquant_amd import workloads as W
    spec = W.config_linears(config, M=64)[0]
    layer, x = W.build_layer(spec, device=DEV, real_quant=True)
    xin = x.to(spec.x_dtype).to(DEV)
    want = layer(xin).clone()
    out = layer(xin[:0])
    assert out.shape == (0, spec.N) and out.dtype == spec.x_dtype
    if config not in (4, 5):  # (group-wise weight scales and unequal K segments run on the fused route only)
        chunks = layer(xin[:0], chunked=True)
        assert chunks.shape[-2] == 0
    torch.cuda.synchronize()
    assert torch.equal(layer(xin), want)


@pytest.mark.parametrize("config", [1, 2, 3, 4, 5])
def test_leading_batch_dimensions(config):
    """(batch, tokens, features) and (a, b, tokens, features) inputs, as the transformer blocks pass
    them: the same values as the flattened 2-D call, in the input's leading shape, on both routes;
    a non-contiguous view (every second token) too."""
    from segquant_amd import workloads as W
    for spec in W.config_linears(config, M=96)[:2]:
        layer, x = W.build_layer(spec, device=DEV, real_quant=True)
        x2 = x.to(spec.x_dtype).to(DEV)
        want = layer(x2)
        for shape in ((2, 48), (2, 3, 16), (1, 96), (96, 1)):
            out = layer(x2.reshape(*shape, spec.K))
            assert out.shape == (*shape, spec.N) and out.dtype == spec.x_dtype
            assert torch.equal(out.reshape(96, spec.N), want), (spec.name, shape)
        every_second = torch.stack([x2, -x2], dim=1)[:, 0]      # rows 2 K apart in memory
        assert not every_second.is_contiguous()
        assert torch.equal(layer(every_second), want), spec.name
        if config in (1, 2, 3):
            chunks2 = layer(x2, chunked=True)
            chunks3 = layer(x2.reshape(2, 48, spec.K), chunked=True)
            assert torch.equal(chunks3.reshape(chunks2.shape), chunks2), spec.name


@pytest.mark.parametrize("config", [2, 3, 5])
def test_one_layer_serves_every_float_input_dtype(config):
    """The reference's models run in fp16; the benchmark configurations in bf16 and fp32.  One
    calibrated layer takes all three: the output comes back in the input's dtype and differs from
    the fp32 call by that dtype's rounding of input and output only (the codes of an fp16 or bf16
    input are those of the rounded values, so the comparison is against the fp32 call on the
    rounded input)."""
    from segquant_amd import workloads as W
    spec = W.config_linears(config, M=80)[0]
    layer, x = W.build_layer(spec, device=DEV, real_quant=True)
    for dt, ulp in ((torch.float16, 2.0 ** -11), (torch.bfloat16, 2.0 ** -8), (torch.float32, 0.0)):
        xin = x.to(dt).to(DEV)
        out = layer(xin)
        assert out.dtype == dt and out.shape == (80, spec.N)
        ref = layer(xin.float())           # the same rounded values, fp32 in and out
        err = (out.float() - ref).abs().max().item() / ref.abs().max().item()
        assert err <= ulp + 1e-6, (spec.name, dt, err)


@pytest.mark.parametrize("fmt", ["fpe4m3", "int8"])
def test_chained_linears_write_the_next_layers_codes(fmt):
    """Config 2's MLP pair (fc1 -> GELU(tanh) -> fc2 with DualScale) through ``forward_into``: fc1's GEMM
    epilogue writes fc2's two code tensors.  Bit for bit the result of the three launches it
    replaces (fc1's GEMM writing bf16, fc2's quantise kernel with the GELU fused, fc2's GEMM), which
    the other tests pin against the oracle; and pairs the epilogue does not serve (an fp32 input)
    take the two ordinary forwards."""
    import dataclasses
    from segquant_amd import workloads as W
    s1, s2 = W.config_linears(2, M=384)
    s1, s2 = dataclasses.replace(s1, act=fmt, weight=fmt), dataclasses.replace(s2, act=fmt, weight=fmt)
    fc1, x = W.build_layer(s1, device=DEV, real_quant=True)
    xd = x.to(torch.bfloat16).to(DEV)
    # calibrate fc2 on what it will see: gelu(fc1(x))
    h = torch.nn.functional.gelu(fc1(xd), approximate="tanh")
    fc2, _ = W.build_layer(s2, device=DEV, real_quant=True, x=h.float().cpu())
    assert fc1.optimizer.writes_codes(xd) and fc2.optimizer.accepts_codes()
    want = fc2(fc1(xd), pre_op="gelu_tanh")
    got = fc1.forward_into(fc2, xd, pre_op="gelu_tanh")
    assert got.shape == want.shape and got.dtype == want.dtype and torch.equal(got, want)
    ref = torch.nn.functional.linear(h.float(), W.make_weight(s2).to(DEV), W.make_bias(s2).to(DEV))
    assert ((got.float() - ref).norm() / ref.norm()).item() < (0.08 if fmt == "fpe4m3" else 0.03)
    # the launches: one quantise and one GEMM for fc1, one GEMM for fc2
    from segquant_amd import ops
    with ops.record_launches() as log:
        fc1.forward_into(fc2, xd, pre_op="gelu_tanh")
        torch.cuda.synchronize()
    assert [k for k, *_ in log] == ["quantize", "gemm", "gemm"]
    x32 = x.to(DEV)
    assert not fc1.optimizer.writes_codes(x32)
    assert torch.equal(fc1.forward_into(fc2, x32, pre_op="gelu_tanh"), fc2(fc1(x32), pre_op="gelu_tanh"))


def test_launch_cache_is_bounded_over_token_counts():
    """A layer fed with many different token counts keeps launch descriptors and buffers for the
    last few only, and still computes every one of them right (bit-equal to a fresh layer's)."""
    from segquant_amd import workloads as W
    from segquant_amd.optimum import optimizer as opt_mod
    spec = W.config_linears(3, M=64)[0]
    layer, x = W.build_layer(spec, device=DEV, real_quant=True)
    fresh, _ = W.build_layer(spec, device=DEV, real_quant=True)
    xs = x.to(spec.x_dtype).to(DEV)
    for m in list(range(16, 64, 4)) + [16, 20]:
        got = layer(xs[:m])
        assert torch.equal(got, fresh.optimizer.forward_fused(xs[:m], fresh.bias_data, addend=None).view_as(got))
        assert len(layer.optimizer._plan["launches"]) <= opt_mod._MAX_CACHED_TOKEN_COUNTS
