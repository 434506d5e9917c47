"""Synthetic workloads: the five benchmark configurations as lists of linears.

Inputs are drawn on the CPU in fp32 from seeded generators so that every run
and every machine sees the same tensors:
``manual_seed(20250 + 10 * config + tensor_index)``.

* activations ~ N(0, 1); 1 % of the channels (the first ceil(0.01 K) of a seeded
  permutation) are outliers: multiplied by 20 or 30, or replaced by Student-t
  (nu = 3) samples;
* a linear that follows an activation function gets ``gelu_tanh`` of such a
  tensor (narrow negative side -> DualScale);
* weights ~ N(0, 0.02^2), bias ~ N(0, 0.01^2).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field
from typing import List, Optional

import torch


@dataclass
class LinearSpec:
    name: str
    config: int
    M: int
    K: int
    N: int
    act: str = "int8"            # int8 | fpe4m3
    weight: str = "int8"         # int8 | fpe4m3 | int4
    seg_mode: str = "weight"
    chunksizes: Optional[List[int]] = None   # None = unsegmented
    act_axis: Optional[int] = None           # None per tensor, -1 per token
    dynamic: bool = False
    weight_axis: Optional[int] = None        # None per tensor / per segment, 1 per channel
    weight_group: Optional[int] = None       # with weight_axis 1: one scale per run of this many input channels
    dual_segments: List[int] = field(default_factory=list)  # K segments (or [0]) that use DualScale
    outlier: str = "x20"                     # x20 | x30 | student_t
    gelu_segments: List[int] = field(default_factory=list)  # segments passed through gelu_tanh
    x_dtype: torch.dtype = torch.bfloat16
    tensor_index: int = 0

    @property
    def ops(self) -> int:
        return 2 * self.M * self.N * self.K

    @property
    def kernel_type(self) -> str:
        return f"W{self.weight}A{self.act}"


def _gen(spec: LinearSpec, idx: int) -> torch.Generator:
    return torch.Generator().manual_seed(20250 + 10 * spec.config + spec.tensor_index * 3 + idx)


def make_input(spec: LinearSpec, M: Optional[int] = None, activated: bool = True) -> torch.Tensor:
    """fp32 (M, K) activation tensor of ``spec`` (optionally only the first M rows' worth).
    ``activated=False`` leaves out the ``gelu_tanh`` of the segments that have one: what their
    producer holds before its activation function."""
    M = spec.M if M is None else M
    g = _gen(spec, 0)
    K = spec.K
    x = torch.randn(M, K, generator=g)
    n_out = math.ceil(0.01 * K)
    chan = torch.randperm(K, generator=g)[:n_out]
    if spec.outlier == "student_t":
        z = torch.randn(M, n_out, generator=g)
        chi = torch.randn(3, M, n_out, generator=g).pow(2).sum(0) / 3.0
        x[:, chan] = z / chi.sqrt()
    else:
        x[:, chan] *= 30.0 if spec.outlier == "x30" else 20.0
    if spec.gelu_segments and activated:
        bounds = segment_bounds(spec)
        for s in spec.gelu_segments:
            a, b = bounds[s], bounds[s + 1]
            x[:, a:b] = torch.nn.functional.gelu(x[:, a:b], approximate="tanh")
    return x


def make_weight(spec: LinearSpec) -> torch.Tensor:
    return torch.randn(spec.N, spec.K, generator=_gen(spec, 1)) * 0.02


def make_bias(spec: LinearSpec) -> torch.Tensor:
    return torch.randn(spec.N, generator=_gen(spec, 2)) * 0.01


def segment_bounds(spec: LinearSpec) -> List[int]:
    """K boundaries for input segmentation, [0, K] otherwise."""
    if spec.seg_mode == "input" and spec.chunksizes:
        b = [0]
        for c in spec.chunksizes:
            b.append(b[-1] + c)
        return b
    return [0, spec.K]


def config_linears(config: int, M: Optional[int] = None) -> List[LinearSpec]:
    """The linears of benchmark configuration 1..5 (the shapes the headline metric is quoted on and its parity cases)."""
    if config == 1:
        return [LinearSpec("adaLN", 1, M or 256, 1536, 9216, chunksizes=[1536] * 6, x_dtype=torch.float32,
                           outlier="x20")]
    if config == 2:
        m = M or 4096
        return [
            LinearSpec("fc1", 2, m, 1536, 6144, act="fpe4m3", weight="fpe4m3", outlier="x30", tensor_index=0),
            LinearSpec("fc2", 2, m, 6144, 1536, act="fpe4m3", weight="fpe4m3", outlier="x30", dual_segments=[0],
                       gelu_segments=[0], tensor_index=1),
        ]
    if config == 3:
        m = M or 4608
        kw = dict(act_axis=-1, dynamic=True, outlier="student_t")
        return [
            LinearSpec("qkv", 3, m, 3072, 9216, chunksizes=[3072] * 3, tensor_index=0, **kw),
            LinearSpec("mlp_up", 3, m, 3072, 12288, weight_axis=1, tensor_index=1, **kw),
            LinearSpec("mlp_down", 3, m, 12288, 3072, weight_axis=1, tensor_index=2, **kw),
        ]
    if config == 4:
        m = M or 8192
        kw = dict(weight="int4", act_axis=-1, dynamic=True, weight_axis=1, weight_group=128, outlier="x20")
        return [
            LinearSpec("geglu_proj", 4, m, 1280, 10240, chunksizes=[5120] * 2, tensor_index=0, **kw),
            LinearSpec("ff_out", 4, m, 5120, 1280, tensor_index=1, **kw),
            LinearSpec("geglu_proj_small_m", 4, 2048 if M is None else M, 1280, 10240, chunksizes=[5120] * 2,
                       tensor_index=2, **kw),
        ]
    if config == 5:
        out = []
        ms = [1024, 4608, 9216] if M is None else [M]
        for i, m in enumerate(ms):
            for j, fmt in enumerate(("int8", "fpe4m3")):
                out.append(LinearSpec(f"proj_out_{fmt}_m{m}", 5, m, 15360, 3072, act=fmt, weight=fmt,
                                      seg_mode="input", chunksizes=[3072, 12288], dual_segments=[1],
                                      gelu_segments=[1], outlier="x20", tensor_index=0))
        return out
    raise ValueError(f"no configuration {config}")


def build_layer(spec: LinearSpec, device="cuda:0", real_quant=True, x: Optional[torch.Tensor] = None, opt_kwargs=None):
    """A calibrated ``SegmentLinear`` for ``spec`` plus the activation tensor it
    was calibrated on (fp32, CPU)."""
    from .layers.SegmentLinear import SegmentLinear

    x = make_input(spec) if x is None else x
    w = make_weight(spec)
    b = make_bias(spec)
    chunks = len(spec.chunksizes) if spec.chunksizes else 1
    n_in = chunks if spec.seg_mode == "input" else 1
    dual = [i in spec.dual_segments for i in range(n_in)] if n_in > 1 else bool(spec.dual_segments)
    layer = SegmentLinear(
        spec.K, spec.N, bias=True, seg_mode=spec.seg_mode, chunks=chunks, chunksizes=spec.chunksizes,
        custom_weight_tensor=w, custom_bias_tensor=b, input_quant_type=spec.act, weight_quant_type=spec.weight,
        input_quant_args={"real_quant": real_quant, "dual_scale": dual, "axis": spec.act_axis,
                          "dynamic": spec.dynamic},
        weight_quant_args={"real_quant": real_quant, "axis": spec.weight_axis,
                           **({"group_size": spec.weight_group} if spec.weight_group else {})}, opt_kwargs=opt_kwargs,
        device=device)
    layer.calibrate(x.to(device))
    layer.finish_calibrate()
    return layer, x
