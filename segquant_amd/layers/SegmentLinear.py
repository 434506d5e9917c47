"""Segmented linear module: the drop-in counterpart of the reference's
``SegmentLinear`` (segquant/layers/SegmentLinear.py:11-269).

Same constructor arguments and defaults, same ``forward(x, chunked=False)``
contract, same calibration life cycle (``calibrate`` -> ``finish_calibrate``).
Differences, all deliberate:

* With ``real_quant`` the un-chunked forward takes the fused route (one
  quantise launch + one GEMM launch, bias in the epilogue) instead of
  replicating the input per segment and recombining in Python.
* ``real_quant`` with a kernel type this build has no GEMM for falls back to
  fake quantisation with a warning, as the reference does (:105-113); but if
  the type IS supported and the library or GPU is missing, construction raises
  instead of silently computing something else.
* Unequal chunk sizes are accepted (the reference refuses them, :80-82): the
  fused route and the fake path handle them; ``chunked=True`` and
  ``segment_forward`` return stacked per-segment tensors and still need equal
  sizes.
* The fake path does not write into the caller's input.
"""
from __future__ import annotations

from typing import Literal

import torch
import torch.nn as nn

from ..calibrator.calibrator import CalibratorRegistry
from ..config import Calibrate, DType, Optimum
from ..optimum.optimizer import OptimizerRegistry
from ..optimum import smooth as _smooth  # noqa: F401  (registers the "smooth" and "svd" optimisers)
from ..utils.extension import _KERNELS, kernels_available
from . import ext_dict
from .segment_tensor_manager import InputSegmentTensorManager, WeightSegmentTensorManager


class SegmentLinear(nn.Module):
    def __init__(self, in_features, out_features, bias=True, seg_mode: Literal["input", "weight"] = "weight",
                 chunks=1, chunksizes=None, custom_weight_tensor=None, custom_bias_tensor=None,
                 input_quant_type=None, weight_quant_type=None, input_quant_args=None, weight_quant_args=None,
                 opt_type: Literal["default", "smooth", "svd"] = "default", opt_kwargs=None,
                 calib_type: Literal["amax", "gptq"] = "amax", calib_kwargs=None, device="cuda:0"):
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        input_quant_args = dict(input_quant_args or {})
        weight_quant_args = dict(weight_quant_args or {})
        opt_kwargs = dict(opt_kwargs or {})
        calib_kwargs = dict(calib_kwargs or {})

        if custom_weight_tensor is not None:
            if tuple(custom_weight_tensor.shape) != (out_features, in_features):
                raise AssertionError(f"Mismatched custom_weight_tensor shape! Expected ({out_features}, {in_features}), "
                                     f"but got {tuple(custom_weight_tensor.shape)}.")
            self.origin_device = custom_weight_tensor.device
            weight = custom_weight_tensor.detach().to(device).clone()
        else:
            self.origin_device = torch.device("cpu")
            weight = torch.randn(out_features, in_features)
        self.bias = bias
        self.bias_data = None
        if bias:
            self.bias_data = (custom_bias_tensor.detach().to(device).clone() if custom_bias_tensor is not None
                              else torch.zeros(out_features, device=device))

        if seg_mode not in ("input", "weight"):
            raise ValueError("seg_mode not found")
        target = in_features if seg_mode == "input" else out_features
        self.seg_mode = seg_mode
        self.chunks = chunks
        if chunksizes is None:
            base, rem = divmod(target, chunks)
            chunksizes = [base + (1 if i < rem else 0) for i in range(chunks)]
        else:
            assert len(chunksizes) == chunks and sum(chunksizes) == target
        self.chunksizes = list(chunksizes)
        self.equal_chunks = len(set(self.chunksizes)) == 1

        real_quant = bool(input_quant_args.get("real_quant", False)) if input_quant_type is not None else False
        # dual_scale: a bool as in the reference, or one bool per input segment
        dual_arg = input_quant_args.get("dual_scale", False) if input_quant_type is not None else False
        n_in = chunks if seg_mode == "input" else 1
        dual_segments = [bool(d) for d in dual_arg] if isinstance(dual_arg, (list, tuple)) else [bool(dual_arg)] * n_in
        if len(dual_segments) != n_in:
            raise ValueError(f"dual_scale lists one flag per input segment ({n_in}), got {len(dual_segments)}")
        dual_scale = any(dual_segments)
        if weight_quant_type is not None:
            if "real_quant" in weight_quant_args:
                assert real_quant == weight_quant_args["real_quant"], \
                    f"Mismatch: real_quant={real_quant}, weight_quant_args['real_quant']={weight_quant_args['real_quant']}"
            if "dual_scale" in weight_quant_args:
                raise ValueError("Dual scale is not supported for weight quantizer in DefaultSegmentLinear.")

        kernel_type = f"W{weight_quant_type}A{input_quant_type}"
        if real_quant:
            entry = ext_dict.get(kernel_type)
            if kernel_type in _KERNELS and not kernels_available():
                raise RuntimeError(f"real_quant needs libsegq.so and a GPU for [{kernel_type}]; neither a CPU path "
                                   "nor a silent fallback exists")
            if entry is None:
                print(f"[Warning] Seglinear need [{kernel_type}] but not found")
                real_quant = False
            elif entry["gemm_scaled_fn"] is None or entry["gemm_dual_scaled_fn"] is None:
                print(f"[Warning] Seglinear need [{kernel_type}] but function is None")
                real_quant = False
        input_quant_args["real_quant"] = real_quant
        weight_quant_args["real_quant"] = real_quant

        self.opt_type = opt_type
        if opt_type not in ("default", "smooth", "svd"):
            raise ValueError(f"Optimizer '{opt_type}' not found in registry.")
        # calibrators per optimiser, as the reference lays them out (SegmentLinear.py:118-128): the
        # default optimiser has one per segment on the segmented side and one on the other, the
        # smoothing ones a pair per chunk
        if opt_type == "default":
            n_w = 1 if seg_mode == "input" else chunks
        else:
            n_w = n_in = chunks
            if len(dual_segments) != chunks:
                dual_segments = dual_segments * chunks

        weight_manager = WeightSegmentTensorManager(weight, seg_mode=seg_mode, segments=chunks,
                                                    segment_size=self.chunksizes[0])
        self.optimizer = OptimizerRegistry.create(
            opt_type, seg_mode=seg_mode, chunks=chunks, chunksizes=self.chunksizes, weight_manager=weight_manager,
            input_calibrators=[CalibratorRegistry.create("amax", data_type="input", quant_type=input_quant_type,
                                                         quant_args={**input_quant_args, "dual_scale": d},
                                                         **calib_kwargs)
                               for d in dual_segments],
            weight_calibrators=[CalibratorRegistry.create(calib_type, data_type="weight", quant_type=weight_quant_type,
                                                          quant_args=weight_quant_args, **calib_kwargs)
                                for _ in range(n_w)],
            real_quant=real_quant, dual_scale=dual_scale, kernel_type=kernel_type, dual_segments=dual_segments,
            **opt_kwargs)

    def _manager(self, x):
        return InputSegmentTensorManager(x, seg_mode=self.seg_mode, segments=self.chunks,
                                         segment_size=self.chunksizes[0])

    def __repr__(self):
        return (f"SegmentLinear(\n  in_features={self.in_features}, out_features={self.out_features}, "
                f"seg_mode={self.seg_mode},\n  chunks={self.chunks}, chunksize={self.chunksizes},\n"
                f"  opt={self.optimizer!r}\n)")

    def trace(self, input_data):
        """Smoothing optimisers only: record the activation maxima of a calibration batch."""
        self.optimizer.trace(self._manager(input_data))

    def smooth(self):
        """Smoothing optimisers only: fix the per-channel factors (and the low-rank split)."""
        self.optimizer.smooth()

    def calibrate(self, input_data):
        self.optimizer.calibrate(self._manager(input_data))

    def finish_calibrate(self):
        self.optimizer.finish_calibrate()

    def segment_forward(self, x, weight):
        """Unquantised per-segment product, used when searching."""
        xs = self._manager(x).iter_view()
        ws = WeightSegmentTensorManager(weight, seg_mode=self.seg_mode, segments=self.chunks,
                                        segment_size=self.chunksizes[0]).iter_view()
        return xs @ ws.unsqueeze(1).transpose(-1, -2)

    def to(self, device):
        device = torch.device(device) if isinstance(device, str) else device
        if device.type == "cuda":
            self.to_cuda()
        elif device.type == "cpu":
            self.to_cpu()
        else:
            raise ValueError(f"Unsupported device type: {device.type}")
        return self

    def to_cpu(self):
        self.optimizer.to_cpu()
        if self.bias_data is not None:
            self.bias_data = self.bias_data.to("cpu")

    def to_cuda(self):
        self.optimizer.to_cuda(self.origin_device)
        if self.bias_data is not None:
            self.bias_data = self.bias_data.to(self.origin_device)

    @staticmethod
    def _activated(x, pre_op, gate):
        """op(x), or x * op(gate), with torch operators (the routes without the fused kernel)."""
        import torch.nn.functional as F
        fn = {"gelu_tanh": lambda t: F.gelu(t, approximate="tanh"), "gelu": F.gelu, "silu": F.silu}[pre_op]
        return fn(x) if gate is None else x * fn(gate)

    def forward(self, x, chunked=False, pre_op=None, gate=None, col_div=None, addend=None):
        """``pre_op`` ("gelu_tanh", "gelu", "silu") and ``gate`` are not in the reference: they
        hand the activation function of the module in front (x -> op(x), or x * op(gate) for
        GEGLU / SwiGLU, backend/torch/layers/activations.py:52-57, :77-80, :110-121) to this
        layer, whose quantise kernel evaluates it on the fly instead of reading back a stored
        activation tensor.  The layer must have been calibrated on the activated input.
        ``col_div`` (per input channel, applied after the activation) and ``addend`` (added to
        the output) are the hooks for the reference's SmoothQuant division and SVD low-rank
        branch (segquant/optimum/optimizer.py:467-470, :731-740), fused into the same kernels."""
        opt = self.optimizer
        if pre_op is not None and getattr(opt, "l1s", None) is not None:
            # a low-rank branch multiplies the layer's input itself: evaluate the activation first
            x, pre_op, gate = self._activated(x, pre_op, gate), None, None
        if col_div is not None and getattr(opt, "s", None) is not None:
            raise RuntimeError("a smoothed layer divides by its own factors: an external col_div is not combined with them")
        if not chunked and opt.fused_available():
            return opt.forward_fused(x, self.bias_data if self.bias else None, pre_op=pre_op, gate=gate,
                                     col_div=col_div, addend=addend)
        if pre_op is not None:
            x = self._activated(x, pre_op, gate)
        if col_div is not None:
            x = x / col_div.to(x.dtype)
        if addend is not None:
            return self.forward(x, chunked=chunked) + addend
        if not chunked and not self.equal_chunks:
            res = opt.forward_fake(x)
            return res + self.bias_data if self.bias else res
        chunks = opt.forward(self._manager(x))
        if chunked:
            return chunks
        if self.seg_mode == "weight":  # (S, ..., n) -> (..., S*n)
            res = chunks.movedim(0, -2).reshape(*chunks.shape[1:-1], -1)
        else:  # (S, ..., out) -> (..., out)
            res = chunks.sum(dim=0)
        return res + self.bias_data if self.bias else res


    def forward_into(self, nxt: "SegmentLinear", x, pre_op=None):
        """``nxt(op(self(x)))`` for two chained linears (an MLP's fc1 -> activation -> fc2) with the
        activation codes of ``nxt`` written by this layer's GEMM epilogue: the epilogue adds the
        bias, rounds to the layer dtype, applies ``pre_op`` ("gelu_tanh" | "gelu" | "silu" | None),
        rounds again, and encodes with the static activation scale(s) of ``nxt`` (two code tensors
        for DualScale), bit for bit what ``nxt``'s quantise kernel would have made of the stored
        tensor.  Neither this layer's float output is written nor a quantise launch reads it back.
        Not in the reference, which runs the activation as a torch operator on the full-size tensor
        and quantises it in a launch of its own (backend/torch/layers/activations.py:52-57 in front
        of segquant/src/real_quant/real_gemm.cu:700-705).  Layers the epilogue does not serve
        (dynamic or per-token scales in ``nxt``, several K ranges, smoothing, int4 weights here,
        fp32 inputs) take the two ordinary forwards."""
        opt, nopt = self.optimizer, nxt.optimizer
        if nxt.in_features != self.out_features:
            raise RuntimeError(f"forward_into: {self.out_features} outputs feed a layer with {nxt.in_features} inputs")
        if getattr(opt, "writes_codes", None) and opt.writes_codes(x) and getattr(nopt, "accepts_codes", None) and nopt.accepts_codes():
            spec = nopt.code_spec(x.device, pre_op)
            q, g, ws = opt.fused_launches(x, self.bias_data if self.bias else None, out_codes=spec)
            if ops_mod().recording_launches():
                ops_mod().quantize_launch(q)
                codes = ops_mod().gemm_launch(g, ws)
            else:
                codes = ops_mod().linear(q, g, ws)
            return nopt.forward_codes(codes, x.shape[:-1], x.dtype, nxt.bias_data if nxt.bias else None)
        return nxt(self(x), pre_op=pre_op)

    def forward_parts(self, parts, pre_ops=None):
        """Forward of an input-segmented layer from the tensors that would have been concatenated
        into its input (one per segment), each optionally still in front of its producer's
        activation function (``pre_ops[s]`` in "gelu_tanh" | "gelu" | "silu" | None).  Not in the
        reference, which runs ``torch.cat([...])`` (and the activation) before the linear
        (backend/torch/modules/transformer_flux.py:91-101): here every part is quantised
        straight into its column range of the code tensor, so neither the activated tensor
        nor the concatenation is written to memory.  The layer must have been calibrated on
        the concatenated, activated input."""
        opt = self.optimizer
        pre_ops = list(pre_ops) if pre_ops is not None else [None] * len(parts)
        if (self.seg_mode == "input" and opt.fused_available() and getattr(opt, "supports_parts", True)
                and getattr(opt.weight_calibrators[0], "group_size", None) is None):
            return opt.forward_parts(parts, self.bias_data if self.bias else None, pre_ops)
        acted = [p if op is None else self._activated(p, op, None) for p, op in zip(parts, pre_ops)]
        return self.forward(torch.cat(acted, dim=-1))


def ops_mod():
    from .. import ops
    return ops


def create_segment_linear(input_dtype: DType, weight_dtype: DType, opt: Optimum, calib: Calibrate, in_features,
                          out_features, opt_kwargs, calib_kwargs, input_quant_args, weight_quant_args, **kwargs):
    return SegmentLinear(in_features, out_features, input_quant_type=input_dtype.value,
                         weight_quant_type=weight_dtype.value, opt_type=opt.value, calib_type=calib.value,
                         opt_kwargs=opt_kwargs, calib_kwargs=calib_kwargs, input_quant_args=input_quant_args,
                         weight_quant_args=weight_quant_args, **kwargs)
