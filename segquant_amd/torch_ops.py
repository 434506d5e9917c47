"""``torch.library`` registration of the two reference-named operators, so that a
model whose linears call them can be traced (``torch.compile``, ``make_fx``,
fake tensors) without the tracer looking inside.

The reference binds its operators with pybind11 as plain functions
(segquant/src/real_quant/seg_utils.h:82-161), which a tracer cannot see
through and breaks the graph at.  Here they are custom operators

    torch.ops.segquant_amd.real_quantized_gemm_scaled(inputs, weights, scale_x, scale_w, fmt_a, fmt_w)
    torch.ops.segquant_amd.real_quantized_gemm_dual_scaled(inputs, weights, pos_scale_x, neg_scale_x, scale_w,
                                                           fmt_a, fmt_w)

with the tensor contract of ``segquant_amd.ops`` and a shape-only implementation
for fake / meta tensors.  ``RealQuantExt`` (utils/extension.py) routes the
``<prefix>_real_quantized_gemm_*`` functions of ``ext_dict`` through them.
"""
from __future__ import annotations

import torch

from . import ops

_NS = "segquant_amd"


def _out_shape(inputs: torch.Tensor, weights: torch.Tensor, fmt_w: str):
    k = inputs.shape[-1]
    n = weights.shape[1] * 2 // k if fmt_w == ops.FMT_INT4 else weights.shape[1]
    return (*inputs.shape[:-1], n)


@torch.library.custom_op(f"{_NS}::real_quantized_gemm_scaled", mutates_args=(), device_types="cuda")
def real_quantized_gemm_scaled(inputs: torch.Tensor, weights: torch.Tensor, scale_x: torch.Tensor,
                               scale_w: torch.Tensor, fmt_a: str, fmt_w: str) -> torch.Tensor:
    return ops.real_quantized_gemm_scaled(fmt_a, fmt_w, inputs, weights, scale_x, scale_w)


@real_quantized_gemm_scaled.register_fake
def _(inputs, weights, scale_x, scale_w, fmt_a, fmt_w):
    return inputs.new_empty(_out_shape(inputs, weights, fmt_w))


@torch.library.custom_op(f"{_NS}::real_quantized_gemm_dual_scaled", mutates_args=(), device_types="cuda")
def real_quantized_gemm_dual_scaled(inputs: torch.Tensor, weights: torch.Tensor, pos_scale_x: torch.Tensor,
                                    neg_scale_x: torch.Tensor, scale_w: torch.Tensor, fmt_a: str,
                                    fmt_w: str) -> torch.Tensor:
    return ops.real_quantized_gemm_dual_scaled(fmt_a, fmt_w, inputs, weights, pos_scale_x, neg_scale_x, scale_w)


@real_quantized_gemm_dual_scaled.register_fake
def _(inputs, weights, pos_scale_x, neg_scale_x, scale_w, fmt_a, fmt_w):
    return inputs.new_empty(_out_shape(inputs, weights, fmt_w))
