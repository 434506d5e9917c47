"""The reference's CPU-runnable fake-quant linear, restated with torch so that
it uses the host's cores.  TEST / BASELINE INFRASTRUCTURE ONLY: the bench times
it as ``cpu_baseline`` and a test checks it against the numpy oracle; the
shipped package never imports it.

Steps, as in the reference: fp32 quantise->de-quantise of the activations
(segquant/quantizers/quantizer.py:250-281, :484-528), ``x_hat @ w_hat^T`` with
weights that were fake-quantised once and are stored de-quantised
(segquant/optimum/optimizer.py:119-123, segquant/layers/segment_tensor_manager.py:83-94),
segment recombination and bias (segquant/layers/SegmentLinear.py:233-241).
"""
from __future__ import annotations

import torch

EPS = 1.0 / (1 << 24)


def _e4m3(v: torch.Tensor) -> torch.Tensor:
    return torch.clamp(v, -448.0, 448.0).to(torch.float8_e4m3fn).float()


def fake_quant(x: torch.Tensor, fmt: str, scale, neg_scale=None) -> torch.Tensor:
    """Quantise->de-quantise in fp32.  ``scale`` broadcasts against ``x``;
    ``neg_scale`` switches DualScale on."""
    if fmt == "fpe4m3":
        if neg_scale is None:
            out = _e4m3(x * scale) / scale
        else:
            pos = x >= 0
            out = torch.where(pos, _e4m3(x * scale) / scale, _e4m3(x * neg_scale) / neg_scale)
        return out.masked_fill(x.abs() < EPS, 0.0)
    bits = 4 if fmt == "int4" else 8
    qmin, qmax = -(2 ** (bits - 1)), 2 ** (bits - 1) - 1
    if neg_scale is None:
        return torch.clamp(torch.round(x * scale), qmin, qmax) / scale
    pos = x >= 0
    q = torch.where(pos, torch.clamp(torch.round(x * scale), 0, qmax), torch.clamp(torch.round(x * neg_scale), qmin, 0))
    return torch.where(pos, q / scale, q / neg_scale)


def scale_of(amax: torch.Tensor, fmt: str, negative_side: bool = False) -> torch.Tensor:
    lim = {"int8": 128.0 if negative_side else 127.0, "int4": 8.0 if negative_side else 7.0, "fpe4m3": 448.0}[fmt]
    return lim / amax.clamp(min=EPS)


def fake_linear(x: torch.Tensor, w_hat: torch.Tensor, bias, fmt: str, bounds, dual_segments, per_token: bool):
    """One forward of the fake-quant segmented linear on fp32 CPU tensors with
    dynamic scales: per token (``per_token``) or per tensor, per K segment."""
    parts = []
    for s in range(len(bounds) - 1):
        xs = x[:, bounds[s]:bounds[s + 1]]
        dims = dict(dim=-1, keepdim=True) if per_token else {}
        if dual_segments[s]:
            zero = torch.zeros_like(xs)
            pa = torch.where(xs > 0, xs, zero).amax(**dims)
            na = torch.where(xs < 0, -xs, zero).amax(**dims)
            parts.append(fake_quant(xs, fmt, scale_of(pa, fmt), scale_of(na, fmt, True)))
        else:
            parts.append(fake_quant(xs, fmt, scale_of(xs.abs().amax(**dims), fmt)))
    y = torch.cat(parts, dim=-1) @ w_hat.T
    return y + bias if bias is not None else y
