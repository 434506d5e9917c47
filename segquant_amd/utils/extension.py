"""Loaders of the real-quantised kernels, shaped like the reference's.

The reference JIT-builds one pybind module per flavour and returns
``(ext, prefixes)`` (segquant/utils/extension.py:85-213); ``ext`` carries
``<prefix>_real_quantized_gemm_scaled``, ``<prefix>_real_quantized_gemm_dual_scaled``,
``real_quantized_quantize_weights`` and ``create_quantized_weights``.  Here the
functions are thin closures over :mod:`segquant_amd.ops`, i.e. over the C ABI of
the prebuilt ``libsegq.so``; nothing is compiled at import time.

When the library or a GPU is missing, a loader returns ``(None, prefixes)``
(``required=False``) or raises ``RuntimeError`` (``required=True``).  The
reference dereferences ``None`` in that case (segquant/utils/extension.py:113);
that defect is not reproduced.
"""
from __future__ import annotations

import os

import torch

from .. import _lib as L
from .. import ops

supported_type = [
    "Wint8Aint8",
    "Wint4Aint8",
    "Wint4Aint4",
    "Wint8Afp16",
    "Wfpe4m3Afpe4m3",
    "Wfp16Afp16",
]

# kernel types this build has MFMA kernels for: prefix -> (activation, weight)
_KERNELS = {
    "Wint8Aint8": (ops.FMT_INT8, ops.FMT_INT8),
    "Wfpe4m3Afpe4m3": (ops.FMT_E4M3, ops.FMT_E4M3),
    "Wint4Aint8": (ops.FMT_INT8, ops.FMT_INT4),
}

_loaded_extensions = {}


def kernels_available() -> bool:
    """True when libsegq.so is built and a GPU is visible."""
    return os.path.exists(L.LIB_PATH) and torch.cuda.is_available()


class RealQuantExt:
    """The object a loader returns; attribute names follow the reference's pybind modules."""

    def __init__(self, name: str, prefixes, weight_fmt):
        self.name = name
        self.weight_fmt = weight_fmt
        for p in prefixes:
            if p not in _KERNELS:
                continue
            fa, fw = _KERNELS[p]
            setattr(self, f"{p}_real_quantized_gemm_scaled", self._scaled(fa, fw))
            setattr(self, f"{p}_real_quantized_gemm_dual_scaled", self._dual(fa, fw))

    @staticmethod
    def _scaled(fa, fw):
        def fn(inputs, weights, scale_x, scale_w):
            from .. import torch_ops
            return torch_ops.real_quantized_gemm_scaled(inputs, weights, scale_x, scale_w, fa, fw)
        return fn

    @staticmethod
    def _dual(fa, fw):
        def fn(inputs, weights, pos_scale_x, neg_scale_x, scale_w):
            from .. import torch_ops
            return torch_ops.real_quantized_gemm_dual_scaled(inputs, weights, pos_scale_x, neg_scale_x, scale_w, fa, fw)
        return fn

    def create_quantized_weights(self, x: torch.Tensor) -> torch.Tensor:
        """Empty code tensor for weights ``x``: same shape (int8 / e4m3 bytes) or
        a flat ``ceil(numel/2)`` byte vector for int4 (segquant/utils/extension.py:110-111,
        :138-139, :166-169)."""
        if self.weight_fmt is None:
            raise RuntimeError(f"{self.name} has no single weight format")
        if self.weight_fmt == ops.FMT_INT4:
            return torch.empty((x.numel() + 1) // 2, dtype=torch.uint8, device=x.device)
        return torch.empty_like(x, dtype=ops.code_dtype(self.weight_fmt))

    def real_quantized_quantize_weights(self, weights, outputs, scale_w):
        if self.weight_fmt is None:
            raise RuntimeError(f"{self.name} has no single weight format")
        ops.real_quantized_quantize_weights(self.weight_fmt, weights, outputs, scale_w)

    def quantize_weights_groups(self, weights, scales, group):
        """Codes for group-wise scales ((k / group, n) float32); not in the reference."""
        if self.weight_fmt is None:
            raise RuntimeError(f"{self.name} has no single weight format")
        return ops.quantize_weights_groups(self.weight_fmt, weights, scales, group)


def _load(name, prefixes, weight_fmt, verbose, required):
    if name in _loaded_extensions:
        return _loaded_extensions[name], prefixes
    if not kernels_available():
        msg = (f"{name}: libsegq.so missing at {L.LIB_PATH}" if not os.path.exists(L.LIB_PATH)
               else f"{name}: no GPU visible")
        if verbose:
            print(f"[ERROR] {msg}")
        if required:
            raise RuntimeError(f"Required extension '{name}' failed to load: {msg}")
        return None, prefixes
    L.lib()
    ext = RealQuantExt(name, prefixes, weight_fmt)
    _loaded_extensions[name] = ext
    if verbose:
        print(f"[INFO] Successfully loaded extension: {name}")
    return ext, prefixes


def load_real_quant_fp8_ext(verbose=False, required=False):
    return _load("segquant_real_quant_fp8", ("Wfpe4m3Afpe4m3",), ops.FMT_E4M3, verbose, required)


def load_real_quant_int8_ext(verbose=False, required=False):
    return _load("segquant_real_quant_int8", ("Wint8Aint8",), ops.FMT_INT8, verbose, required)


def load_real_quant_int4_ext(verbose=False, required=False):
    """Int4 weight codes.  The W4A4 GEMM of the reference has no counterpart
    here, so the returned object has no ``Wint4Aint4_*`` functions and a layer
    asking for that type takes the reference's warn-and-fake-quantise route."""
    return _load("segquant_real_quant_int4", ("Wint4Aint4",), ops.FMT_INT4, verbose, required)


def load_real_quant_mix_ext(verbose=False, required=False):
    return _load("segquant_real_quant_mix", tuple(supported_type), None, verbose, required)


class FakeQuantFp8Ext:
    """``fake_e4m3fy``: float -> e4m3 -> float (segquant/src/fake_quant/quantizer_fp8.cpp:25-39).
    GPU tensors go through the HIP kernel; CPU tensors through torch's own
    float8 cast on saturated input, as the reference's CPU loop is also a plain
    cast."""

    @staticmethod
    def fake_e4m3fy(inputs: torch.Tensor) -> torch.Tensor:
        if inputs.is_cuda:
            return ops.fake_e4m3fy(inputs)
        x = inputs.float()
        y = torch.clamp(x, -448.0, 448.0).to(torch.float8_e4m3fn).float()
        return torch.where(torch.isnan(x), x, y).to(inputs.dtype)


def load_fake_quant_fp8_ext(verbose=False, required=False):
    return FakeQuantFp8Ext()
