"""Kernel registry of the segmented linear.

``ext_dict`` has the reference's shape (segquant/layers/__init__.py:3-22):
``{kernel_type: {"gemm_scaled_fn": f or None, "gemm_dual_scaled_fn": f or None}}``
with kernel types ``W{weight}A{input}``.  Later loaders overwrite earlier keys.
When no GPU or no built library is present the functions are ``None``.
"""
from ..utils.extension import (load_real_quant_fp8_ext, load_real_quant_int4_ext, load_real_quant_int8_ext,
                               load_real_quant_mix_ext)


def build_ext_dict():
    table = {}
    for loader in (load_real_quant_mix_ext, load_real_quant_fp8_ext, load_real_quant_int8_ext,
                   load_real_quant_int4_ext):
        ext, prefixes = loader(required=False)
        for p in prefixes:
            table[p] = {
                "gemm_scaled_fn": getattr(ext, f"{p}_real_quantized_gemm_scaled", None),
                "gemm_dual_scaled_fn": getattr(ext, f"{p}_real_quantized_gemm_dual_scaled", None),
            }
    return table


ext_dict = build_ext_dict()
