"""Enumerations and the default configuration of ``quantize()``.

Same names and string values as the reference (segquant/config.py:18-97): the
kernel registry is keyed by ``W{weight}A{input}`` built from ``DType.value``.
"""
from enum import Enum


class DType(Enum):
    INT4 = "int4"
    INT6 = "int6"
    INT8 = "int8"
    INT16 = "int16"
    FP8E5M2 = "fpe5m2"
    FP8E4M3 = "fpe4m3"
    FP16 = "fp16"
    BF16 = "bf16"


class Optimum(Enum):
    DEFAULT = "default"
    SMOOTH = "smooth"
    SVD = "svd"


class Calibrate(Enum):
    AMAX = "amax"
    GPTQ = "gptq"


class SegPattern(Enum):
    LINEAR2CHUNK = "linear_to_chunk"
    LINEAR2SPLIT = "linear_to_split"
    CONCAT2LINEAR = "concat_to_linear"
    STACK2LINEAR = "stack_to_linear"
    RESHAPE2LINEAR = "reshape_to_linear"
    ACTIVATION2LINEAR = "activation_to_linear"

    @classmethod
    def seg(cls):
        return [cls.LINEAR2CHUNK, cls.LINEAR2SPLIT, cls.CONCAT2LINEAR, cls.STACK2LINEAR, cls.RESHAPE2LINEAR]

    @classmethod
    def all(cls):
        return cls.seg() + [cls.ACTIVATION2LINEAR]


# The reference's default optimiser is "smooth" (segquant/config.py:80-84); this
# build implements the kernel path, whose optimiser is "default".
default_quantize_config = {
    "default": {
        "enable": True,
        "seglinear": True,
        "search_patterns": SegPattern.all(),
        "real_quant": False,
        "opt": {"type": Optimum.DEFAULT},
        "calib": {"type": Calibrate.AMAX},
        "input_quant": {"type": DType.INT8, "axis": None},
        "weight_quant": {"type": DType.INT8, "axis": None},
    },
}
