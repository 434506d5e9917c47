"""ctypes binding of libsegq.so (the C ABI declared in include/segq.h).

The library is built in-tree by ``segquant_amd/csrc/Makefile``.  Loading fails
loudly when it is missing: there is no CPU fallback for the real-quantised path.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libsegq.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

SEGQ_MAX_KSEG = 8
SEGQ_MAX_RANGES = 64

# enum segq_dtype
F32, F16, BF16, ACC = 0, 1, 2, 3
# enum segq_code
CODE_I8, CODE_E4M3, CODE_I4 = 0, 1, 2


class QuantDesc(C.Structure):
    _fields_ = [
        ("x", C.c_void_p), ("x_dtype", C.c_int32), ("code_fmt", C.c_int32),
        ("rows", C.c_int64), ("cols", C.c_int64), ("ldx", C.c_int64),
        ("codes", C.c_void_p), ("codes_neg", C.c_void_p), ("ld_codes", C.c_int64),
        ("scale", C.c_void_p), ("scale_neg", C.c_void_p),
        ("seg_rows", C.c_int64), ("seg_stride", C.c_int64), ("row_stride", C.c_int64),
        ("kseg_stride", C.c_int64),
        ("n_kseg", C.c_int32), ("dual", C.c_int32), ("dual_kseg_mask", C.c_uint32), ("dynamic", C.c_int32),
        ("kseg_bounds", C.c_int64 * (SEGQ_MAX_KSEG + 1)),
        ("pre_op", C.c_int32), ("gate", C.c_void_p), ("ld_gate", C.c_int64), ("col_div", C.c_void_p),
    ]


class KRange(C.Structure):
    _fields_ = [
        ("k_begin", C.c_int64), ("k_len", C.c_int64),
        ("a_sel", C.c_int32), ("sx_row_stride", C.c_int32), ("sw_col_stride", C.c_int32), ("reserved", C.c_int32),
        ("sx", C.c_void_p), ("sw", C.c_void_p),
    ]


class GemmDesc(C.Structure):
    _fields_ = [
        ("a_fmt", C.c_int32), ("b_fmt", C.c_int32), ("out_dtype", C.c_int32), ("bias_dtype", C.c_int32),
        ("m", C.c_int64), ("n", C.c_int64),
        ("a", C.c_void_p), ("a_neg", C.c_void_p), ("lda", C.c_int64),
        ("b", C.c_void_p), ("ldb", C.c_int64),
        ("out", C.c_void_p), ("ldo", C.c_int64),
        ("bias", C.c_void_p),
        ("batch", C.c_int64), ("batch_stride_a", C.c_int64), ("batch_stride_b", C.c_int64),
        ("batch_stride_out", C.c_int64), ("batch_stride_sx", C.c_int64), ("batch_stride_sw", C.c_int64),
        ("n_ranges", C.c_int32), ("tile", C.c_int32), ("workspace", C.c_void_p), ("workspace_bytes", C.c_int64),
        ("group_dequant", C.c_void_p), ("group_dequant_stride", C.c_int64),
        ("addend", C.c_void_p), ("ld_addend", C.c_int64), ("split_k", C.c_int64),
        ("lowrank_t", C.c_void_p), ("ld_lowrank_t", C.c_int64), ("lowrank_l2t", C.c_void_p), ("ld_lowrank_l2t", C.c_int64),
        ("lowrank_rank", C.c_int32), ("out_pre_op", C.c_int32),
        ("out_codes", C.c_void_p), ("out_codes_neg", C.c_void_p), ("ld_out_codes", C.c_int64),
        ("out_scale", C.c_void_p), ("out_scale_neg", C.c_void_p), ("out_code_fmt", C.c_int32), ("reserved2", C.c_int32),
        ("ranges", KRange * SEGQ_MAX_RANGES),
    ]


EXPORTS = (
    "segq_version", "segq_last_error", "segq_quantize", "segq_quantize_many", "segq_quantize_weights_scalar",
    "segq_quantize_weights_rows", "segq_quantize_weights_groups", "segq_repack_int4_cols_to_rows", "segq_gemm", "segq_gemm_tile_count", "segq_gemm_workspace_bytes", "segq_gemm_plan", "segq_linear", "segq_fake_e4m3",
    "segq_gemm_noalloc", "segq_noalloc_scratch_bytes", "segq_init", "segq_device_info",
)

_lib = None


def build(verbose: bool = False) -> str:
    """Compile libsegq.so for gfx950 with hipcc (works without a GPU)."""
    out = subprocess.run(["make", "-C", CSRC_DIR, "-j8"], capture_output=True, text=True)
    if verbose or out.returncode != 0:
        print(out.stdout[-4000:])
        print(out.stderr[-4000:])
    if out.returncode != 0:
        raise RuntimeError("building libsegq.so failed")
    return LIB_PATH


def lib() -> C.CDLL:
    """The loaded library.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    # torch ships its own HIP runtime; it has to be in the process before this
    # library is, so that both resolve to the same runtime (two runtimes in one
    # process do not see each other's devices and streams)
    import torch  # noqa: F401
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
            "(the real-quantised path has no fallback)")
    L = C.CDLL(LIB_PATH)
    L.segq_version.restype = C.c_int
    L.segq_last_error.restype = C.c_char_p
    L.segq_quantize.argtypes = [C.POINTER(QuantDesc), C.c_void_p]
    L.segq_quantize_many.argtypes = [C.POINTER(QuantDesc), C.c_int32, C.c_void_p]
    L.segq_quantize_weights_scalar.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p,
                                               C.c_int32, C.c_float, C.c_void_p]
    L.segq_quantize_weights_rows.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p,
                                             C.c_int32, C.c_void_p, C.c_void_p]
    L.segq_quantize_weights_groups.argtypes = [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_void_p, C.c_int32,
                                               C.c_void_p, C.c_int64, C.c_void_p]
    L.segq_repack_int4_cols_to_rows.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_void_p]
    L.segq_gemm.argtypes = [C.POINTER(GemmDesc), C.c_void_p]
    L.segq_gemm_tile_count.restype = C.c_int
    L.segq_gemm_workspace_bytes.argtypes = [C.POINTER(GemmDesc), C.POINTER(C.c_int64)]
    L.segq_gemm_plan.argtypes = [C.POINTER(GemmDesc), C.POINTER(C.c_int32), C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    L.segq_gemm_plan.restype = C.c_int
    L.segq_gemm_noalloc.argtypes = [C.POINTER(GemmDesc), C.c_void_p]
    L.segq_gemm_noalloc.restype = C.c_int
    L.segq_noalloc_scratch_bytes.restype = C.c_int64
    L.segq_init.restype = C.c_int
    L.segq_device_info.argtypes = [C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    L.segq_device_info.restype = C.c_int
    L.segq_linear.argtypes = [C.POINTER(QuantDesc), C.POINTER(GemmDesc), C.c_void_p]
    L.segq_fake_e4m3.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_void_p]
    for name in ("segq_quantize", "segq_quantize_weights_scalar", "segq_quantize_weights_rows", "segq_gemm",
                 "segq_quantize_weights_groups", "segq_repack_int4_cols_to_rows",
                 "segq_gemm_workspace_bytes", "segq_gemm_plan", "segq_linear", "segq_fake_e4m3"):
        getattr(L, name).restype = C.c_int
    _lib = L
    return L


def check(rc: int) -> None:
    """Turn a non-zero status into the RuntimeError the reference's bindings raise."""
    if rc != 0:
        raise RuntimeError(f"libsegq error {rc}: {lib().segq_last_error().decode()}")
