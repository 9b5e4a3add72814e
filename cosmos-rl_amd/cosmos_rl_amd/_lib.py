"""ctypes binding of ``libcosmosfp8.so`` (declared in ``include/cosmos_fp8.h``).

There is no CPU fallback: if the library is missing, or a call fails, an
exception is raised.  Loading the library needs no GPU; calling into it does.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_void_p, POINTER
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libcosmosfp8.so"

OUT_BF16 = 0
OUT_F32 = 1
GROUP_MODE_DIV = 0
GROUP_MODE_DEEPEP = 1
SCALE_F32, SCALE_E8M0 = 0, 1
TENSORWISE_AMAX_SLOTS = 64
TENSORWISE_STATIC_MAX_TENSORS = 512
IN_BF16, IN_F16, IN_F32 = 0, 1, 2
COMBINE_BF16_STEPS, COMBINE_F32 = 0, 1

EINVAL, EARCH, ELAUNCH, EWORKSPACE = -1, -2, -3, -4


class TensorDesc(ctypes.Structure):
    _fields_ = [("x", c_void_p), ("q", c_void_p), ("scale", c_void_p), ("numel", c_int64)]


class RowwiseDesc(ctypes.Structure):
    _fields_ = [("x", c_void_p), ("q", c_void_p), ("scales", c_void_p), ("rows", c_int64), ("cols", c_int64),
                ("ld_x", c_int64), ("ld_q", c_int64), ("x_dtype", c_int32), ("reserved", c_int32)]


# name -> (restype, argtypes); must list every symbol the header declares
SIGNATURES = {
    "cfp8_version": (c_int, []),
    "cfp8_last_error": (c_char_p, []),
    "cfp8_quant_rowwise": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "cfp8_quant_rowwise_from": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "cfp8_quant_rowwise_multi": (c_int, [POINTER(RowwiseDesc), c_int64, c_void_p]),
    "cfp8_quant_tensorwise_multi": (c_int, [POINTER(TensorDesc), c_int64, c_void_p, c_void_p]),
    "cfp8_quant_tensorwise_multi_static": (c_int, [POINTER(TensorDesc), c_int64, c_void_p]),
    "cfp8_tensorwise_resident": (c_int, [c_int]),
    "cfp8_tensorwise_status": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "cfp8_tensorwise_resident_tuning": (c_int, [c_int64, c_int]),
    "cfp8_tensorwise_amax_multi": (c_int, [POINTER(TensorDesc), c_int64, c_void_p, c_void_p]),
    "cfp8_tensorwise_cast_multi": (c_int, [POINTER(TensorDesc), c_int64, c_void_p, c_void_p]),
    "cfp8_quant_tensorwise": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "cfp8_quant_block128": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p]),
    "cfp8_quant_group128": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int, c_void_p]),
    "cfp8_swiglu_quant_group128": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "cfp8_gemm_grouped_swiglu_quant": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                               c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "cfp8_generate_permute_indices": (c_int, [c_void_p, c_int, c_int, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "cfp8_gather_rows": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "cfp8_combine_rows": (c_int, [c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int64, c_int, c_int64, c_int,
                                  c_void_p, c_int64, c_void_p]),
    "cfp8_quant_mxfp4": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p]),
    "cfp8_gemm_mxfp4": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                c_int, c_int64, c_int64, c_int64, c_void_p]),
    "cfp8_linear_mxfp4": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int, c_int64, c_int64, c_int64,
                                  c_void_p, c_size_t, c_void_p]),
    "cfp8_gather_quant_group128": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_void_p]),
    "cfp8_scatter_quant_group128": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64,
                                            c_void_p, c_void_p]),
    "cfp8_dequant_block128": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "cfp8_dequant_group128": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int, c_int64, c_int64, c_void_p, c_int64, c_int, c_void_p]),
    "cfp8_scaled_mm_rowwise": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64,
                                       c_int, c_int64, c_int64, c_int64, c_void_p]),
    "cfp8_linear_workspace_bytes": (c_size_t, [c_int64, c_int64]),
    "cfp8_linear_workspace_bytes_split": (c_size_t, [c_int64, c_int64, c_int64]),
    "cfp8_linear_rowwise": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_int,
                                    c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "cfp8_gemm_block128": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_int64,
                                   c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p]),
    "cfp8_gemm_dispatch_info": (c_int, [c_int, c_int64, c_int64, c_int64, c_int, c_int, c_int, c_char_p, c_size_t]),
    "cfp8_gemm_grouped_block128": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_int64, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m cosmos_rl_amd._build` "
            "(hipcc, gfx950). There is no CPU fallback for the FP8 path.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the export is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


DISPATCH_ROWWISE, DISPATCH_LINEAR, DISPATCH_BLOCK, DISPATCH_GROUPED, DISPATCH_GROUPED_SWIGLU = range(5)


def gemm_dispatch_info(kind: int, M: int, N: int, K: int, out_dtype: int = OUT_BF16, cus: int = 256,
                       with_split_workspace: bool = False) -> str:
    """The kernels a GEMM entry point would launch for a problem ("name grid=.. block=.. lds=..; ..."); needs no GPU."""
    buf = ctypes.create_string_buffer(1024)
    check(load().cfp8_gemm_dispatch_info(kind, M, N, K, out_dtype, cus, int(with_split_workspace), buf, len(buf)))
    return buf.value.decode()


def last_error() -> str:
    msg = load().cfp8_last_error()
    return msg.decode() if msg else ""


def check(rc: int) -> None:
    """Translate a C return code into the exception the reference's Python path raises."""
    if rc == 0:
        return
    msg = last_error()
    if rc == EINVAL:
        raise ValueError(f"cosmos_fp8: {msg}")
    raise RuntimeError(f"cosmos_fp8 error {rc}: {msg}")
