"""The C-ABI library loads without a GPU, exports every symbol the header declares, and rejects
bad arguments with error codes (never an abort) before it touches a device."""
import ctypes
import re
from pathlib import Path

import pytest
import torch

from cosmos_rl_amd import _lib, ops

HEADER = Path(__file__).resolve().parent.parent / "include" / "cosmos_fp8.h"


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(cfp8_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound():
    syms = declared_symbols()
    assert len(syms) >= 15
    lib = _lib.load()
    for s in syms:
        assert hasattr(lib, s), f"{s} declared in the header but not exported"
        assert s in _lib.SIGNATURES, f"{s} has no ctypes prototype"
    assert set(_lib.SIGNATURES) == set(syms), "python binds symbols the header does not declare"
    assert lib.cfp8_version() >= 100


def test_header_constants_match_binding():
    text = HEADER.read_text()
    val = lambda name: int(re.search(rf"#define {name}\s+\(?(-?\d+)\)?", text).group(1))
    assert val("CFP8_EINVAL") == _lib.EINVAL and val("CFP8_EARCH") == _lib.EARCH
    assert val("CFP8_ELAUNCH") == _lib.ELAUNCH and val("CFP8_EWORKSPACE") == _lib.EWORKSPACE
    assert val("CFP8_OUT_BF16") == _lib.OUT_BF16 and val("CFP8_OUT_F32") == _lib.OUT_F32
    assert val("CFP8_GROUP_MODE_DIV") == _lib.GROUP_MODE_DIV and val("CFP8_GROUP_MODE_DEEPEP") == _lib.GROUP_MODE_DEEPEP
    assert val("CFP8_TENSORWISE_AMAX_SLOTS") == _lib.TENSORWISE_AMAX_SLOTS
    assert val("CFP8_TENSORWISE_STATIC_MAX_TENSORS") == _lib.TENSORWISE_STATIC_MAX_TENSORS
    assert (val("CFP8_IN_BF16"), val("CFP8_IN_F16"), val("CFP8_IN_F32")) == (_lib.IN_BF16, _lib.IN_F16, _lib.IN_F32)
    assert (val("CFP8_COMBINE_BF16_STEPS"), val("CFP8_COMBINE_F32")) == (_lib.COMBINE_BF16_STEPS, _lib.COMBINE_F32)
    assert ctypes.sizeof(_lib.TensorDesc) == 32


def test_argument_errors_need_no_device():
    lib = _lib.load()
    # null pointers / bad shapes are rejected before any HIP call
    assert lib.cfp8_quant_rowwise(None, 4, 16, 16, None, 16, None, None) == _lib.EINVAL
    assert "null pointer" in _lib.last_error()
    assert lib.cfp8_quant_rowwise_from(None, _lib.IN_F32, 4, 16, 16, None, 16, None, None) == _lib.EINVAL
    assert lib.cfp8_quant_rowwise_from(None, 7, 0, 16, 16, None, 16, None, None) == _lib.EINVAL  # unknown dtype
    assert lib.cfp8_quant_rowwise_from(None, _lib.IN_F16, 0, 16, 16, None, 16, None, None) == 0  # nothing to do
    assert lib.cfp8_quant_rowwise_from(None, 7, 4, 16, 16, None, 16, None, None) == _lib.EINVAL
    assert "unknown source dtype" in _lib.last_error()
    assert lib.cfp8_swiglu_quant_group128(None, 128, None, 128, 4, 128, None, 128, None, None) == _lib.EINVAL
    assert lib.cfp8_swiglu_quant_group128(None, 128, None, 128, 0, 128, None, 128, None, None) == 0
    assert lib.cfp8_quant_rowwise(None, -1, 16, 16, None, 16, None, None) == _lib.EINVAL
    assert lib.cfp8_quant_block128(None, 1, 128, 128, None, None, 0, None) == _lib.EINVAL
    assert lib.cfp8_quant_group128(None, 4, 128, 128, None, 128, None, 0, None) == _lib.EINVAL
    assert lib.cfp8_scaled_mm_rowwise(None, 128, None, None, 128, None, None, 64, 0, 16, 64, 128, None) == _lib.EINVAL
    assert lib.cfp8_gemm_block128(None, 128, None, None, 128, None, 1, 1, None, 64, 0, 16, 64, 128, None) == _lib.EINVAL
    assert lib.cfp8_quant_tensorwise_multi(None, 3, None, None) == _lib.EINVAL
    # the entry point with the library's own amax slots: its capacity is checked before any device call
    many = (_lib.TensorDesc * (_lib.TENSORWISE_STATIC_MAX_TENSORS + 1))()
    assert lib.cfp8_quant_tensorwise_multi_static(many, _lib.TENSORWISE_STATIC_MAX_TENSORS + 1, None) == _lib.EWORKSPACE
    assert "exceed" in _lib.last_error()
    assert lib.cfp8_quant_tensorwise_multi_static(None, 0, None) == 0
    assert lib.cfp8_quant_tensorwise_multi_static(None, 2, None) == _lib.EINVAL
    assert lib.cfp8_quant_tensorwise_multi_static(None, -1, None) == _lib.EINVAL
    # shape checks come before any device access: host pointers are never dereferenced here
    buf = ctypes.create_string_buffer(4096)
    ptr = (ctypes.addressof(buf) + 255) & ~255
    assert lib.cfp8_scaled_mm_rowwise(ptr, 128, ptr, ptr, 128, ptr, ptr, 64, 0, 16, 64, 0, None) == _lib.EINVAL   # K = 0
    assert "positive multiple of 16" in _lib.last_error()
    assert lib.cfp8_scaled_mm_rowwise(ptr, 1 << 24, ptr, ptr, 128, ptr, ptr, 64, 0, 16, 64, 128, None) == _lib.EINVAL
    assert "supported range" in _lib.last_error()
    # weighted combine: topk range, mode / dtype pairing, row width
    assert lib.cfp8_combine_rows(ptr, 64, 4, ptr, ptr, _lib.IN_BF16, 4, 65, 64, 0, ptr, 64, None) == _lib.EINVAL
    assert "topk" in _lib.last_error()
    assert lib.cfp8_combine_rows(ptr, 64, 4, ptr, ptr, _lib.IN_F32, 4, 2, 64, _lib.COMBINE_BF16_STEPS, ptr, 64, None) == _lib.EINVAL
    assert lib.cfp8_combine_rows(ptr, 64, 4, ptr, ptr, _lib.IN_F16, 4, 2, 64, _lib.COMBINE_F32, ptr, 64, None) == _lib.EINVAL
    assert lib.cfp8_combine_rows(ptr, 60, 4, ptr, ptr, _lib.IN_BF16, 4, 2, 60, 0, ptr, 60, None) == _lib.EINVAL
    assert lib.cfp8_combine_rows(ptr, 64, 4, ptr, ptr, _lib.IN_BF16, 4, 2, 64, 2, ptr, 64, None) == _lib.EINVAL
    assert lib.cfp8_combine_rows(None, 64, 4, None, None, _lib.IN_BF16, 4, 2, 64, 0, None, 64, None) == _lib.EINVAL
    assert lib.cfp8_combine_rows(None, 64, 0, None, None, _lib.IN_BF16, 0, 2, 64, 0, None, 64, None) == 0
    assert lib.cfp8_quant_mxfp4(ptr, 4, 48, 48, ptr, 24, ptr, 2, None) == _lib.EINVAL     # cols % 32
    assert "multiple of 32" in _lib.last_error()
    assert lib.cfp8_quant_mxfp4(ptr, 4, 64, 64, ptr, 30, ptr, 2, None) == _lib.EINVAL     # q pitch
    assert lib.cfp8_quant_mxfp4(None, 4, 64, 64, None, 32, None, 2, None) == _lib.EINVAL
    assert lib.cfp8_quant_mxfp4(None, 0, 64, 64, None, 32, None, 2, None) == 0
    assert lib.cfp8_gemm_grouped_swiglu_quant(ptr, 128, ptr, ptr, ptr, ptr, ptr, 100, ptr, 128, 100, 128, 2, None) == _lib.EINVAL   # I % 128
    assert lib.cfp8_gemm_grouped_swiglu_quant(ptr, 128, ptr, ptr, ptr, ptr, ptr, 128, ptr, 64, 128, 128, 2, None) == _lib.EINVAL    # M % 128
    assert lib.cfp8_gemm_grouped_swiglu_quant(None, 128, None, None, None, None, None, 128, None, 0, 128, 128, 2, None) == 0
    assert lib.cfp8_gather_quant_group128(ptr, 60, ptr, 4, 60, ptr, 64, ptr, None) == _lib.EINVAL
    assert lib.cfp8_gather_quant_group128(None, 64, None, 4, 64, None, 64, None, None) == _lib.EINVAL
    assert lib.cfp8_gather_quant_group128(None, 64, None, 0, 64, None, 64, None, None) == 0
    assert lib.cfp8_scatter_quant_group128(ptr, 64, 4, 60, ptr, 2, ptr, 8, ptr, 64, ptr, None) == _lib.EINVAL      # cols % 8
    assert lib.cfp8_scatter_quant_group128(ptr, 64, 4, 64, ptr, 65, ptr, 8, ptr, 64, ptr, None) == _lib.EINVAL     # topk
    assert "topk" in _lib.last_error()
    assert lib.cfp8_scatter_quant_group128(None, 64, 4, 64, None, 2, ptr, 8, ptr, 64, ptr, None) == _lib.EINVAL
    assert lib.cfp8_scatter_quant_group128(None, 64, 4, 64, None, 2, None, 0, None, 64, None, None) == 0
    # empty problems succeed without pointers
    assert lib.cfp8_quant_rowwise(None, 0, 16, 16, None, 16, None, None) == 0
    assert lib.cfp8_scaled_mm_rowwise(None, 128, None, None, 128, None, None, 64, 0, 0, 64, 128, None) == 0
    assert lib.cfp8_quant_tensorwise_multi(None, 0, None, None) == 0
    with pytest.raises(ValueError):
        _lib.check(_lib.EINVAL)
    with pytest.raises(RuntimeError):
        _lib.check(_lib.ELAUNCH)


def test_linear_workspace_bytes():
    lib = _lib.load()
    assert lib.cfp8_linear_workspace_bytes(0, 128) == 0
    n = lib.cfp8_linear_workspace_bytes(64, 3584)
    assert n >= 64 * 3584 + 64 * 4 and n % 256 == 0
    # the split-K size adds room for partial sums only where the library would split: 17..64 tokens, at most
    # 4096 weight rows, K of at least 14 steps
    assert lib.cfp8_linear_workspace_bytes_split(64, 3584, 18944) == lib.cfp8_linear_workspace_bytes(64, 18944) + 8 * 64 * 3584 * 4
    for M, N, K in [(16, 3584, 18944), (65, 3584, 18944), (64, 18944, 3584), (64, 3584, 1024), (0, 64, 128)]:
        assert lib.cfp8_linear_workspace_bytes_split(M, N, K) == lib.cfp8_linear_workspace_bytes(M, K)
    # too small a workspace is an error code of its own
    rc = lib.cfp8_linear_rowwise(None, 3584, None, 3584, None, None, 64, 0, 64, 64, 3584, None, 0, None)
    assert rc == _lib.EWORKSPACE


def test_no_cpu_fallback():
    """Operators refuse CPU tensors instead of computing somewhere else."""
    x = torch.zeros(4, 128, dtype=torch.bfloat16)
    for fn in (ops.quant_rowwise, ops.quant_tensorwise, ops.per_block_cast_to_fp8, ops.groupwise_activation_quant,
               ops.per_token_cast_to_fp8):
        with pytest.raises(RuntimeError, match="GPU only"):
            fn(x)
    with pytest.raises(NotImplementedError):
        ops.scaled_fp8_quant(x, scale=torch.ones(1))


def test_product_does_not_import_the_oracle():
    pkg = Path(_lib.__file__).resolve().parent
    for f in list(pkg.rglob("*.py")) + list((pkg.parent / "csrc").glob("*")):
        if f.is_file() and f.suffix in (".py", ".hip", ".h"):
            assert "oracle" not in f.read_text(), f"{f} mentions the oracle"
