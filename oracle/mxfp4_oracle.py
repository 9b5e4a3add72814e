"""CPU oracle for MXFP4 weight quantisation.  TEST INFRASTRUCTURE ONLY (imported by tests/ alone; the
shipped package never comes here).

PARITY UNPINNED against the reference.  The reference quantises GPT-OSS expert weights with
``downcast_to_mxfp(w.to(torch.bfloat16), torch.uint8, axis=1)`` from the third-party package
``triton_kernels`` (cosmos_rl/rollout/vllm_rollout/monkey_patch_for_mxfp4.py:18-24, called from
vllm_rollout.py:1018-1029 between two transposes, so that blocks run along the last axis of the
[experts, out, in] weight).  That package is not vendored, not pinned to a version in the reference's files
and not importable here, and the reference holds no fixture for it.  ``downcast`` below restates the
algorithm of that function as published in the triton repository (python/triton_kernels/triton_kernels/
numerics_details/mxfp_details/_downcast_to_mxfp.py, default DequantScaleRoundingMode.ROUND_UP):

    max_val   = max |x| over the 32 elements of a block               (fp32)
    dequant   = max_val / 6.0
    exponent  = (bits(dequant) + 0x007FFFFF) & 0x7F800000             -> 2^ceil(log2(dequant))
    scale     = exponent >> 23                                        (e8m0 byte)
    q         = x * (1 / 2^.. , or 0 when the exponent field is 0)
    e2m1 code from the fp32 bits of q: sign, exponent rebiased 127 -> 1, two mantissa bits, one extra bit
    added for rounding ("nearest, ties up" in magnitude), saturated at 7; even element in the low nibble.

What tests/test_mxfp4.py pins is therefore the published algorithm, not the package: the e2m1 rounding
against a brute-force nearest-value search with ties away from zero, the scale against 2^ceil(log2(max/6))
computed with math.frexp, the packing order, and the bound |x - dequant(q)| <= scale / 2 * step.
Whether triton's fp32 division there is IEEE or approximate is not known (it matters only when max/6 lies
within an ulp of a power of two); IEEE division is assumed.
"""
from __future__ import annotations

from typing import Tuple

import numpy as np
import torch

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)


def e2m1_codes(q_f32: np.ndarray) -> np.ndarray:
    """4-bit codes (sign in bit 3) of fp32 values, by the bit manipulation of the published kernel."""
    b = np.ascontiguousarray(q_f32, dtype=np.float32).view(np.uint32).astype(np.uint64)
    signs = b & 0x80000000
    exponents = (b >> 23) & 0xFF
    mantissas = b & 0x7FFFFF
    adjusted = np.minimum(126 - np.minimum(exponents, 126), 63)            # shift of 32 or more gives 0
    sub = (0x400000 | (mantissas >> 1)) >> adjusted
    mantissas = np.where(exponents < 127, sub, mantissas)
    exponents = np.maximum(exponents, 126) - 126
    tmp = np.minimum((((exponents << 2) | (mantissas >> 21)) + 1) >> 1, 7)
    return ((signs >> 28) | tmp).astype(np.uint8)


def downcast(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [..., K] bf16, K % 32 == 0 -> (packed uint8 [..., K/2], scales uint8 [..., K/32])."""
    assert x.dtype == torch.bfloat16 and x.shape[-1] % 32 == 0
    f = x.float().numpy().reshape(-1, x.shape[-1] // 32, 32)
    max_val = np.abs(f).max(axis=2, keepdims=True)
    dequant = (max_val / np.float32(6.0)).astype(np.float32)
    exponent = ((dequant.view(np.uint32).astype(np.uint64) + 0x007FFFFF) & 0x7F800000).astype(np.uint32)
    rounded = exponent.view(np.float32)
    with np.errstate(divide="ignore", over="ignore", invalid="ignore"):
        quant_scale = np.where(rounded == 0, np.float32(0), np.float32(1.0) / rounded).astype(np.float32)
        q = (f * quant_scale).astype(np.float32)
    codes = e2m1_codes(q).reshape(-1, x.shape[-1])
    packed = codes[:, 0::2] | (codes[:, 1::2] << 4)
    scales = (exponent >> 23).astype(np.uint8).reshape(-1, x.shape[-1] // 32)
    lead = tuple(x.shape[:-1])
    return (torch.from_numpy(packed).reshape(*lead, x.shape[-1] // 2),
            torch.from_numpy(scales).reshape(*lead, x.shape[-1] // 32))


def upcast(packed: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """fp32 values of (packed, scales): value = (+-) E2M1_VALUES[code & 7] * 2^(scale - 127)."""
    p = packed.numpy()
    codes = np.stack([p & 0xF, p >> 4], axis=-1).reshape(*p.shape[:-1], p.shape[-1] * 2)
    vals = E2M1_VALUES[codes & 7] * np.where(codes & 8, np.float32(-1), np.float32(1))
    s = np.ldexp(np.float64(1.0), scales.numpy().astype(np.int64) - 127)
    return torch.from_numpy((vals.astype(np.float64) * np.repeat(s, 32, axis=-1)).astype(np.float32))


def gemm(xq: torch.Tensor, sx: torch.Tensor, packed: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """out[m, n] = sx[m] * sum_k xq[m, k] * upcast(packed, scales)[n, k] in float64: the product the rollout engine
    forms with the weights of ``downcast`` (vllm_rollout.py:1018-1033 hands them to its FusedMoE layers), here on
    per-token FP8 activations (xq e4m3 [M, K], sx fp32 [M]).  Every product xq * code * 2^e is exact in fp32 and
    so is this sum in float64 for any K a test uses; the kernel under test may differ by its fp32 accumulation."""
    w = upcast(packed, scales).double()
    return (xq.float().double() @ w.t()) * sx.double().reshape(-1, 1)

