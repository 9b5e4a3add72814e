"""MXFP4 weight quantisation for GPT-OSS experts - counterpart of ``quantize_mx4`` in
cosmos_rl/rollout/vllm_rollout/monkey_patch_for_mxfp4.py:18-24 and of the quantisation step of
``vLLMRollout.mxfp4_quantization`` (cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:1001-1029)."""
from __future__ import annotations

from typing import Tuple

import torch

from cosmos_rl_amd import ops

__all__ = ["quantize_mx4", "mxfp4_quantization"]


def quantize_mx4(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``downcast_to_mxfp(w.to(torch.bfloat16), torch.uint8, axis=1)`` of a 3-D tensor: blocks of 32 run along
    axis 1.  Returns (uint8 [d0, d1/2, d2], uint8 [d0, d1/32, d2]).  The kernel works along the last axis,
    so this entry point pays two transposes; ``mxfp4_quantization`` is the one that does not."""
    if w.dim() != 3:
        raise ValueError("quantize_mx4 expects a 3-D tensor")
    q, s = ops.quant_mxfp4(w.to(torch.bfloat16).transpose(1, 2).contiguous())
    return q.transpose(1, 2).contiguous(), s.transpose(1, 2).contiguous()


def mxfp4_quantization(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """The quantisation step of the reference's ``mxfp4_quantization``: its transpose, ``quantize_mx4`` and
    transpose back (vllm_rollout.py:1018-1029) cancel into one pass along the last axis of the
    [experts, out, in] weight.  Returns (uint8 [experts, out, in/2], uint8 [experts, out, in/32]); the
    engine-specific swizzle the reference applies next (:1037-1045) belongs to the engine."""
    return ops.quant_mxfp4(weight.to(torch.bfloat16))
