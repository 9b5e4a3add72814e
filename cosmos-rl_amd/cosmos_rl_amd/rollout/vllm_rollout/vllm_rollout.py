"""``fp8_quantization`` of the vLLM rollout (cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:989-999)
and the FP8 halves of its weight-sync hooks (:354-427), without the engine around them."""
from __future__ import annotations

from typing import Dict, Tuple

import torch

from cosmos_rl_amd import ops
from cosmos_rl_amd.rollout.vllm_rollout import monkey_patch_for_fp8 as fp8_patch


def fp8_quantization(weight: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rowwise dynamic quantisation of a weight [out_dim, in_dim].

    Returns ``(qweight.t(), weight_scale)``: the fp8 bytes as the [in_dim, out_dim] transposed
    view of a contiguous [out_dim, in_dim] buffer - the layout of the engine's parameter, so the
    later ``copy_`` is a flat byte copy - and fp32 scales [out_dim, 1]."""
    qweight, weight_scale = ops.scaled_fp8_quant(weight, scale=None, use_per_token_if_dynamic=True)
    return qweight.t(), weight_scale


class FP8RolloutMixin:
    """Methods a rollout backend mixes in to serve an FP8 engine: the quantiser and the two
    hooks of ``RolloutBase`` (cosmos_rl/rollout/rollout_base.py:138-185) as vLLMRollout fills
    them for ``quantization_type == "fp8"``.  The host class provides ``get_underlying_model()``."""

    def fp8_quantization(self, weight: torch.Tensor):
        return fp8_quantization(weight)

    def pre_get_params_for_sync_hook(self, quantization_type, weight_mapper, parallel_dims=None,
                                     promotion_dtype: torch.dtype = torch.bfloat16, **kwargs
                                     ) -> Tuple[Dict[str, torch.Tensor], Dict[str, torch.Tensor]]:
        if quantization_type != "fp8":
            return {}, {}
        model = self.get_underlying_model()
        hp_map, quantized_map = fp8_patch.cache_weight_of_quantized_module(
            model, promotion_dtype, weight_mapper, parallel_dims)
        # receive into the high-precision buffers while the view map is built
        fp8_patch.replace_weight_of_quantized_module(model, hp_map, weight_mapper)
        return hp_map, quantized_map

    def post_get_params_for_sync_hook(self, quantization_type, weight_mapper, weight_view_map,
                                      quantized_weight_map, **kwargs) -> Dict[str, torch.Tensor]:
        if quantization_type != "fp8":
            return weight_view_map
        view_map = fp8_patch.post_process_view_map_for_fp8(weight_view_map)
        # the engine computes with the quantised parameters again
        fp8_patch.replace_weight_of_quantized_module(self.get_underlying_model(), quantized_weight_map,
                                                     weight_mapper)
        return view_map
