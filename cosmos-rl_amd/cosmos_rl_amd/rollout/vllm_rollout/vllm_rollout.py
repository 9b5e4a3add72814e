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
    them for ``quantization_type == "fp8"``, and the parameter map weight sync copies into
    (rollout_base.py:186-230).  The host class provides ``get_underlying_model()`` and sets
    ``_engine_initialized`` once its engine is up, as ``RolloutBase`` does."""

    _engine_initialized: bool = False
    _model_param_map = None  # key: compatible name, value: param

    def fp8_quantization(self, weight: torch.Tensor):
        return fp8_quantization(weight)

    def is_engine_initialized(self) -> bool:
        return self._engine_initialized

    def get_quantized_tensors(self, weight_mapper) -> Dict[str, torch.Tensor]:
        """rollout_base.py:211-230: quantised tensors that live outside the model's state dict.  For FP8 the
        engine's fp8 weights and ``weight_scale`` tensors are ordinary parameters, so the map is empty (the
        reference fills it for MXFP4 only, vllm_rollout.py:1088-1120)."""
        if not self._engine_initialized:
            raise RuntimeError("[Rollout] Engine is not initialized, please call init_engine first.")
        return {}

    def model_param_map(self, weight_mapper) -> Dict[str, torch.Tensor]:
        """rollout_base.py:186-209: every parameter of the rollout model under its HF-compatible name, plus
        the quantised tensors; built once and cached."""
        if not self._engine_initialized:
            raise RuntimeError("[Rollout] Engine is not initialized, please call init_engine first.")
        if self._model_param_map:
            return self._model_param_map
        model = self.get_underlying_model()
        param_map = {}
        for name, param in model.state_dict().items():
            param_map[weight_mapper.rollout_map_local_key_to_hf_key(name)] = param
        param_map.update(self.get_quantized_tensors(weight_mapper))
        self._model_param_map = param_map
        return self._model_param_map

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
