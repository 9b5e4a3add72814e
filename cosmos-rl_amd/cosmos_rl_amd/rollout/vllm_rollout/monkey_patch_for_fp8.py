"""Rowwise FP8 linear for the rollout engine, with the helper names and signatures of
cosmos_rl/rollout/vllm_rollout/monkey_patch_for_fp8.py.

The reference patches vLLM classes in place; vLLM is not part of this build, so the two
classes it patches (``Fp8LinearMethod``, ``Fp8LinearOp``) are provided here with the
behaviour the patches give them, and modules are recognised by ``isinstance(quant_method,
Fp8LinearMethod)`` exactly as the reference does.  An engine adopts the path by giving each
quantised linear a ``quant_method = Fp8LinearMethod()``.
"""
from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch
from torch.nn import Parameter

from cosmos_rl_amd import ops


class Fp8LinearOp:
    """Per-token dynamic activation quantisation feeding the rowwise scaled mm - what
    ``Fp8LinearOp(cutlass_fp8_supported=False, use_per_token_if_dynamic=True).apply`` does after
    the dispatch patch (monkey_patch_for_fp8.py:26-34, 74-79)."""

    def __init__(self, cutlass_fp8_supported: bool = False, use_per_token_if_dynamic: bool = True):
        if not use_per_token_if_dynamic:
            raise NotImplementedError("only the per-token (rowwise) FP8 linear is on this path")
        self.cutlass_fp8_supported = cutlass_fp8_supported
        self.use_per_token_if_dynamic = use_per_token_if_dynamic
        # the scaled-mm kernel comes from the dispatch function, as in the engine the reference patches
        self.w8a8_scaled_mm = _dispatch["dispatch_w8a8_scaled_mm"](cutlass_fp8_supported, True, use_per_token_if_dynamic)

    def apply(self, input: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
              out_dtype: Optional[torch.dtype] = None, input_scale: Optional[torch.Tensor] = None,
              input_scale_ub: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        if input_scale is not None:
            raise NotImplementedError("static activation scales are not on this path")
        if self.w8a8_scaled_mm is torch_per_token_w8a8_scaled_mm:
            # the per-token rowwise kernel: quantisation and GEMM as one library call
            return ops.fp8_linear(input, weight, weight_scale, bias=bias, out_dtype=out_dtype or input.dtype)
        x2 = input.reshape(-1, input.shape[-1])
        qinput, x_scale = ops.scaled_fp8_quant(x2, scale=None, use_per_token_if_dynamic=True)
        out = self.w8a8_scaled_mm(qinput=qinput, weight=weight, out_dtype=out_dtype or input.dtype, scale_a=x_scale,
                                  scale_b=weight_scale, bias=bias)
        return out.reshape(*input.shape[:-1], out.shape[-1])


class Fp8LinearMethod:
    """Marker + behaviour of the (patched) vLLM ``Fp8LinearMethod`` for one linear layer."""

    def __init__(self) -> None:
        self.fp8_linear = Fp8LinearOp(cutlass_fp8_supported=False, use_per_token_if_dynamic=True)

    def process_weights_after_loading(self, layer: torch.nn.Module) -> None:
        _simplified_process_weights_after_loading(self, layer)

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
        return self.fp8_linear.apply(input=x, weight=layer.weight, weight_scale=layer.weight_scale,
                                     out_dtype=x.dtype, input_scale=getattr(layer, "input_scale", None), bias=bias)


def torch_per_token_w8a8_scaled_mm(*, qinput: torch.Tensor, weight: torch.Tensor, out_dtype: torch.dtype,
                                   scale_a: torch.Tensor, scale_b: torch.Tensor,
                                   bias: Optional[torch.Tensor] = None, **kwargs: Any) -> torch.Tensor:
    """The kernel the reference forces the dispatch to (monkey_patch_for_fp8.py:28-31):
    ``torch._scaled_mm(qinput, weight, scale_a, scale_b.t(), out_dtype)``."""
    return ops.scaled_mm(qinput, weight, scale_a, scale_b, out_dtype=out_dtype, bias=bias)


def dispatch_w8a8_scaled_mm(cutlass_fp8_supported: bool, per_tensor_weights: bool, per_tensor_activations: bool):
    """The engine's kernel choice for an FP8 linear.  Only one kernel exists on this path, so the unpatched
    choice is already the per-token rowwise mm; the name is kept because the reference replaces it."""
    return torch_per_token_w8a8_scaled_mm


# what ``Fp8LinearOp.__init__`` asks for its scaled-mm kernel; ``apply_patch_to_dispatch`` replaces the entry
_dispatch = {"dispatch_w8a8_scaled_mm": dispatch_w8a8_scaled_mm}


def apply_patch_to_dispatch():
    """monkey_patch_for_fp8.py:26-34: every FP8 linear constructed from now on goes through the per-token
    rowwise mm, whatever the engine's own dispatch would have picked."""
    def dispatch_fp8_linear_kernel_to_torch_scaled_mm(*args, **kwargs):
        return torch_per_token_w8a8_scaled_mm

    _dispatch["dispatch_w8a8_scaled_mm"] = dispatch_fp8_linear_kernel_to_torch_scaled_mm


apply_patch_to_dispatch()


def _simplified_process_weights_after_loading(self, layer: torch.nn.Module) -> None:
    # monkey_patch_for_fp8.py:45-54 - rowwise only
    qweight, weight_scale = ops.scaled_fp8_quant(layer.weight, scale=None, use_per_token_if_dynamic=True)
    layer.weight = Parameter(qweight.t(), requires_grad=False)
    layer.weight_scale = Parameter(weight_scale, requires_grad=False)
    layer.input_scale = None


def simplify_process_weights_after_loading():
    """monkey_patch_for_fp8.py:37-59: quantise linear weights in ``rowwise`` mode only."""
    Fp8LinearMethod.process_weights_after_loading = _simplified_process_weights_after_loading


def _fp8_linears(model: torch.nn.Module):
    """(module name, module) of every linear whose quant method is the FP8 one."""
    for name, module in model.named_modules():
        if isinstance(getattr(module, "quant_method", None), Fp8LinearMethod):
            yield name, module


def apply_fp8_linear_patch(model: torch.nn.Module):
    """monkey_patch_for_fp8.py:63-82: give every FP8 linear the per-token rowwise op; other
    quant methods are left alone."""
    for _, module in _fp8_linears(model):
        module.quant_method.fp8_linear = Fp8LinearOp(cutlass_fp8_supported=False, use_per_token_if_dynamic=True)


def replace_weight_of_quantized_module(vllm_model: torch.nn.Module, cached_weight_map: Dict[str, torch.Tensor],
                                       weight_mapper):
    """monkey_patch_for_fp8.py:85-100: swap a cached tensor (high-precision staging buffer, or
    the quantised parameter on the way back) into every module whose HF-compatible weight name
    is a key of ``cached_weight_map``."""
    for name, module in vllm_model.named_modules():
        key = weight_mapper.rollout_map_local_key_to_hf_key(f"{name}.weight")
        cached = cached_weight_map.get(key)
        if cached is not None:
            module.weight = cached


def cache_weight_of_quantized_module(vllm_model: torch.nn.Module, promotion_dtype: torch.dtype, weight_mapper,
                                     parallel_dims=None) -> Tuple[Dict[str, torch.Tensor], Dict[str, torch.Tensor]]:
    """monkey_patch_for_fp8.py:103-129.  Returns ``(hp_weight_map, original_weight_map)``:
    for every FP8 linear, a fresh ``promotion_dtype`` parameter shaped [out_dim, in_dim] that
    weight sync receives into, and the engine's own quantised parameter ([in_dim, out_dim], the
    transposed view of a contiguous [out_dim, in_dim] buffer)."""
    hp_weight_map: Dict[str, torch.Tensor] = {}
    original_weight_map: Dict[str, torch.Tensor] = {}
    for name, module in _fp8_linears(vllm_model):
        key = weight_mapper.rollout_map_local_key_to_hf_key(f"{name}.weight")
        qweight = module.weight
        original_weight_map[key] = qweight
        hp_weight_map[key] = Parameter(qweight.t().to(promotion_dtype).contiguous(), requires_grad=False)
    return hp_weight_map, original_weight_map


def post_process_view_map_for_fp8(vllm_weight_inplace_view_map: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    """monkey_patch_for_fp8.py:132-147: scales are derived on the rollout side, never received,
    so every ``weight_scale`` entry leaves the recv view map."""
    return {k: v for k, v in vllm_weight_inplace_view_map.items() if "weight_scale" not in k}
