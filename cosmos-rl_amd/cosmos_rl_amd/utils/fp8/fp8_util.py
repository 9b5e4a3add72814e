"""FP8 recipes, module filter and model converter with the names and behaviour of
cosmos_rl/utils/fp8/fp8_util.py.

The reference hands the converted modules to torchao's ``Float8Linear``; here the converted
module is ``Float8Linear`` below, whose forward quantises activation and weight with the chosen
recipe (rowwise: one scale per token / per output feature; tensorwise: one scale per tensor)
and runs the FP8 MFMA GEMM.  Only the forward (rollout / inference) direction is on this path;
gradients of the FP8 matmul are outside it and ``Float8Linear`` refuses to run under autograd.
"""
from __future__ import annotations

from dataclasses import dataclass
from enum import Enum
from functools import partial
from typing import List, Optional, Union

import torch
import torch.nn as nn

from cosmos_rl_amd import ops
from cosmos_rl_amd.utils.model_converter import ModelConverter


class _StrEnum(str, Enum):
    def __str__(self) -> str:
        return str(self.value)


class FP8Recipe(_StrEnum):
    DYNAMIC_SCALING = "dynamic_scaling"
    DELAYED_SCALING = "delayed_scaling"


def is_valid_fp8_recipe(value: str) -> bool:
    return value in [m.value for m in FP8Recipe]


class FP8QuantRecipe(_StrEnum):
    ROWWISE = "rowwise"
    TENSORWISE = "tensorwise"


def is_valid_fp8_quant_recipe(value: str) -> bool:
    return value in [m.value for m in FP8QuantRecipe]


@dataclass
class FP8Config:
    """Field names of ``FP8Config`` (cosmos_rl/policy/config/__init__.py:752-763)."""
    enable_fp8: bool = False
    fp8_recipe: str = "dynamic_scaling"
    quant_recipe: str = "rowwise"


def module_filter_fn(mod: nn.Module, fqn: str, filter_fqns: List[str]) -> bool:
    """fp8_util.py:62-87: convert only ``nn.Linear`` whose two dimensions are multiples of 16
    and whose fully qualified name contains none of ``filter_fqns``.  (The FP8 GEMM takes any such
    ``in_features``: a K that is not a multiple of its 128-wide step runs with the last step masked.)"""
    if not isinstance(mod, nn.Linear):
        return False
    out_features, in_features = mod.weight.shape
    if out_features % 16 or in_features % 16:
        return False
    return not any(f in fqn for f in filter_fqns)


def is_gfx950_available() -> bool:
    if not torch.cuda.is_available():
        return False
    name = getattr(torch.cuda.get_device_properties(torch.cuda.current_device()), "gcnArchName", "")
    return name.startswith("gfx950")


class Float8Linear(nn.Linear):
    """``nn.Linear`` whose forward runs in FP8 with dynamic scaling of both operands."""

    quant_recipe: str = "rowwise"

    @classmethod
    def from_float(cls, mod: nn.Linear, quant_recipe: str) -> "Float8Linear":
        with torch.device("meta"):
            new = cls(mod.in_features, mod.out_features, bias=False)
        new.weight = mod.weight
        new.bias = mod.bias
        new.quant_recipe = str(quant_recipe)
        return new

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if torch.is_grad_enabled() and (input.requires_grad or self.weight.requires_grad):
            raise NotImplementedError(
                "Float8Linear covers the forward (rollout) direction only; call it under torch.no_grad()")
        x2 = input.reshape(-1, self.in_features)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        w = self.weight if self.weight.dtype == torch.bfloat16 else self.weight.to(torch.bfloat16)
        if self.quant_recipe == FP8QuantRecipe.ROWWISE:
            qw, sw = ops.quant_rowwise(w)
            out = ops.fp8_linear(x2, qw.t(), sw, bias=None, out_dtype=torch.bfloat16)
        else:
            qw, sw = ops.quant_tensorwise(w)
            qx, sx = ops.quant_tensorwise(x2)
            out = ops.scaled_mm(qx, qw.t(), sx, sw, out_dtype=torch.bfloat16)
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out.reshape(*input.shape[:-1], self.out_features).to(input.dtype)


def convert_to_float8_training(model: nn.Module, quant_recipe: str, module_filter_fn=None) -> nn.Module:
    """Swap eligible ``nn.Linear`` children for ``Float8Linear`` in place (the root itself is
    never swapped), calling ``module_filter_fn(module, fqn)`` like torchao's helper of that name."""
    def visit(parent: nn.Module, prefix: str) -> None:
        for name, child in list(parent.named_children()):
            fqn = f"{prefix}.{name}" if prefix else name
            if isinstance(child, nn.Linear) and not isinstance(child, Float8Linear):
                if module_filter_fn is None or module_filter_fn(child, fqn):
                    setattr(parent, name, Float8Linear.from_float(child, quant_recipe))
            else:
                visit(child, fqn)
    visit(model, "")
    return model


class FP8ModelConverter(ModelConverter):
    """fp8_util.py:90-166.  ``config.train.fp8`` carries ``enable_fp8 / fp8_recipe / quant_recipe``."""

    def __init__(self, config, parallel_dims=None):
        super().__init__(config, parallel_dims)
        if not is_gfx950_available():
            raise RuntimeError("FP8 is only supported on gfx950 (MI355X) devices by this build")
        self.fp8_config = config.train.fp8
        assert is_valid_fp8_quant_recipe(self.fp8_config.quant_recipe)
        assert is_valid_fp8_recipe(self.fp8_config.fp8_recipe)
        if self.fp8_config.fp8_recipe == FP8Recipe.DELAYED_SCALING:
            raise NotImplementedError("[FP8] Delayed scaling is not supported yet.")
        self.precompute_scale = False

    def convert_model(self, model: torch.nn.Module) -> None:
        """fp8_util.py:139-152: converts in place and returns nothing."""
        if not self.fp8_config.enable_fp8:
            return
        filter_fqns = model.fqn_filter_for_quantization() if hasattr(model, "fqn_filter_for_quantization") else []
        convert_to_float8_training(model, self.fp8_config.quant_recipe,
                                   module_filter_fn=partial(module_filter_fn, filter_fqns=filter_fqns))

    def post_optimizer_hook(self, model: Union[nn.Module, List[nn.Module]]):
        # scales are dynamic (recomputed from the weights at every forward); nothing to refresh
        if not self.fp8_config.enable_fp8 or not self.precompute_scale:
            return
