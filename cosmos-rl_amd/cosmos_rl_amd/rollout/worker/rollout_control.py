"""Quantise-on-receive step of policy->rollout weight sync.

Counterpart of the low-precision branch of ``recv_weight_shard.completion_lambda``
(cosmos_rl/rollout/worker/rollout_control.py:684-695, 822-898) without the transport around
it: the NCCL receive that fills the high-precision staging buffers, the instruction planner and
the command loop stay with their owner; this class is what runs once every shard of one full
weight has landed.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Optional

import torch


class QuantizedWeightReceiver:
    """Holds the maps the rollout worker builds at ``prepare_shard_infos_for_weight_sync_insts``
    (rollout_control.py:374-438) and performs "quantise the full weight, check it on the first
    sync, copy bytes and scales into the engine's parameters".

    rollout            object with ``fp8_quantization(weight) -> (q_t, scale)`` and
                       ``model_param_map(weight_mapper) -> {name: tensor}``
    weight_mapper      object with ``get_unsplited_weight_name(name)``
    hp_weight_map      full weight name -> bf16 staging parameter [out_dim, in_dim]
    quantized_weight_map  full weight name -> the engine's fp8 parameter
    """

    def __init__(self, rollout, weight_mapper, hp_weight_map: Dict[str, torch.Tensor],
                 quantized_weight_map: Dict[str, torch.Tensor], quantization_type: Optional[str] = "fp8"):
        if quantization_type not in (None, "fp8"):
            raise NotImplementedError(f"quantization_type={quantization_type!r} is not on this path")
        self.rollout = rollout
        self.weight_mapper = weight_mapper
        self.hp_weight_map = hp_weight_map
        self.quantized_weight_map = quantized_weight_map
        self.quantization_type = quantization_type

    # -- rollout_control.py:684-695 -------------------------------------------------------
    def full_weight_name_of_group(self, param_names: Iterable[str]) -> str:
        """An instruction group carries every split (q/k/v, gate/up) of one engine parameter;
        any of its names identifies the unsplit weight."""
        first = next(iter(param_names))
        return self.weight_mapper.get_unsplited_weight_name(first)

    def check_inside_group(self, param_names: Iterable[str], do_weight_sync_check: bool) -> bool:
        """The plain element-wise recv check only applies to weights that are not re-quantised."""
        if self.quantization_type is None:
            return do_weight_sync_check
        full = self.full_weight_name_of_group(param_names)
        return do_weight_sync_check and full not in self.quantized_weight_map

    def plan_group(self, param_names: List[str], do_weight_sync_check: bool = False) -> Callable[[], None]:
        """Returns the completion callback for one instruction group, to be run (on the copy
        stream) after every shard of the group has been received - rollout_control.py:822-827."""
        post: List[str] = []
        if self.quantization_type is not None and not self.check_inside_group(param_names, do_weight_sync_check):
            post.append(self.full_weight_name_of_group(param_names))

        def completion() -> None:
            for name in post:
                self.quantize_full_weight(name, do_weight_sync_check)

        return completion

    # -- rollout_control.py:856-898 -------------------------------------------------------
    def quantize_full_weight(self, full_weight_name: str, do_weight_sync_check: bool = False) -> bool:
        """Quantise one fully received weight into the engine.  Returns False when the name is
        not a quantised weight (nothing to do)."""
        if self.quantization_type != "fp8" or full_weight_name not in self.hp_weight_map:
            return False
        weight_to_quantize = self.hp_weight_map[full_weight_name]  # [out_dim, in_dim]
        quantized_weight, weight_scale = self.rollout.fp8_quantization(weight_to_quantize)
        model_param_map = self.rollout.model_param_map(self.weight_mapper)
        native = model_param_map[full_weight_name]
        if do_weight_sync_check:
            # allclose has no fp8 kernel: promote both sides
            if not torch.allclose(native.to(torch.bfloat16), quantized_weight.to(torch.bfloat16)):
                raise ValueError(
                    "FP8 weight doesn't match after weight sync and dynamic quantization for full weight "
                    f"name: {full_weight_name}.")
        native.copy_(quantized_weight)
        scale_key = full_weight_name.replace(".weight", ".weight_scale")
        scale_tensor = model_param_map[scale_key]
        assert scale_tensor.shape == weight_scale.shape, (
            f"scale_tensor.shape: {scale_tensor.shape}, weight_scale.shape: {weight_scale.shape}")
        scale_tensor.copy_(weight_scale)
        return True

    # -- rollout_control.py:1308-1319: the completions of a flush group, run together ---------------------
    def flush_completions(self, groups: Iterable[List[str]], do_weight_sync_check: bool = False) -> List[str]:
        """Quantise the full weights of several instruction groups whose shards have all landed, as the
        reference's ``flush_completions`` runs its queued completion lambdas together on the copy stream.
        Without the first-sync check the weights of the batch that share a row length go through ONE launch
        each way (``cfp8_quant_rowwise_multi``), straight from the staging parameters into the engine's fp8
        parameters and ``weight_scale`` tensors - same bytes as one ``quantize_full_weight`` per group.
        With the check every weight takes ``quantize_full_weight`` (the check compares old and new bytes).
        Returns the full weight names that were quantised."""
        from cosmos_rl_amd import ops

        names: List[str] = []
        for param_names in groups:
            if self.quantization_type is None or self.check_inside_group(param_names, do_weight_sync_check):
                continue
            full = self.full_weight_name_of_group(param_names)
            if self.quantization_type == "fp8" and full in self.hp_weight_map and full not in names:
                names.append(full)
        if do_weight_sync_check:
            for name in names:
                self.quantize_full_weight(name, True)
            return names
        model_param_map = self.rollout.model_param_map(self.weight_mapper)
        weights, natives, scales = [], [], []
        for name in names:
            weight = self.hp_weight_map[name]                            # [out_dim, in_dim]
            native = model_param_map[name]                               # [in_dim, out_dim], strides (1, in_dim)
            scale_tensor = model_param_map[name.replace(".weight", ".weight_scale")]
            assert tuple(scale_tensor.shape) == (weight.shape[0], 1), (
                f"scale_tensor.shape: {scale_tensor.shape}, weight_scale.shape: {(weight.shape[0], 1)}")
            weights.append(weight.data)
            natives.append(native.data)
            scales.append(scale_tensor.data)
        ops.quant_rowwise_multi_into(weights, natives, scales)
        return names

    # -- fused form of base.py:1053-1069 + rollout_control.py:856-898 --------------------------
    def quantize_received_rows(self, full_weight_name: str, recv_tensor: torch.Tensor, row_start: int = 0) -> bool:
        """Quantise a received shard that holds whole rows ``[row_start, row_start + n)`` of a weight
        straight into the engine's fp8 parameter and its ``weight_scale``: no cast into the bf16 staging
        parameter, no temporary fp8 tensor, no strided copies.  Rowwise scales depend on their own row
        only, so shards that split a weight along dim 0 (column-parallel layers, q/k/v and gate/up
        splits, unsharded weights) can each be quantised as they land.  Shards that split rows
        (row-parallel layers) must go through the staging parameter and ``quantize_full_weight``.
        The first-sync check of the reference compares old and new bytes and therefore needs the
        unfused path.  Returns False when the name is not a quantised weight."""
        from cosmos_rl_amd import ops

        if self.quantization_type != "fp8" or full_weight_name not in self.hp_weight_map:
            return False
        model_param_map = self.rollout.model_param_map(self.weight_mapper)
        native = model_param_map[full_weight_name]                       # [in_dim, out_dim], strides (1, in_dim)
        scale_tensor = model_param_map[full_weight_name.replace(".weight", ".weight_scale")]
        out_dim, in_dim = self.hp_weight_map[full_weight_name].shape
        n = recv_tensor.shape[0]
        if recv_tensor.dim() != 2 or recv_tensor.shape[1] != in_dim or row_start < 0 or row_start + n > out_dim:
            raise ValueError(
                f"received rows [{row_start}, {row_start + n}) x {tuple(recv_tensor.shape[1:])} do not fit "
                f"{full_weight_name} [{out_dim}, {in_dim}]")
        assert tuple(scale_tensor.shape) == (out_dim, 1), (
            f"scale_tensor.shape: {scale_tensor.shape}, weight_scale.shape: {(out_dim, 1)}")
        ops.quant_rowwise_into(recv_tensor, native[:, row_start:row_start + n], scale_tensor[row_start:row_start + n])
        return True
