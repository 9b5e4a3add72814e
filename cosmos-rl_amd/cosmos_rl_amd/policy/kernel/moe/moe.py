"""Token routing around the grouped experts - counterpart of ``GroupedExperts.forward`` in
cosmos_rl/policy/kernel/moe/moe.py:179-285.

The reference loops over experts: gather the expert's tokens, run its MLP, multiply by the routing
weight, ``scatter_add_`` into ``y``.  Here all experts run as one grouped GEMM, so the loop becomes
three steps: ``route_tokens`` lays the (token, slot) pairs out by expert, ``permute_tokens`` +
``GroupGEMMStrategy.execute`` compute every expert row, and ``combine_expert_outputs`` accumulates each
token's rows in ascending expert order with the same bf16 roundings as the loop - the result is bit for
bit what the loop gives for the same expert rows.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

from cosmos_rl_amd import _lib
from cosmos_rl_amd.policy.kernel.moe.indices import generate_permute_indices, permute_tokens

__all__ = ["TokenRouting", "route_tokens", "combine_expert_outputs", "grouped_experts_forward"]


@dataclass
class TokenRouting:
    row_tokens: torch.Tensor   # int32 [rows]: token that feeds each row of the expert-grouped matrix, -1 = padding
    row_map: torch.Tensor      # int32 [tokens, topk]: row of each (token, slot), slots by ascending expert, -1 = masked
    slot_order: torch.Tensor   # int64 [tokens, topk]: the slot permutation behind row_map (apply it to the weights)
    m_sizes: torch.Tensor      # int32 [experts]: padded group sizes
    m_offsets: torch.Tensor    # int32 [experts]: their inclusive cumulative sum


def route_tokens(indices: torch.Tensor, token_mask: Optional[torch.Tensor], n_experts: int, alignment: int = 128,
                 max_rows: Optional[int] = None) -> TokenRouting:
    """Expert-grouped layout of the routed (token, slot) pairs: groups in expert order, tokens ascending
    inside a group (the order ``torch.where`` gives the reference, moe.py:244-245), every group padded to
    ``alignment`` rows.  No host synchronisation: the row count is the bound ``max_rows`` (default
    tokens * topk + n_experts * alignment); rows past the real end are padding."""
    if indices.dim() != 2 or not indices.is_cuda:
        raise ValueError("indices must be a [tokens, topk] GPU tensor")
    T, K = indices.shape
    dev = indices.device
    idx64 = indices.to(torch.int64)
    if token_mask is not None:
        idx64 = torch.where(token_mask.to(torch.bool).unsqueeze(-1), idx64, torch.full_like(idx64, n_experts))
    key = idx64.reshape(-1)                                   # masked slots fall into a bin past the last expert
    order = torch.argsort(key, stable=True)
    # (torch.bincount reads its result size back from the device; a scatter-add does not, so this can be graph-captured)
    counts = torch.zeros(n_experts + 1, dtype=torch.int64, device=dev).scatter_add_(0, key, torch.ones_like(key))[:n_experts]
    capacity = int(max_rows) if max_rows is not None else T * K + n_experts * alignment
    permuted, m_sizes, m_offsets = generate_permute_indices(counts, n_experts, 1, alignment, max_len=capacity)
    valid_row = permuted >= 0
    src_slot = order[permuted.clamp_min(0).to(torch.int64)]  # flat (token, slot) behind every row
    row_tokens = torch.where(valid_row, (src_slot // K).to(torch.int32), torch.full_like(permuted, -1))
    row_of_slot = torch.full((T * K + 1,), -1, dtype=torch.int32, device=dev)
    row_of_slot.scatter_(0, torch.where(valid_row, src_slot, torch.full_like(src_slot, T * K)),
                         torch.arange(capacity, dtype=torch.int32, device=dev))
    row_of_slot[T * K:].fill_(-1)                             # the slot that caught the padding rows
    _, slot_order = torch.sort(idx64, dim=1, stable=True)
    row_map = torch.gather(row_of_slot[:T * K].view(T, K), 1, slot_order).contiguous()
    return TokenRouting(row_tokens, row_map, slot_order, m_sizes, m_offsets)


def combine_expert_outputs(expert_out: torch.Tensor, routing: TokenRouting, weights: torch.Tensor,
                           accumulate: str = "bf16") -> torch.Tensor:
    """y[t] = sum over the token's experts, ascending, of weights[t, slot] * expert_out[row].

    ``accumulate="bf16"`` rounds every product and partial sum to bf16 like ``expert_out * weights[idx, top,
    None]`` followed by ``y.scatter_add_`` (moe.py:259-263); ``"fp32"`` keeps an fp32 accumulator like the
    un-permute kernel of megatron_moe/permutation.py:336-428."""
    if expert_out.dtype != torch.bfloat16 or expert_out.dim() != 2 or expert_out.stride(1) != 1 or not expert_out.is_cuda:
        raise ValueError("expert_out must be a 2-D bf16 GPU tensor with unit column stride")
    T, K = routing.row_map.shape
    if weights.shape != (T, K):
        raise ValueError(f"weights must be [{T}, {K}]")
    w = torch.gather(weights, 1, routing.slot_order)
    if accumulate == "bf16":
        mode, w, wd = _lib.COMBINE_BF16_STEPS, w.to(torch.bfloat16).contiguous(), _lib.IN_BF16
    elif accumulate == "fp32":
        mode = _lib.COMBINE_F32
        if w.dtype == torch.bfloat16:
            w, wd = w.contiguous(), _lib.IN_BF16
        else:
            w, wd = w.to(torch.float32).contiguous(), _lib.IN_F32
    else:
        raise ValueError("accumulate must be 'bf16' or 'fp32'")
    H = expert_out.shape[1]
    out = torch.empty((T, H), dtype=torch.bfloat16, device=expert_out.device)
    _lib.check(_lib.load().cfp8_combine_rows(expert_out.data_ptr(), expert_out.stride(0), expert_out.shape[0],
                                             routing.row_map.data_ptr(), w.data_ptr(), wd, T, K, H, mode,
                                             out.data_ptr(), H, torch.cuda.current_stream().cuda_stream))
    return out


def grouped_experts_forward(x: torch.Tensor, token_mask: Optional[torch.Tensor], weights: torch.Tensor,
                            indices: torch.Tensor, strategy, module, n_experts: int, alignment: int = 128) -> torch.Tensor:
    """``GroupedExperts.forward(x, token_mask, weights, indices)`` (moe.py:179-285) on one rank, with the
    experts of ``module`` run by ``strategy`` (a ``GroupGEMMStrategy``) instead of the per-expert loop."""
    routing = route_tokens(indices, token_mask, n_experts, alignment)
    if hasattr(strategy, "execute_from_tokens") and x.dtype == torch.bfloat16:
        # the FP8 strategy quantises while it gathers: the expert-grouped bf16 copy of the tokens is never built
        out = strategy.execute_from_tokens(x, routing.row_tokens, routing.m_sizes, routing.m_offsets, module, row_map=routing.row_map)
    else:
        contig = permute_tokens(x, routing.row_tokens)
        out = strategy.execute(contig, routing.m_sizes, routing.m_offsets, module)
    return combine_expert_outputs(out, routing, weights)
