"""CPU oracle for the expert-grouping index generation.  TEST INFRASTRUCTURE ONLY (imported by
tests/ alone; the shipped package never comes here).

Restates the CPU path of cosmos_rl/policy/kernel/moe/indices.py: ``generate_permute_indices``
(:147-220) with ``fill_indices_cpu`` (:112-144).  Pinned in tests/test_moe_indices.py by the two
cases the reference's own self-tests use (:225-261 all counts 4, alignment 32; :264-330 counts
[4,0,2,3,1,0,0,5], alignment 8, with their assertions: sizes are multiples of the alignment, an expert
without tokens gets `alignment` slots all -1), by the worked example of the docstring (:166-171), and
by ``brute_force`` below, which builds the same answer from explicit python lists with no prefix sums.

``grouped_experts_combine`` restates the output side of ``GroupedExperts.forward``
(cosmos_rl/policy/kernel/moe/moe.py:240-262) with the expert MLP replaced by given rows; it is pinned
by the scalar C restatement ``fp8ref_combine_rows`` (explicit bf16 rounding of every product and partial
sum, rounding by neighbour search in double arithmetic) in tests/test_moe_indices.py.
"""
from __future__ import annotations

from typing import List, Tuple

import torch


def generate_permute_indices(tokens_per_expert_group: torch.Tensor, experts_per_rank: int, num_ranks: int,
                             alignment: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """(permuted_indices int32 [sum(m_sizes)], m_sizes int32 [E], m_offsets int32 [E])."""
    counts = tokens_per_expert_group.to(torch.int64).cpu()
    start_index_values = torch.cumsum(counts, 0) - counts                      # indices.py:175-177
    total = counts.view(num_ranks, -1).sum(0)                                  # :180
    total = torch.clamp_min(total, alignment)                                  # :183
    m_sizes = ((total + alignment - 1) // alignment * alignment).to(torch.int32)  # :186-188
    m_offsets = torch.cumsum(m_sizes, 0)                                       # :191
    write_offsets = m_offsets - m_sizes
    total_size = int(m_offsets[-1])
    out = torch.full((total_size,), -1, dtype=torch.int32)                     # :122-126
    for e in range(experts_per_rank):                                          # :129-143
        write_start = int(write_offsets[e])
        for r in range(num_ranks):
            i = r * experts_per_rank + e
            start, length = int(start_index_values[i]), int(counts[i])
            if length > 0:
                end = min(write_start + length, total_size)
                out[write_start:end] = torch.arange(start, start + (end - write_start), dtype=torch.int32)
            write_start += length
    return out, m_sizes, m_offsets.to(torch.int32)


def brute_force(counts: List[int], experts_per_rank: int, num_ranks: int, alignment: int) -> List[int]:
    """The same permutation from first principles: number the incoming rows 0.. in (rank, expert) order, hand
    each row to its expert, lay the experts out one after the other, pad each to the alignment (at least one
    aligned block) with -1."""
    rows_of_expert: List[List[int]] = [[] for _ in range(experts_per_rank)]
    row = 0
    for r in range(num_ranks):
        for e in range(experts_per_rank):
            for _ in range(counts[r * experts_per_rank + e]):
                rows_of_expert[e].append(row)
                row += 1
    out: List[int] = []
    for e in range(experts_per_rank):
        n = max(len(rows_of_expert[e]), alignment)
        n = -(-n // alignment) * alignment
        out.extend(rows_of_expert[e] + [-1] * (n - len(rows_of_expert[e])))
    return out


def grouped_experts_combine(expert_rows: List[torch.Tensor], token_mask: torch.Tensor, weights: torch.Tensor,
                            indices: torch.Tensor, hidden: int) -> torch.Tensor:
    """y [T, hidden] as GroupedExperts.forward builds it (moe.py:240-262), where expert_rows[i] stands for
    ``swiglu(x_idx, ...)`` of expert i: one row per token routed to it, tokens in ascending order."""
    T = indices.shape[0]
    y = torch.zeros(T, hidden, dtype=expert_rows[0].dtype if expert_rows else weights.dtype)  # :240
    for i in range(len(expert_rows)):                                                       # :243
        indices_mask = torch.logical_and(indices == i, token_mask.unsqueeze(-1))           # :244
        idx, top = torch.where(indices_mask)                                                # :245
        if idx.numel() == 0:                                                                # :247
            continue
        idx_b = idx[:, None].expand(-1, hidden)                                             # :256
        expert_out = expert_rows[i] * weights[idx, top, None]                               # :259-261
        y.scatter_add_(dim=0, index=idx_b, src=expert_out)                                  # :263
    return y
