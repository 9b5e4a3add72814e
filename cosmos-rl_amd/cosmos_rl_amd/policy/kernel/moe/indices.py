"""Expert-grouping permutation indices - counterpart of cosmos_rl/policy/kernel/moe/indices.py.

Same entry point and return values as the reference's ``generate_permute_indices`` (:147-220); the
Triton fill kernel and the torch prefix sums around it (:24-118, :174-196) are one call into the HIP
library (two launches, no intermediate tensors).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from cosmos_rl_amd import _lib

__all__ = ["generate_permute_indices", "permute_tokens", "permute_quantize_tokens"]


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def generate_permute_indices(tokens_per_expert_group: torch.Tensor, experts_per_rank: int, num_ranks: int,
                             alignment: int, use_cpu: bool = False, max_len: Optional[int] = None
                             ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (permuted_indices, m_sizes, m_offsets) as indices.py:147-220 does.

    permuted_indices has ``sum(m_sizes)`` entries like the reference's (which reads that sum back to
    size its output, :194-196).  Pass ``max_len`` (any bound >= sum(m_sizes), e.g. tokens + experts *
    alignment) to get a tensor of that length instead, -1 past the end, with no host synchronisation.
    ``use_cpu`` selected a python loop in the reference; there is no CPU path here."""
    if use_cpu or not tokens_per_expert_group.is_cuda:
        raise RuntimeError("generate_permute_indices runs on the GPU only")
    if tokens_per_expert_group.numel() != experts_per_rank * num_ranks:
        raise ValueError(f"expected {experts_per_rank * num_ranks} counts, got {tokens_per_expert_group.numel()}")
    dev = tokens_per_expert_group.device
    counts = tokens_per_expert_group.to(torch.int64).contiguous()
    m_sizes = torch.empty(experts_per_rank, dtype=torch.int32, device=dev)
    m_offsets = torch.empty(experts_per_rank, dtype=torch.int32, device=dev)
    start = torch.empty(experts_per_rank * num_ranks, dtype=torch.int64, device=dev)
    lib = _lib.load()
    if max_len is None:
        # sizes first (capacity 0 skips the fill), one read-back, then the fill at the exact length
        _lib.check(lib.cfp8_generate_permute_indices(counts.data_ptr(), experts_per_rank, num_ranks, alignment,
                                                     None, 0, m_sizes.data_ptr(), m_offsets.data_ptr(),
                                                     start.data_ptr(), _stream()))
        capacity = int(m_offsets[-1])
    else:
        capacity = int(max_len)
    out = torch.empty(capacity, dtype=torch.int32, device=dev)
    _lib.check(lib.cfp8_generate_permute_indices(counts.data_ptr(), experts_per_rank, num_ranks, alignment,
                                                 out.data_ptr(), capacity, m_sizes.data_ptr(), m_offsets.data_ptr(),
                                                 start.data_ptr(), _stream()))
    return out, m_sizes, m_offsets


def permute_tokens(tokens: torch.Tensor, permuted_indices: torch.Tensor) -> torch.Tensor:
    """``tokens[permuted_indices]`` with zero rows where the index is -1: the contiguous, padded,
    expert-grouped matrix that GroupGEMMStrategy.execute takes (group_gemms.py:152-156)."""
    if not tokens.is_cuda or tokens.dim() != 2 or tokens.stride(1) != 1:
        raise ValueError("expected a 2-D GPU tensor with unit column stride")
    row_bytes = tokens.shape[1] * tokens.element_size()
    out = torch.empty((permuted_indices.numel(), tokens.shape[1]), dtype=tokens.dtype, device=tokens.device)
    idx = permuted_indices.to(torch.int32).contiguous()
    _lib.check(_lib.load().cfp8_gather_rows(tokens.data_ptr(), tokens.stride(0) * tokens.element_size(), idx.data_ptr(),
                                            idx.numel(), row_bytes, out.data_ptr(), row_bytes, _stream()))
    return out


def permute_quantize_tokens(tokens: torch.Tensor, permuted_indices: torch.Tensor,
                            row_map: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """``groupwise_activation_quant(tokens[permuted_indices])`` (zero rows for -1) in one pass: the 1x128-quantised
    input of the first grouped GEMM (group_gemms.py:188-191) straight from the token matrix, without the gathered
    bf16 copy.  Returns (fp8 [rows, H], fp32 [rows, ceil(H/128)]).

    ``row_map`` (int32 [tokens, topk], the rows each token feeds, -1 for none: ``TokenRouting.row_map``) selects the
    scatter form, which quantises every token once and stores the result to all of its rows - same bits, an eighth
    of the reads and of the arithmetic at top-8.  It must describe the same layout as ``permuted_indices``."""
    if not tokens.is_cuda or tokens.dim() != 2 or tokens.stride(1) != 1 or tokens.dtype != torch.bfloat16:
        raise ValueError("expected a 2-D bf16 GPU tensor with unit column stride")
    H = tokens.shape[1]
    idx = permuted_indices.to(torch.int32).contiguous()
    q = torch.empty((idx.numel(), H), dtype=torch.float8_e4m3fn, device=tokens.device)
    s = torch.empty((idx.numel(), (H + 127) // 128), dtype=torch.float32, device=tokens.device)
    if row_map is not None:
        if row_map.dim() != 2 or row_map.shape[0] != tokens.shape[0] or row_map.dtype != torch.int32 or not row_map.is_cuda:
            raise ValueError(f"row_map must be an int32 GPU tensor [tokens, topk], got {tuple(row_map.shape)} {row_map.dtype}")
        rm = row_map.contiguous()
        _lib.check(_lib.load().cfp8_scatter_quant_group128(tokens.data_ptr(), tokens.stride(0), tokens.shape[0], H, rm.data_ptr(),
                                                          rm.shape[1], idx.data_ptr(), idx.numel(), q.data_ptr(), H, s.data_ptr(),
                                                          _stream()))
        return q, s
    _lib.check(_lib.load().cfp8_gather_quant_group128(tokens.data_ptr(), tokens.stride(0), idx.data_ptr(), idx.numel(), H,
                                                     q.data_ptr(), H, s.data_ptr(), _stream()))
    return q, s
