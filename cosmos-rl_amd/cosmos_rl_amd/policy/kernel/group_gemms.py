"""Grouped-GEMM strategies for MoE experts with the interface of
cosmos_rl/policy/kernel/group_gemms.py (``GroupGEMMStrategy`` :32-69, ``TorchBF16GroupGEMM``
:80-118, ``DSGroupGEMM`` :121-233).  ``DSGroupGEMM`` runs 128x128 block-quantised weights,
1x128 group-quantised activations and the grouped FP8 MFMA GEMM of this library."""
from __future__ import annotations

import torch
import torch.nn as nn

from cosmos_rl_amd import _lib, ops

__all__ = ["GroupGEMMStrategy", "DSGroupGEMM", "TorchBF16GroupGEMM"]


class GroupGEMMStrategy:
    """Base class for group gemm strategies."""

    def __init__(self, custom_activation):
        self.activation_function = custom_activation

    def arrange_expert_weights(self, all_weights, submod_name, module):
        """Turn the per-expert weight list of ``submod_name`` ('gate_proj', 'up_proj',
        'down_proj') into the layout the strategy computes with; may register extra
        parameters on ``module``.  Returns the arranged weight tensor."""
        raise NotImplementedError("Requires arrange_expert_weights method")

    def execute(self, contig_tokens, m_sizes, m_offsets, module):
        """Run gate/up/activation/down over tokens laid out contiguously by expert."""
        raise NotImplementedError("GroupGEMM strategy must implement execute method")

    @staticmethod
    def is_available() -> bool:
        return False


class TorchBF16GroupGEMM(GroupGEMMStrategy):
    """bf16 baseline (group_gemms.py:80-118): ``torch._grouped_mm`` with int32 ``m_offsets``, which stay on the
    device; where this torch build has no grouped kernel for the operands (the CPU, notably) one matmul per
    expert group, which reads the offsets back."""

    _native = None  # None: not tried yet; True / False: torch._grouped_mm works / does not for these operands

    def arrange_expert_weights(self, all_weights, submod_name, module):
        return torch.stack(all_weights)

    @classmethod
    def _grouped(cls, x, w, m_offsets):
        if cls._native is not False and x.is_cuda and hasattr(torch, "_grouped_mm"):
            offs = m_offsets if m_offsets.dtype == torch.int32 else m_offsets.to(torch.int32)
            try:
                out = torch._grouped_mm(x, w.transpose(-2, -1), offs, out_dtype=torch.bfloat16)
                cls._native = True
                return out
            except (RuntimeError, NotImplementedError):
                if cls._native:
                    raise
                cls._native = False
        out = torch.zeros(x.shape[0], w.shape[1], dtype=torch.bfloat16, device=x.device)
        start = 0
        for e, end in enumerate(m_offsets.tolist()):
            if end > start:
                out[start:end] = x[start:end] @ w[e].t()
            start = end
        return out

    def execute(self, contig_tokens, m_sizes, m_offsets, module):
        w_gate = module.get_parameter("gate_proj_weight")
        w_up = module.get_parameter("up_proj_weight")
        w_down = module.get_parameter("down_proj_weight")
        hidden = self.activation_function(self._grouped(contig_tokens, w_gate, m_offsets)) * \
            self._grouped(contig_tokens, w_up, m_offsets)
        return self._grouped(hidden, w_down, m_offsets)

    @staticmethod
    def is_available() -> bool:
        return True


class DSGroupGEMM(GroupGEMMStrategy):
    """FP8 grouped GEMM: block-quantised expert weights, 1x128 activation groups."""

    def __init__(self, custom_activation, use_triton_quant=True, fuse_swiglu=True, fuse_gate_up=False, fuse_epilogue=True):
        # ``use_triton_quant`` selected between two third-party quantisers in the reference
        # (group_gemms.py:188-191); both map to the one HIP group quantiser here.
        # fuse_swiglu: when the activation is SiLU, ``act(gate) * up`` and the 1x128 quantisation of the
        # product (group_gemms.py:209-218) run as one kernel and the bf16 product is never written.
        # fuse_gate_up: the gate and up projections (two GEMMs on the same input, :194-207) run as one
        # GEMM over the concatenated weights; costs a second copy of those weights.
        # With both, the intermediate size a multiple of 128 and token rows padded to 128, the SwiGLU and
        # the quantisation become the epilogue of that one GEMM (weights interleaved in 128-row blocks of
        # gate and up): the [rows, 2 I] product never reaches memory.  Same bits as the unfused chain.
        # ``fuse_epilogue=False`` keeps the GEMM and the SwiGLU quantiser as two launches.
        self.activation_function = custom_activation
        self.use_triton_quant = use_triton_quant
        self.fuse_swiglu = fuse_swiglu and self._is_silu(custom_activation)
        self.fuse_gate_up = fuse_gate_up
        self.fuse_epilogue = fuse_epilogue

    @staticmethod
    def _is_silu(fn) -> bool:
        return isinstance(fn, nn.SiLU) or fn is torch.nn.functional.silu

    def arrange_expert_weights(self, all_weights, submod_name, module):
        combined_weights = torch.stack(all_weights)
        fp8, scales = ops.prepare_fp8_weight(combined_weights)
        module.register_parameter(f"{submod_name}_fp8", nn.Parameter(fp8, requires_grad=False))
        module.register_parameter(f"{submod_name}_scales", nn.Parameter(scales, requires_grad=False))
        self.invalidate_fused_weights(module)
        return combined_weights

    def _quant(self, x):
        return ops.groupwise_activation_quant(x) if self.use_triton_quant else ops.prepare_fp8_input(x)

    def execute(self, contig_tokens, m_sizes, m_offsets, module):
        rows = contig_tokens.shape[0]
        if rows % ops.BLOCK == 0 and contig_tokens.is_contiguous():
            # The row count of the buffer already bounds the valid rows (group_gemms.py:154 slices it with
            # m_offsets[-1], a host read-back): every row is quantised, rows past the last group get expert -1,
            # which the GEMMs skip, and the down projection writes straight into ``contig_tokens`` - the rows the
            # reference's final copy (:228) leaves alone stay untouched, and nothing waits for the device.
            m_indices = ops.create_indices_from_offsets_nosync(m_offsets, rows, n_experts=m_offsets.numel())
            self._run(self._quant(contig_tokens), m_indices, rows, module, contig_tokens.dtype, out=contig_tokens)
            return contig_tokens
        total = int(m_offsets[-1])
        valid_tokens = contig_tokens[:total]
        m_indices = ops.create_indices_from_offsets_nosync(m_offsets, total)
        contig_tokens[:total] = self._run(self._quant(valid_tokens), m_indices, total, module, contig_tokens.dtype)
        return contig_tokens

    def execute_from_tokens(self, tokens, row_tokens, m_sizes, m_offsets, module, row_map=None):
        """``execute`` on ``tokens[row_tokens]`` (zero rows for -1) without building that matrix: the gather and the
        1x128 quantisation of the first GEMM's input are one pass over the token matrix.  Returns the expert outputs
        [rows, hidden] for the rows of the expert-grouped layout (``row_tokens``: token behind each row).  When
        ``row_tokens`` has a multiple of 128 entries (a capacity bound, as ``route_tokens`` returns) nothing is read
        back from the device: rows past the last group are padding to the GEMMs and come back as zeros.
        ``row_map`` (``TokenRouting.row_map``: the rows of every token) lets the pass quantise each token once and
        store it to all its rows instead of once per row; same bits."""
        from cosmos_rl_amd.policy.kernel.moe.indices import permute_quantize_tokens
        rows = row_tokens.numel()
        if rows % ops.BLOCK == 0:
            m_indices = ops.create_indices_from_offsets_nosync(m_offsets, rows, n_experts=m_offsets.numel())
            hidden_size = module.get_parameter("down_proj_weight").shape[1]
            out = torch.zeros((rows, hidden_size), device=tokens.device, dtype=tokens.dtype)
            return self._run(permute_quantize_tokens(tokens, row_tokens, row_map), m_indices, rows, module, tokens.dtype, out=out)
        total = int(m_offsets[-1])
        m_indices = ops.create_indices_from_offsets_nosync(m_offsets, total)
        # (rows of row_map at or past `total` would be padding; the scatter form skips rows beyond its output)
        return self._run(permute_quantize_tokens(tokens, row_tokens[:total], row_map), m_indices, total, module, tokens.dtype)

    @staticmethod
    def _weights_key(*tensors):
        # address and in-place version of every tensor a fused copy was built from: an in-place update (copy_,
        # load_state_dict) keeps the address and bumps the version.  A write through ``tensor.data`` bumps nothing:
        # whoever updates the expert weights that way calls ``invalidate_fused_weights`` afterwards.
        return tuple((t.data_ptr(), t._version) for t in tensors)

    @staticmethod
    def invalidate_fused_weights(module) -> None:
        """Drop the fused / interleaved copies of the gate and up weights kept on ``module``; the next ``execute``
        rebuilds them.  ``arrange_expert_weights`` calls it, so re-arranged weights are always picked up."""
        for attr in ("_gate_up_fp8_interleaved", "_gate_up_fp8_fused"):
            if hasattr(module, attr):
                delattr(module, attr)

    def _run(self, gate_up_input, m_indices, total, module, dt, out=None):
        """gate/up GEMMs, activation, requantisation, down GEMM on the quantised expert-grouped rows; the result
        goes to ``out`` ([total, hidden], rows of padding untouched) when given"""

        gate_fp8, gate_s = module.get_parameter("gate_proj_fp8"), module.get_parameter("gate_proj_scales")
        up_fp8, up_s = module.get_parameter("up_proj_fp8"), module.get_parameter("up_proj_scales")
        down_fp8, down_s = module.get_parameter("down_proj_fp8"), module.get_parameter("down_proj_scales")

        intermediate_size = module.get_parameter("gate_proj_weight").shape[1]
        hidden_size = module.get_parameter("down_proj_weight").shape[1]
        dev = gate_up_input[0].device

        down_out = out if out is not None else torch.empty((total, hidden_size), device=dev, dtype=dt)
        # padding rows (m_indices < 0) are not written by the GEMMs: start from zeros so that what the
        # activation reads there is defined
        hidden_quantized = None
        if self.fuse_gate_up and self.fuse_swiglu and self.fuse_epilogue and intermediate_size % 128 == 0 and total % 128 == 0:
            key = self._weights_key(gate_fp8, up_fp8, gate_s, up_s)
            inter = getattr(module, "_gate_up_fp8_interleaved", None)
            if inter is None or inter[2] != key:
                inter = (*ops.interleave_gate_up((gate_fp8, gate_s), (up_fp8, up_s)), key)
                module._gate_up_fp8_interleaved = inter
            hidden_quantized = ops.grouped_gemm_swiglu_quant(gate_up_input, (inter[0], inter[1]), m_indices)
        elif self.fuse_gate_up and intermediate_size % 128 == 0:
            key = self._weights_key(gate_fp8, up_fp8, gate_s, up_s)
            fused = getattr(module, "_gate_up_fp8_fused", None)
            if fused is None or fused[2] != key:
                fused = (torch.cat([gate_fp8, up_fp8], dim=1), torch.cat([gate_s, up_s], dim=1), key)
                module._gate_up_fp8_fused = fused
            gate_up_out = torch.zeros((total, 2 * intermediate_size), device=dev, dtype=dt)
            ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(gate_up_input, (fused[0], fused[1]), gate_up_out, m_indices)
            gate_out, up_out = gate_up_out[:, :intermediate_size], gate_up_out[:, intermediate_size:]
        else:
            gate_out = torch.zeros((total, intermediate_size), device=dev, dtype=dt)
            up_out = torch.zeros_like(gate_out)
            ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(gate_up_input, (gate_fp8, gate_s), gate_out, m_indices)
            ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(gate_up_input, (up_fp8, up_s), up_out, m_indices)
        if hidden_quantized is not None:
            pass
        elif self.fuse_swiglu:
            hidden_quantized = ops.swiglu_quant(gate_out, up_out)
        else:
            hidden_quantized = self._quant(self.activation_function(gate_out) * up_out)
        ops.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(hidden_quantized, (down_fp8, down_s), down_out, m_indices)
        return down_out

    @staticmethod
    def is_available() -> bool:
        if not _lib.LIB_PATH.exists() or not torch.cuda.is_available():
            return False
        name = getattr(torch.cuda.get_device_properties(torch.cuda.current_device()), "gcnArchName", "")
        return name.startswith("gfx950")
