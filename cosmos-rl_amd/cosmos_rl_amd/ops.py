"""Torch-facing operators of the FP8 hot path, named after the third-party ops the
reference calls, each a thin shim over one C-ABI entry point.

The shim allocates every output and workspace as a torch tensor, passes raw
device pointers plus the current HIP stream, and never synchronises.  Inputs
must live on the GPU; nothing here computes on the CPU.
"""
from __future__ import annotations

import contextlib
import ctypes
from typing import List, Optional, Sequence, Tuple

import torch

from . import _lib

FP8_DTYPE = torch.float8_e4m3fn
FP8_MAX = 448.0
BLOCK = 128


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _need_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError(
                "cosmos_fp8 operators run on the GPU only (got a tensor on "
                f"{t.device}); there is no CPU path")


def _ptr(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _out_code(dtype: torch.dtype) -> int:
    if dtype == torch.bfloat16:
        return _lib.OUT_BF16
    if dtype == torch.float32:
        return _lib.OUT_F32
    raise ValueError(f"out_dtype must be bfloat16 or float32, got {dtype}")


# ---------------------------------------------------------------------------
# quantizers
# ---------------------------------------------------------------------------
def scaled_fp8_quant(input: torch.Tensor, scale: Optional[torch.Tensor] = None,
                     use_per_token_if_dynamic: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dynamic FP8 quantisation with the call shape of ``vllm._custom_ops.scaled_fp8_quant``
    (reference call sites: cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:995-997,
    monkey_patch_for_fp8.py:47-49).

    ``use_per_token_if_dynamic=True``: one scale per row, returns (fp8 [R, C], fp32 [R, 1]).
    ``False``: one scale for the tensor, returns (fp8 [R, C], fp32 [1]).
    Static scales (``scale`` given) are not part of this path.
    """
    if scale is not None:
        raise NotImplementedError("static-scale quantisation is not on the cosmos-rl FP8 path")
    if input.dim() != 2:
        raise ValueError(f"expected a 2-D tensor, got {tuple(input.shape)}")
    if not use_per_token_if_dynamic:
        q, s = quant_tensorwise(input)
        return q, s
    return quant_rowwise(input)


def quant_rowwise(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    _need_gpu(x)
    if x.dtype != torch.bfloat16:
        raise ValueError(f"rowwise FP8 quantisation takes bfloat16 input, got {x.dtype}")
    if x.dim() != 2:
        raise ValueError(f"expected a 2-D tensor, got {tuple(x.shape)}")
    if x.stride(1) != 1 and x.shape[1] > 1:
        x = x.contiguous()
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=FP8_DTYPE, device=x.device)
    s = torch.empty((rows, 1), dtype=torch.float32, device=x.device)
    ld_x = x.stride(0) if rows > 1 else max(cols, 1)
    _lib.check(_lib.load().cfp8_quant_rowwise(x.data_ptr(), rows, cols, ld_x, q.data_ptr(), cols,
                                             s.data_ptr(), _stream()))
    return q, s


_IN_DTYPE = {torch.bfloat16: _lib.IN_BF16, torch.float16: _lib.IN_F16, torch.float32: _lib.IN_F32}


def quant_rowwise_into(recv: torch.Tensor, q_out: torch.Tensor, scale_out: torch.Tensor) -> None:
    """Rowwise quantisation of ``recv.to(bfloat16)`` written straight into caller-owned storage.

    One kernel for what the reference does in three passes when a received shard holds whole rows of
    a weight: the dtype cast into the bf16 staging view (cosmos_rl/policy/model/base.py:1053-1069),
    ``fp8_quantization`` (vllm_rollout.py:989-999) and the copies into the engine's weight and
    ``weight_scale`` parameters (rollout_control.py:889-898).

    recv       [R, C] bf16 / fp16 / fp32, unit stride along C
    q_out      fp8 storage of the same logical shape, given row-major: either an [R, C] tensor with
               unit stride along C, or the engine's transposed parameter ``[C, R]`` with strides
               ``(1, pitch)`` (the ``.t()`` view of a row-major buffer, monkey_patch_for_fp8.py:52)
    scale_out  fp32 [R, 1] or [R], contiguous
    """
    _need_gpu(recv, q_out, scale_out)
    if recv.dim() != 2 or recv.dtype not in _IN_DTYPE:
        raise ValueError(f"expected a 2-D bf16/fp16/fp32 tensor, got {tuple(recv.shape)} {recv.dtype}")
    if q_out.dtype != FP8_DTYPE or scale_out.dtype != torch.float32:
        raise ValueError("q_out must be float8_e4m3fn and scale_out float32")
    rows, cols = recv.shape
    q_rm = _row_major_q(q_out, rows, cols)
    if scale_out.numel() != rows or not scale_out.is_contiguous():
        raise ValueError(f"scale_out must hold {rows} contiguous floats, got {tuple(scale_out.shape)}")
    if recv.stride(1) != 1 and cols > 1:
        recv = recv.contiguous()
    ld_x = recv.stride(0) if rows > 1 else max(cols, 1)
    ld_q = q_rm.stride(0) if rows > 1 else max(cols, 1)
    _lib.check(_lib.load().cfp8_quant_rowwise_from(recv.data_ptr(), _IN_DTYPE[recv.dtype], rows, cols, ld_x,
                                                  q_rm.data_ptr(), ld_q, scale_out.data_ptr(), _stream()))


def _row_major_q(q_out: torch.Tensor, rows: int, cols: int) -> torch.Tensor:
    """The [rows, cols] row-major view of fp8 storage given either that way or as the engine's
    transposed parameter [cols, rows] with strides (1, pitch)."""
    if q_out.dim() == 2 and tuple(q_out.shape) == (rows, cols) and (q_out.stride(1) == 1 or cols == 1):
        return q_out
    if q_out.dim() == 2 and tuple(q_out.shape) == (cols, rows) and (q_out.stride(0) == 1 or cols == 1):
        return q_out.t()
    raise ValueError(f"q_out {tuple(q_out.shape)} strides {q_out.stride()} is not row-major storage for {(rows, cols)}")


def quant_rowwise_multi_into(recvs: Sequence[torch.Tensor], q_outs: Sequence[torch.Tensor],
                             scale_outs: Sequence[torch.Tensor]) -> None:
    """``quant_rowwise_into`` for a batch of weights in as few launches as their shapes allow (weights of one
    row length and dtype share a launch): the completions a weight sync runs together once their shards have
    landed (cosmos_rl/rollout/worker/rollout_control.py:1308-1319).  Same bits as per-weight calls."""
    n = len(recvs)
    if len(q_outs) != n or len(scale_outs) != n:
        raise ValueError("one output and one scale tensor per weight")
    if n == 0:
        return
    _need_gpu(*recvs, *q_outs, *scale_outs)
    descs = (_lib.RowwiseDesc * n)()
    keep = []
    for i, (recv, q_out, scale_out) in enumerate(zip(recvs, q_outs, scale_outs)):
        if recv.dim() != 2 or recv.dtype not in _IN_DTYPE:
            raise ValueError(f"weight {i}: expected a 2-D bf16/fp16/fp32 tensor, got {tuple(recv.shape)} {recv.dtype}")
        if q_out.dtype != FP8_DTYPE or scale_out.dtype != torch.float32:
            raise ValueError(f"weight {i}: q_out must be float8_e4m3fn and scale_out float32")
        rows, cols = recv.shape
        q_rm = _row_major_q(q_out, rows, cols)
        if scale_out.numel() != rows or not scale_out.is_contiguous():
            raise ValueError(f"weight {i}: scale_out must hold {rows} contiguous floats, got {tuple(scale_out.shape)}")
        if recv.stride(1) != 1 and cols > 1:
            recv = recv.contiguous()
        keep.append(recv)
        d = descs[i]
        d.x, d.q, d.scales = recv.data_ptr(), q_rm.data_ptr(), scale_out.data_ptr()
        d.rows, d.cols = rows, cols
        d.ld_x = recv.stride(0) if rows > 1 else max(cols, 1)
        d.ld_q = q_rm.stride(0) if rows > 1 else max(cols, 1)
        d.x_dtype = _IN_DTYPE[recv.dtype]
    _lib.check(_lib.load().cfp8_quant_rowwise_multi(descs, n, _stream()))


def quant_rowwise_multi(tensors: Sequence[torch.Tensor]) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """Rowwise quantisation of a list of 2-D weights; returns (fp8 tensors [R, C], fp32 scales [R, 1])."""
    qs = [torch.empty(t.shape, dtype=FP8_DTYPE, device=t.device) for t in tensors]
    ss = [torch.empty((t.shape[0], 1), dtype=torch.float32, device=t.device) for t in tensors]
    quant_rowwise_multi_into(tensors, qs, ss)
    return qs, ss


@contextlib.contextmanager
def gpu_is_mine():
    """While active, ``quant_tensorwise_multi`` may use the launch that reads large tensors once and needs every
    compute unit of the GPU at the same time (``cfp8_tensorwise_resident``).  For a process that owns the GPU while
    it quantises, e.g. a trainer casting its weights; process-wide, restores the previous setting on exit."""
    lib = _lib.load()
    prev = lib.cfp8_tensorwise_resident(1)
    try:
        yield
    finally:
        lib.cfp8_tensorwise_resident(prev)


def quant_tensorwise_multi(tensors: Sequence[torch.Tensor], return_status: bool = False):
    """Tensorwise dynamic quantisation of a list of bf16 tensors in two launches per
    batch.  Returns (list of fp8 tensors shaped like the inputs, fp32 scales [n]); with ``return_status`` also a
    device int32 scalar, the number of tensors that the read-once launch (see ``gpu_is_mine``) gave up and the
    two ordinary passes redid - nonzero means that the GPU was not the caller's alone; results are right either way."""
    n = len(tensors)
    if n == 0:
        empty = ([], torch.empty(0, dtype=torch.float32))
        return (*empty, torch.zeros((), dtype=torch.int32)) if return_status else empty
    _need_gpu(*tensors)
    dev = tensors[0].device
    scales = torch.empty(n, dtype=torch.float32, device=dev)
    amax_ws = torch.empty(n * _lib.TENSORWISE_AMAX_SLOTS, dtype=torch.float32, device=dev)
    outs: List[torch.Tensor] = []
    keep = []
    descs = (_lib.TensorDesc * n)()
    sbase = scales.data_ptr()
    for i, t in enumerate(tensors):
        if t.dtype != torch.bfloat16:
            raise ValueError(f"tensorwise FP8 quantisation takes bfloat16 input, got {t.dtype}")
        tc = t if t.is_contiguous() else t.contiguous()
        keep.append(tc)
        q = torch.empty(t.shape, dtype=FP8_DTYPE, device=dev)
        outs.append(q)
        descs[i].x = tc.data_ptr()
        descs[i].q = q.data_ptr()
        descs[i].scale = sbase + 4 * i
        descs[i].numel = tc.numel()
    _lib.check(_lib.load().cfp8_quant_tensorwise_multi(descs, n, amax_ws.data_ptr(), _stream()))
    if return_status:
        given_up = torch.empty((), dtype=torch.int32, device=dev)
        _lib.check(_lib.load().cfp8_tensorwise_status(amax_ws.data_ptr(), n, given_up.data_ptr(), _stream()))
        return outs, scales, given_up
    return outs, scales


def quant_tensorwise_multi_static(tensors: Sequence[torch.Tensor], outs: Sequence[torch.Tensor],
                                  scales: torch.Tensor) -> None:
    """``quant_tensorwise_multi`` into caller-owned ``outs`` (fp8, shaped like the inputs, contiguous)
    and ``scales`` (fp32 [n]) through the entry point that allocates nothing: the amax slots are the
    library's own fixed device array, so at most ``_lib.TENSORWISE_STATIC_MAX_TENSORS`` tensors per
    call, and calls that overlap on one GPU race on that array.  Nothing is allocated here either;
    non-contiguous inputs are refused instead of copied."""
    n = len(tensors)
    if len(outs) != n or scales.numel() != n or scales.dtype != torch.float32 or not scales.is_contiguous():
        raise ValueError("outs and scales must match the tensors: one fp8 tensor and one fp32 scale each")
    if n == 0:
        return
    _need_gpu(scales, *tensors, *outs)
    descs = (_lib.TensorDesc * n)()
    sbase = scales.data_ptr()
    for i, (t, q) in enumerate(zip(tensors, outs)):
        if t.dtype != torch.bfloat16 or q.dtype != FP8_DTYPE:
            raise ValueError(f"tensor {i}: expected bfloat16 in and float8_e4m3fn out, got {t.dtype} and {q.dtype}")
        if not t.is_contiguous() or not q.is_contiguous() or q.numel() != t.numel():
            raise ValueError(f"tensor {i}: input and output must be contiguous and of equal size")
        descs[i].x = t.data_ptr()
        descs[i].q = q.data_ptr()
        descs[i].scale = sbase + 4 * i
        descs[i].numel = t.numel()
    _lib.check(_lib.load().cfp8_quant_tensorwise_multi_static(descs, n, _stream()))


def quant_tensorwise(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """One global amax, one fp32 scale (shape [1]), saturated cast: the tensorwise recipe
    selected at cosmos_rl/utils/fp8/fp8_util.py:121-137."""
    outs, scales = quant_tensorwise_multi([x])
    return outs[0], scales


def per_block_cast_to_fp8(w: torch.Tensor, transpose_out: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """128x128 block quantisation of [R, C] or a stack [E, R, C].
    Returns (fp8 like w - or with the last two dims swapped when ``transpose_out`` -,
    fp32 scales [..., ceil(R/128), ceil(C/128)])."""
    _need_gpu(w)
    if w.dtype != torch.bfloat16:
        raise ValueError(f"block FP8 quantisation takes bfloat16 input, got {w.dtype}")
    if w.dim() not in (2, 3):
        raise ValueError(f"expected a 2-D or 3-D tensor, got {tuple(w.shape)}")
    w = w.contiguous()
    lead = w.shape[:-2]
    rows, cols = w.shape[-2:]
    batch = int(lead[0]) if lead else 1
    oshape = (*lead, cols, rows) if transpose_out else (*lead, rows, cols)
    q = torch.empty(oshape, dtype=FP8_DTYPE, device=w.device)
    s = torch.empty((*lead, -(-rows // BLOCK), -(-cols // BLOCK)), dtype=torch.float32, device=w.device)
    _lib.check(_lib.load().cfp8_quant_block128(w.data_ptr(), batch, rows, cols, q.data_ptr(), s.data_ptr(),
                                              1 if transpose_out else 0, _stream()))
    return q, s


def prepare_fp8_weight(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``dsgemm_utils.prepare_fp8_weight`` (cosmos_rl/policy/kernel/group_gemms.py:132)."""
    return per_block_cast_to_fp8(w)


def _group128(x: torch.Tensor, mode: int) -> Tuple[torch.Tensor, torch.Tensor]:
    _need_gpu(x)
    if x.dtype != torch.bfloat16:
        raise ValueError(f"1x128 FP8 quantisation takes bfloat16 input, got {x.dtype}")
    if x.dim() != 2:
        raise ValueError(f"expected a 2-D tensor, got {tuple(x.shape)}")
    if x.stride(1) != 1 and x.shape[1] > 1:
        x = x.contiguous()
    rows, cols = x.shape
    q = torch.empty((rows, cols), dtype=FP8_DTYPE, device=x.device)
    s = torch.empty((rows, -(-cols // BLOCK)), dtype=torch.float32, device=x.device)
    ld_x = x.stride(0) if rows > 1 else max(cols, 1)
    _lib.check(_lib.load().cfp8_quant_group128(x.data_ptr(), rows, cols, ld_x, q.data_ptr(), cols,
                                              s.data_ptr(), mode, _stream()))
    return q, s


def groupwise_activation_quant(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``dsgemm_kernels.groupwise_activation_quant`` (group_gemms.py:188-189): 1x128 groups,
    returns (fp8 [M, K], fp32 [M, K/128]) ready to feed the block GEMM."""
    return _group128(x, _lib.GROUP_MODE_DIV)


def prepare_fp8_input(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``dsgemm_utils.prepare_fp8_input`` (group_gemms.py:190-191)."""
    return _group128(x, _lib.GROUP_MODE_DIV)


def swiglu_quant(gate: torch.Tensor, up: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``silu(gate) * up`` and the 1x128 quantisation of the product in one kernel; the bf16 product is
    never written.  Takes the two expert-GEMM outputs of cosmos_rl/policy/kernel/group_gemms.py:194-207
    (or the two column halves of one fused gate_up output: any row pitch, unit column stride) and returns
    what ``groupwise_activation_quant(activation(gate) * up)`` returns at :209-218: (fp8 [M, I], fp32 [M, I/128])."""
    _need_gpu(gate, up)
    if gate.dtype != torch.bfloat16 or up.dtype != torch.bfloat16 or gate.dim() != 2 or gate.shape != up.shape:
        raise ValueError(f"expected two bf16 [M, I] tensors, got {tuple(gate.shape)} {gate.dtype} and {tuple(up.shape)} {up.dtype}")
    rows, cols = gate.shape
    if cols > 1 and gate.stride(1) != 1:
        gate = gate.contiguous()
    if cols > 1 and up.stride(1) != 1:
        up = up.contiguous()
    q = torch.empty((rows, cols), dtype=FP8_DTYPE, device=gate.device)
    s = torch.empty((rows, (cols + 127) // 128), dtype=torch.float32, device=gate.device)
    ldg = gate.stride(0) if rows > 1 else max(cols, 1)
    ldu = up.stride(0) if rows > 1 else max(cols, 1)
    _lib.check(_lib.load().cfp8_swiglu_quant_group128(gate.data_ptr(), ldg, up.data_ptr(), ldu, rows, cols,
                                                     q.data_ptr(), cols, s.data_ptr(), _stream()))
    return q, s


def quant_mxfp4(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """MXFP4 along the last axis of a bf16 tensor [..., K], K % 32 == 0: (uint8 [..., K/2] with two e2m1
    codes per byte, even element low; uint8 [..., K/32] e8m0 scales)."""
    _need_gpu(w)
    if w.dtype != torch.bfloat16 or w.dim() < 1 or w.shape[-1] % 32:
        raise ValueError(f"expected a bf16 tensor whose last dimension is a multiple of 32, got {tuple(w.shape)} {w.dtype}")
    w = w.contiguous()
    K = w.shape[-1]
    rows = w.numel() // K if K else 0
    q = torch.empty((*w.shape[:-1], K // 2), dtype=torch.uint8, device=w.device)
    s = torch.empty((*w.shape[:-1], K // 32), dtype=torch.uint8, device=w.device)
    _lib.check(_lib.load().cfp8_quant_mxfp4(w.data_ptr(), rows, K, K, q.data_ptr(), K // 2, s.data_ptr(), K // 32, _stream()))
    return q, s


def gemm_mxfp4(lhs: Tuple[torch.Tensor, torch.Tensor], rhs: Tuple[torch.Tensor, torch.Tensor],
               out_dtype: torch.dtype = torch.bfloat16, m_indices: Optional[torch.Tensor] = None,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Product of per-token FP8 activations with MXFP4 weights as ``quant_mxfp4`` (``quantize_mx4``,
    monkey_patch_for_mxfp4.py:18-24) writes them.  lhs = (fp8 [M, K], fp32 [M] or [M, 1]); rhs = (uint8 [N, K/2],
    uint8 [N, K/32]) or, with ``m_indices`` (int32 [M], groups contiguous and 128-row aligned, negative =
    padding, rows left untouched), ([E, N, K/2], [E, N, K/32]).  K % 32 == 0, N % 16 == 0."""
    a, sa = lhs
    w, ws = rhs
    _need_gpu(a, sa, w, ws)
    if a.dim() != 2 or a.dtype != FP8_DTYPE or w.dtype != torch.uint8 or ws.dtype != torch.uint8:
        raise ValueError("expected fp8 [M, K] activations and uint8 weight codes / scales")
    M, K = a.shape
    grouped = m_indices is not None
    if w.dim() != (3 if grouped else 2):
        raise ValueError("weights must be [N, K/2] (or [E, N, K/2] with m_indices)")
    E = w.shape[0] if grouped else 1
    N = w.shape[-2]
    if K % 32 or w.shape[-1] != K // 2 or tuple(ws.shape) != (*w.shape[:-1], K // 32) or sa.numel() != M:
        raise ValueError("shape mismatch in MXFP4 GEMM")
    if sa.dtype != torch.float32:
        raise ValueError("activation scales must be fp32")
    a, sa, w, ws = a.contiguous(), sa.contiguous(), w.contiguous(), ws.contiguous()
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    elif tuple(out.shape) != (M, N) or not out.is_contiguous():
        raise ValueError("out must be a contiguous [M, N] tensor")
    mi = 0
    if grouped:
        _need_gpu(m_indices)
        if m_indices.numel() != M:
            raise ValueError("m_indices must have one entry per row")
        m_indices = m_indices.to(torch.int32).contiguous()
        mi = m_indices.data_ptr()
    _lib.check(_lib.load().cfp8_gemm_mxfp4(a.data_ptr(), K, sa.data_ptr(), w.data_ptr(), K // 2, ws.data_ptr(), K // 32,
                                          mi, E if grouped else 0, out.data_ptr(), N, _out_code(out.dtype), M, N, K, _stream()))
    return out


def linear_mxfp4(x: torch.Tensor, weight: Tuple[torch.Tensor, torch.Tensor],
                 out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """x [..., K] bf16 times MXFP4 weights (codes [N, K/2], scales [N, K/32]): per-token dynamic FP8
    quantisation of x (as in ``fp8_linear``) and ``gemm_mxfp4``, one launch for up to 4 tokens."""
    w, ws = weight
    _need_gpu(x, w, ws)
    K = x.shape[-1]
    if x.dtype != torch.bfloat16 or w.dtype != torch.uint8 or ws.dtype != torch.uint8 or w.dim() != 2:
        raise ValueError("expected bf16 activations and uint8 [N, K/2] codes / [N, K/32] scales")
    N = w.shape[0]
    if K % 32 or w.shape[1] != K // 2 or tuple(ws.shape) != (N, K // 32):
        raise ValueError("shape mismatch in MXFP4 linear")
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1 or x2.stride(0) % 8 or x2.data_ptr() % 16:
        x2 = x2.contiguous()
    M = x2.shape[0]
    w, ws = w.contiguous(), ws.contiguous()
    out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    lib = _lib.load()
    wsb = lib.cfp8_linear_workspace_bytes(M, K)
    work = torch.empty(max(wsb, 1), dtype=torch.uint8, device=x.device)
    ld_x = x2.stride(0) if M > 1 else K
    _lib.check(lib.cfp8_linear_mxfp4(x2.data_ptr(), ld_x, w.data_ptr(), K // 2, ws.data_ptr(), K // 32, out.data_ptr(), N,
                                     _out_code(out.dtype), M, N, K, work.data_ptr(), wsb, _stream()))
    return out.reshape(*x.shape[:-1], N)


def per_token_cast_to_fp8(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``per_token_cast_to_fp8`` of the reference's tests/test_deepep.py:75-85, including its
    formula ``x * (448 / amax.clamp(1e-4))`` with scales ``amax / 448``."""
    return _group128(x, _lib.GROUP_MODE_DEEPEP)


def per_token_cast_back(x_fp8: torch.Tensor, x_scales: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``per_token_cast_back`` of the reference's tests/test_deepep.py:86-108: ``bf16(fp32(x_fp8) * scale)`` with one
    scale per row and group of 128 columns.  ``x_scales`` is fp32 ``[m, ceil(n / 128)]`` or, as in the reference's
    ``x_scales.dtype == torch.int`` branch (:97-99), int32 holding four E8M0 exponent bytes each, lowest byte first
    (``[m, ceil(n / 128) / 4]``)."""
    if x_fp8.numel() == 0:
        return x_fp8.to(out_dtype)
    _need_gpu(x_fp8, x_scales)
    assert x_fp8.dim() == 2 and x_fp8.dtype == FP8_DTYPE
    m, n = x_fp8.shape
    groups = -(-n // BLOCK)
    q = x_fp8 if x_fp8.is_contiguous() else x_fp8.contiguous()
    if x_scales.dtype == torch.int32:
        sc = x_scales.contiguous().view(torch.uint8).view(m, -1)
        kind = _lib.SCALE_E8M0
    elif x_scales.dtype == torch.float32:
        sc = x_scales.contiguous().view(m, -1)
        kind = _lib.SCALE_F32
    else:
        raise ValueError(f"scales must be float32 or packed int32, got {x_scales.dtype}")
    if sc.shape[1] < groups:
        raise ValueError(f"{sc.shape[1]} scales per row do not cover {n} columns")
    y = torch.empty((m, n), dtype=out_dtype, device=x_fp8.device)
    _lib.check(_lib.load().cfp8_dequant_group128(q.data_ptr(), n, sc.data_ptr(), sc.shape[1], kind, m, n, y.data_ptr(), n,
                                                _out_code(out_dtype), _stream()))
    return y


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128,
                   out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``weight_dequant`` (cosmos_rl/policy/model/deepseek_v3/weight_mapper.py:246-259):
    y = fp8 * s[i // 128, j // 128]; output in the default dtype unless given."""
    _need_gpu(x, s)
    assert x.is_contiguous() and s.is_contiguous()
    assert x.dim() == 2 and s.dim() == 2
    if block_size != BLOCK:
        raise ValueError("only 128x128 blocks are supported")
    dt = out_dtype or torch.get_default_dtype()
    M, N = x.shape
    if tuple(s.shape) != (-(-M // BLOCK), -(-N // BLOCK)):
        raise ValueError(f"scale shape {tuple(s.shape)} does not match weight {tuple(x.shape)}")
    y = torch.empty((M, N), dtype=dt, device=x.device)
    _lib.check(_lib.load().cfp8_dequant_block128(x.data_ptr(), s.data_ptr(), M, N, y.data_ptr(),
                                                _out_code(dt), _stream()))
    return y


# ---------------------------------------------------------------------------
# GEMMs
# ---------------------------------------------------------------------------
def scaled_mm(a: torch.Tensor, b: torch.Tensor, scale_a: torch.Tensor, scale_b: torch.Tensor,
              out_dtype: torch.dtype = torch.bfloat16, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rowwise ``torch._scaled_mm``: a fp8 [M, K] row-major, b fp8 [K, N] column-major (the
    ``.t()`` of a contiguous [N, K] weight, monkey_patch_for_fp8.py:52), scale_a [M, 1],
    scale_b [1, N] (or [N, 1]); out = (a @ b) * scale_a * scale_b (+ bias).  A scale of one element
    (the tensorwise form of ``torch._scaled_mm``) stands for every row / column: the kernels read one
    scale per row and per column, so it is spread into a vector here."""
    _need_gpu(a, b, scale_a, scale_b)
    if a.dtype != FP8_DTYPE or b.dtype != FP8_DTYPE:
        raise ValueError("scaled_mm takes float8_e4m3fn operands")
    if a.dim() != 2 or b.dim() != 2 or a.shape[1] != b.shape[0]:
        raise ValueError(f"shape mismatch: {tuple(a.shape)} @ {tuple(b.shape)}")
    M, K = a.shape
    N = b.shape[1]
    if not (a.stride(1) == 1 or K == 1):
        raise ValueError("a must be row-major")
    if not (b.stride(0) == 1 or K == 1):
        raise ValueError("b must be column-major (pass weight.t() of a contiguous [N, K] weight)")
    if scale_a.numel() not in (1, M) or scale_b.numel() not in (1, N):
        raise ValueError("scaled_mm needs rowwise scales, scale_a [M, 1] and scale_b [1, N], or scales of one element")
    sa = scale_a.reshape(-1).float()
    sb = scale_b.reshape(-1).float()
    sa = sa.expand(M).contiguous() if sa.numel() != M else sa.contiguous()
    sb = sb.expand(N).contiguous() if sb.numel() != N else sb.contiguous()
    out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    ld_a = a.stride(0) if M > 1 else K
    ld_b = b.stride(1) if N > 1 else K
    _lib.check(_lib.load().cfp8_scaled_mm_rowwise(a.data_ptr(), ld_a, sa.data_ptr(), b.data_ptr(), ld_b,
                                                 sb.data_ptr(), out.data_ptr(), N, _out_code(out_dtype),
                                                 M, N, K, _stream()))
    if bias is not None:
        out = out + bias
    return out


def fp8_linear(x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
               bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.bfloat16,
               workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``Fp8LinearOp(use_per_token_if_dynamic=True).apply`` (monkey_patch_for_fp8.py:74-79):
    per-token dynamic quantisation of x, then the rowwise scaled mm.

    weight: fp8 [K, N] column-major, i.e. ``qweight.t()`` as the reference stores it;
    weight_scale [N, 1]; x bf16 [..., K].  Returns [..., N]."""
    _need_gpu(x, weight, weight_scale)
    if x.dtype != torch.bfloat16:
        raise ValueError(f"fp8_linear takes bfloat16 activations, got {x.dtype}")
    K, N = weight.shape
    if weight.stride(0) != 1 and K > 1:
        raise ValueError("weight must be the transposed view of a contiguous [N, K] fp8 tensor")
    x2 = x.reshape(-1, K)
    if x2.stride(1) != 1 and K > 1:
        x2 = x2.contiguous()
    M = x2.shape[0]
    lib = _lib.load()
    need = lib.cfp8_linear_workspace_bytes(M, K)
    if workspace is None or workspace.numel() * workspace.element_size() < need:
        # the larger size lets the library split K where that pays (few weight rows, long K, 17..64 tokens)
        workspace = torch.empty(max(lib.cfp8_linear_workspace_bytes_split(M, N, K), 256), dtype=torch.uint8, device=x.device)
    sw = weight_scale.reshape(-1)
    if sw.dtype != torch.float32 or not sw.is_contiguous():
        sw = sw.contiguous().float()
    out = torch.empty((M, N), dtype=out_dtype, device=x.device)
    ld_x = x2.stride(0) if M > 1 else K
    ld_w = weight.stride(1) if N > 1 else K
    _lib.check(lib.cfp8_linear_rowwise(x2.data_ptr(), ld_x, weight.data_ptr(), ld_w, sw.data_ptr(),
                                      out.data_ptr(), N, _out_code(out_dtype), M, N, K,
                                      workspace.data_ptr(), workspace.numel() * workspace.element_size(),
                                      _stream()))
    if bias is not None:
        out = out + bias
    return out.reshape(*x.shape[:-1], N)


def gemm_fp8_fp8_bf16_nt(lhs: Tuple[torch.Tensor, torch.Tensor], rhs: Tuple[torch.Tensor, torch.Tensor],
                         out: torch.Tensor, rhs_scale_kn: bool = False) -> torch.Tensor:
    """Dense block-scaled GEMM.  lhs = (fp8 [M, K], fp32 [M, K/128]); rhs = (fp8 [N, K],
    fp32 [ceil(N/128), K/128]) or, with ``rhs_scale_kn``, scales laid out [K/128, ceil(N/128)]
    (what quantising a [K, N] weight produces).  Writes into ``out`` [M, N]."""
    a, sa = lhs
    b, sb = rhs
    _need_gpu(a, sa, b, sb, out)
    M, K = a.shape
    N = b.shape[0]
    if b.shape[1] != K or tuple(out.shape) != (M, N):
        raise ValueError("shape mismatch in block-scaled GEMM")
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    nb, kb = -(-N // BLOCK), K // BLOCK
    if rhs_scale_kn:
        if tuple(sb.shape) != (kb, nb):
            raise ValueError(f"rhs scales must be [{kb}, {nb}], got {tuple(sb.shape)}")
        stride_n, stride_k = 1, nb
    else:
        if tuple(sb.shape) != (nb, kb):
            raise ValueError(f"rhs scales must be [{nb}, {kb}], got {tuple(sb.shape)}")
        stride_n, stride_k = kb, 1
    if tuple(sa.shape) != (M, kb):
        raise ValueError(f"lhs scales must be [{M}, {kb}], got {tuple(sa.shape)}")
    if not out.is_contiguous():
        raise ValueError("out must be contiguous")
    _lib.check(_lib.load().cfp8_gemm_block128(a.data_ptr(), K, sa.data_ptr(), b.data_ptr(), K, sb.data_ptr(),
                                             stride_n, stride_k, out.data_ptr(), N, _out_code(out.dtype),
                                             M, N, K, _stream()))
    return out


def m_grouped_gemm_fp8_fp8_bf16_nt_contiguous(lhs: Tuple[torch.Tensor, torch.Tensor],
                                              rhs: Tuple[torch.Tensor, torch.Tensor],
                                              out: torch.Tensor, m_indices: torch.Tensor) -> torch.Tensor:
    """``deep_gemm.m_grouped_gemm_fp8_fp8_bf16_nt_contiguous`` (group_gemms.py:194-225).
    lhs = (fp8 [M, K], fp32 [M, K/128]); rhs = (fp8 [E, N, K], fp32 [E, ceil(N/128), K/128]);
    m_indices int32 [M], groups contiguous and 128-row aligned, negative = padding (rows left
    untouched).  Writes into ``out`` [M, N]."""
    a, sa = lhs
    b, sb = rhs
    _need_gpu(a, sa, b, sb, out, m_indices)
    M, K = a.shape
    E, N, Kb = b.shape
    if Kb != K or tuple(out.shape) != (M, N) or m_indices.numel() != M:
        raise ValueError("shape mismatch in grouped GEMM")
    if m_indices.dtype != torch.int32:
        m_indices = m_indices.to(torch.int32)
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    if tuple(sb.shape) != (E, -(-N // BLOCK), K // BLOCK) or tuple(sa.shape) != (M, K // BLOCK):
        raise ValueError("scale shape mismatch in grouped GEMM")
    if not out.is_contiguous():
        raise ValueError("out must be contiguous")
    _lib.check(_lib.load().cfp8_gemm_grouped_block128(a.data_ptr(), K, sa.data_ptr(), b.data_ptr(), sb.data_ptr(),
                                                     m_indices.contiguous().data_ptr(), out.data_ptr(), N,
                                                     _out_code(out.dtype), M, N, K, E, _stream()))
    return out


def interleave_gate_up(gate: Tuple[torch.Tensor, torch.Tensor], up: Tuple[torch.Tensor, torch.Tensor]
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gate and up expert weights (fp8 [E, I, K], block scales [E, I/128, K/128] each) as one [E, 2I, K] weight in
    the layout ``grouped_gemm_swiglu_quant`` takes: rows alternate in units of 16 - 16 gate rows, the 16 up rows of
    the same intermediate features, the next 16 gate rows ... - so every 256 rows hold one 128-feature block of both
    projections; scale rows alternate per block: gate block j, up block j.  Done once, when the weights are arranged."""
    (qg, sg), (qu, su) = gate, up
    E, I, K = qg.shape
    if I % BLOCK or qu.shape != qg.shape or sg.shape != su.shape:
        raise ValueError("gate and up must have the same shape with I a multiple of 128")
    q = torch.stack([qg.view(torch.uint8).view(E, I // 16, 16, K), qu.view(torch.uint8).view(E, I // 16, 16, K)], dim=2)
    s = torch.stack([sg, su], dim=2)
    return q.reshape(E, 2 * I, K).view(FP8_DTYPE), s.reshape(E, 2 * I // BLOCK, K // BLOCK).contiguous()


def grouped_gemm_swiglu_quant(lhs: Tuple[torch.Tensor, torch.Tensor], rhs_interleaved: Tuple[torch.Tensor, torch.Tensor],
                              m_indices: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Grouped gate_up GEMM, SiLU(gate) * up and the 1x128 quantisation of the product in one launch
    (group_gemms.py:194-218): returns (fp8 [M, I], fp32 [M, I/128]) - the input of the down GEMM.  Rows whose
    m_indices is negative are left as allocated."""
    a, sa = lhs
    b, sb = rhs_interleaved
    _need_gpu(a, sa, b, sb, m_indices)
    M, K = a.shape
    E, N2, Kb = b.shape
    I = N2 // 2
    if Kb != K or m_indices.numel() != M or tuple(sa.shape) != (M, K // BLOCK) or tuple(sb.shape) != (E, N2 // BLOCK, K // BLOCK):
        raise ValueError("shape mismatch in grouped GEMM")
    if m_indices.dtype != torch.int32:
        m_indices = m_indices.to(torch.int32)
    a, b, sa, sb = a.contiguous(), b.contiguous(), sa.contiguous(), sb.contiguous()
    q = torch.empty((M, I), dtype=FP8_DTYPE, device=a.device)
    s = torch.empty((M, I // BLOCK), dtype=torch.float32, device=a.device)
    _lib.check(_lib.load().cfp8_gemm_grouped_swiglu_quant(a.data_ptr(), K, sa.data_ptr(), b.data_ptr(), sb.data_ptr(),
                                                         m_indices.contiguous().data_ptr(), q.data_ptr(), I, s.data_ptr(),
                                                         M, I, K, E, _stream()))
    return q, s


def create_indices_from_offsets_nosync(m_offsets: torch.Tensor, total: Optional[int] = None,
                                       n_experts: Optional[int] = None) -> torch.Tensor:
    """``dsgemm_utils.create_indices_from_offsets_nosync`` (group_gemms.py:157): expert id per
    row from the inclusive cumulative group ends.  Pass ``total`` (the number of rows, which the
    caller already knows from its own slice at group_gemms.py:154) to stay free of a host sync;
    without it the last offset is read back.  With ``n_experts`` given, ``total`` may be any bound on
    the row count: rows past the last group get -1 (padding to the grouped GEMMs)."""
    if total is None:
        total = int(m_offsets[-1])
    rows = torch.arange(total, device=m_offsets.device, dtype=m_offsets.dtype)
    idx = torch.searchsorted(m_offsets, rows, right=True).to(torch.int32)
    if n_experts is not None:
        idx = torch.where(idx < n_experts, idx, torch.full_like(idx, -1))
    return idx
