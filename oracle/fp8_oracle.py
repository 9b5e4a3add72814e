"""CPU oracle for the FP8 hot path.  TEST INFRASTRUCTURE ONLY.

This module is a checker.  Only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import it; the shipped package never
does, and it raises when its HIP library is missing instead of coming here.

The reference (nvidia-cosmos/cosmos-rl) owns no arithmetic on this path: every
call site hands the work to a third-party wheel that is not vendored in the
reference tree:

  * rowwise weight quant       cosmos_rl/rollout/vllm_rollout/vllm_rollout.py:989-999
                               cosmos_rl/rollout/vllm_rollout/monkey_patch_for_fp8.py:45-54
                               -> vllm._custom_ops.scaled_fp8_quant        (vllm 0.11.0 / 0.17.0)
  * per-token act quant + mm   monkey_patch_for_fp8.py:26-34, 63-82
                               -> torch._scaled_mm rowwise                  (torch 2.8.0 / 2.10.0)
  * tensorwise / rowwise       cosmos_rl/utils/fp8/fp8_util.py:110-152
                               -> torchao.float8                            (torchao 0.13.0 / 0.16.0)
  * 128x128 block / 1x128      cosmos_rl/policy/kernel/group_gemms.py:128-229
    quant + grouped GEMM       -> deep_gemm / dsgemm_utils / dsgemm_kernels (unpinned)

so this file restates the *published* algorithm of those ops with the one
scale formula the build adopts for all granularities:

    amax  = max |x|                 over the reduction set, exact in fp32
    scale = max(amax, 1e-12) / 448  fp32 IEEE division, stored
    q     = e4m3fn_rne(clamp(fp32(x) / scale, -448, 448))

NaN contract: a NaN anywhere in a reduction set makes its scale NaN and all
its bytes NaN.  The sign / payload of a NaN is platform noise (x86 produces a
negative default NaN for inf/inf), so both the oracle and the kernels emit the
canonical byte 0x7F and the canonical scale 0x7FC00000.

Two fragments of the path *are* stated in the reference tree and are followed
to the letter:

  * ``per_token_cast_to_fp8`` / ``per_token_cast_back``  tests/test_deepep.py:75-109
    (1x128 groups, ``x * (448 / amax)``, ``amax.clamp(1e-4)``, scales ``amax / 448``
    laid out ``[m, n/128]``, zero padded tail group) -> ``group128_cast_deepep``.
  * ``weight_dequant``  cosmos_rl/policy/model/deepseek_v3/weight_mapper.py:232-259
    (``y = fp8 * s[i // 128, j // 128]``, scales row-major
    ``[ceil(M/128), ceil(N/128)]``) -> ``weight_dequant``.

What pins each function (tests/test_oracle.py, tests/test_c_oracle.py):

  e4m3 cast        known-answer table, exhaustive 65536 bf16 patterns against an
                   independent integer RNE encoder (oracle/fp8_ref.c) and against
                   a brute-force nearest-value search over the 256 e4m3 codes
  amax / scale     closed forms (zero row -> 0x2720D7C5), brute force on tiny inputs
  quantizers       invariants: every non-zero set holds a +-0x7E byte, error
                   <= half an e4m3 ulp, idempotent re-quantisation, permutation
                   commutation; C restatement agrees byte for byte
  transfer dtype   quant_rowwise_from: fp32 -> bf16 rounding of oracle/fp8_ref.c (integer RNE)
                   against torch's own cast on ties, overflow, NaN, subnormals; then
                   it is quant_rowwise
  SwiGLU + requant exp32 of oracle/fp8_ref.c against fp64 exp (< 2 ulp on a dense grid), closed
                   forms silu(0) = 0, silu(x) -> x and -> -0 at the ends, hidden state within one
                   bf16 ulp of torch's silu(g) * u on <= 0.1 % of elements and equal elsewhere
  block layout     round trip through weight_dequant (the in-tree inverse)
  1x128 layout     round trip through per_token_cast_back (in-tree)
  GEMMs            fp64 matmul of dequantised operands, one-hot operands,
                   power-of-two scales, brute-force python loop over experts

The upstream wheels themselves are absent here (no vllm / torchao / deep_gemm in
the image and no reference test holds an FP8 golden vector), so agreement with
*their* bits is "parity unpinned"; agreement with the formula above is pinned.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import torch

E4M3_MAX = 448.0
AMAX_FLOOR = 1e-12
DEEPEP_AMAX_FLOOR = 1e-4
BLOCK = 128

_F8 = torch.float8_e4m3fn


# --------------------------------------------------------------------------
# primitives
# --------------------------------------------------------------------------
def _canon_nan_bytes(q_u8: torch.Tensor) -> torch.Tensor:
    """0xFF (negative NaN) -> 0x7F; e4m3fn has no other NaN codes."""
    return torch.where((q_u8 & 0x7F) == 0x7F, torch.full_like(q_u8, 0x7F), q_u8)


def _canon_nan_scale(s: torch.Tensor) -> torch.Tensor:
    return torch.where(torch.isnan(s), torch.full_like(s, float("nan")), s)


def e4m3_bytes(v_f32: torch.Tensor) -> torch.Tensor:
    """fp32 -> OCP e4m3fn bytes (uint8), RNE, via torch's CPU cast."""
    return _canon_nan_bytes(v_f32.to(torch.float32).to(_F8).view(torch.uint8))


def e4m3_to_f32(q_u8: torch.Tensor) -> torch.Tensor:
    return q_u8.view(_F8).to(torch.float32)


def scale_from_amax(amax_f32: torch.Tensor) -> torch.Tensor:
    """scale = max(amax, 1e-12) / 448 in fp32; NaN propagates (torch.clamp does)."""
    s = torch.clamp(amax_f32.to(torch.float32), min=AMAX_FLOOR) / E4M3_MAX
    return _canon_nan_scale(s)


def _cast_with_scale(x: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
    """bytes = e4m3_rne(clamp(fp32(x) / scale, +-448)); ``scale`` broadcasts."""
    y = x.to(torch.float32) / scale
    y = torch.clamp(y, -E4M3_MAX, E4M3_MAX)
    return e4m3_bytes(y)


# --------------------------------------------------------------------------
# quantizers
# --------------------------------------------------------------------------
def quant_rowwise(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``scaled_fp8_quant(x, scale=None, use_per_token_if_dynamic=True)`` as used at
    vllm_rollout.py:995-997 and monkey_patch_for_fp8.py:47-49.

    x: [R, C] (bf16 / fp16 / fp32).  Returns (uint8 [R, C], fp32 [R, 1]).
    """
    assert x.dim() == 2
    amax = x.to(torch.float32).abs().amax(dim=1, keepdim=True) if x.shape[1] else \
        torch.zeros(x.shape[0], 1)
    scale = scale_from_amax(amax)
    return _cast_with_scale(x, scale), scale


def quant_rowwise_from(recv: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rowwise quantisation of a received weight in its transfer dtype (bf16 / fp16 / fp32):
    the three steps ``recv.to(view.dtype)`` + ``view.copy_`` (policy/model/base.py:1053-1069, the
    staging view is bf16, monkey_patch_for_fp8.py:122-125), ``fp8_quantization``
    (vllm_rollout.py:989-999) and the copies into the engine's parameters
    (rollout_control.py:889-898) as one function of the received values."""
    return quant_rowwise(recv.to(torch.bfloat16))


def quant_tensorwise(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Tensorwise dynamic scaling (fp8_util.py:121-137 selects this recipe): one
    global amax, one fp32 scale, saturated cast.  Returns (uint8 like x, fp32 [1])."""
    if x.numel() == 0:
        amax = torch.zeros(())
    else:
        amax = x.to(torch.float32).abs().amax()
    scale = scale_from_amax(amax).reshape(1)
    return _cast_with_scale(x, scale), scale


def quant_block128(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """128x128 block scaling of [..., R, C] (``prepare_fp8_weight`` at
    group_gemms.py:132; layout of the scales pinned by weight_mapper.py:236-243).

    Returns (uint8 [..., R, C], fp32 [..., ceil(R/128), ceil(C/128)]).
    """
    *lead, R, C = w.shape
    rb, cb = -(-R // BLOCK), -(-C // BLOCK)
    xf = w.to(torch.float32)
    pad = torch.zeros(*lead, rb * BLOCK, cb * BLOCK, dtype=torch.float32)
    pad[..., :R, :C] = xf
    tiles = pad.view(*lead, rb, BLOCK, cb, BLOCK)
    amax = tiles.abs().amax(dim=(-3, -1))                      # [..., rb, cb]
    scale = scale_from_amax(amax)
    y = tiles / scale[..., :, None, :, None]
    y = torch.clamp(y, -E4M3_MAX, E4M3_MAX).reshape(*lead, rb * BLOCK, cb * BLOCK)
    q = e4m3_bytes(y[..., :R, :C].contiguous())
    return q, scale


def quant_group128(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """1x128 group scaling of activations [M, K] with the build's formula
    (``prepare_fp8_input`` / ``groupwise_activation_quant`` at group_gemms.py:188-191).

    Returns (uint8 [M, K], fp32 [M, ceil(K/128)])."""
    assert x.dim() == 2
    M, K = x.shape
    kb = -(-K // BLOCK)
    pad = torch.zeros(M, kb * BLOCK, dtype=torch.float32)
    pad[:, :K] = x.to(torch.float32)
    g = pad.view(M, kb, BLOCK)
    scale = scale_from_amax(g.abs().amax(dim=2))               # [M, kb]
    y = torch.clamp(g / scale[:, :, None], -E4M3_MAX, E4M3_MAX).reshape(M, kb * BLOCK)
    return e4m3_bytes(y[:, :K].contiguous()), scale


def swiglu_quant_group128(gate: torch.Tensor, up: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``hidden = activation(gate_out) * up_out`` on bf16 tensors followed by the 1x128 quantiser
    (cosmos_rl/policy/kernel/group_gemms.py:209-218) for the SiLU activation, with torch's own ops.

    The fused kernel and oracle/fp8_ref.c define exp by a fixed fp32 operation sequence; torch's
    vectorised exp may differ from it in the last fp32 bit, which moves the bf16 rounding of
    silu(g) for about one element in 10^4.  Tests therefore hold the kernel bit-exact against the
    C restatement and within one bf16 ulp of the hidden state (rare) against this function."""
    h = torch.nn.functional.silu(gate.to(torch.bfloat16)) * up.to(torch.bfloat16)
    return quant_group128(h)


def swiglu_hidden(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.silu(gate.to(torch.bfloat16)) * up.to(torch.bfloat16)


def group128_cast_deepep(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``per_token_cast_to_fp8`` exactly as tests/test_deepep.py:75-85 states it:
    multiply by ``448 / clamp(amax, 1e-4)``, no saturation clamp before the cast,
    scales ``amax / 448``.  Note that torch evaluates ``python_float / tensor`` as
    ``tensor.reciprocal() * python_float`` (Tensor.__rtruediv__), so the multiplier is
    fl(fl(1/amax) * 448), not fl(448/amax); the expression below keeps that form."""
    assert x.dim() == 2
    M, K = x.shape
    kb = -(-K // BLOCK)
    xp = torch.nn.functional.pad(x, (0, kb * BLOCK - K), mode="constant", value=0)
    v = xp.view(M, kb, BLOCK)
    amax = v.abs().float().amax(dim=2).view(M, -1).clamp(DEEPEP_AMAX_FLOOR)
    y = v.float() * (E4M3_MAX / amax.unsqueeze(2))
    q = e4m3_bytes(y).view(M, kb * BLOCK)[:, :K].contiguous()
    return q, _canon_nan_scale((amax / E4M3_MAX).view(M, -1))


# --------------------------------------------------------------------------
# inverses (in-tree statements)
# --------------------------------------------------------------------------
def weight_dequant(q_u8: torch.Tensor, s: torch.Tensor, block_size: int = BLOCK) -> torch.Tensor:
    """weight_mapper.py:232-259: y[i, j] = fp8[i, j] * s[i // bs, j // bs] in fp32."""
    *lead, R, C = q_u8.shape
    se = s.repeat_interleave(block_size, dim=-2).repeat_interleave(block_size, dim=-1)
    return e4m3_to_f32(q_u8) * se[..., :R, :C]


def group128_dequant(q_u8: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    """``per_token_cast_back`` (tests/test_deepep.py:88-109) without the final bf16 cast."""
    M, K = q_u8.shape
    se = s.repeat_interleave(BLOCK, dim=1)[:, :K]
    return e4m3_to_f32(q_u8) * se


def per_token_cast_back(q_u8: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
    """``per_token_cast_back`` (tests/test_deepep.py:86-108) in full: the columns are padded to a multiple of 128, a
    scale tensor of dtype int32 holds four E8M0 exponent bytes per element (viewed as uint8 and shifted into the
    exponent field of an fp32, :97-99), the product is formed in fp32 and cast to bf16."""
    m, n = q_u8.shape
    if q_u8.numel() == 0:
        return torch.empty(m, n, dtype=torch.bfloat16)
    aligned = (n + BLOCK - 1) // BLOCK * BLOCK
    x = torch.zeros(m, aligned, dtype=torch.float32)
    x[:, :n] = e4m3_to_f32(q_u8)
    if scales.dtype == torch.int32:
        scales = (scales.contiguous().view(torch.uint8).to(torch.int32) << 23).view(torch.float32)
    sc = scales.reshape(m, -1, 1)
    return (x.view(m, -1, BLOCK) * sc).view(m, aligned).to(torch.bfloat16)[:, :n].contiguous()


def rowwise_dequant(q_u8: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    return e4m3_to_f32(q_u8) * s.reshape(-1, 1)


# --------------------------------------------------------------------------
# GEMMs.  All return fp32; callers compare bf16(kernel) with bf16(oracle) or an
# fp32-epilogue kernel with the fp32 oracle (bf16 rounding alone is 1.65e-3
# relative Frobenius error, above the 1e-3 bar).
# --------------------------------------------------------------------------
def scaled_mm_rowwise(qa: torch.Tensor, sa: torch.Tensor,
                      qb: torch.Tensor, sb: torch.Tensor,
                      accum: torch.dtype = torch.float32) -> torch.Tensor:
    """``torch._scaled_mm(a[M,K], b.t()[K,N], scale_a[M,1], scale_b[1,N])`` as forced
    by monkey_patch_for_fp8.py:26-34.  qa: uint8 [M, K]; qb: uint8 [N, K] (the
    contiguous buffer whose ``.t()`` the reference passes); sa [M,1]; sb [N,1]."""
    a = e4m3_to_f32(qa).to(accum)
    b = e4m3_to_f32(qb).to(accum)
    acc = a @ b.t()
    return (acc * sa.reshape(-1, 1).to(accum) * sb.reshape(1, -1).to(accum)).to(torch.float32)


def fp8_linear_rowwise(x: torch.Tensor, qw: torch.Tensor, sw: torch.Tensor,
                       accum: torch.dtype = torch.float32) -> torch.Tensor:
    """Per-token dynamic activation quant followed by the rowwise scaled mm
    (``Fp8LinearOp.apply`` installed at monkey_patch_for_fp8.py:74-79)."""
    qx, sx = quant_rowwise(x)
    return scaled_mm_rowwise(qx, sx, qw, sw, accum)


def scaled_mm_block128(qa: torch.Tensor, sa: torch.Tensor,
                       qb: torch.Tensor, sb: torch.Tensor,
                       accum: torch.dtype = torch.float32) -> torch.Tensor:
    """Block-scaled "nt" GEMM: qa uint8 [M, K] with sa [M, K/128]; qb uint8 [N, K]
    with sb [ceil(N/128), K/128]; out[m, n] = sum_kb (a_kb . b_kb) sa[m,kb] sb[n//128,kb]."""
    a = group128_dequant(qa, sa).to(accum)
    b = weight_dequant(qb, sb).to(accum)
    return (a @ b.t()).to(torch.float32)


def grouped_mm_block128(qa: torch.Tensor, sa: torch.Tensor,
                        qb: torch.Tensor, sb: torch.Tensor,
                        m_indices: torch.Tensor,
                        accum: torch.dtype = torch.float32) -> torch.Tensor:
    """``m_grouped_gemm_fp8_fp8_bf16_nt_contiguous`` (group_gemms.py:194-225): row r
    of qa is multiplied with expert ``m_indices[r]`` of qb [E, N, K]; rows whose
    index is negative are padding and produce zeros here (kernels leave them
    untouched)."""
    M, K = qa.shape
    E, N, _ = qb.shape
    out = torch.zeros(M, N, dtype=torch.float32)
    a = group128_dequant(qa, sa).to(accum)
    for e in range(E):
        rows = (m_indices == e).nonzero().flatten()
        if rows.numel() == 0:
            continue
        b = weight_dequant(qb[e], sb[e]).to(accum)
        out[rows] = (a[rows] @ b.t()).to(torch.float32)
    return out


def calc_diff(x: torch.Tensor, y: torch.Tensor) -> float:
    """The similarity metric of the reference's own FP8 tests (tests/test_deepep.py:62-67):
    1 - 2<x+1, y+1> / (|x+1|^2 + |y+1|^2) in fp64."""
    x, y = x.double() + 1, y.double() + 1
    return float(1 - 2 * (x * y).sum() / (x * x + y * y).sum())


def rel_frobenius(got: torch.Tensor, want: torch.Tensor) -> float:
    g, w = got.double(), want.double()
    denom = w.norm().item()
    return (g - w).norm().item() / (denom if denom > 0 else 1.0)


# --------------------------------------------------------------------------
# routing helpers for the MoE config (semantics of Gate + generate_permute_indices,
# cosmos_rl/policy/kernel/moe/moe.py:582-614 and moe/indices.py:177-220)
# --------------------------------------------------------------------------
def route_topk_contiguous(logits: torch.Tensor, top_k: int, alignment: int
                          ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns (token_of_row [M_pad] with -1 for padding, m_indices [M_pad] with -1 for
    padding, m_sizes [E] padded sizes, m_offsets [E] inclusive cumulative ends).
    Empty experts are clamped up to ``alignment`` rows of padding (indices.py:186-191)."""
    T, E = logits.shape
    topi = torch.topk(logits, top_k, dim=1).indices            # [T, k]
    flat_e = topi.reshape(-1)
    flat_t = torch.arange(T).repeat_interleave(top_k)
    order = torch.argsort(flat_e, stable=True)
    counts = torch.bincount(flat_e, minlength=E)
    padded = torch.clamp_min(((counts + alignment - 1) // alignment) * alignment, alignment)
    offsets = torch.cumsum(padded, 0)
    total = int(offsets[-1])
    token_of_row = torch.full((total,), -1, dtype=torch.int64)
    m_indices = torch.full((total,), -1, dtype=torch.int32)
    src = 0
    for e in range(E):
        start = int(offsets[e] - padded[e])
        c = int(counts[e])
        token_of_row[start:start + c] = flat_t[order[src:src + c]]
        m_indices[start:start + c] = e
        src += c
    return token_of_row, m_indices, padded.to(torch.int32), offsets.to(torch.int32)


# --------------------------------------------------------------------------
# seeded synthetic inputs of the five benchmark configurations
# --------------------------------------------------------------------------
def make_weight(shape: Sequence[int], seed: int, std: float = 0.02,
                outlier_frac: float = 0.0, outlier_mul: float = 1.0) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(*shape, generator=g, dtype=torch.float32) * std
    if outlier_frac > 0:
        mask = torch.rand(*shape, generator=g) < outlier_frac
        w = torch.where(mask, w * outlier_mul, w)
    return w.to(torch.bfloat16)


def make_activation(M: int, K: int, seed: int, chan_outlier_frac: float = 0.0,
                    outlier_mul: float = 1.0) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(M, K, generator=g, dtype=torch.float32)
    if chan_outlier_frac > 0:
        chan = torch.rand(K, generator=g) < chan_outlier_frac
        x = torch.where(chan[None, :], x * outlier_mul, x)
    return x.to(torch.bfloat16)


QWEN25_7B_LINEAR_SHAPES: List[Tuple[str, Tuple[int, int], int]] = [
    ("q_proj", (3584, 3584), 28), ("o_proj", (3584, 3584), 28),
    ("k_proj", (512, 3584), 28), ("v_proj", (512, 3584), 28),
    ("gate_proj", (18944, 3584), 28), ("up_proj", (18944, 3584), 28),
    ("down_proj", (3584, 18944), 28), ("lm_head", (152064, 3584), 1),
]


def qwen25_7b_numel() -> int:
    return sum(r * c * n for _, (r, c), n in QWEN25_7B_LINEAR_SHAPES)


assert qwen25_7b_numel() == 7_070_285_824
