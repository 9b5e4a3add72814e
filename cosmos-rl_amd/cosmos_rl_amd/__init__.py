"""cosmos_rl_amd: the FP8 hot path of cosmos-rl on MI355X (gfx950).

Layout mirrors the reference's module paths for the files on this path:

  ops                                      C-ABI shims named after the third-party ops replaced
  rollout/vllm_rollout/monkey_patch_for_fp8  rowwise FP8 linear method, weight caching helpers
  rollout/vllm_rollout/vllm_rollout          ``fp8_quantization``
  rollout/worker/rollout_control             quantise-on-receive step of weight sync
  utils/fp8/fp8_util                         recipes, module filter, model converter
  policy/kernel/group_gemms                  grouped GEMM strategies for MoE experts
"""
from . import _lib  # noqa: F401
from . import ops  # noqa: F401

__all__ = ["ops", "_lib"]
__version__ = "0.1.0"
