"""The tensorwise quantiser that allocates nothing (amax slots inside the library's device image)
gives the bits of the workspace-taking entry point, call after call on one GPU."""
import pytest
import torch

from cosmos_rl_amd import _lib, ops
from oracle import fp8_oracle as O

pytestmark = pytest.mark.gpu


def _run_both(dev, shapes, seed):
    ws = [O.make_weight(sh, seed=seed + i, std=0.02 * (1 + i % 5)).to(dev) for i, sh in enumerate(shapes)]
    want_q, want_s = ops.quant_tensorwise_multi(ws)
    outs = [torch.full(w.shape, 0x55, dtype=torch.uint8, device=dev).view(ops.FP8_DTYPE) for w in ws]
    scales = torch.full((len(ws),), -1.0, dtype=torch.float32, device=dev)
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    ops.quant_tensorwise_multi_static(ws, outs, scales)
    after = torch.cuda.memory_stats(dev)["allocation.all.allocated"]
    torch.cuda.synchronize()
    assert after == before, "the no-allocation entry point went through torch's allocator"
    assert torch.equal(scales.view(torch.int32), want_s.view(torch.int32)), "scales differ"
    for i, (q, wq) in enumerate(zip(outs, want_q)):
        assert torch.equal(q.view(torch.uint8), wq.view(torch.uint8)), f"tensor {i} bytes differ"
    return ws, outs, scales


def test_static_slots_match_workspace_entry_point_on_consecutive_calls(dev):
    # first call: more tensors than one descriptor table holds, large amax values left in the slots
    big = [(3584, 512), (512, 512), (1184, 512), (512, 1184), (300, 72), (2048 * 8 + 8,), (0, 16), (1, 8)] + \
          [(16 + 8 * (i % 5), 64) for i in range(60)]
    ws, _, _ = _run_both(dev, big, seed=900)
    # second call, right behind it on the same GPU: fewer and smaller tensors with much smaller values, so a
    # slot that kept the first call's maximum would change the scale
    small = [(64, 64), (8, 8), (128, 24)]
    tiny = [O.make_weight(sh, seed=77 + i, std=1e-4).to(dev) for i, sh in enumerate(small)]
    want_q, want_s = ops.quant_tensorwise_multi(tiny)
    outs = [torch.empty(w.shape, dtype=ops.FP8_DTYPE, device=dev) for w in tiny]
    scales = torch.empty(len(tiny), dtype=torch.float32, device=dev)
    ops.quant_tensorwise_multi_static(tiny, outs, scales)
    assert torch.equal(scales.view(torch.int32), want_s.view(torch.int32)), "second call: scales differ"
    for i, (q, wq) in enumerate(zip(outs, want_q)):
        assert torch.equal(q.view(torch.uint8), wq.view(torch.uint8)), f"second call: tensor {i} bytes differ"
    # and against the oracle, so both entry points cannot be wrong together
    for i, w in enumerate(tiny):
        qo, so = O.quant_tensorwise(w.cpu())
        assert torch.equal(outs[i].view(torch.uint8).cpu(), qo) and torch.equal(scales[i:i + 1].view(torch.int32).cpu(), so.view(torch.int32))
    # a third call at the capacity limit
    cap = [(8, 8)] * _lib.TENSORWISE_STATIC_MAX_TENSORS
    _run_both(dev, cap, seed=3000)


def test_static_slots_capacity_is_an_error(dev):
    n = _lib.TENSORWISE_STATIC_MAX_TENSORS + 1
    ws = [torch.zeros(8, 8, dtype=torch.bfloat16, device=dev)] * n
    outs = [torch.empty(8, 8, dtype=ops.FP8_DTYPE, device=dev) for _ in range(n)]
    scales = torch.empty(n, dtype=torch.float32, device=dev)
    with pytest.raises(RuntimeError, match="exceed"):
        ops.quant_tensorwise_multi_static(ws, outs, scales)
