"""The reference-named Python entry points running on the HIP kernels (through the C ABI)."""
from types import SimpleNamespace

import pytest
import torch
import torch.nn as nn

from oracle import fp8_oracle as O
from cosmos_rl_amd import ops
from cosmos_rl_amd.policy.kernel import group_gemms
from cosmos_rl_amd.rollout.vllm_rollout import monkey_patch_for_fp8 as mp
from cosmos_rl_amd.rollout.vllm_rollout.vllm_rollout import FP8RolloutMixin, fp8_quantization
from cosmos_rl_amd.rollout.worker.rollout_control import QuantizedWeightReceiver
from cosmos_rl_amd.utils.fp8 import fp8_util

pytestmark = pytest.mark.gpu


class Lin(nn.Module):
    def __init__(self, w):
        super().__init__()
        self.weight = nn.Parameter(w, requires_grad=False)
        self.quant_method = mp.Fp8LinearMethod()

    def forward(self, x):
        return self.quant_method.apply(self, x)


class Model(nn.Module):
    def __init__(self, dev):
        super().__init__()
        self.qkv_proj = Lin(O.make_weight((4608, 3584), seed=1).to(dev))
        self.down_proj = Lin(O.make_weight((3584, 2048), seed=2).to(dev))


class Mapper:
    def rollout_map_local_key_to_hf_key(self, n):
        return n

    def get_unsplited_weight_name(self, n):
        for p in ("q_proj.", "k_proj.", "v_proj."):
            if n.startswith(p):
                return "qkv_proj." + n[len(p):]
        return n


class Rollout(FP8RolloutMixin):
    def __init__(self, model):
        self.model = model
        self._engine_initialized = True

    def get_underlying_model(self):
        return self.model


def recv_view_map(model, mapper):
    # what cosmos_rollout_prepare_recv builds between the two hooks (rollout_control.py:382-384)
    return {mapper.rollout_map_local_key_to_hf_key(k): v for k, v in model.state_dict().items()}


def test_weight_sync_end_to_end(dev):
    """Engine load -> patch -> forward -> a weight sync of the packed qkv weight -> forward."""
    model = Model(dev)
    w_qkv = model.qkv_proj.weight.detach().clone()
    mp.simplify_process_weights_after_loading()
    for m in model.children():
        m.quant_method.process_weights_after_loading(m)
    mp.apply_fp8_linear_patch(model)
    qo, so = O.quant_rowwise(w_qkv.cpu())
    assert torch.equal(model.qkv_proj.weight.t().contiguous().view(torch.uint8).cpu(), qo)
    assert torch.equal(model.qkv_proj.weight_scale.cpu(), so)

    x = O.make_activation(48, 3584, seed=3, chan_outlier_frac=0.005, outlier_mul=30.0)
    y = model.qkv_proj(x.to(dev))
    ref = O.fp8_linear_rowwise(x, qo, so, accum=torch.float64)
    assert y.dtype == torch.bfloat16 and O.rel_frobenius(y.float().cpu(), ref.to(torch.bfloat16).float()) <= 1e-3

    mapper, rollout = Mapper(), Rollout(model)
    hp, quantized = rollout.pre_get_params_for_sync_hook("fp8", mapper, None)
    view = rollout.post_get_params_for_sync_hook("fp8", mapper, recv_view_map(model, mapper), quantized)
    assert "qkv_proj.weight_scale" not in view
    recv = QuantizedWeightReceiver(rollout, mapper, hp, quantized, "fp8")
    # first sync: the policy sends the very weights the engine was loaded with -> self check passes
    hp["qkv_proj.weight"].data.copy_(w_qkv)
    recv.plan_group(["q_proj.weight", "k_proj.weight", "v_proj.weight"], do_weight_sync_check=True)()
    # later sync: new weights
    w_new = O.make_weight((4608, 3584), seed=9, std=0.03)
    hp["qkv_proj.weight"].data.copy_(w_new.to(dev))
    assert recv.quantize_full_weight("qkv_proj.weight") is True
    qn, sn = O.quant_rowwise(w_new)
    assert torch.equal(model.qkv_proj.weight.t().contiguous().view(torch.uint8).cpu(), qn)
    assert torch.equal(model.qkv_proj.weight_scale.cpu(), sn)
    y2 = model.qkv_proj(x.to(dev))
    ref2 = O.fp8_linear_rowwise(x, qn, sn, accum=torch.float64)
    assert O.rel_frobenius(y2.float().cpu(), ref2.to(torch.bfloat16).float()) <= 1e-3
    # a mismatching engine weight fails the first-sync check with the reference's error
    hp["qkv_proj.weight"].data.mul_(2.0).add_(0.01)
    with pytest.raises(ValueError, match="FP8 weight doesn't match"):
        recv.quantize_full_weight("qkv_proj.weight", do_weight_sync_check=True)


def test_fused_receive_quantises_row_shards_in_place(dev):
    """q/k/v shards arrive in fp32, each holds whole rows of the packed qkv weight: quantise-on-receive writes
    the engine's fp8 parameter and weight_scale directly; the result equals the unfused path bit for bit."""
    model = Model(dev)
    mp.simplify_process_weights_after_loading()
    for m in model.children():
        m.quant_method.process_weights_after_loading(m)
    mapper, rollout = Mapper(), Rollout(model)
    hp, quantized = rollout.pre_get_params_for_sync_hook("fp8", mapper, None)
    rollout.post_get_params_for_sync_hook("fp8", mapper, recv_view_map(model, mapper), quantized)
    recv = QuantizedWeightReceiver(rollout, mapper, hp, quantized, "fp8")
    g = torch.Generator().manual_seed(11)
    w32 = torch.randn(4608, 3584, generator=g) * 0.03                       # transfer dtype fp32
    for a, b in ((0, 3584), (3584, 4096), (4096, 4608)):                    # q, k, v row ranges
        assert recv.quantize_received_rows("qkv_proj.weight", w32[a:b].to(dev), row_start=a) is True
    qo, so = O.quant_rowwise_from(w32)
    assert torch.equal(model.qkv_proj.weight.t().contiguous().view(torch.uint8).cpu(), qo)
    assert torch.equal(model.qkv_proj.weight_scale.cpu().view(torch.int32), so.view(torch.int32))
    # same bytes as the reference's three-pass route through the bf16 staging parameter
    hp["qkv_proj.weight"].data.copy_(w32.to(dev).to(torch.bfloat16))
    before = model.qkv_proj.weight.t().contiguous().view(torch.uint8).clone()
    recv.quantize_full_weight("qkv_proj.weight")
    assert torch.equal(model.qkv_proj.weight.t().contiguous().view(torch.uint8), before)
    assert recv.quantize_received_rows("not_quantised.weight", w32[:8].to(dev)) is False
    with pytest.raises(ValueError, match="do not fit"):
        recv.quantize_received_rows("qkv_proj.weight", w32[:64].to(dev), row_start=4600)


def test_flush_completions_quantises_a_batch_in_place(dev):
    """The completions of a flush group run together: both weights go from their staging parameters into the
    engine's fp8 parameters and weight_scale tensors through the table-driven quantiser; same bytes as one
    quantize_full_weight per group, and the first-sync check still takes the per-weight path."""
    model = Model(dev)
    mp.simplify_process_weights_after_loading()
    for m in model.children():
        m.quant_method.process_weights_after_loading(m)
    mapper, rollout = Mapper(), Rollout(model)
    hp, quantized = rollout.pre_get_params_for_sync_hook("fp8", mapper, None)
    rollout.post_get_params_for_sync_hook("fp8", mapper, recv_view_map(model, mapper), quantized)
    recv = QuantizedWeightReceiver(rollout, mapper, hp, quantized, "fp8")
    w_qkv = O.make_weight((4608, 3584), seed=21, std=0.03)
    w_down = O.make_weight((3584, 2048), seed=22, std=0.01)
    hp["qkv_proj.weight"].data.copy_(w_qkv.to(dev))
    hp["down_proj.weight"].data.copy_(w_down.to(dev))
    groups = [["q_proj.weight", "k_proj.weight", "v_proj.weight"], ["down_proj.weight"], ["norm.weight"]]
    assert recv.flush_completions(groups) == ["qkv_proj.weight", "down_proj.weight"]
    for lin, w in ((model.qkv_proj, w_qkv), (model.down_proj, w_down)):
        qo, so = O.quant_rowwise(w)
        assert torch.equal(lin.weight.t().contiguous().view(torch.uint8).cpu(), qo)
        assert torch.equal(lin.weight_scale.cpu().view(torch.int32), so.view(torch.int32))
        assert lin.weight.stride() == (1, w.shape[1])
    # the engine now holds these weights: the first-sync check passes, and fails once the policy's differ
    assert recv.flush_completions(groups, do_weight_sync_check=True) == ["qkv_proj.weight", "down_proj.weight"]
    hp["down_proj.weight"].data.mul_(2.0).add_(0.01)
    with pytest.raises(ValueError, match="FP8 weight doesn't match"):
        recv.flush_completions(groups, do_weight_sync_check=True)


def test_fp8_quantization_layout(dev):
    w = O.make_weight((3584, 18944), seed=4).to(dev)
    qt, s = fp8_quantization(w)
    assert tuple(qt.shape) == (18944, 3584) and qt.stride() == (1, 18944) and tuple(s.shape) == (3584, 1)
    param = torch.empty(3584, 18944, dtype=torch.float8_e4m3fn, device=dev).t()
    param.copy_(qt)                                      # same strides: a flat byte copy
    assert torch.equal(param.t().contiguous().view(torch.uint8), qt.t().contiguous().view(torch.uint8))


def test_float8_linear_recipes(dev):
    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.up = nn.Linear(512, 1024, bias=True)
            self.odd = nn.Linear(1200, 48, bias=True)    # multiples of 16 only: the GEMM's masked last K step
            self.lm_head = nn.Linear(512, 256, bias=False)

        def fqn_filter_for_quantization(self):
            return ["lm_head"]

    x = O.make_activation(40, 512, seed=5)
    for recipe in ("rowwise", "tensorwise"):
        torch.manual_seed(0)
        net = Net().to(dev).to(torch.bfloat16)
        cfg = SimpleNamespace(train=SimpleNamespace(fp8=fp8_util.FP8Config(enable_fp8=True, quant_recipe=recipe)))
        fp8_util.FP8ModelConverter(cfg, None).convert_model(net)
        assert isinstance(net.up, fp8_util.Float8Linear) and type(net.lm_head) is nn.Linear
        with torch.no_grad():
            y = net.up(x.to(dev))
        w, b = net.up.weight.detach().cpu(), net.up.bias.detach().cpu()
        if recipe == "rowwise":
            qw, sw = O.quant_rowwise(w)
            ref = O.fp8_linear_rowwise(x, qw, sw, accum=torch.float64)
        else:
            qw, sw = O.quant_tensorwise(w)
            qx, sx = O.quant_tensorwise(x)
            ref = O.scaled_mm_rowwise(qx, sx.expand(40, 1), qw, sw.expand(1024, 1), accum=torch.float64)
        ref = (ref.to(torch.bfloat16) + b).float()
        assert y.dtype == torch.bfloat16 and O.rel_frobenius(y.float().cpu(), ref) <= 2e-3
        if recipe == "rowwise":
            assert isinstance(net.odd, fp8_util.Float8Linear)
            x2 = O.make_activation(33, 1200, seed=6)
            with torch.no_grad():
                y2 = net.odd(x2.to(dev))
            qw2, sw2 = O.quant_rowwise(net.odd.weight.detach().cpu())
            ref2 = (O.fp8_linear_rowwise(x2, qw2, sw2, accum=torch.float64).to(torch.bfloat16) + net.odd.bias.detach().cpu()).float()
            assert O.rel_frobenius(y2.float().cpu(), ref2) <= 2e-3


def test_ds_group_gemm_strategy(dev):
    """DSGroupGEMM.arrange_expert_weights + execute against the oracle pipeline
    (1x128 quant -> grouped gate/up GEMMs -> silu*up -> 1x128 quant -> grouped down GEMM)."""
    assert group_gemms.DSGroupGEMM.is_available()
    E, H, I, T, topk = 8, 512, 256, 200, 2
    g = torch.Generator().manual_seed(11)
    act = torch.nn.functional.silu
    strat = group_gemms.DSGroupGEMM(act)
    mod = nn.Module()
    weights = {}
    for name, shape in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
        ws = [O.make_weight(shape, seed=100 + 10 * e + len(name), std=0.05) for e in range(E)]
        weights[name] = torch.stack(ws)
        stacked = strat.arrange_expert_weights([w.to(dev) for w in ws], name, mod)
        mod.register_parameter(f"{name}_weight", nn.Parameter(stacked, requires_grad=False))
        qo, so = O.quant_block128(weights[name])
        assert torch.equal(mod.get_parameter(f"{name}_fp8").view(torch.uint8).cpu(), qo)
        assert torch.equal(mod.get_parameter(f"{name}_scales").cpu(), so)
    logits = torch.rand(T, E, generator=g)
    tok, m_idx, m_sizes, m_offsets = O.route_topk_contiguous(logits, topk, 128)
    x = O.make_activation(T, H, seed=12)
    xs = torch.zeros(tok.numel(), H, dtype=torch.bfloat16)
    xs[tok >= 0] = x[tok[tok >= 0]]
    out = strat.execute(xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod).cpu()
    # the same module through the other kernel choices: one fused gate_up GEMM gives the very same bits as two
    # GEMMs; the unfused activation (torch silu, mul, then the quantiser) may differ by a bf16 ulp in the hidden state
    assert strat.fuse_swiglu and not strat.fuse_gate_up
    out_gu = group_gemms.DSGroupGEMM(act, fuse_gate_up=True).execute(
        xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod).cpu()
    assert torch.equal(out_gu, out)                      # SwiGLU + requantisation as the epilogue of the one GEMM
    out_gu2 = group_gemms.DSGroupGEMM(act, fuse_gate_up=True, fuse_epilogue=False).execute(
        xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod).cpu()
    assert torch.equal(out_gu2, out)                     # one fused GEMM, then the SwiGLU quantiser
    # straight from the token matrix: the gather and the first quantisation in one pass
    out_ft = strat.execute_from_tokens(x.to(dev), tok.to(torch.int32).to(dev), m_sizes.to(dev), m_offsets.to(dev), mod).cpu()
    assert torch.equal(out_ft, out[:out_ft.shape[0]])
    out_plain = group_gemms.DSGroupGEMM(act, fuse_swiglu=False).execute(
        xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod).cpu()
    assert O.rel_frobenius(out_plain.float(), out.float()) <= 5e-3
    assert not group_gemms.DSGroupGEMM(torch.nn.functional.gelu).fuse_swiglu

    # oracle pipeline; execute() treats every row of a padded group as belonging to that expert
    full_idx = ops.create_indices_from_offsets_nosync(m_offsets, tok.numel())
    qx, sx = O.quant_group128(xs)
    def gmm(name, qa, sa):
        qb, sb = O.quant_block128(weights[name])
        return O.grouped_mm_block128(qa, sa, qb, sb, full_idx, accum=torch.float64).to(torch.bfloat16)
    hidden = act(gmm("gate_proj", qx, sx)) * gmm("up_proj", qx, sx)
    qh, sh = O.quant_group128(hidden)
    ref = gmm("down_proj", qh, sh)
    valid = tok >= 0
    # bf16 intermediates may differ by an ulp between kernel and oracle, which re-quantisation
    # can amplify to one e4m3 step on isolated entries: compare in Frobenius norm
    assert O.rel_frobenius(out[valid].float(), ref[valid].float()) <= 5e-3
    assert bool((out[~valid] == 0).all())               # zero tokens in, zeros out

    # a buffer with more rows than the groups fill (a capacity bound): nothing is read back from the device, the
    # rows of the groups equal the exact-size call and the rows past the last group keep what they held
    cap = torch.full((tok.numel() + 256, H), 7.0, dtype=torch.bfloat16, device=dev)
    cap[:tok.numel()] = xs.to(dev)
    for kw in ({}, {"fuse_gate_up": True}, {"fuse_swiglu": False}):
        want = group_gemms.DSGroupGEMM(act, **kw).execute(xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod)
        got = group_gemms.DSGroupGEMM(act, **kw).execute(cap.clone(), m_sizes.to(dev), m_offsets.to(dev), mod)
        assert torch.equal(got[:tok.numel()], want) and bool((got[tok.numel():] == 7.0).all())
    # a row count that is no multiple of 128 takes the reference's route (slice by m_offsets[-1])
    odd = torch.cat([xs.to(dev), torch.full((40, H), 7.0, dtype=torch.bfloat16, device=dev)])
    got = strat.execute(odd, m_sizes.to(dev), m_offsets.to(dev), mod)
    assert torch.equal(got[:tok.numel()].cpu(), out) and bool((got[tok.numel():] == 7.0).all())

    # the fused copies of the gate / up weights follow in-place updates of the parameters they were built from
    for kw in ({"fuse_gate_up": True}, {"fuse_gate_up": True, "fuse_epilogue": False}):
        st2 = group_gemms.DSGroupGEMM(act, **kw)
        before = st2.execute(xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod)
        saved = mod.gate_proj_fp8.detach().clone()
        with torch.no_grad():
            mod.gate_proj_fp8.copy_(mod.up_proj_fp8)                       # same storage, new contents
        after = st2.execute(xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod)
        fresh = group_gemms.DSGroupGEMM(act).execute(xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod)
        assert not torch.equal(after, before) and torch.equal(after, fresh)
        mod.gate_proj_fp8.data.copy_(saved)                                # a write that no version counter sees ...
        st2.invalidate_fused_weights(mod)                                  # ... is announced by the writer
        assert torch.equal(st2.execute(xs.to(dev).clone(), m_sizes.to(dev), m_offsets.to(dev), mod), before)
