"""Host-side mirror of the reference's Python callers, on the CPU.  The HIP operators are
GPU-only, so these tests stand an oracle-backed stub in for ``ops.scaled_fp8_quant`` - the same
move the reference's own worker tests make with mocks - and check the protocol around it."""
from types import SimpleNamespace

import pytest
import torch
import torch.nn as nn

from oracle import fp8_oracle as O
from cosmos_rl_amd import ops
from cosmos_rl_amd.policy.kernel import group_gemms
from cosmos_rl_amd.rollout.vllm_rollout import monkey_patch_for_fp8 as mp
from cosmos_rl_amd.rollout.vllm_rollout import vllm_rollout
from cosmos_rl_amd.rollout.worker.rollout_control import QuantizedWeightReceiver
from cosmos_rl_amd.utils.fp8 import fp8_util


@pytest.fixture
def stub_quant(monkeypatch):
    calls = []

    def fake(input, scale=None, use_per_token_if_dynamic=False):
        assert scale is None and use_per_token_if_dynamic
        calls.append(tuple(input.shape))
        q, s = O.quant_rowwise(input)
        return q.view(torch.float8_e4m3fn), s

    monkeypatch.setattr(ops, "scaled_fp8_quant", fake)
    return calls


class ToyLinear(nn.Module):
    def __init__(self, out_f, in_f, quantized=True):
        super().__init__()
        self.weight = nn.Parameter(torch.randn(out_f, in_f).to(torch.bfloat16) * 0.02, requires_grad=False)
        if quantized:
            self.quant_method = mp.Fp8LinearMethod()


class ToyModel(nn.Module):
    def __init__(self):
        super().__init__()
        self.qkv_proj = ToyLinear(48, 32)
        self.o_proj = ToyLinear(32, 32)
        self.norm = ToyLinear(32, 32, quantized=False)
        self.other = ToyLinear(16, 32, quantized=False)
        self.other.quant_method = object()  # some other quantisation method: left alone


class Mapper:
    def rollout_map_local_key_to_hf_key(self, name):
        return "model." + name

    def get_unsplited_weight_name(self, name):
        for part in (".q_proj.", ".k_proj.", ".v_proj."):
            if part in name:
                return name.replace(part, ".qkv_proj.")
        return name


def load_fp8(model):
    for m in model.modules():
        qm = getattr(m, "quant_method", None)
        if isinstance(qm, mp.Fp8LinearMethod):
            qm.process_weights_after_loading(m)


def test_process_weights_after_loading_and_patches(stub_quant):
    torch.manual_seed(0)
    model = ToyModel()
    w0 = model.qkv_proj.weight.detach().clone()
    mp.simplify_process_weights_after_loading()
    load_fp8(model)
    lin = model.qkv_proj
    assert lin.weight.dtype == torch.float8_e4m3fn and tuple(lin.weight.shape) == (32, 48)
    assert lin.weight.stride() == (1, 32)                 # transposed view of a contiguous [out, in] buffer
    assert tuple(lin.weight_scale.shape) == (48, 1) and lin.input_scale is None
    qo, so = O.quant_rowwise(w0)
    assert torch.equal(lin.weight.t().contiguous().view(torch.uint8), qo) and torch.equal(lin.weight_scale, so)
    assert model.norm.weight.dtype == torch.bfloat16
    mp.apply_fp8_linear_patch(model)
    assert isinstance(lin.quant_method.fp8_linear, mp.Fp8LinearOp)
    assert lin.quant_method.fp8_linear.use_per_token_if_dynamic and not lin.quant_method.fp8_linear.cutlass_fp8_supported
    assert mp._dispatch["dispatch_w8a8_scaled_mm"]() is mp.torch_per_token_w8a8_scaled_mm
    assert lin.quant_method.fp8_linear.w8a8_scaled_mm is mp.torch_per_token_w8a8_scaled_mm   # the op reads the dispatch
    with pytest.raises(NotImplementedError):
        mp.Fp8LinearOp(use_per_token_if_dynamic=False)


def test_cache_replace_and_view_map(stub_quant):
    torch.manual_seed(1)
    model = ToyModel()
    load_fp8(model)
    mapper = Mapper()
    hp, orig = mp.cache_weight_of_quantized_module(model, torch.bfloat16, mapper, None)
    assert set(hp) == {"model.qkv_proj.weight", "model.o_proj.weight"} == set(orig)
    assert hp["model.qkv_proj.weight"].dtype == torch.bfloat16 and tuple(hp["model.qkv_proj.weight"].shape) == (48, 32)
    assert hp["model.qkv_proj.weight"].is_contiguous() and not hp["model.qkv_proj.weight"].requires_grad
    assert orig["model.qkv_proj.weight"] is model.qkv_proj.weight
    # the staging buffer holds the dequantised-without-scale bytes of the engine weight
    assert torch.equal(hp["model.o_proj.weight"], model.o_proj.weight.t().to(torch.bfloat16))
    mp.replace_weight_of_quantized_module(model, hp, mapper)
    assert model.qkv_proj.weight is hp["model.qkv_proj.weight"] and model.norm.weight.dtype == torch.bfloat16
    mp.replace_weight_of_quantized_module(model, orig, mapper)
    assert model.qkv_proj.weight is orig["model.qkv_proj.weight"]
    vm = {"a.weight": 1, "a.weight_scale": 2, "b.bias": 3}
    assert mp.post_process_view_map_for_fp8(vm) == {"a.weight": 1, "b.bias": 3}


class ToyRollout(vllm_rollout.FP8RolloutMixin):
    def __init__(self, model):
        self.model = model
        self._engine_initialized = True

    def get_underlying_model(self):
        return self.model


def test_model_param_map_and_quantized_tensors(stub_quant):
    """rollout_base.py:186-230: refuses before the engine is up, maps every state-dict entry to its HF name,
    caches the map."""
    model = ToyModel()
    load_fp8(model)
    mapper = Mapper()
    rollout = ToyRollout(model)
    rollout._engine_initialized = False
    assert rollout.is_engine_initialized() is False
    with pytest.raises(RuntimeError, match="Engine is not initialized, please call init_engine first"):
        rollout.model_param_map(mapper)
    with pytest.raises(RuntimeError, match="Engine is not initialized, please call init_engine first"):
        rollout.get_quantized_tensors(mapper)
    rollout._engine_initialized = True
    assert rollout.get_quantized_tensors(mapper) == {}
    pm = rollout.model_param_map(mapper)
    assert set(pm) == {"model.qkv_proj.weight", "model.qkv_proj.weight_scale", "model.o_proj.weight",
                       "model.o_proj.weight_scale", "model.norm.weight", "model.other.weight"}
    assert pm["model.qkv_proj.weight"].data_ptr() == model.qkv_proj.weight.data_ptr()
    assert pm["model.qkv_proj.weight"].stride() == (1, 32)
    assert rollout.model_param_map(mapper) is pm                       # cached


def test_sync_hooks_and_quantize_on_receive(stub_quant):
    """q/k/v shards arrive separately; the packed qkv weight is quantised once, after the group."""
    torch.manual_seed(2)
    model = ToyModel()
    load_fp8(model)
    stub_quant.clear()
    mapper = Mapper()
    rollout = ToyRollout(model)
    hp, quantized = rollout.pre_get_params_for_sync_hook("fp8", mapper, None)
    assert model.qkv_proj.weight is hp["model.qkv_proj.weight"]       # engine exposes hp buffers to the recv planner
    # (the recv view map is built from the model between the two hooks, as cosmos_rollout_prepare_recv does at
    # rollout_control.py:382-384; model_param_map is first asked for by a completion, after the second hook)
    view_map = {mapper.rollout_map_local_key_to_hf_key(k): v for k, v in model.state_dict().items()}
    view_map = rollout.post_get_params_for_sync_hook("fp8", mapper, view_map, quantized)
    assert not any("weight_scale" in k for k in view_map)
    assert model.qkv_proj.weight is quantized["model.qkv_proj.weight"]  # engine computes in fp8 again
    assert rollout.pre_get_params_for_sync_hook(None, mapper, None) == ({}, {})

    recv = QuantizedWeightReceiver(rollout, mapper, hp, quantized, "fp8")
    new_qkv = (torch.randn(48, 32) * 0.05).to(torch.bfloat16)
    group = ["model.q_proj.weight", "model.k_proj.weight", "model.v_proj.weight"]
    assert recv.full_weight_name_of_group(group) == "model.qkv_proj.weight"
    done = recv.plan_group(group, do_weight_sync_check=False)
    for i, _ in enumerate(group):                                      # the three "NCCL receives"
        hp["model.qkv_proj.weight"].data[i * 16:(i + 1) * 16].copy_(new_qkv[i * 16:(i + 1) * 16])
        assert stub_quant == []                                        # nothing quantised mid-group
    done()
    assert stub_quant == [(48, 32)]                                    # one quantisation of the packed weight
    qo, so = O.quant_rowwise(new_qkv)
    assert torch.equal(model.qkv_proj.weight.t().contiguous().view(torch.uint8), qo)
    assert torch.equal(model.qkv_proj.weight_scale, so)
    assert model.qkv_proj.weight.stride() == (1, 32)                   # copy_ kept the engine's layout

    # first-sync self check: passes when the engine already holds the same weights ...
    assert recv.check_inside_group(group, True) is False               # quantised weights skip the plain check
    recv.plan_group(group, do_weight_sync_check=True)()
    # ... and raises with the reference's message when it does not
    hp["model.qkv_proj.weight"].data.mul_(3.0).add_(0.01)
    with pytest.raises(ValueError, match="FP8 weight doesn't match after weight sync"):
        recv.plan_group(group, do_weight_sync_check=True)()
    # a non-quantised weight is not touched, and keeps the plain check
    assert recv.quantize_full_weight("model.norm.weight") is False
    assert recv.check_inside_group(["model.norm.weight"], True) is True
    # scale shape assert (rollout_control.py:895)
    model.o_proj.weight_scale = nn.Parameter(torch.zeros(32), requires_grad=False)
    rollout._model_param_map = None                                    # the map is cached: rebuild it for the new parameter
    with pytest.raises(AssertionError, match="scale_tensor.shape"):
        recv.quantize_full_weight("model.o_proj.weight")
    with pytest.raises(NotImplementedError):
        QuantizedWeightReceiver(rollout, mapper, hp, quantized, "mxfp4")


def test_flush_completions_batches_the_groups(stub_quant, monkeypatch):
    """rollout_control.py:1308-1319: the completions of a flush group run together - here as one table-driven
    quantiser call over the quantised weights of the batch, written into the engine's own parameters."""
    torch.manual_seed(4)
    model = ToyModel()
    load_fp8(model)
    mapper, rollout = Mapper(), ToyRollout(model)
    hp, quantized = rollout.pre_get_params_for_sync_hook("fp8", mapper, None)
    view_map = {mapper.rollout_map_local_key_to_hf_key(k): v for k, v in model.state_dict().items()}
    rollout.post_get_params_for_sync_hook("fp8", mapper, view_map, quantized)
    recv = QuantizedWeightReceiver(rollout, mapper, hp, quantized, "fp8")
    stub_quant.clear()
    batches = []

    def fake_multi(weights, q_outs, scale_outs):
        batches.append([tuple(w.shape) for w in weights])
        for w, q, sc in zip(weights, q_outs, scale_outs):
            qo, so = O.quant_rowwise(w)
            assert tuple(q.shape) == (w.shape[1], w.shape[0]) and q.stride() == (1, w.shape[1])   # the engine's layout
            q.copy_(qo.view(torch.float8_e4m3fn).t())
            sc.copy_(so)

    monkeypatch.setattr(ops, "quant_rowwise_multi_into", fake_multi)
    new_qkv = (torch.randn(48, 32) * 0.05).to(torch.bfloat16)
    new_o = (torch.randn(32, 32) * 0.02).to(torch.bfloat16)
    hp["model.qkv_proj.weight"].data.copy_(new_qkv)
    hp["model.o_proj.weight"].data.copy_(new_o)
    groups = [["model.q_proj.weight", "model.k_proj.weight", "model.v_proj.weight"], ["model.o_proj.weight"],
              ["model.norm.weight"], ["model.o_proj.weight"]]
    assert recv.flush_completions(groups) == ["model.qkv_proj.weight", "model.o_proj.weight"]
    assert batches == [[(48, 32), (32, 32)]] and stub_quant == []       # one batch, no per-weight call
    for lin, w in ((model.qkv_proj, new_qkv), (model.o_proj, new_o)):
        qo, so = O.quant_rowwise(w)
        assert torch.equal(lin.weight.t().contiguous().view(torch.uint8), qo) and torch.equal(lin.weight_scale, so)
    # with the first-sync check every weight takes the per-weight path (the check compares old and new bytes)
    assert recv.flush_completions(groups, do_weight_sync_check=True) == ["model.qkv_proj.weight", "model.o_proj.weight"]
    assert stub_quant == [(48, 32), (32, 32)] and len(batches) == 1
    assert QuantizedWeightReceiver(rollout, mapper, hp, quantized, None).flush_completions(groups) == []


def test_fp8_quantization_returns_transposed_view(stub_quant):
    w = O.make_weight((64, 32), seed=3)
    qt, s = vllm_rollout.fp8_quantization(w)
    assert tuple(qt.shape) == (32, 64) and qt.stride() == (1, 32) and tuple(s.shape) == (64, 1)


def test_recipes_filter_and_converter(monkeypatch):
    assert fp8_util.is_valid_fp8_recipe("dynamic_scaling") and fp8_util.is_valid_fp8_recipe("delayed_scaling")
    assert not fp8_util.is_valid_fp8_recipe("static")
    assert fp8_util.is_valid_fp8_quant_recipe("rowwise") and fp8_util.is_valid_fp8_quant_recipe("tensorwise")
    assert not fp8_util.is_valid_fp8_quant_recipe("blockwise")
    assert fp8_util.FP8QuantRecipe.ROWWISE == "rowwise" and str(fp8_util.FP8Recipe.DYNAMIC_SCALING) == "dynamic_scaling"
    f = fp8_util.module_filter_fn
    assert f(nn.Linear(128, 64), "model.layers.0.mlp.up_proj", ["lm_head"])
    assert not f(nn.Linear(128, 64), "lm_head", ["lm_head"])
    assert not f(nn.Linear(120, 64), "x", []) and not f(nn.Linear(128, 40), "x", [])
    # every multiple of 16 converts, as in the reference: the GEMM masks a last K step shorter than 128
    assert f(nn.Linear(80, 64), "x", []) and f(nn.Linear(1200, 64), "x", []) and f(nn.Linear(1280, 48), "x", [])
    assert not f(nn.LayerNorm(32), "x", [])

    def cfg(**kw):
        return SimpleNamespace(train=SimpleNamespace(fp8=fp8_util.FP8Config(**kw)))

    # no gfx950 device in this process: the converter refuses, like the reference does below sm89
    if not fp8_util.is_gfx950_available():
        with pytest.raises(RuntimeError, match="FP8 is only supported"):
            fp8_util.FP8ModelConverter(cfg(enable_fp8=True), None)
    monkeypatch.setattr(fp8_util, "is_gfx950_available", lambda: True)
    with pytest.raises(NotImplementedError, match="Delayed scaling"):
        fp8_util.FP8ModelConverter(cfg(enable_fp8=True, fp8_recipe="delayed_scaling"), None)
    with pytest.raises(AssertionError):
        fp8_util.FP8ModelConverter(cfg(enable_fp8=True, quant_recipe="blockwise"), None)

    class Net(nn.Module):
        def __init__(self):
            super().__init__()
            self.body = nn.Sequential(nn.Linear(128, 256), nn.ReLU(), nn.Linear(256, 24), nn.Linear(80, 64))
            self.lm_head = nn.Linear(128, 128)

        def fqn_filter_for_quantization(self):
            return ["lm_head"]

    net = Net()
    conv = fp8_util.FP8ModelConverter(cfg(enable_fp8=False), None)
    assert conv.convert_model(net) is None and type(net.body[0]) is nn.Linear
    conv = fp8_util.FP8ModelConverter(cfg(enable_fp8=True, quant_recipe="tensorwise"), None)
    w_before = net.body[0].weight
    conv.convert_model(net)
    assert isinstance(net.body[0], fp8_util.Float8Linear) and net.body[0].quant_recipe == "tensorwise"
    assert net.body[0].weight is w_before
    assert type(net.body[2]) is nn.Linear            # 24 is not a multiple of 16
    assert isinstance(net.body[3], fp8_util.Float8Linear)  # in_features 80: a multiple of 16, not of the GEMM's K step
    assert type(net.lm_head) is nn.Linear            # filtered by FQN
    assert conv.post_optimizer_hook(net) is None
    with pytest.raises(NotImplementedError):         # forward direction only
        net.body[0](torch.randn(2, 128, requires_grad=True))


def test_group_gemm_strategies_on_cpu():
    base = group_gemms.GroupGEMMStrategy(torch.nn.functional.silu)
    with pytest.raises(NotImplementedError):
        base.arrange_expert_weights([], "gate_proj", None)
    with pytest.raises(NotImplementedError):
        base.execute(None, None, None, None)
    assert group_gemms.GroupGEMMStrategy.is_available() is False
    assert group_gemms.TorchBF16GroupGEMM.is_available() is True
    if not torch.cuda.is_available():
        assert group_gemms.DSGroupGEMM.is_available() is False

    E, H, I = 3, 32, 16
    g = torch.Generator().manual_seed(0)
    mod = nn.Module()
    strat = group_gemms.TorchBF16GroupGEMM(torch.nn.functional.silu)
    for name, shape in (("gate_proj", (I, H)), ("up_proj", (I, H)), ("down_proj", (H, I))):
        ws = [(torch.randn(*shape, generator=g) * 0.1).to(torch.bfloat16) for _ in range(E)]
        mod.register_parameter(f"{name}_weight", nn.Parameter(strat.arrange_expert_weights(ws, name, mod), requires_grad=False))
    x = torch.randn(10, H, generator=g).to(torch.bfloat16)
    offs = torch.tensor([4, 4, 10], dtype=torch.int32)                 # expert 1 is empty
    out = strat.execute(x, None, offs, mod)
    for e, (a, b) in enumerate([(0, 4), (4, 4), (4, 10)]):
        if b > a:
            h = torch.nn.functional.silu(x[a:b] @ mod.gate_proj_weight[e].t()) * (x[a:b] @ mod.up_proj_weight[e].t())
            assert torch.equal(out[a:b], h @ mod.down_proj_weight[e].t())


def test_create_indices_from_offsets():
    offs = torch.tensor([128, 128, 384], dtype=torch.int32)
    idx = ops.create_indices_from_offsets_nosync(offs, 384)
    assert idx.dtype == torch.int32 and idx.numel() == 384
    assert bool((idx[:128] == 0).all()) and bool((idx[128:] == 2).all())
    assert torch.equal(idx, ops.create_indices_from_offsets_nosync(offs))
    # a row bound instead of the exact count: rows past the last group are padding (-1), nothing is read back
    cap = ops.create_indices_from_offsets_nosync(offs, 640, n_experts=3)
    assert torch.equal(cap[:384], idx) and bool((cap[384:] == -1).all())
