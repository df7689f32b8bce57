"""Host-side behaviour of the transform and the training-context decision table
(no GPU needed).  Mirrors what the reference's tests check with mocks:
tests/model/test_transformer_engine_transform.py:206-229 (disabled => identity),
:231-295,:322-403 (top-level and nested swaps, in place);
tests/optim/test_fp8_context.py:31-53 (dict keys), :152-228 (fallbacks, scaler off)."""
from contextlib import nullcontext

import pytest
import torch
import torch.nn as nn

from optimus_dl_amd.core.registry import RegistryConfig, RegistryConfigStrict, make_registry
from optimus_dl_amd.modules.amp import AmpConfig, Fp8Config, OptimizationConfig, fp8_autocast, fp8_backward
from optimus_dl_amd.modules.fp8_linear import FP8Linear
from optimus_dl_amd.modules.model import GPT2, GPT2Config, Llama, LlamaConfig, Qwen3, Qwen3Config
from optimus_dl_amd.modules.model_transforms import build_model_transform
from optimus_dl_amd.modules.model_transforms import fp8_linear_transform as T
from optimus_dl_amd.recipe import TrainingContext, execute_backward_pass, execute_forward_pass


class Nested(nn.Module):
    def __init__(self):
        super().__init__()
        self.fc = nn.Linear(16, 32)
        self.inner = nn.Sequential(nn.Linear(32, 32, bias=False), nn.LayerNorm(32), nn.ModuleList([nn.Linear(32, 16)]))

    def forward(self, x):
        return self.inner[2][0](self.inner[1](self.inner[0](self.fc(x))))


class MyLinear(nn.Linear):
    pass


def test_disabled_is_identity():
    m = Nested()
    before = {n: id(mod) for n, mod in m.named_modules()}
    out = build_model_transform({"_name": "transformer_engine", "enabled": False}).apply(m, device=None, collective=None)
    assert out is m and before == {n: id(mod) for n, mod in m.named_modules()}


def test_backend_missing_is_identity(monkeypatch):
    monkeypatch.setattr(T, "_HAVE_TE", False)
    m = Nested()
    out = build_model_transform({"_name": "transformer_engine"}).apply(m)
    assert out is m and type(m.fc) is nn.Linear


def test_swap_nested_in_place_and_share_parameters(monkeypatch):
    monkeypatch.setattr(T, "_HAVE_TE", True)
    m = Nested()
    m.sub = MyLinear(4, 4)                       # exact class match only: subclasses stay
    w_before, b_before = m.fc.weight, m.fc.bias
    keys_before = sorted(m.state_dict().keys())
    x = torch.randn(3, 16)
    y_before = m(x)
    t = build_model_transform({"_name": "transformer_engine", "verbose": True})
    out = t.apply(m, collective=None, device=torch.device("cpu"), is_restart=False, checkpoint_manager=None)
    assert out is m
    assert isinstance(m.fc, FP8Linear) and isinstance(m.inner[0], FP8Linear) and isinstance(m.inner[2][0], FP8Linear)
    assert type(m.sub) is MyLinear
    # the LayerNorm is the same object, still an nn.LayerNorm, with the fused forward mixed in
    assert isinstance(m.inner[1], nn.LayerNorm) and type(m.inner[1]).__name__ == "LayerNorm" and m.inner[1]._odl_fused_layernorm
    assert t.last_replacements == {"Linear": 3, "RMSNorm": 0, "LayerNorm": 1, "Attention": 0}
    assert m.fc.weight is w_before and m.fc.bias is b_before                 # same Parameter objects
    assert sorted(m.state_dict().keys()) == keys_before                     # no key renames
    assert m.inner[0].bias is None and m.fc.in_features == 16 and m.fc.out_features == 32 and m.fc.use_bias is True
    assert m.fc._te_linear is m.fc
    torch.testing.assert_close(m(x), y_before)                              # outside FP8 autocast: a plain Linear
    assert isinstance(m.fc, nn.Linear)


def test_replace_linear_false_and_not_inplace(monkeypatch):
    monkeypatch.setattr(T, "_HAVE_TE", True)
    m = Nested()
    build_model_transform({"_name": "fp8_linear", "replace_linear": False}).apply(m)
    assert type(m.fc) is nn.Linear
    t = build_model_transform({"_name": "fp8_linear", "replace_inplace": False})
    t.apply(m)
    assert type(m.fc) is nn.Linear and t.last_replacements["Linear"] == 3    # counted, not installed


def test_linear_kwargs_are_forwarded(monkeypatch):
    monkeypatch.setattr(T, "_HAVE_TE", True)
    m = Nested()
    build_model_transform({"_name": "transformer_engine", "linear_kwargs": {"sequence_parallel": True}}).apply(m)
    assert m.fc.kwargs == {"sequence_parallel": True}


@pytest.mark.parametrize("family", ["llama", "qwen3", "gpt2"])
def test_swap_on_model_families(monkeypatch, family):
    monkeypatch.setattr(T, "_HAVE_TE", True)
    if family == "llama":
        m = Llama(LlamaConfig(vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=64, intermediate_size=128))
        per_block, tied = 7, False
    elif family == "qwen3":
        m = Qwen3(Qwen3Config(vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=64, head_dim=32, intermediate_size=128))
        per_block, tied = 7, True
    else:
        m = GPT2(GPT2Config(vocab_size=256, n_layer=2, n_head=4, n_embd=64, block_size=32))
        per_block, tied = 6, True
    keys = sorted(m.state_dict().keys())
    n_params = sum(p.numel() for p in m.parameters())
    t = build_model_transform({"_name": "transformer_engine"})
    t.apply(m)
    assert t.last_replacements["Linear"] == 2 * per_block + 1
    blk = m.transformer.h[0]
    for name in ("wq", "wk", "wv", "wo"):
        assert isinstance(getattr(blk.attn, name), FP8Linear)
    if family == "gpt2":
        assert isinstance(blk.mlp.c_fc, FP8Linear) and isinstance(blk.mlp.c_proj, FP8Linear)
    else:
        assert isinstance(blk.mlp.w1, FP8Linear) and isinstance(blk.mlp.w2, FP8Linear) and isinstance(blk.mlp.c_proj, FP8Linear)
    assert isinstance(m.lm_head, FP8Linear)
    assert (m.transformer.wte.weight is m.lm_head.weight) == tied           # tying survives the swap
    assert sorted(m.state_dict().keys()) == keys and sum(p.numel() for p in m.parameters()) == n_params
    out = m(torch.randint(0, 256, (2, 16)))["logits"]
    assert out.shape == (2, 16, 256)
    out.float().mean().backward()
    assert blk.attn.wq.weight.grad is not None


def test_registry_basics():
    table, register, build = make_registry("unit_test_registry")

    from dataclasses import dataclass

    @dataclass
    class Cfg(RegistryConfig):
        a: int = 1

    @dataclass
    class Strict(RegistryConfigStrict):
        b: int = 2

    @register("thing", Cfg)
    class Thing:
        def __init__(self, cfg, **kw):
            self.cfg, self.kw = cfg, kw

    @register("strict", Strict)
    class StrictThing(Thing):
        pass

    t = build({"_name": "thing", "a": 5, "extra": "x"}, device="d")
    assert t.cfg.a == 5 and t.cfg["extra"] == "x" and t.kw == {"device": "d"}
    assert build(Cfg(_name="thing")).cfg.a == 1
    with pytest.raises(ValueError):
        build({"_name": "strict", "zzz": 1})
    with pytest.raises(ValueError, match="unknown"):
        build({"_name": "nope"})
    with pytest.raises(ValueError):
        build({"a": 1})
    assert build(None) is None


# ------------------------------------------------------------- training context
class FakeCuda:
    type = "cuda"


def opt(dtype, enabled=True, fp8_enabled=True, **fp8):
    return OptimizationConfig(amp=AmpConfig(enabled=enabled, dtype=dtype, fp8=Fp8Config(enabled=fp8_enabled, **fp8)))


def test_context_keys_and_bf16_path():
    ctx = TrainingContext(opt("torch.bfloat16", fp8_enabled=False)).setup_training_context(torch.device("cpu"))
    assert set(ctx) == {"scaler", "amp_ctx", "amp_cfg", "device", "fp8_recipe", "fp8_enabled", "is_fp8_dtype", "fp8_backward_ctx"}
    assert ctx["fp8_recipe"] is None and ctx["fp8_enabled"] is False and ctx["is_fp8_dtype"] is False
    assert isinstance(ctx["fp8_backward_ctx"], nullcontext) and not ctx["scaler"].is_enabled()


def test_fp8_on_cpu_raises():
    with pytest.raises(ValueError, match="FP8 training is only supported on CUDA devices"):
        TrainingContext(opt("torch.float8_e4m3fn")).setup_training_context(torch.device("cpu"))


def test_fp8_dtype_but_fp8_disabled_falls_back_to_amp(monkeypatch):
    monkeypatch.setattr(torch.cuda, "is_bf16_supported", lambda *a, **k: True)
    ctx = TrainingContext(opt("torch.float8_e4m3fn", fp8_enabled=False)).setup_training_context(FakeCuda())
    assert ctx["is_fp8_dtype"] is True and ctx["fp8_enabled"] is False and ctx["fp8_recipe"] is None
    assert isinstance(ctx["amp_ctx"], torch.autocast) and ctx["amp_ctx"].fast_dtype == torch.bfloat16
    assert not ctx["scaler"].is_enabled()                                    # FP8 dtype always switches the loss scaler off


def test_fp8_requested_without_backend_falls_back(monkeypatch):
    import optimus_dl_amd.recipe.training_context as tc

    monkeypatch.setattr(tc, "is_transformer_engine_available", lambda: False)
    monkeypatch.setattr(torch.cuda, "is_bf16_supported", lambda *a, **k: True)
    ctx = TrainingContext(opt("torch.float8_e4m3fn")).setup_training_context(FakeCuda())
    assert ctx["fp8_enabled"] is False and isinstance(ctx["amp_ctx"], torch.autocast)


def test_scaler_for_fp16_only():
    c16 = TrainingContext(opt("torch.float16", fp8_enabled=False)).setup_training_context(torch.device("cpu"))
    assert c16["amp_cfg"].resolved_enable_scaler() is True
    cbf = TrainingContext(opt("torch.bfloat16", fp8_enabled=False)).setup_training_context(torch.device("cpu"))
    assert not cbf["scaler"].is_enabled()


def test_create_recipe_returns_none_without_backend():
    from optimus_dl_amd.modules.amp import FP8Recipe, create_fp8_recipe, is_transformer_engine_available

    if is_transformer_engine_available():
        pytest.skip("a GPU backend is present here")
    assert create_fp8_recipe("delayed", "hybrid") is None
    with pytest.raises(ImportError):
        FP8Recipe()


def test_autocast_helpers_without_recipe_are_plain_amp():
    lin = nn.Linear(8, 8)
    x = torch.randn(4, 8)
    with fp8_autocast(torch.device("cpu"), None, dtype=torch.bfloat16):
        assert lin(x).dtype == torch.bfloat16
    with fp8_autocast(torch.device("cpu"), None, enabled=False):
        assert lin(x).dtype == torch.float32
    with fp8_backward(None):
        lin(x).sum().backward()
    assert lin.weight.grad is not None


def test_forward_backward_helpers_accept_instance_or_factory():
    lin = nn.Linear(8, 8)
    batch = torch.randn(4, 8)
    crit = lambda model, b: model(b).float().pow(2).mean()
    calls = []

    def factory():
        calls.append(1)
        return nullcontext()

    loss = execute_forward_pass(lin, batch, crit, factory)
    execute_backward_pass(loss, None, factory)
    loss = execute_forward_pass(lin, batch, crit, nullcontext())
    execute_backward_pass(loss, None, nullcontext())
    assert len(calls) == 2 and lin.weight.grad is not None


def test_first_and_last_blocks_can_stay_out_of_fp8(monkeypatch):
    """first_last_layers_bf16 / num_layers_at_{start,end}_in_bf16 (optimus_dl/modules/optim/config.py:62-66): the block
    list is found by structure, the Linears of the chosen blocks are marked and nothing else is touched."""
    from optimus_dl_amd.modules.fp8_linear import keep_layers_in_bf16

    monkeypatch.setattr(T, "_HAVE_TE", True)
    m = Llama(LlamaConfig(vocab_size=256, n_layer=5, n_head=4, n_kv_head=2, n_embd=64, intermediate_size=128))
    build_model_transform({"_name": "transformer_engine"}).apply(m)
    names = keep_layers_in_bf16(m, at_start=1, at_end=2)
    assert len(names) == 3 * 7 and "transformer.h.0.attn.wq" in names and "transformer.h.4.mlp.c_proj" in names
    off = {i for i in range(5) if not m.transformer.h[i].attn.wq.fp8_enabled}
    assert off == {0, 3, 4}
    for i in range(5):
        flags = {mod.fp8_enabled for mod in m.transformer.h[i].modules() if isinstance(mod, FP8Linear)}
        assert flags == {i not in off}
    assert m.lm_head.fp8_enabled                                          # the head is not a block
    assert keep_layers_in_bf16(nn.Sequential(nn.Linear(4, 4)), 1, 1) == []  # no block list: nothing to do
    # more layers asked for than there are: all of them, each once
    m2 = GPT2(GPT2Config(vocab_size=256, n_layer=2, n_head=4, n_embd=64, block_size=32))
    build_model_transform({"_name": "transformer_engine"}).apply(m2)
    assert len(keep_layers_in_bf16(m2, at_start=3, at_end=3)) == 2 * 6
    # the training context reads the keys; without an FP8 recipe (this machine has no GPU) it does nothing
    ctx = TrainingContext(opt("torch.bfloat16", fp8_enabled=False, first_last_layers_bf16=True))
    ctx.setup_training_context(torch.device("cpu"))
    assert ctx.apply_fp8_layer_policy(m) == []
    # a Linear that is switched off is a plain Linear even inside an FP8 context
    out = m(torch.randint(0, 256, (2, 16)))["logits"]
    assert out.shape == (2, 16, 256)


# ------------------------------------------------- fused producers: transform and hand-over (host side)
def _llama_tree():
    from optimus_dl_amd.modules.model import Llama, LlamaConfig

    torch.manual_seed(0)
    return Llama(LlamaConfig(vocab_size=64, n_layer=2, n_head=2, n_kv_head=1, n_embd=32, intermediate_size=64))


def test_transform_fuses_swiglu_and_rmsnorm_in_place(monkeypatch):
    from optimus_dl_amd.modules.model.blocks import RMSNorm, SwiGLUMLP

    monkeypatch.setattr(T, "_HAVE_TE", True)
    m = _llama_tree()
    keys = sorted(m.state_dict().keys())
    mlp, norm = m.transformer.h[0].mlp, m.transformer.h[0].ln_1
    ids = torch.randint(0, 64, (2, 8))
    before = m(ids)["logits"]
    t = build_model_transform({"_name": "transformer_engine"})
    assert t.apply(m) is m
    n_lin = sum(isinstance(x, FP8Linear) for x in m.modules())
    assert t.last_replacements == {"Linear": n_lin, "RMSNorm": 5, "LayerNorm": 0, "Attention": 0, "SwiGLU": 2}
    assert m.transformer.h[0].mlp is mlp and m.transformer.h[0].ln_1 is norm          # same objects
    assert isinstance(mlp, SwiGLUMLP) and isinstance(norm, RMSNorm)
    assert type(mlp).__name__ == "SwiGLUMLP" and type(norm).__module__ == RMSNorm.__module__
    assert getattr(mlp, "_odl_fused_swiglu", False) and getattr(norm, "_odl_fused_rmsnorm", False)
    assert sorted(m.state_dict().keys()) == keys
    torch.testing.assert_close(m(ids)["logits"], before)                              # no recipe active: own forwards
    again = build_model_transform({"_name": "transformer_engine"})
    again.apply(m)
    assert again.last_replacements == {"Linear": 0, "RMSNorm": 0, "LayerNorm": 0, "Attention": 0}


def test_transform_fusion_switches(monkeypatch):
    monkeypatch.setattr(T, "_HAVE_TE", True)
    m = _llama_tree()
    t = build_model_transform({"_name": "fp8_linear", "replace_norm": False, "fuse_swiglu": False})
    t.apply(m)
    assert t.last_replacements["RMSNorm"] == 0 and "SwiGLU" not in t.last_replacements
    assert not hasattr(m.transformer.h[0].mlp, "_odl_fused_swiglu") and not hasattr(m.transformer.ln_f, "_odl_fused_rmsnorm")
    m = _llama_tree()
    t = build_model_transform({"_name": "fp8_linear", "replace_linear": False})
    t.apply(m)
    assert "SwiGLU" not in t.last_replacements and t.last_replacements["RMSNorm"] == 5   # MLP projections are plain Linears
    m = _llama_tree()
    t = build_model_transform({"_name": "fp8_linear", "replace_inplace": False})
    t.apply(m)
    assert not hasattr(m.transformer.ln_f, "_odl_fused_rmsnorm") and not hasattr(m.transformer.h[0].mlp, "_odl_fused_swiglu")


def test_producer_parts_hand_over(monkeypatch):
    from optimus_dl_amd.modules import amp as A
    from optimus_dl_amd.modules.amp import fp8 as fp8_mod

    monkeypatch.setattr(fp8_mod, "is_native_backend_available", lambda: True)   # bookkeeping only, no kernel runs
    r = A.FP8Recipe(recipe_type="tensorwise")
    x = torch.zeros(4, 6)
    parts = torch.ones(3)
    r.offer_parts(x, parts)
    assert r.take_parts(torch.zeros(4, 6)) is None                    # another tensor
    assert r.take_parts(x.reshape(2, 12)) is parts                    # a view of all of it
    assert r.take_parts(x) is None                                    # handed over once
    r.offer_parts(x, parts)
    x.add_(1)                                                         # changed in place since
    assert r.take_parts(x) is None
    for i in range(12):
        r.offer_parts(torch.zeros(1), parts)
    assert len(r.producer_parts) == 8
    with r.autocast():
        pass
    assert r.producer_parts == []
    d = A.FP8Recipe(recipe_type="delayed")
    d.offer_parts(x, parts)
    assert d.producer_parts == []                                     # only current scaling reads an amax per tensor


def test_converted_and_fused_modules_survive_deepcopy_and_pickling():
    """An EMA copy (copy.deepcopy) and torch.save of a whole module: the FP8 Linears and the modules re-classed in
    place for the fused forwards come back as the same types with the same state-dict keys and the same outputs."""
    import copy
    import io

    from optimus_dl_amd.modules.fp8_linear import FP8Linear
    from optimus_dl_amd.modules.model.blocks import GPT2Block, LlamaBlock
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    for blk in (LlamaBlock(64, 4, 2, 128), GPT2Block(64, 4)):
        build_model_transform({"_name": "transformer_engine"}).apply(blk)
        x = torch.randn(2, 8, 64)
        want = blk(x)
        buf = io.BytesIO()
        torch.save(blk, buf)
        buf.seek(0)
        for other in (copy.deepcopy(blk), torch.load(buf, weights_only=False)):
            assert type(other.ln_1) is type(blk.ln_1) and type(other.mlp) is type(blk.mlp)
            assert all(isinstance(m, FP8Linear) for m in other.modules() if isinstance(m, torch.nn.Linear))
            assert list(other.state_dict().keys()) == list(blk.state_dict().keys())
            assert torch.equal(other(x), want)
            again = build_model_transform({"_name": "transformer_engine"})
            again.apply(other)                                  # already converted: nothing left to do
            assert not any(again.last_replacements.values())


# ---------------------------------------------------------------- evaluation forward context
def test_forward_context_fallbacks_follow_the_reference_evaluator(monkeypatch):
    """optimus_dl/recipe/train/mixins/managers/evaluation_manager.py:98-144: nothing when AMP is off; plain
    autocast in the AMP dtype; bf16 autocast standing in for an FP8 dtype when ``fp8.enabled`` is off or the
    backend is missing; an FP8 recipe only with dtype + flag + backend together."""
    import optimus_dl_amd.recipe.training_context as tc

    cpu = torch.device("cpu")
    lin, x = nn.Linear(8, 8), torch.randn(4, 8)
    with tc.forward_context(opt("torch.bfloat16", enabled=False).amp, cpu):
        assert not torch.is_autocast_enabled("cpu") and lin(x).dtype == torch.float32
    with tc.forward_context(opt("torch.bfloat16", fp8_enabled=False).amp, cpu):
        assert torch.is_autocast_enabled("cpu") and lin(x).dtype == torch.bfloat16
    with tc.forward_context(opt("torch.float16", fp8_enabled=False).amp, cpu):
        assert torch.get_autocast_dtype("cpu") == torch.float16
    with tc.forward_context(opt("torch.float8_e4m3fn", fp8_enabled=False).amp, cpu):          # FP8 dtype, flag off
        assert torch.get_autocast_dtype("cpu") == torch.bfloat16 and lin(x).dtype == torch.bfloat16
    monkeypatch.setattr(tc, "is_transformer_engine_available", lambda: False)                    # FP8 asked for, no backend
    made = []
    monkeypatch.setattr(tc, "create_fp8_recipe", lambda **kw: made.append(kw))
    with tc.forward_context(opt("torch.float8_e4m3fn").amp, cpu):
        assert torch.get_autocast_dtype("cpu") == torch.bfloat16
    assert made == []
    # dtype + flag + backend: a recipe is built from the config's keys, once per distinct configuration
    monkeypatch.setattr(tc, "is_transformer_engine_available", lambda: True)
    monkeypatch.setattr(tc, "_eval_recipes", {})

    class Rec:
        def __init__(self, **kw):
            self.kw, self.entered = kw, 0

        def autocast(self):
            self.entered += 1
            return nullcontext()

    monkeypatch.setattr(tc, "create_fp8_recipe", lambda **kw: made.append(Rec(**kw)) or made[-1])
    cfg = opt("torch.float8_e4m3fn", recipe="tensorwise", format="e4m3", margin=1, amax_history_len=8).amp
    for _ in range(3):
        with tc.forward_context(cfg, FakeCuda()):
            pass
    assert len(made) == 1 and made[0].entered == 3
    assert made[0].kw == dict(recipe_type="tensorwise", format="e4m3", margin=1, amax_history_len=8, amax_compute_algo="max",
                              reduce_amax=True, fp8_dpa=False, fp8_mha=False)
    with tc.forward_context(opt("torch.float8_e4m3fn", recipe="delayed").amp, FakeCuda()):
        pass
    assert len(made) == 2                                          # another configuration, another recipe
    with tc.forward_context(cfg, cpu):                             # a recipe off the GPU: ordinary bf16 autocast (fp8.py:488)
        assert torch.get_autocast_dtype("cpu") == torch.bfloat16
