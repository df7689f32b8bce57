"""GPU parity of the whole FP8 Linear (module + autograd + recipes) vs the oracle.

GEMM outputs: max|out-ref|/max|ref| <= 1e-2 (bf16 out).  Scales and histories:
bit-exact.  The module is driven exactly as a training loop drives it: through
the FP8Recipe contexts.
"""
import pytest
import torch
import torch.nn as nn

from oracle import oracle as O
from tests.helpers import assert_f32_bits_equal, max_rel_err, seeded_bf16

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def amp():
    from optimus_dl_amd.modules import amp as A

    return A


def make_linear(w: torch.Tensor, bias: torch.Tensor | None = None, dtype=torch.bfloat16):
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    lin = nn.Linear(w.shape[1], w.shape[0], bias=bias is not None)
    with torch.no_grad():
        lin.weight.copy_(w.float())
        if bias is not None:
            lin.bias.copy_(bias.float())
    lin = lin.to("cuda", dtype)
    return FP8Linear.from_linear(lin)


def run_step(lin, recipe, x, dy):
    xd = x.cuda().requires_grad_(True)
    lin.weight.grad = None
    with recipe.autocast():
        y = lin(xd)
    with recipe.backward():
        y.backward(dy.cuda())
    return y.detach(), xd.grad.detach(), lin.weight.grad.detach()


@pytest.mark.parametrize("fmt", ["hybrid", "e4m3"])
def test_tensorwise_matches_oracle(amp, fmt):
    M, K, N = 512, 1024, 768
    x, w, dy = seeded_bf16((M, K), 1.0, 0), seeded_bf16((N, K), 0.02, 1), seeded_bf16((M, N), 1e-3, 2)
    recipe = amp.create_fp8_recipe("tensorwise", fmt)
    lin = make_linear(w)
    y, dx, dw = run_step(lin, recipe, x, dy)
    fb = O.E5M2 if fmt == "hybrid" else O.E4M3
    ref = O.linear_fwd_bwd(x, w, dy, O.E4M3, fb)
    assert y.dtype == torch.bfloat16 and dx.dtype == torch.bfloat16 and dw.dtype == torch.bfloat16
    for name, got in (("y", y), ("dx", dx), ("dw", dw)):
        err = max_rel_err(got, ref[name])
        assert err <= TOL, f"{name}: {err}"
    assert lin.fp8_calls == 1


def test_three_dimensional_input_bias_and_fp32_master_weights(amp):
    B, S, K, N = 4, 64, 256, 512
    x = seeded_bf16((B * S, K), 1.0, 3)
    w32 = torch.randn(N, K, generator=torch.Generator().manual_seed(4)) * 0.02
    bias = torch.randn(N, generator=torch.Generator().manual_seed(5)) * 0.1
    dy = seeded_bf16((B * S, N), 1e-2, 6)
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    lin = make_linear(w32, bias, dtype=torch.float32)
    xd = x.cuda().reshape(B, S, K).requires_grad_(True)
    with amp.fp8_autocast(torch.device("cuda"), recipe, dtype=torch.bfloat16):
        y = lin(xd)
    assert y.shape == (B, S, N) and y.dtype == torch.bfloat16
    with amp.fp8_backward(recipe):
        y.backward(dy.cuda().reshape(B, S, N))
    # oracle: the weight is quantised from its fp32 values
    sx, sw, sg = O.t_scale(O.t_amax(x), O.E4M3), O.t_scale(w32.abs().amax().reshape(1), O.E4M3), O.t_scale(O.t_amax(dy), O.E5M2)
    xq, wq, gq = O.t_cast(x, sx, O.E4M3), O.t_cast(w32, sw, O.E4M3), O.t_cast(dy, sg, O.E5M2)
    y_ref = (O.t_gemm_nt(xq, wq, O.E4M3, O.E4M3, 1 / sx, 1 / sw, want_f32=True)[1] + bias).bfloat16()
    dx_ref = O.t_gemm_nt(gq, wq.t().contiguous(), O.E5M2, O.E4M3, 1 / sg, 1 / sw)
    dw_ref = O.t_gemm_nt(gq.t().contiguous(), xq.t().contiguous(), O.E5M2, O.E4M3, 1 / sg, 1 / sx, want_f32=True)[1]
    assert max_rel_err(y.reshape(-1, N), y_ref) <= TOL
    assert max_rel_err(xd.grad.reshape(-1, K), dx_ref) <= TOL
    assert lin.weight.grad.dtype == torch.float32 and max_rel_err(lin.weight.grad, dw_ref) <= TOL
    torch.testing.assert_close(lin.bias.grad.cpu(), dy.float().sum(0), rtol=1e-5, atol=1e-6)


def test_rowwise_with_outlier_channels_matches_oracle(amp):
    M, K, N = 1024, 512, 768
    x = seeded_bf16((M, K), 1.0, 0)
    g = torch.Generator().manual_seed(0)
    idx = torch.randperm(K, generator=g)[:2]
    x[:, idx] = (x[:, idx].float() * 100).bfloat16()
    w, dy = seeded_bf16((N, K), 0.02, 1), seeded_bf16((M, N), 1e-3, 2)
    recipe = amp.create_fp8_recipe("rowwise", "hybrid")
    lin = make_linear(w)
    y, dx, dw = run_step(lin, recipe, x, dy)
    ref = O.linear_fwd_bwd(x, w, dy, rowwise=True)
    for name, got in (("y", y), ("dx", dx), ("dw", dw)):
        err = max_rel_err(got, ref[name])
        assert err <= TOL, f"{name}: {err}"
    # row isolation: scaling one row of X by 2^3 scales that row of Y by 2^3 exactly and nothing else
    x2 = x.clone()
    x2[5] = (x2[5].float() * 8).bfloat16()
    y2, _, _ = run_step(lin, recipe, x2, dy)
    assert torch.equal(y2[5].float(), y[5].float() * 8) and torch.equal(y2[6], y[6])


def test_delayed_scaling_twenty_steps_with_drift(amp):
    """Benchmark configuration 5 in miniature: history 16, 20 steps, input std 1.0 -> 1.5."""
    M, K, N, H, STEPS = 256, 512, 384, 16, 20
    w = seeded_bf16((N, K), 0.01, 100)
    recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    lin = make_linear(w)
    fwd = O.DelayedState([O.E4M3] * 3, H)
    bwd = O.DelayedState([O.E5M2] * 2, H)
    for step in range(STEPS):
        std = 1.0 + 0.5 * step / (STEPS - 1)
        x, dy = seeded_bf16((M, K), std, step), seeded_bf16((M, N), 1e-3 * std, 1000 + step)
        stale = (fwd.scale[0], fwd.scale[1], bwd.scale[0])
        y, dx, dw = run_step(lin, recipe, x, dy)
        ref = O.linear_fwd_bwd(x, w, dy, scales=stale)
        for name, got in (("y", y), ("dx", dx), ("dw", dw)):
            err = max_rel_err(got, ref[name])
            # the first step runs with scale 1: gradients of 1e-3 sit in e5m2 subnormals, as they do in the oracle
            assert err <= TOL, f"step {step} {name}: {err}"
        fwd.record(0, O.t_amax(x).item()); fwd.record(1, O.t_amax(w).item()); fwd.update()
        bwd.record(0, O.t_amax(dy).item()); bwd.update()
        mf, mb = lin.fp8_meta["scaling_fwd"], lin.fp8_meta["scaling_bwd"]
        assert mf.amax_history.shape == (H, 3) and mb.amax_history.shape == (H, 2)
        assert_f32_bits_equal(mf.amax_history, torch.from_numpy(fwd.history), f"fwd history step {step}")
        assert_f32_bits_equal(mb.amax_history, torch.from_numpy(bwd.history), f"bwd history step {step}")
        assert_f32_bits_equal(mf.scale, torch.from_numpy(fwd.scale), f"fwd scale step {step}")
        assert_f32_bits_equal(mb.scale, torch.from_numpy(bwd.scale), f"bwd scale step {step}")
        assert_f32_bits_equal(mf.scale_inv, torch.from_numpy(fwd.scale_inv), f"fwd scale_inv step {step}")
    # the window has evicted the first steps: the scale depends on the last 16 amaxes only
    assert (lin.fp8_meta["scaling_fwd"].amax_history > 0).any()


def test_history_has_a_value_after_one_step_like_the_reference_test(amp):
    """tests/optim/test_fp8.py:567-625 of the reference: TELinear(32, 64), x [16, 32],
    2-D amax histories with some element > 0 after one forward+backward."""
    from optimus_dl_amd.modules.model_transforms.transformer_engine import TELinear

    recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=16)
    lin = TELinear(32, 64).to("cuda", torch.bfloat16)
    x = torch.randn(16, 32, device="cuda", dtype=torch.bfloat16, requires_grad=True)
    # during the step the casts' maxima wait with the roles; leaving the context folds them into the history and rolls it
    with recipe.autocast():
        y = lin(x)
        meta = lin._te_linear.fp8_meta["scaling_fwd"]
        assert meta.pending_amax.shape == (3,) and (meta.pending_amax > 0).sum() == 2      # input and weight; the output role is unused
        assert not (meta.amax_history > 0).any()
    hist = lin._te_linear.fp8_meta["scaling_fwd"].amax_history
    assert hist.dim() == 2 and hist.shape == (16, 3) and (hist > 0).any() and not meta.pending_amax.any()
    with recipe.backward():
        y.sum().backward()
    hb = lin.fp8_meta["scaling_bwd"].amax_history
    assert hb.shape == (16, 2) and (hb > 0).any()
    assert (lin.fp8_meta["scaling_fwd"].amax_history > 0).any() and x.grad is not None and lin.weight.grad is not None


def test_nested_contexts_and_plain_linear_outside(amp):
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    w = seeded_bf16((64, 64), 0.02, 1)
    lin = make_linear(w)
    x = seeded_bf16((32, 64), 1.0, 2).cuda()
    y_plain = lin(x)
    assert lin.fp8_calls == 0
    with amp.fp8_autocast(torch.device("cuda"), recipe):
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            y1 = lin(x)
        y2 = lin(x)
    assert lin.fp8_calls == 2 and torch.equal(y1, y2)
    assert max_rel_err(y1, y_plain) < 0.1 and not torch.equal(y1, y_plain)
    assert torch.equal(lin(x), y_plain)
    with amp.fp8_autocast(torch.device("cuda"), recipe, enabled=False):
        assert torch.equal(lin(x), y_plain)


def test_weight_cache_requantises_only_when_the_parameter_changes(amp):
    from optimus_dl_amd import native

    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    lin = make_linear(seeded_bf16((128, 256), 0.02, 1))
    x = seeded_bf16((64, 256), 1.0, 2).cuda().requires_grad_(True)
    with recipe.autocast():
        lin(x)
        wq_first = lin._wcache.wq
        lin(x)                                          # a second microbatch
        assert lin._wcache.wq is wq_first
        with torch.no_grad():
            lin.weight.mul_(1.5)                        # what an optimizer step does
        lin(x)
        assert lin._wcache.wq is not wq_first
    want = O.t_cast(lin.weight.detach().cpu(), O.t_scale(O.t_amax(lin.weight.detach().cpu()), O.E4M3), O.E4M3)
    assert torch.equal(lin._wcache.wq.cpu(), want)
    del native


def test_unsupported_shapes_run_as_plain_linear(amp):
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    lin = make_linear(seeded_bf16((40, 24), 0.02, 1))      # 24, 40 are not multiples of 16
    x = seeded_bf16((16, 24), 1.0, 2).cuda()
    with recipe.autocast():
        y = lin(x)
    assert lin.fp8_calls == 0 and y.shape == (16, 40)
    lin2 = make_linear(seeded_bf16((64, 64), 0.02, 1))
    with recipe.autocast():
        lin2(seeded_bf16((7, 64), 1.0, 3).cuda())           # 7 tokens
    assert lin2.fp8_calls == 0


def test_e5m2_delayed_is_refused_and_every_recipe_type_constructs(amp):
    with pytest.raises(ValueError, match="Pure E5M2 format is not supported"):
        amp.FP8Recipe("delayed", "e5m2")
    r = amp.FP8Recipe("tensorwise", "e5m2")
    assert r.format == amp.Fp8Format.E5M2 and r.recipe.fmt_fwd == O.E5M2
    assert amp.FP8Recipe("mxfp8", "hybrid").recipe.kind == "mxfp8"
    assert amp.FP8Recipe("blockwise", "hybrid").recipe.kind == "blockwise"
    rec = amp.create_fp8_recipe("delayed", "hybrid", margin=2, amax_history_len=32, amax_compute_algo="most_recent", reduce_amax=False)
    assert (rec.margin, rec.amax_history_len, rec.amax_compute_algo, rec.reduce_amax, rec.fp8_dpa, rec.fp8_mha) == (2, 32, "most_recent", False, False, False)
    assert rec.recipe_type == amp.Fp8RecipeType.DELAYED and rec.format == amp.Fp8Format.HYBRID and rec.recipe is not None


def test_first_and_last_blocks_stay_in_bf16_when_the_config_says_so(amp):
    """amp.fp8.first_last_layers_bf16 with one layer at each end (optimus_dl/modules/optim/config.py:62-66): the Linears
    of blocks 0 and 3 of a 4-block model never take the FP8 path, those of blocks 1 and 2 and the head do, and a
    training step still runs through the reference-shaped glue."""
    from optimus_dl_amd.modules.fp8_linear import FP8Linear
    from optimus_dl_amd.modules.model import Llama, LlamaConfig
    from optimus_dl_amd.modules.model_transforms import build_model_transform
    from optimus_dl_amd.modules.optim.config import AmpConfig, Fp8Config, OptimizationConfig
    from optimus_dl_amd.recipe import TrainingContext, execute_backward_pass, execute_forward_pass

    torch.manual_seed(0)
    model = Llama(LlamaConfig(vocab_size=512, n_layer=4, n_head=4, n_kv_head=2, n_embd=128, intermediate_size=256)).cuda()
    model = build_model_transform({"_name": "transformer_engine"}).apply(model, device=torch.device("cuda"))
    cfg = OptimizationConfig(amp=AmpConfig(enabled=True, dtype="torch.float8_e4m3fn", fp8=Fp8Config(
        enabled=True, recipe="tensorwise", first_last_layers_bf16=True, num_layers_at_start_in_bf16=1, num_layers_at_end_in_bf16=1)))
    tc = TrainingContext(cfg)
    ctx = tc.setup_training_context(torch.device("cuda"))
    names = tc.apply_fp8_layer_policy(model)
    assert len(names) == 2 * 7 and all(n.startswith(("transformer.h.0.", "transformer.h.3.")) for n in names)

    def crit(m, batch):
        logits = m(batch["input_ids"])["logits"].float()
        return torch.nn.functional.cross_entropy(logits.view(-1, logits.shape[-1]), batch["labels"].view(-1))

    ids = torch.randint(0, 512, (8, 33), generator=torch.Generator().manual_seed(1))
    batch = {"input_ids": ids[:, :-1].cuda(), "labels": ids[:, 1:].cuda()}
    loss = execute_forward_pass(model, batch, crit, ctx["amp_ctx"])
    execute_backward_pass(loss, ctx["scaler"], ctx["fp8_backward_ctx"])
    assert torch.isfinite(loss)
    for i, blk in enumerate(model.transformer.h):
        calls = [m.fp8_calls for m in blk.modules() if isinstance(m, FP8Linear)]
        assert all(c == 0 for c in calls) if i in (0, 3) else all(c == 1 for c in calls), (i, calls)
        assert all(m.weight.grad is not None for m in blk.modules() if isinstance(m, FP8Linear))
    assert model.lm_head.fp8_calls == 1


def test_wgrad_false_keeps_weight_gradient_in_bf16(amp):
    M, K, N = 128, 256, 128
    x, w, dy = seeded_bf16((M, K), 1.0, 0), seeded_bf16((N, K), 0.02, 1), seeded_bf16((M, N), 1e-3, 2)
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid", wgrad=False)
    lin = make_linear(w)
    _, _, dw = run_step(lin, recipe, x, dy)
    want = (dy.float().t() @ x.float()).bfloat16()
    assert max_rel_err(dw, want) <= 1e-2


@pytest.mark.parametrize("family,recipe_name", [("llama", "delayed"), ("qwen3", "delayed"), ("gpt2", "delayed"),
                                                ("llama", "mxfp8"), ("gpt2", "mxfp8"), ("qwen3", "tensorwise"), ("llama", "blockwise")])
def test_training_loop_through_the_reference_shaped_glue(amp, family, recipe_name):
    """Transform -> training context -> a few optimizer steps, FP8 vs bf16 on the same init."""
    from optimus_dl_amd.modules.model import GPT2, GPT2Config, Llama, LlamaConfig, Qwen3, Qwen3Config
    from optimus_dl_amd.modules.model_transforms import build_model_transform
    from optimus_dl_amd.modules.optim.config import AmpConfig, Fp8Config, OptimizationConfig
    from optimus_dl_amd.recipe import TrainingContext, execute_backward_pass, execute_forward_pass

    def build():
        torch.manual_seed(0)
        if family == "llama":
            return Llama(LlamaConfig(vocab_size=512, n_layer=2, n_head=4, n_kv_head=2, n_embd=128, intermediate_size=256))
        if family == "qwen3":
            return Qwen3(Qwen3Config(vocab_size=512, n_layer=2, n_head=4, n_kv_head=2, n_embd=128, head_dim=32, intermediate_size=256))
        return GPT2(GPT2Config(vocab_size=512, n_layer=2, n_head=4, n_embd=128, block_size=64))

    def crit(model, batch):
        logits = model(batch["input_ids"])["logits"].float()
        return torch.nn.functional.cross_entropy(logits.view(-1, logits.shape[-1]), batch["labels"].view(-1))

    g = torch.Generator().manual_seed(1)
    ids = torch.randint(0, 512, (8, 33), generator=g)
    batch = {"input_ids": ids[:, :-1].cuda(), "labels": ids[:, 1:].cuda()}
    losses = {}
    for mode in ("bf16", "fp8"):
        model = build().cuda()
        if mode == "fp8":
            t = build_model_transform({"_name": "transformer_engine"})
            model = t.apply(model, device=torch.device("cuda"), collective=None, is_restart=False, checkpoint_manager=None)
            cfg = OptimizationConfig(amp=AmpConfig(enabled=True, dtype="torch.float8_e4m3fn", fp8=Fp8Config(enabled=True, recipe=recipe_name, amax_history_len=4)))
        else:
            cfg = OptimizationConfig(amp=AmpConfig(enabled=True, dtype="torch.bfloat16"))
        ctx = TrainingContext(cfg).setup_training_context(torch.device("cuda"))
        assert ctx["fp8_enabled"] == (mode == "fp8")
        optim = torch.optim.AdamW(model.parameters(), lr=3e-3)
        trace = []
        for _ in range(8):
            optim.zero_grad(set_to_none=True)
            loss = execute_forward_pass(model, batch, crit, ctx["amp_ctx"])
            execute_backward_pass(loss, ctx["scaler"], ctx["fp8_backward_ctx"])
            optim.step()
            trace.append(loss.item())
        losses[mode] = trace
        if mode == "fp8":
            n_fp8 = sum(m.fp8_calls for m in model.modules() if hasattr(m, "fp8_calls"))
            assert n_fp8 > 0, "no Linear took the FP8 path"
    assert losses["fp8"][-1] < losses["fp8"][0] - 0.5, losses
    assert abs(losses["fp8"][-1] - losses["bf16"][-1]) < 0.25, losses


def _count_calls(monkeypatch, native, name):
    calls = []
    orig = getattr(native, name)

    def counted(*a, **kw):
        calls.append(a[0].shape)
        return orig(*a, **kw)

    monkeypatch.setattr(native, name, counted)
    return calls


@pytest.mark.parametrize("in_dtype", [torch.bfloat16, torch.float32])
def test_linears_fed_by_the_same_tensor_quantise_it_once(amp, monkeypatch, in_dtype):
    """gate/up of an MLP (q/k/v of an attention block): same input tensor, one amax and one cast of it.
    Results are bit-identical to quantising it per Linear."""
    from optimus_dl_amd import native

    M, K, N = 256, 512, 384
    x = seeded_bf16((M, K), 1.0, 40)
    wg, wu = seeded_bf16((N, K), 0.02, 41), seeded_bf16((N, K), 0.02, 42)
    dy = seeded_bf16((M, N), 1e-3, 43).cuda()

    def run(share):
        recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
        recipe.share_inputs = share
        gate, up = make_linear(wg), make_linear(wu)
        xd = x.to(in_dtype).cuda().requires_grad_(True)
        with amp.fp8_autocast(torch.device("cuda"), recipe, dtype=torch.bfloat16):
            h = gate(xd) * up(xd)
        with recipe.backward():
            h.backward(dy)
        assert recipe.shared_input is None                      # dropped when the context was left
        return h.detach(), xd.grad.detach(), gate.weight.grad.detach(), up.weight.grad.detach()

    calls = _count_calls(monkeypatch, native, "amax_parts")
    shared = run(True)
    n_shared = len([s for s in calls if tuple(s) == (M, K)])
    calls.clear()
    separate = run(False)
    n_separate = len([s for s in calls if tuple(s) == (M, K)])
    assert (n_shared, n_separate) == (1, 2)
    for i, (a, b) in enumerate(zip(shared, separate)):
        if i == 1 and in_dtype == torch.float32:
            # the two input gradients meet in bf16 (behind the shared conversion) instead of in fp32
            assert max_rel_err(a, b) <= 1e-2
        else:
            assert torch.equal(a, b)


def test_rowwise_linears_fed_by_the_same_tensor_quantise_it_once(amp, monkeypatch):
    """The rowwise recipe quantises an input in two passes (row scales for the forward, column scales and the transposed
    codes for wgrad): Linears fed the very same tensor share them; same bits as quantising per Linear; Linears with frozen
    weights (no wgrad) take the row pass only and share that."""
    from optimus_dl_amd import native

    M, K, N = 256, 512, 384
    x = seeded_bf16((M, K), 1.0, 44)
    wg, wu = seeded_bf16((N, K), 0.02, 45), seeded_bf16((N, K), 0.02, 46)
    dy = seeded_bf16((M, N), 1e-3, 47).cuda()

    def count_of(fn):
        calls = []
        orig = getattr(native, fn)
        monkeypatch.setattr(native, fn, lambda *a, **k: (calls.append(tuple(a[0].shape)), orig(*a, **k))[1])
        return calls

    def run(share):
        recipe = amp.create_fp8_recipe("rowwise", "hybrid")
        recipe.share_inputs = share
        gate, up = make_linear(wg), make_linear(wu)
        xd = x.cuda().requires_grad_(True)
        with recipe.autocast():
            h = gate(xd) * up(xd)
        with recipe.backward():
            h.backward(dy)
        assert recipe.shared_input is None
        gate.weight.requires_grad_(False)
        up.weight.requires_grad_(False)
        with recipe.autocast():
            e = gate(xd) + up(xd)
        return h.detach(), xd.grad.detach(), gate.weight.grad.detach(), up.weight.grad.detach(), e.detach()

    both, rows_only = count_of("quantize_rowcol"), count_of("amax")
    shared = run(True)
    n_shared = (len([c for c in both if c == (M, K)]), len([c for c in rows_only if c == (M, K)]))
    both.clear(); rows_only.clear()
    separate = run(False)
    n_separate = (len([c for c in both if c == (M, K)]), len([c for c in rows_only if c == (M, K)]))
    assert n_shared == (1, 1) and n_separate == (2, 2), (n_shared, n_separate)
    for a, b in zip(shared, separate):
        assert torch.equal(a, b)


def test_shared_input_is_not_reused_after_an_in_place_change_or_for_another_tensor(amp, monkeypatch):
    from optimus_dl_amd import native

    M, K, N = 128, 256, 128
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    lin = make_linear(seeded_bf16((N, K), 0.02, 50))
    x = seeded_bf16((M, K), 1.0, 51).cuda()
    calls = _count_calls(monkeypatch, native, "amax_parts")
    with torch.no_grad(), recipe.autocast():
        y1 = lin(x)
        y1_again = lin(x)                                       # hit
        n_after_hit = len(calls)
        x.mul_(2.0)                                             # same address, new contents
        y2 = lin(x)
        other = x.clone()
        y3 = lin(other)
    assert n_after_hit == 2                                     # weight + x, once each
    assert len(calls) == 4                                      # + x after the change + the clone
    assert torch.equal(y1, y1_again) and torch.equal(y2, y3)
    assert not torch.equal(y1, y2)


@pytest.mark.parametrize("recipe_name", ["tensorwise", "mxfp8"])
def test_forward_backward_can_be_captured_in_a_graph_and_replayed(amp, recipe_name):
    """Small Linears are launch-bound; callers capture them.  Every native call takes the capture
    stream and allocates nothing itself, so a captured forward+backward must replay correctly:
    three replays on new data, eager work and synchronisations in between, each against eager."""
    M, K, N = 256, 512, 384
    recipe = amp.create_fp8_recipe(recipe_name, "hybrid")
    lin = make_linear(seeded_bf16((N, K), 0.02, 90))
    x_static = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda", requires_grad=True)
    dy_static = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")

    def fwd_bwd():
        lin._wcache.key = None
        lin._wcache_rowwise.clear()
        with recipe.autocast():
            y = lin(x_static)
        with recipe.backward():
            gx, gw = torch.autograd.grad(y, (x_static, lin.weight), dy_static)
        return y, gx, gw

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up off the default stream, as capture requires
        for _ in range(2):
            fwd_bwd()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g, gx_g, gw_g = fwd_bwd()
    for rep in range(3):
        x_new, dy_new = seeded_bf16((M, K), 1.0 + rep, 91 + rep).cuda(), seeded_bf16((M, N), 1e-3 * (rep + 1), 95 + rep).cuda()
        with torch.no_grad():
            x_static.copy_(x_new)
            dy_static.copy_(dy_new)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in (y_g, gx_g, gw_g)]
        want = fwd_bwd()                                # eager, same buffers
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "dx", "dw"), got, want):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from eager"


def test_delayed_scaling_step_replays_from_a_graph_like_the_eager_twin(amp):
    """Delayed scaling keeps state between steps (histories, scales): they are refreshed in place, so a captured step
    carries them forward from replay to replay.  A twin layer runs the same steps eagerly; every replay must give the
    twin's bits, and the scaling state must be the same afterwards."""
    M, K, N = 256, 512, 384
    w = seeded_bf16((N, K), 0.02, 190)
    setups = []
    for _ in range(2):
        recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=4)
        lin = make_linear(w)
        x_s = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda", requires_grad=True)
        dy_s = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
        setups.append((recipe, lin, x_s, dy_s))

    def fwd_bwd(recipe, lin, x_s, dy_s):
        lin._wcache.key = None
        with recipe.autocast():
            y = lin(x_s)
        with recipe.backward():
            gx, gw = torch.autograd.grad(y, (x_s, lin.weight), dy_s)
        return y, gx, gw

    def feed(step):
        x_new, dy_new = seeded_bf16((M, K), 1.0 + step, 191 + step).cuda(), seeded_bf16((M, N), 1e-3 * (step + 1), 195 + step).cuda()
        with torch.no_grad():
            for _, _, x_s, dy_s in setups:
                x_s.copy_(x_new)
                dy_s.copy_(dy_new)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # two real steps each, off the default stream
        for step in range(2):
            feed(step)
            for s_ in setups:
                fwd_bwd(*s_)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs_g = fwd_bwd(*setups[0])
    for step in range(2, 6):                            # more replays than the history is long
        feed(step)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs_g]
        want = fwd_bwd(*setups[1])
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "dx", "dw"), got, want):
            assert torch.equal(a, b), f"step {step}: {name} from the replay differs from the eager twin"
    for direction in ("scaling_fwd", "scaling_bwd"):
        ma, mb = setups[0][1].fp8_meta[direction], setups[1][1].fp8_meta[direction]
        assert torch.equal(ma.scale, mb.scale) and torch.equal(ma.amax_history, mb.amax_history)
        assert ma.scale[0] != 1.0                       # the scales did move (the reserved output roles keep 1.0)


@pytest.mark.parametrize("recipe_name,fmt,margin", [("tensorwise", "e5m2", 0), ("tensorwise", "hybrid", 2), ("rowwise", "e4m3", 1)])
def test_other_formats_and_margins_match_the_oracle(amp, recipe_name, fmt, margin):
    """Pure E5M2 (allowed for current scaling), a margin (scales divided by 2^margin) and rowwise E4M3 gradients."""
    M, K, N = 256, 512, 384
    x, w, dy = seeded_bf16((M, K), 1.0, 130), seeded_bf16((N, K), 0.02, 131), seeded_bf16((M, N), 1e-3, 132)
    recipe = amp.create_fp8_recipe(recipe_name, fmt, margin=margin)
    lin = make_linear(w)
    y, dx, dw = run_step(lin, recipe, x, dy)
    ff = O.E5M2 if fmt == "e5m2" else O.E4M3
    fb = O.E4M3 if fmt == "e4m3" else O.E5M2
    if recipe_name == "rowwise":
        ref = O.linear_fwd_bwd(x, w, dy, ff, fb, rowwise=True) if margin == 0 else None
    else:
        scales = tuple(O.t_scale(O.t_amax(t), f, margin) for t, f in ((x, ff), (w, ff), (dy, fb)))
        ref = O.linear_fwd_bwd(x, w, dy, ff, fb, scales=scales)
    if ref is not None:
        for name, got in (("y", y), ("dx", dx), ("dw", dw)):
            err = max_rel_err(got, ref[name])
            assert err <= TOL, f"{name}: {err}"
    else:
        # a margin only moves every scale by a power of two: codes stay far from the clamp, results match margin 0 closely
        y0, dx0, dw0 = run_step(make_linear(w), amp.create_fp8_recipe(recipe_name, fmt), x, dy)
        for name, a, b in (("y", y, y0), ("dx", dx, dx0), ("dw", dw, dw0)):
            assert max_rel_err(a, b) <= 2e-2, name


def test_nan_and_inf_inputs_do_not_poison_the_scales(amp):
    """A NaN in the activation: its amax is NaN, the scale falls back to 1, the NaN element becomes the NaN code and
    reaches exactly one output row; an Inf saturates.  The other rows stay finite."""
    M, K, N = 128, 256, 128
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    lin = make_linear(seeded_bf16((N, K), 0.02, 140))
    x = seeded_bf16((M, K), 1.0, 141)
    x[7, 11] = float("nan")
    with torch.no_grad(), recipe.autocast():
        y = lin(x.cuda())
    assert torch.isnan(y[7]).all()
    keep = torch.ones(M, dtype=torch.bool); keep[7] = False
    assert torch.isfinite(y[keep.cuda()].float()).all()
    x[7, 11] = float("inf")
    with torch.no_grad(), recipe.autocast():
        y = lin(x.cuda())
    assert torch.isfinite(y.float()).all()              # amax = Inf -> scale 1, the Inf element clamps to 448


def test_cache_weights_switch_requantises_after_a_data_write(amp, monkeypatch):
    from optimus_dl_amd import native

    w = seeded_bf16((256, 512), 0.02, 1)
    lin = make_linear(w)
    x = seeded_bf16((256, 512), 1.0, 2).cuda()
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    with recipe.autocast():
        y0 = lin(x)
    lin.weight.data.mul_(2.0)                      # does not move weight._version
    with recipe.autocast():
        stale = lin(x)
    assert torch.equal(stale, y0)                  # the cached codes were used: the documented caveat
    recipe.cache_weights = False
    calls = _count_calls(monkeypatch, native, "amax_parts")
    with recipe.autocast():
        fresh = lin(x)
        again = lin(x)
    assert calls.count((256, 512)) >= 2            # the weight (and x, same shape here) quantised on every forward
    assert torch.equal(fresh, again) and max_rel_err(fresh, 2 * y0.float()) <= TOL


@pytest.mark.parametrize("wdtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("recipe_name", ["tensorwise", "delayed"])
def test_wgrad_reads_dy_as_stored_and_matches_the_transposed_copy_route(amp, monkeypatch, wdtype, recipe_name):
    """With whole 256 x 256 tiles the weight gradient is computed from the row-major codes of dy
    (no transposed copy), in the weight's own type (fp32 master weights get an fp32 gradient): the
    result equals the route over the transposed copy bit for bit."""
    from optimus_dl_amd import native

    M, K, N = 1024, 512, 768
    x, w, dy = seeded_bf16((M, K), 1.0, 50), seeded_bf16((N, K), 0.02, 51), seeded_bf16((M, N), 1e-3, 52)
    results = {}
    for direct in (True, False):
        recipe = amp.create_fp8_recipe(recipe_name, "hybrid", amax_history_len=4)
        recipe.direct_layouts = direct
        lin = make_linear(w, dtype=wdtype)
        run_step(lin, recipe, x, dy)               # delayed scaling: the second step runs on measured scales
        seen = []
        real = native.gemm_layouts
        monkeypatch.setattr(native, "gemm_layouts", lambda *a, **k: (seen.append(k.get("out_dtype")), real(*a, **k))[1])
        y, dx, dw = run_step(lin, recipe, x, dy)
        monkeypatch.setattr(native, "gemm_layouts", real)
        assert dw.dtype == wdtype and y.dtype == torch.bfloat16
        assert seen == ([wdtype] if direct else [])
        results[direct] = (y, dx, dw)
    for got, want in zip(results[True], results[False]):
        assert torch.equal(got, want)
    ref = O.linear_fwd_bwd(x, w, dy) if recipe_name == "tensorwise" else None
    if ref is not None:
        assert max_rel_err(results[True][2], ref["dw"]) <= TOL


def test_mid_sized_weight_gradients_take_the_transposed_copy(amp, monkeypatch):
    """A gradient whose 256 x 256 tiles neither fill the chip nor are few enough not to matter is computed from a
    transposed copy of dy (native.wgrad_direct_pays); the two routes give the same bits."""
    from optimus_dl_amd import native

    assert native.wgrad_direct_pays(14336, 4096, 8192) and native.wgrad_direct_pays(4096, 4096, 8192)
    assert native.wgrad_direct_pays(768, 768, 8192) and native.wgrad_direct_pays(2304, 768, 8192)
    assert not native.wgrad_direct_pays(1024, 4096, 8192) and not native.wgrad_direct_pays(2048, 4096, 8192)
    M, K, N = 512, 4096, 1024
    x, w, dy = seeded_bf16((M, K), 1.0, 60), seeded_bf16((N, K), 0.02, 61), seeded_bf16((M, N), 1e-3, 62)
    results = {}
    for force_direct in (False, True):
        if force_direct:
            monkeypatch.setattr(native, "wgrad_direct_pays", lambda *a: True)
        calls = _count_calls(monkeypatch, native, "gemm_layouts")
        recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
        results[force_direct] = run_step(make_linear(w), recipe, x, dy)
        assert (len(calls) == 1) == force_direct
    for got, want in zip(results[False], results[True]):
        assert torch.equal(got, want)


@pytest.mark.parametrize("seed", range(24))
def test_seeded_random_linears_match_the_oracle(amp, seed):
    """Layer sizes on the grids the kernels distinguish, tokens likewise, bf16 or fp32 master weights, with and
    without bias, per-tensor or rowwise scaling: forward, dgrad, wgrad and the bias gradient against the oracle."""
    g = torch.Generator().manual_seed(500 + seed)
    def draw(grids, hi):
        step = grids[int(torch.randint(0, len(grids), (1,), generator=g))]
        return step * int(torch.randint(1, hi // step + 1, (1,), generator=g))
    M, K, N = draw((16, 128, 256), 1024), draw((16, 128, 256), 1024), draw((16, 128, 256), 1024)
    if seed % 6 == 5:
        M = 128 * int(torch.randint(16, 40, (1,), generator=g))          # long token axis: wgrad is cut into K runs
    rowwise, with_bias, w_f32 = seed % 3 == 2, seed % 2 == 1, seed % 4 >= 2
    x, w, dy = seeded_bf16((M, K), 1.0, 600 + seed), seeded_bf16((N, K), 0.02, 700 + seed), seeded_bf16((M, N), 1e-3, 800 + seed)
    bias = seeded_bf16((N,), 0.1, 900 + seed) if with_bias else None
    recipe = amp.create_fp8_recipe("rowwise" if rowwise else "tensorwise", "hybrid")
    lin = make_linear(w, bias, dtype=torch.float32 if w_f32 else torch.bfloat16)
    y, dx, dw = run_step(lin, recipe, x, dy)
    assert lin.fp8_calls == 1 and y.dtype == torch.bfloat16 and dw.dtype == lin.weight.dtype
    ref = O.linear_fwd_bwd(x, w, dy, rowwise=rowwise)
    want_y = ref["y"] if bias is None else (ref["y"].float() + bias.float()).bfloat16()
    what = f"{M}x{K}->{N} rowwise={rowwise} bias={with_bias} fp32 weights={w_f32}"
    for name, got, want in (("y", y, want_y), ("dx", dx, ref["dx"]), ("dw", dw, ref["dw"])):
        err = max_rel_err(got, want)
        assert err <= TOL, f"{what}: {name} {err}"
    if with_bias:
        want_db = dy.float().sum(0)
        err = (lin.bias.grad.float().cpu() - want_db).abs().max().item() / max(want_db.abs().max().item(), 1e-30)
        assert err <= (1e-2 if lin.bias.dtype == torch.bfloat16 else 1e-5), f"{what}: db {err}"
