"""Where the delayed-scaling state lives and who sees it: evaluation forwards, checkpoints,
activation checkpointing.

The reference's backend keeps ``fp8_meta`` on every layer, so a recipe object built per evaluation
forward (optimus_dl/recipe/train/mixins/managers/evaluation_manager.py:98-144) continues with the
scales training measured, and the layer's state travels with the model.  These tests pin the same
behaviour here.
"""
import copy

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


def make_linear(w: torch.Tensor, dtype=torch.bfloat16):
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    lin = nn.Linear(w.shape[1], w.shape[0], bias=False)
    with torch.no_grad():
        lin.weight.copy_(w.float())
    return FP8Linear.from_linear(lin.to("cuda", dtype))


def train_step(lin, recipe, x, dy):
    xd = x.cuda().requires_grad_(True)
    lin.weight.grad = None
    with recipe.autocast():
        y = lin(xd)
    with recipe.backward():
        y.backward(dy.cuda())
    return y.detach(), xd.grad.detach(), lin.weight.grad.detach()


def fp8_cfg(recipe: str, **kw):
    from optimus_dl_amd.modules.optim.config import AmpConfig, Fp8Config

    return AmpConfig(enabled=True, dtype="torch.float8_e4m3fn", fp8=Fp8Config(enabled=True, recipe=recipe, **kw))


def arena_count():
    """Arenas alive in the process (they are what delayed scaling allocates)."""
    import gc

    from optimus_dl_amd.modules.amp import state

    gc.collect()
    return sum(1 for o in gc.get_objects() if isinstance(o, state.MetaArena))


def test_eval_forward_context_takes_the_fp8_path_with_the_training_bits(amp):
    """Tensorwise scaling keeps no state: the evaluation forward (its own recipe object, module in eval
    mode, no grad) must give exactly the bits of the training forward, and both must be the oracle's."""
    from optimus_dl_amd.recipe.training_context import forward_context

    M, K, N = 256, 512, 384
    x, w, dy = seeded_bf16((M, K), 1.0, 300), seeded_bf16((N, K), 0.02, 301), seeded_bf16((M, N), 1e-3, 302)
    lin = make_linear(w)
    y_train, _, _ = train_step(lin, amp.create_fp8_recipe("tensorwise", "hybrid"), x, dy)
    calls = lin.fp8_calls
    lin.eval()
    with torch.no_grad(), forward_context(fp8_cfg("tensorwise"), torch.device("cuda")):
        y_eval = lin(x.cuda())
    assert lin.fp8_calls == calls + 1, "the evaluation forward did not take the FP8 path"
    assert y_eval.dtype == torch.bfloat16 and torch.equal(y_eval, y_train)
    assert max_rel_err(y_eval, O.linear_fwd_bwd(x, w, dy)["y"]) <= TOL


def test_eval_forward_after_delayed_training_uses_the_trained_scales(amp):
    """Delayed scaling: an evaluation forward after N training steps quantises with the scales those
    steps measured (not with the initial 1), leaves histories and scales untouched, and reserves
    nothing: no new arena, no new roles, however often it is called."""
    from optimus_dl_amd.recipe.training_context import forward_context

    M, K, N, H = 256, 512, 384, 4
    w = seeded_bf16((N, K), 0.02, 310)
    lin = make_linear(w)
    recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    sim = O.DelayedState([O.E4M3] * 3, H)
    for step in range(3):
        x, dy = seeded_bf16((M, K), 1.0 + step, 311 + step), seeded_bf16((M, N), 1e-3, 320 + step)
        train_step(lin, recipe, x, dy)
        sim.record(0, O.t_amax(x).item()); sim.record(1, O.t_amax(w).item()); sim.update()
    meta = lin.fp8_meta["scaling_fwd"]
    assert_f32_bits_equal(meta.scale, torch.from_numpy(sim.scale), "trained forward scales")
    hist_before, scale_before = meta.amax_history.clone(), meta.scale.clone()
    arenas_before, used_before = arena_count(), meta.arena.used
    cfg = fp8_cfg("delayed", amax_history_len=H)
    x_eval = seeded_bf16((M, K), 2.0, 330)
    lin.eval()
    outs = []
    for _ in range(3):
        with torch.no_grad(), forward_context(cfg, torch.device("cuda")):
            outs.append(lin(x_eval.cuda()))
    assert arena_count() == arenas_before and meta.arena.used == used_before, "an evaluation forward reserved scaling state"
    assert lin.fp8_meta["scaling_fwd"] is meta, "the evaluation recipe did not find the module's state"
    assert torch.equal(meta.amax_history, hist_before) and torch.equal(meta.scale, scale_before)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    # what the trained scales give, from the oracle: x and w cast with them, GEMM, bf16
    sx, sw = float(sim.scale[0]), float(sim.scale[1])
    want = O.t_gemm_nt(O.t_cast(x_eval, sx, O.E4M3), O.t_cast(w, sw, O.E4M3), O.E4M3, O.E4M3,
                       torch.tensor(1.0 / sx), torch.tensor(1.0 / sw))
    assert max_rel_err(outs[0], want) <= TOL
    # with the initial scale 1 the weight (std 0.02) would sit in E4M3's subnormals: far off
    coarse = O.t_gemm_nt(O.t_cast(x_eval, 1.0, O.E4M3), O.t_cast(w, 1.0, O.E4M3), O.E4M3, O.E4M3, torch.tensor(1.0), torch.tensor(1.0))
    assert max_rel_err(coarse, want) > 5 * TOL
    # and training goes on from the same state afterwards
    lin.train()
    x, dy = seeded_bf16((M, K), 4.0, 340), seeded_bf16((M, N), 1e-3, 341)
    train_step(lin, recipe, x, dy)
    sim.record(0, O.t_amax(x).item()); sim.record(1, O.t_amax(w).item()); sim.update()
    assert_f32_bits_equal(meta.scale, torch.from_numpy(sim.scale), "forward scales after evaluation + one more step")
    # a NEW recipe object of the same shape that trains on: it adopts the module's arena and keeps refreshing it
    recipe_b = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    x, dy = seeded_bf16((M, K), 0.5, 342), seeded_bf16((M, N), 1e-3, 343)
    train_step(lin, recipe_b, x, dy)
    sim.record(0, O.t_amax(x).item()); sim.record(1, O.t_amax(w).item()); sim.update()
    assert lin.fp8_meta["scaling_fwd"] is meta and arena_count() == arenas_before
    assert_f32_bits_equal(meta.scale, torch.from_numpy(sim.scale), "forward scales after a step under a second recipe object")


def test_eval_forward_of_an_untrained_delayed_module_scales_from_its_own_amax(amp):
    """No training step has run: the roles still carry the initial scale 1.  An evaluation forward
    then scales every tensor from its own amax (current scaling) instead of crushing the weight."""
    from optimus_dl_amd.recipe.training_context import forward_context

    M, K, N = 128, 256, 128
    x, w = seeded_bf16((M, K), 1.0, 350), seeded_bf16((N, K), 0.02, 351)
    lin = make_linear(w).eval()
    before = arena_count()
    with torch.no_grad(), forward_context(fp8_cfg("delayed", amax_history_len=8), torch.device("cuda")):
        y = lin(x.cuda())
    assert lin.fp8_calls == 1
    want = O.linear_fwd_bwd(x, w, seeded_bf16((M, N), 1e-3, 352))["y"]
    assert max_rel_err(y, want) <= TOL
    assert lin.fp8_meta == {} and arena_count() == before, "an evaluation forward of an untrained module reserved scaling state"


def test_scaling_state_survives_save_and_reload_into_a_fresh_model(amp):
    """Checkpoint / resume of a delayed-scaling run: recipe.state_dict(model) after 3 steps, loaded into a
    freshly built model + recipe BEFORE its first forward; the next step of the resumed pair equals the
    next step of the original bit for bit, and so does the scaling state afterwards."""
    M, K, N, H = 256, 512, 384, 4

    def build():
        torch.manual_seed(0)
        from optimus_dl_amd.modules.fp8_linear import FP8Linear

        net = nn.Sequential(nn.Linear(K, N, bias=False), nn.Linear(N, K, bias=False)).to("cuda", torch.bfloat16)
        net[0], net[1] = FP8Linear.from_linear(net[0]), FP8Linear.from_linear(net[1])
        return net

    def step(net, recipe, x, dy):
        xd = x.cuda().requires_grad_(True)
        for p in net.parameters():
            p.grad = None
        with recipe.autocast():
            y = net(xd)
        with recipe.backward():
            y.backward(dy.cuda())
        return [y.detach().clone(), xd.grad.clone()] + [p.grad.clone() for p in net.parameters()]

    net, recipe = build(), amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    for s in range(3):
        step(net, recipe, seeded_bf16((M, K), 1.0 + s, 360 + s), seeded_bf16((M, K), 1e-3, 370 + s))
    blob = copy.deepcopy(recipe.state_dict(net))
    weights = copy.deepcopy(net.state_dict())
    assert sorted(blob["modules"]) == ["0", "1"] and blob["modules"]["0"]["fwd"]["amax_history"].shape == (H, 3)
    assert all(not k.endswith("_extra_state") for k in weights), "the model's own state dict must keep its plain keys"

    net2, recipe2 = build(), amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    net2.load_state_dict(weights)
    recipe2.load_state_dict(net2, blob)                       # before any forward of net2
    x, dy = seeded_bf16((M, K), 5.0, 380), seeded_bf16((M, K), 1e-3, 381)
    got, want = step(net2, recipe2, x, dy), step(net, recipe, x, dy)
    for name, a, b in zip(("y", "dx", "dw0", "dw1"), got, want):
        assert torch.equal(a, b), f"{name} of the resumed run differs"
    for i in (0, 1):
        for key in ("scaling_fwd", "scaling_bwd"):
            a, b = net2[i].fp8_meta[key], net[i].fp8_meta[key]
            assert torch.equal(a.amax_history, b.amax_history) and torch.equal(a.scale, b.scale) and torch.equal(a.scale_inv, b.scale_inv)
    # a resumed run that skips the load starts from scale 1 and must differ (the test would otherwise prove nothing)
    net3, recipe3 = build(), amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    net3.load_state_dict(weights)
    assert not torch.equal(step(net3, recipe3, x, dy)[0], want[0])
    # names that do not match are reported, not skipped
    with pytest.raises(KeyError):
        recipe2.load_state_dict(nn.Sequential(net2[0]), blob)
    with pytest.raises(ValueError):
        amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H + 1).load_state_dict(net2, blob)


def test_activation_checkpointing_drops_the_saved_fp8_tensors(amp):
    """The tensors a Linear keeps for its backward (transposed codes of x and w) go through
    autograd's saved-tensor machinery, so non-reentrant activation checkpointing drops them after the
    forward: a checkpointed stack must peak lower than the plain one, with identical gradients."""
    from torch.utils.checkpoint import checkpoint

    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    D, M, L = 1024, 4096, 6
    torch.manual_seed(0)
    blocks = nn.ModuleList([nn.Sequential(FP8Linear(D, 4 * D, bias=False), nn.GELU(), FP8Linear(4 * D, D, bias=False)) for _ in range(L)])
    blocks = blocks.to("cuda", torch.bfloat16)
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    x = seeded_bf16((M, D), 1.0, 390).cuda().requires_grad_(True)
    dy = seeded_bf16((M, D), 1e-3, 391).cuda()

    def run(use_ckpt):
        for p in blocks.parameters():
            p.grad = None
        x.grad = None
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        base = torch.cuda.memory_allocated()
        with recipe.autocast():
            h = x
            for blk in blocks:
                h = checkpoint(blk, h, use_reentrant=False) if use_ckpt else blk(h)
            after_fwd = torch.cuda.memory_allocated() - base
        with recipe.backward():
            h.backward(dy)
        torch.cuda.synchronize()
        peak = torch.cuda.max_memory_allocated() - base
        return after_fwd, peak, x.grad.clone(), [p.grad.clone() for p in blocks.parameters()]

    run(False)                                                  # warm the weight caches: both timed runs see the same state
    held_plain, peak_plain, gx_plain, gw_plain = run(False)
    held_ckpt, peak_ckpt, gx_ckpt, gw_ckpt = run(True)
    # plain: every block holds h [M, 4D] in bf16 for GELU plus 1-byte transposed codes of both Linear inputs;
    # checkpointed: one bf16 [M, D] input per block
    assert held_ckpt < 0.4 * held_plain, (held_ckpt, held_plain)
    assert peak_ckpt < 0.8 * peak_plain, (peak_ckpt, peak_plain)
    assert torch.equal(gx_plain, gx_ckpt)
    for a, b in zip(gw_plain, gw_ckpt):
        assert torch.equal(a, b)


def test_no_grad_forward_in_training_mode_leaves_the_histories_alone(amp):
    """A validation pass under torch.no_grad() WITHOUT model.eval(): the reference's backend refreshes its scaling
    state only when grad mode is on, so such a pass reads the trained scales and records nothing."""
    M, K, N, H = 128, 256, 128, 4
    lin = make_linear(seeded_bf16((N, K), 0.02, 601))
    recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    for s in range(2):
        train_step(lin, recipe, seeded_bf16((M, K), 1.0 + s, 602 + s), seeded_bf16((M, N), 1e-3, 610 + s))
    meta = lin.fp8_meta["scaling_fwd"]
    hist, scale = meta.amax_history.clone(), meta.scale.clone()
    assert lin.training
    with torch.no_grad(), recipe.autocast():
        y = lin(seeded_bf16((M, K), 50.0, 620).cuda())          # much larger than anything training saw
    assert torch.equal(meta.amax_history, hist) and torch.equal(meta.scale, scale)
    assert float(meta.pending_amax.max()) == 0.0
    assert torch.isfinite(y.float()).all()


def test_first_use_under_stream_capture_is_refused_until_the_device_is_set_up(monkeypatch):
    """The per-device look-ups of the library must not run under stream capture: a wrapper that needs them raises,
    in words, when its first use on a device would fall into a capture; after native.init_device() it goes through."""
    from optimus_dl_amd import native as N

    x = seeded_bf16((64, 128), 1.0, 630).cuda()
    out, dyn = torch.empty((64, 128), dtype=torch.uint8, device="cuda"), torch.empty(3, device="cuda")
    monkeypatch.setattr(N, "_devices_ready", set())
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: True)
    with pytest.raises(N.NativeError, match="init_device"):
        N.cast_dynamic_noalloc(x, N.E4M3, 0, out, None, dyn)
    monkeypatch.undo()
    N.init_device()
    N.cast_dynamic_noalloc(x, N.E4M3, 0, out, None, dyn)
    want, _, _, _, _ = N.quantize_dynamic(x, N.E4M3, 0, want_transposed=False)
    assert torch.equal(out, want)
