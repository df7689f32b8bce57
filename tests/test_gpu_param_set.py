"""Many weights quantised in two launches (odl_fp8_multi_amax_parts + odl_fp8_multi_cast_dynamic) and the
``fp8.param`` parameter set built on them: the same bits as the per-tensor route, and no weight quantisation
launches in the forwards between optimizer steps."""
import pytest
import torch
import torch.nn as nn

from oracle import oracle as O
from tests.helpers import assert_bytes_equal, assert_f32_bits_equal, seeded_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def N():
    from optimus_dl_amd import native

    native.load()
    return native


@pytest.fixture(scope="module")
def amp():
    from optimus_dl_amd.modules import amp as A

    return A


SHAPES = [(1024, 768, torch.bfloat16, 0.02), (16, 8, torch.float32, 1.0), (3072, 1024, torch.float32, 0.02),
          (4096, 4096, torch.bfloat16, 0.5), (144, 200, torch.bfloat16, 3.0), (2048, 64, torch.float32, 1e-3)]


@pytest.mark.parametrize("fmt,margin", [(O.E4M3, 0), (O.E5M2, 2)])
def test_multi_tensor_route_equals_the_per_tensor_route_and_the_oracle(N, fmt, margin):
    xs = [seeded_bf16((r, c), std, 40 + i).to(dt).cuda() for i, (r, c, dt, std) in enumerate(SHAPES)]
    xs[3][4095, 4095] = 77.0                                       # the amax of the big one sits in its last block
    plan = N.MultiTensorPlan(xs, fmt, margin)
    for trip in range(2):
        plan.run()
        torch.cuda.synchronize()
        for i, x in enumerate(xs):
            q, q_t, amax, scale, s_inv = N.quantize_dynamic(x, fmt, margin)
            assert_bytes_equal(plan.codes[i], q, f"tensor {i}: codes")
            assert_bytes_equal(plan.codes_t[i], q_t, f"tensor {i}: transposed codes")
            assert_f32_bits_equal(plan.dyn[i], torch.cat([amax, scale, s_inv]), f"tensor {i}: amax / scale / 1/scale")
            if x.numel() <= 1 << 20:                               # and the oracle, where it takes no time
                a = O.t_amax(x.cpu())
                assert float(plan.dyn[i, 0]) == float(a)
                assert_bytes_equal(plan.codes[i], O.t_cast(x.cpu(), O.t_scale(a, fmt, margin), fmt), f"tensor {i}: codes vs oracle")
            assert plan.parts[i].max().item() == plan.dyn[i, 0].item()
        for x in xs:                                               # second trip: new contents, same buffers
            x.mul_(-1.7)
    assert not plan.stale()
    xs[0].data = xs[0].data.clone()
    assert plan.stale()


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_multi_tensor_delayed_cast_equals_the_single_tensor_call(N, fmt):
    """One launch for all tensors under delayed scaling: codes, transposed codes, recorded maxima and 1/scale as
    odl_fp8_cast_delayed gives them per tensor; the strips accumulate over two runs."""
    xs = [seeded_bf16((r, c), std, 60 + i).to(dt).cuda() for i, (r, c, dt, std) in enumerate(SHAPES)]
    n = len(xs)
    scales = torch.tensor([2.0, 0.5, 448.0 / 3, 1.0, 64.0, 3000.0], device="cuda")
    strips = torch.zeros((n, N.AMAX_PARTS), device="cuda")
    plan = N.MultiTensorPlan(xs, fmt, scales=[scales[i:i + 1] for i in range(n)], parts=[strips[i] for i in range(n)])
    plan.run()
    torch.cuda.synchronize()
    for i, x in enumerate(xs):
        own = torch.zeros(N.AMAX_PARTS, device="cuda")
        q, q_t, s_inv = N.cast_delayed(x, scales[i:i + 1], fmt, amax_parts=own, want_transposed=True)
        assert_bytes_equal(plan.codes[i], q, f"tensor {i}: codes")
        assert_bytes_equal(plan.codes_t[i], q_t, f"tensor {i}: transposed codes")
        assert_f32_bits_equal(plan.dyn[i, 2:3], s_inv, f"tensor {i}: 1/scale")
        assert plan.dyn[i, 1].item() == scales[i].item()
        assert strips[i].max().item() == own.max().item() == x.float().abs().max().item()
        if x.numel() <= 1 << 20:
            assert_bytes_equal(plan.codes[i], O.t_cast(x.cpu(), scales[i:i + 1].cpu(), fmt), f"tensor {i}: codes vs oracle")
    before = strips.amax(dim=1).clone()
    for x in xs:
        x.mul_(0.25)
    plan.run()                                                     # smaller values: the strips keep the earlier maxima
    assert torch.equal(strips.amax(dim=1), before)


def test_multi_tensor_plan_refuses_what_the_kernels_cannot_take(N):
    ok = torch.zeros((32, 16), dtype=torch.bfloat16, device="cuda")
    for bad in (torch.zeros((30, 16), dtype=torch.bfloat16, device="cuda"), torch.zeros((32, 12), dtype=torch.bfloat16, device="cuda"),
                torch.zeros((32, 16), dtype=torch.float16, device="cuda"), torch.zeros((64, 16), dtype=torch.bfloat16, device="cuda")[::2],
                torch.zeros((32, 16), dtype=torch.bfloat16)):
        assert not N.MultiTensorPlan.eligible(bad)
        with pytest.raises(N.NativeError):
            N.MultiTensorPlan([ok, bad], O.E4M3)
    with pytest.raises(N.NativeError):
        N.MultiTensorPlan([], O.E4M3)


class Net(nn.Module):
    def __init__(self):
        super().__init__()
        self.a, self.b = nn.Linear(256, 512, bias=False), nn.Linear(512, 256, bias=True)
        self.odd = nn.Linear(256, 24, bias=False)                  # 24 output channels: no FP8 for this one, and the set skips it
        self.tied = nn.Linear(256, 512, bias=False)
        self.tied.weight = self.a.weight

    def forward(self, x):
        return self.b(torch.relu(self.a(x)) + self.tied(x)), self.odd(x)


def build(seed=0):
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(seed)
    net = Net().cuda()                                             # fp32 master weights, the usual AMP set-up
    build_model_transform({"_name": "fp8_linear"}).apply(net)
    return net


def count_weight_quantisations(N, monkeypatch):
    calls = {"n": 0}
    real = N.quantize_dynamic

    def counted(x, *a, **kw):
        if x.dim() == 2 and x.dtype == torch.float32:              # weights here are fp32, activations bf16
            calls["n"] += 1
        return real(x, *a, **kw)

    monkeypatch.setattr(N, "quantize_dynamic", counted)
    return calls


def test_param_set_trains_like_the_per_module_route_without_weight_launches(N, amp, monkeypatch):
    from optimus_dl_amd.modules.fp8_linear import Fp8ParamSet

    plain, kept = build(), build()
    recipe_a, recipe_b = amp.create_fp8_recipe("tensorwise", "hybrid"), amp.create_fp8_recipe("tensorwise", "hybrid")
    opt_a, opt_b = torch.optim.SGD(plain.parameters(), lr=0.05), torch.optim.SGD(kept.parameters(), lr=0.05)
    ps = recipe_b.attach_params(kept, opt_b)
    assert isinstance(ps, Fp8ParamSet) and len(ps.modules) == 3 and len(ps.skipped) == 1 and ps.syncs == 1
    assert len(ps._plan.sources) == 2                              # a and tied share one Parameter: quantised once
    calls = count_weight_quantisations(N, monkeypatch)
    for step in range(4):
        x = seeded_bf16((64, 256), 1.0, 300 + step).cuda()
        outs = []
        for net, recipe, opt in ((plain, recipe_a, opt_a), (kept, recipe_b, opt_b)):
            before = calls["n"]
            for micro in range(2):                                 # two microbatches per optimizer step
                with amp.fp8_autocast(torch.device("cuda"), recipe):
                    y, z = net(x)
                    loss = y.float().square().mean() + z.float().square().mean()
                with amp.fp8_backward(recipe):
                    loss.backward()
            outs.append((y.detach().clone(), z.detach().clone(), calls["n"] - before))
            opt.step()
            opt.zero_grad(set_to_none=True)
        assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1]), f"step {step}: outputs differ"
        assert outs[0][2] == 3 and outs[1][2] == 0, outs           # per module: a, tied and b once per optimizer step; kept: none
    assert ps.syncs == 5                                           # once at attach, once after each optimizer step
    for pa, pb in zip(plain.parameters(), kept.parameters()):
        assert torch.equal(pa, pb)
    # a weight changed behind the set's back is quantised by its module on the next forward (and matches again after a sync)
    with torch.no_grad():
        kept.b.weight.mul_(0.5)
        plain.b.weight.mul_(0.5)
    x = seeded_bf16((64, 256), 1.0, 999).cuda()
    with amp.fp8_autocast(torch.device("cuda"), recipe_a), torch.no_grad():
        want = plain(x)[0]
    before = calls["n"]
    with amp.fp8_autocast(torch.device("cuda"), recipe_b), torch.no_grad():
        got = kept(x)[0]
    assert torch.equal(got, want) and calls["n"] - before == 1
    # parameters that move (here: to bf16 and back is a new storage) are picked up by the next sync
    kept.b.weight.data = kept.b.weight.data.clone()
    ps.sync()
    assert ps._plan.sources[ps._index[ps.modules.index(kept.b)]].data_ptr() == kept.b.weight.data_ptr()
    with amp.fp8_autocast(torch.device("cuda"), recipe_b), torch.no_grad():
        assert torch.equal(kept(x)[0], want)


def test_training_context_attaches_the_set_when_the_config_says_param(amp):
    from optimus_dl_amd.modules.optim.config import AmpConfig, Fp8Config, OptimizationConfig
    from optimus_dl_amd.recipe.training_context import TrainingContext

    def ctx_for(**kw):
        tc = TrainingContext(OptimizationConfig(amp=AmpConfig(enabled=True, dtype="torch.float8_e4m3fn", fp8=Fp8Config(enabled=True, **kw))))
        tc.setup_training_context(torch.device("cuda"))
        return tc

    net = build()
    opt = torch.optim.SGD(net.parameters(), lr=0.1)
    assert ctx_for(recipe="tensorwise", param=False).attach_fp8_params(net, opt) is None
    assert ctx_for(recipe="rowwise", param=True).attach_fp8_params(net, opt) is None        # per-module route for that recipe
    delayed = ctx_for(recipe="delayed", param=True, amax_history_len=8).attach_fp8_params(build(), None)
    assert delayed is not None and delayed._plan.delayed
    ps = ctx_for(recipe="tensorwise", param=True).attach_fp8_params(net, opt)
    assert ps is not None and ps.syncs == 1
    opt.step()
    assert ps.syncs == 2
    bf16 = TrainingContext(OptimizationConfig(amp=AmpConfig(enabled=True, dtype="torch.bfloat16", fp8=Fp8Config(enabled=True, param=True))))
    bf16.setup_training_context(torch.device("cuda"))
    assert bf16.attach_fp8_params(net, opt) is None


def test_param_set_under_delayed_scaling_matches_the_per_module_route(N, amp):
    """One forward per optimizer step: the set casts every weight right after the step with the scale the next forward
    would use and records its amax for the same refresh, so outputs, histories and scales are the bits of the
    per-module route.  With two microbatches the set's codes are reused (no weight launches), where the per-module
    route casts again with the refreshed scale."""
    plain, kept = build(), build()
    recipe_a = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=4)
    recipe_b = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=4)
    opt_a, opt_b = torch.optim.SGD(plain.parameters(), lr=0.05), torch.optim.SGD(kept.parameters(), lr=0.05)
    ps = recipe_b.attach_params(kept, opt_b)
    assert ps is not None and len(ps.modules) == 3 and ps._plan.delayed and len(ps._plan.sources) == 2
    calls = {"n": 0}
    real = N.cast_delayed

    def counted(x, *a, **kw):
        if x.dtype == torch.float32:                               # weights here are fp32, activations bf16
            calls["n"] += 1
        return real(x, *a, **kw)

    try:
        N.cast_delayed = counted
        for step in range(6):
            x = seeded_bf16((64, 256), 1.0 + 0.2 * step, 400 + step).cuda()
            outs = []
            for net, recipe, opt in ((plain, recipe_a, opt_a), (kept, recipe_b, opt_b)):
                before = calls["n"]
                with amp.fp8_autocast(torch.device("cuda"), recipe):
                    y, z = net(x)
                    loss = y.float().square().mean() + z.float().square().mean()
                with amp.fp8_backward(recipe):
                    loss.backward()
                outs.append((y.detach().clone(), calls["n"] - before))
                opt.step()
                opt.zero_grad(set_to_none=True)
            assert torch.equal(outs[0][0], outs[1][0]), f"step {step}: outputs differ"
            assert outs[0][1] == 3 and outs[1][1] == 0, outs
            for name in ("a", "b"):
                for direction in ("scaling_fwd", "scaling_bwd"):
                    ma, mb = getattr(plain, name).fp8_meta[direction], getattr(kept, name).fp8_meta[direction]
                    assert torch.equal(ma.amax_history, mb.amax_history) and torch.equal(ma.scale, mb.scale), (step, name, direction)
        assert (kept.a.fp8_meta["scaling_fwd"].scale != 1.0).any()
        # two microbatches per optimizer step: nothing is launched for the weights in either forward
        before = calls["n"]
        for micro in range(2):
            with amp.fp8_autocast(torch.device("cuda"), recipe_b):
                y, z = kept(x)
            with amp.fp8_backward(recipe_b):
                (y.float().square().mean() + z.float().square().mean()).backward()
        assert calls["n"] == before
        opt_b.step()
    finally:
        N.cast_delayed = real


def test_param_set_records_the_weight_amax_in_every_microbatch_under_delayed_scaling(N, amp):
    """The kept codes launch nothing for the weights, and every microbatch ends in a refresh that clears the strips of
    partial maxima: the set folds the maxima of its last sync back in before each refresh, so the weight role's history
    gets one real entry per refresh (as on the per-module route, which folds its cached amax on every reuse) instead
    of one real entry and then zeros."""
    kept = build()
    recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=4)
    opt = torch.optim.SGD(kept.parameters(), lr=0.05)
    ps = recipe.attach_params(kept, opt)
    assert ps is not None
    x = seeded_bf16((64, 256), 1.0, 470).cuda()
    for micro in range(3):                                       # three microbatches, no optimizer step in between
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            y, z = kept(x)
        with amp.fp8_backward(recipe):
            (y.float().square().mean() + z.float().square().mean()).backward()
    for name in ("a", "b"):
        mod = getattr(kept, name)
        hist = mod.fp8_meta["scaling_fwd"].amax_history[:, 1]    # role 1 = the weight
        want = mod.weight.detach().float().abs().max()
        # the refresh rolls the history: after three refreshes three of the four rows hold the weight's amax
        assert int((hist == want).sum()) == 3, (name, hist.tolist(), float(want))


def test_loading_scaling_state_drops_the_codes_the_param_set_kept(N, amp):
    """Resume order: load the weights, attach the set (which casts every weight at the initial scale 1), then load the
    scaling state.  The codes the set made under scale 1 must not survive the load: the first step of the resumed run
    equals the next step of the uninterrupted one bit for bit."""
    import copy

    def step(net, recipe, x):
        for p in net.parameters():
            p.grad = None
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            y, z = net(x)
            loss = y.float().square().mean() + z.float().square().mean()
        with amp.fp8_backward(recipe):
            loss.backward()
        return [y.detach().clone(), z.detach().clone()] + [p.grad.detach().clone() for p in net.parameters()]

    net, recipe = build(), amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=4)
    ps = recipe.attach_params(net)
    for s in range(3):
        step(net, recipe, seeded_bf16((64, 256), 1.0 + 0.3 * s, 480 + s).cuda())
        ps.sync()                                                # where the optimizer step would be (weights unchanged here)
    blob, weights = copy.deepcopy(recipe.state_dict(net)), copy.deepcopy(net.state_dict())

    net2, recipe2 = build(), amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=4)
    net2.load_state_dict(weights)
    ps2 = recipe2.attach_params(net2)                            # casts at scale 1: a weight of std 0.02 lands in the subnormals
    recipe2.load_state_dict(net2, blob)
    for i in range(len(ps._plan.codes)):                         # cast again under the restored scales, not left at scale 1
        assert torch.equal(ps2._plan.codes[i], ps._plan.codes[i]) and torch.equal(ps2._plan.dyn[i], ps._plan.dyn[i])
    x = seeded_bf16((64, 256), 2.0, 490).cuda()
    got, want = step(net2, recipe2, x), step(net, recipe, x)
    for i, (a, b) in enumerate(zip(got, want)):
        assert torch.equal(a, b), f"tensor {i} of the resumed step differs"
