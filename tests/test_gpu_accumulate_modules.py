"""The GEMM's accumulate flag at module level: data gradients of Linears fed by one tensor summed by the GEMMs
(``linear_group`` / ``SiblingGroup``; the reference's attention.py:317-319 and mlp.py:76-78 feed q/k/v and gate/up the
same tensor), and weight gradients added into ``.grad`` over microbatches (``fuse_wgrad_accumulation``; the reference
runs ``acc_steps`` microbatches per optimizer step, iteration_mixin.py:332)."""
import pytest
import torch
import torch.nn as nn

from tests.helpers import seeded_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amp():
    from optimus_dl_amd.modules import amp as A

    return A


class Attn(nn.Module):
    """The projections of the reference's attention block, fed the way its forward feeds them."""

    def __init__(self, d=512, kv=256, bias=False):
        super().__init__()
        self.wq, self.wk, self.wv = nn.Linear(d, d, bias=bias), nn.Linear(d, kv, bias=bias), nn.Linear(d, kv, bias=bias)

    def forward(self, x):
        return self.wq(x), self.wk(x), self.wv(x)


def build(bias=False, group=True, dtype=torch.bfloat16):
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(0)
    net = Attn(bias=bias).to("cuda", dtype)
    cfg = {"_name": "fp8_linear"} if group else {"_name": "fp8_linear", "group_siblings": ()}
    build_model_transform(cfg).apply(net)
    return net


def run(net, recipe, x, dys):
    xd = x.clone().requires_grad_(True)
    for p in net.parameters():
        p.grad = None
    with recipe.autocast():
        outs = net(xd)
    with recipe.backward():
        torch.autograd.backward(outs, dys)
    return [o.detach() for o in outs], xd.grad, [p.grad for p in net.parameters()]


@pytest.mark.parametrize("kind", ["tensorwise", "delayed", "rowwise"])
@pytest.mark.parametrize("bias", [False, True])
def test_sibling_group_equals_separate_linears(amp, kind, bias):
    """Outputs and weight gradients are the same bits (same kernels on the same operands); the data gradient is the sum
    formed by the GEMMs, each addition rounded once: within one bf16 unit of the sum autograd forms from the three
    rounded products, and closer to the fp32 sum."""
    grouped, plain = build(bias, True), build(bias, False)
    assert grouped.wq._siblings is not None and grouped.wq._siblings is grouped.wv._siblings and plain.wq._siblings is None
    kw = {"amax_history_len": 4} if kind == "delayed" else {}
    ra, rb = amp.create_fp8_recipe(kind, "hybrid", **kw), amp.create_fp8_recipe(kind, "hybrid", **kw)
    probe = build(bias, False)
    rp = amp.create_fp8_recipe(kind, "hybrid", **kw)
    for step in range(3):
        x = seeded_bf16((4, 96, 512), 1.0, 700 + step).cuda()
        dys = [seeded_bf16((4, 96, n), 1e-3, 710 + 3 * step + i).cuda() for i, n in enumerate((512, 256, 256))]
        got, want = run(grouped, ra, x, dys), run(plain, rb, x, dys)
        for a, b in zip(got[0], want[0]):
            assert torch.equal(a, b)
        for a, b in zip(got[2], want[2]):
            assert torch.equal(a, b)
        if kind == "delayed":
            # (the scales depend on the history, which a probe run would disturb: the sums are compared as they are,
            # against the largest gradient, three roundings of an intermediate sum at most apart)
            assert (got[1].float() - want[1].float()).abs().max().item() <= 3 * 2.0 ** -8 * want[1].float().abs().max().item()
            continue
        # the three products one by one: the plain model with two of the three grad_outputs zeroed
        parts = []
        for i in range(3):
            sel = [dys[j] if j == i else torch.zeros_like(dys[j]) for j in range(3)]
            parts.append(run(probe, rp, x, sel)[1].float())
        exact = parts[0] + parts[1] + parts[2]
        # every rounding (of a product to bf16, of an intermediate sum) is off by at most 2^-9 of a value no larger than the sum of
        # the magnitudes: a few of them stay far inside 2^-5 of that sum, a dropped or doubled product does not
        bound = (parts[0].abs() + parts[1].abs() + parts[2].abs()) * 2.0 ** -5 + 1e-12
        assert bool(((got[1].float() - want[1].float()).abs() <= bound).all())
        assert bool(((got[1].float() - exact).abs() <= bound).all())
        assert (got[1].float() - exact).abs().max().item() <= (want[1].float() - exact).abs().max().item() * 1.5 + 1e-12
    assert grouped.wq.fp8_calls == 3 and grouped.wk.fp8_calls == 3


def test_sibling_group_launches_no_separate_adds(amp, monkeypatch):
    """Two of the three dgrad GEMMs run with the accumulate flag, and an unused output costs nothing in the backward."""
    from optimus_dl_amd import native as N

    net, recipe = build(), amp.create_fp8_recipe("tensorwise", "hybrid")
    calls = []
    real = N.gemm_nt

    def spy(*a, **kw):
        calls.append(bool(kw.get("accumulate", False)))
        return real(*a, **kw)

    monkeypatch.setattr(N, "gemm_nt", spy)
    x = seeded_bf16((128, 512), 1.0, 720).cuda().requires_grad_(True)
    with recipe.autocast():
        q, k, v = net(x)
    with recipe.backward():
        torch.autograd.backward([q, k, v], [torch.ones_like(q), torch.ones_like(k), torch.ones_like(v)])
    assert calls.count(True) == 2, calls
    calls.clear()
    x.grad = None
    with recipe.autocast():
        q, k, v = net(x)
    with recipe.backward():
        (q.float().sum() + v.float().sum()).backward()             # k is not used: its Linear has no backward at all
    assert calls.count(True) == 1 and net.wk.weight.grad is not None
    assert len(calls) == 3 + 2 + 1                                  # 3 forwards, a dgrad each for q and v, ONE wgrad for both (128 tokens: no K-slow wgrad)


def test_sibling_group_stands_down_when_members_get_different_inputs(amp):
    net, recipe = build(), amp.create_fp8_recipe("tensorwise", "hybrid")
    x = seeded_bf16((64, 512), 1.0, 730).cuda().requires_grad_(True)
    y = seeded_bf16((64, 512), 1.0, 731).cuda().requires_grad_(True)
    with recipe.autocast():
        q = net.wq(x)
        k = net.wk(y)                   # cross-attention style: another tensor
        v = net.wv(y)
    grp = net.wq._siblings
    assert grp.misses >= 1 and not grp.pending
    want_k = None
    plain = build(group=False)
    with recipe.autocast():
        want_k = plain.wk(y)
    assert torch.equal(k, want_k)
    with recipe.backward():
        (q.float().sum() + k.float().sum() + v.float().sum()).backward()
    assert x.grad is not None and y.grad is not None
    before = grp.misses
    with recipe.autocast():             # from now on every member runs on its own
        net.wq(x), net.wk(x), net.wv(x)
    assert grp.misses == before and not grp.pending


@pytest.mark.parametrize("wdtype", [torch.float32, torch.bfloat16])
def test_fused_wgrad_accumulation_over_microbatches(amp, wdtype):
    """Four microbatches: with ``fuse_wgrad_accumulation`` the weight gradients of microbatches 2..4 are added into
    ``.grad`` by the GEMM (autograd gets None), equal to the unfused route within one rounding of the gradient type per
    microbatch (exactly equal for fp32 gradients, where both routes add the same fp32 product once)."""
    from optimus_dl_amd import native as N
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    torch.manual_seed(0)
    M, K, Nn = 1024, 512, 768            # 1024 tokens: wgrad reads dY as stored (K-slow) -> the workspace route
    lin_a = FP8Linear(K, Nn, bias=True, device="cuda", dtype=wdtype)
    lin_b = FP8Linear(K, Nn, bias=True, device="cuda", dtype=wdtype)
    lin_b.load_state_dict(lin_a.state_dict())
    ra, rb = amp.create_fp8_recipe("tensorwise", "hybrid"), amp.create_fp8_recipe("tensorwise", "hybrid")
    rb.fuse_wgrad_accumulation = True
    for micro in range(4):
        x = seeded_bf16((M, K), 1.0, 740 + micro).cuda()
        dy = seeded_bf16((M, Nn), 1e-3, 750 + micro).cuda()
        for lin, recipe in ((lin_a, ra), (lin_b, rb)):
            with amp.fp8_autocast(torch.device("cuda"), recipe):
                y = lin(x)
            with amp.fp8_backward(recipe):
                y.backward(dy.to(y.dtype))
    ga, gb = lin_a.weight.grad, lin_b.weight.grad
    if wdtype == torch.float32:
        assert torch.equal(ga, gb)
    else:
        # four roundings to bf16 of running sums on either route: a few units of the largest intermediate value apart
        assert (ga.float() - gb.float()).abs().max().item() <= 2.0 ** -6 * ga.float().abs().max().item()
    assert torch.equal(lin_a.bias.grad, lin_b.bias.grad)


class WideAttn(nn.Module):
    """The same three projections at a size whose data gradient fills the chip with 256 x 256 tiles."""

    def __init__(self, d=2304, q=1024, kv=512):
        super().__init__()
        self.wq, self.wk, self.wv = nn.Linear(d, q, bias=False), nn.Linear(d, kv, bias=False), nn.Linear(d, kv, bias=False)

    def forward(self, x):
        return self.wq(x), self.wk(x), self.wv(x)


def build_wide(group=True):
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(1)
    net = WideAttn().to("cuda", torch.bfloat16)
    build_model_transform({"_name": "fp8_linear"} if group else {"_name": "fp8_linear", "group_siblings": ()}).apply(net)
    return net


@pytest.mark.parametrize("kind", ["tensorwise", "delayed"])
def test_sibling_group_data_gradient_from_one_gemm(amp, kind, monkeypatch):
    """4096 tokens x 2304 features (144 tiles): the group's data gradient comes from ONE launch over the three members'
    operands (no GEMM with the accumulate flag, no dgrad of a member's own), outputs and weight gradients are the bits of
    the separate Linears, and the data gradient lies as close to the fp32 sum of the three products as the sum that the
    accumulate flag forms (``fuse_dgrad_gemm = False``) and as the one autograd forms, or closer."""
    from optimus_dl_amd import native as N

    kw = {"amax_history_len": 4} if kind == "delayed" else {}
    grouped, stepwise, plain = build_wide(), build_wide(), build_wide(False)
    r1, r2, r3 = (amp.create_fp8_recipe(kind, "hybrid", **kw) for _ in range(3))
    r2.fuse_dgrad_gemm = False
    sums, accs = [], []
    real_sum, real_nt = N.gemm_nt_sum, N.gemm_nt
    monkeypatch.setattr(N, "gemm_nt_sum", lambda *a, **k: (sums.append(len(a[0])), real_sum(*a, **k))[1])
    monkeypatch.setattr(N, "gemm_nt", lambda *a, **k: (accs.append(bool(k.get("accumulate", False))), real_nt(*a, **k))[1])
    x = seeded_bf16((4096, 2304), 1.0, 900).cuda()
    dys = [seeded_bf16((4096, n), 1e-3 * (4.0 ** i), 910 + i).cuda() for i, n in enumerate((1024, 512, 512))]
    got = run(grouped, r1, x, dys)
    assert sums == [3] and accs.count(True) == 0
    sums.clear(); accs.clear()
    mid = run(stepwise, r2, x, dys)
    assert sums == [] and accs.count(True) == 2
    want = run(plain, r3, x, dys)
    for a, b in zip(got[0] + got[2], want[0] + want[2]):
        assert torch.equal(a, b)
    if kind == "tensorwise":
        probe, rp = build_wide(False), amp.create_fp8_recipe(kind, "hybrid")
        parts = []
        for i in range(3):
            sel = [dys[j] if j == i else torch.zeros_like(dys[j]) for j in range(3)]
            parts.append(run(probe, rp, x, sel)[1].float())
        exact = parts[0] + parts[1] + parts[2]                      # (each part rounded to bf16 once: 2^-9 relative)
        err = lambda t: (t.float() - exact).abs().max().item()
        assert err(got[1]) <= err(mid[1]) * 1.05 + 1e-12 and err(got[1]) <= err(want[1]) * 1.05 + 1e-12
        bound = (parts[0].abs() + parts[1].abs() + parts[2].abs()) * 2.0 ** -6 + 1e-12
        assert bool(((got[1].float() - exact).abs() <= bound).all())
    else:
        assert (got[1].float() - want[1].float()).abs().max().item() <= 3 * 2.0 ** -8 * want[1].float().abs().max().item()


def test_one_gemm_data_gradient_replays_from_a_graph(amp):
    """The call that sums the members' products takes host arrays of device pointers and hands them to the kernel by value:
    captured in a graph it must replay on new data like everything else (three replays, eager work and synchronisations
    in between, each against eager on the same buffers)."""
    net, recipe = build_wide(), amp.create_fp8_recipe("tensorwise", "hybrid")
    x_static = torch.zeros((4096, 2304), dtype=torch.bfloat16, device="cuda", requires_grad=True)
    dy_static = [torch.zeros((4096, n), dtype=torch.bfloat16, device="cuda") for n in (1024, 512, 512)]
    params = [net.wq.weight, net.wk.weight, net.wv.weight]

    def fwd_bwd():
        for lin in (net.wq, net.wk, net.wv):
            lin._wcache.key = None
        with recipe.autocast():
            ys = net(x_static)
        with recipe.backward():
            grads = torch.autograd.grad(ys, (x_static, *params), dy_static)
        return (*ys, *grads)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fwd_bwd()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs_g = fwd_bwd()
    for rep in range(3):
        with torch.no_grad():
            x_static.copy_(seeded_bf16((4096, 2304), 1.0 + rep, 950 + rep).cuda())
            for i, d in enumerate(dy_static):
                d.copy_(seeded_bf16(tuple(d.shape), 1e-3 * (rep + 1) * 3.0 ** i, 960 + 3 * rep + i).cuda())
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs_g]
        want = fwd_bwd()
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, want)):
            assert torch.equal(a, b), f"replay {rep}: output {i} differs from eager"
