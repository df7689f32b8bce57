"""GPU: the fused SwiGLU / RMSNorm forwards inside real module trees.  What must hold:
the hand-over of partial maxima changes no bit (same codes, same outputs as the amax pass it
replaces), the amax passes it replaces are really gone, and the fused modules agree with the
modules' own PyTorch forwards to within a bf16 unit here and there (GEMM tolerance downstream)."""
import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

from oracle import oracle as O
from tests.helpers import max_rel_err, seeded_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def amp():
    from optimus_dl_amd.modules import amp as A

    return A


def make_mlp(n_embd=256, hidden=512, fuse=True, seed=0):
    from optimus_dl_amd.modules.model.blocks import SwiGLUMLP
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(seed)
    mlp = SwiGLUMLP(n_embd, hidden).to("cuda", torch.bfloat16)
    t = build_model_transform({"_name": "fp8_linear", "fuse_swiglu": fuse})
    t.apply(mlp)
    return mlp, t


def step(module, recipe, x, dy):
    xd = x.clone().requires_grad_(True)
    for p in module.parameters():
        p.grad = None
    with recipe.autocast():
        y = module(xd)
    with recipe.backward():
        y.backward(dy)
    return [y.detach(), xd.grad.detach()] + [p.grad.detach().clone() for p in module.parameters()]


def count_calls(monkeypatch, native, name):
    calls = []
    orig = getattr(native, name)

    def counted(*a, **kw):
        calls.append(tuple(a[0].shape))
        return orig(*a, **kw)

    monkeypatch.setattr(native, name, counted)
    return calls


def test_fused_mlp_skips_three_amax_passes_and_changes_no_bit(amp, monkeypatch):
    from optimus_dl_amd import native

    M, C, H = 384, 256, 512
    x = seeded_bf16((M, C), 1.0, 1).cuda()
    dy = seeded_bf16((M, C), 1e-3, 2).cuda()
    mlp, t = make_mlp(C, H, fuse=True)
    assert t.last_replacements.get("SwiGLU") == 1
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    amax_calls = count_calls(monkeypatch, native, "amax_parts")
    fused = step(mlp, recipe, x, dy)
    # x (shared by w1/w2), three weights, dy of c_proj: h, d_gate and d_up come with their maxima
    assert sorted(amax_calls) == sorted([(M, C), (H, C), (H, C), (C, H), (M, C)])
    assert recipe.producer_parts == []                                   # all three were taken
    # same modules, hand-over switched off: every tensor gets its own amax pass, results identical
    monkeypatch.setattr(type(recipe), "offer_parts", lambda self, t_, p_: None)
    amax_calls.clear()
    plain = step(mlp, recipe, x, dy)
    # the weights' codes are cached (unchanged Parameters): x, h, dy and the two gradients remain
    assert sorted(amax_calls) == sorted([(M, C), (M, H), (M, C), (M, H), (M, H)])
    for a, b in zip(fused, plain):
        assert torch.equal(a, b)


def test_fused_mlp_agrees_with_the_eager_activation(amp):
    M, C, H = 512, 256, 768
    x = seeded_bf16((M, C), 1.0, 3).cuda()
    dy = seeded_bf16((M, C), 1e-3, 4).cuda()
    fused_mlp, _ = make_mlp(C, H, fuse=True, seed=5)
    eager_mlp, t = make_mlp(C, H, fuse=False, seed=5)
    assert "SwiGLU" not in t.last_replacements
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    got = step(fused_mlp, recipe, x, dy)
    want = step(eager_mlp, recipe, x, dy)
    for name, a, b in zip(["y", "dx", "dw1", "dw2", "dwc"], got, want):
        assert max_rel_err(a, b) <= 1e-2, name


def test_swiglu_function_matches_torch_autograd(amp):
    from optimus_dl_amd.modules.fused import swiglu

    g = seeded_bf16((64, 256), 1.5, 6).cuda().requires_grad_(True)
    u = seeded_bf16((64, 256), 1.0, 7).cuda().requires_grad_(True)
    dh = seeded_bf16((64, 256), 1e-2, 8).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    with recipe.autocast():
        h = swiglu(g, u)
    h.backward(dh)
    gc, uc, dhc = g.detach().cpu(), u.detach().cpu(), dh.cpu()
    assert torch.equal(h.detach().cpu().view(torch.int16), O.c_swiglu_fwd(gc, uc).view(torch.int16))
    wg, wu = O.c_swiglu_bwd(dhc, gc, uc)
    assert torch.equal(g.grad.cpu().view(torch.int16), wg.view(torch.int16))
    assert torch.equal(u.grad.cpu().view(torch.int16), wu.view(torch.int16))
    # outside a recipe: plain PyTorch
    h2 = swiglu(g.detach(), u.detach())
    assert torch.equal(h2, F.silu(g.detach()) * u.detach())


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
def test_fused_rmsnorm_feeds_the_linear_and_backpropagates(amp, monkeypatch, in_dtype):
    from optimus_dl_amd import native
    from optimus_dl_amd.modules.model.blocks import RMSNorm
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    class Pre(nn.Module):
        def __init__(self):
            super().__init__()
            self.ln = RMSNorm(256, 1e-5)
            self.wq = nn.Linear(256, 320, bias=False)
            self.wk = nn.Linear(256, 128, bias=False)

        def forward(self, x):
            n = self.ln(x)
            return self.wq(n).float().sum(-1) + self.wk(n).float().sum(-1)

    torch.manual_seed(0)
    net = Pre().cuda()
    with torch.no_grad():
        net.ln.weight.copy_(torch.linspace(0.5, 1.5, 256))
    ref = Pre().cuda()
    ref.load_state_dict(net.state_dict())
    t = build_model_transform({"_name": "transformer_engine"})
    t.apply(net)
    assert t.last_replacements["RMSNorm"] == 1 and t.last_replacements["Linear"] == 2
    build_model_transform({"_name": "transformer_engine", "replace_norm": False}).apply(ref)
    x = (torch.randn(4, 96, 256, generator=torch.Generator().manual_seed(1)) * 2).to(in_dtype).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    amax_calls = count_calls(monkeypatch, native, "amax_parts")
    outs = {}
    for name, m in (("fused", net), ("plain", ref)):
        xd = x.clone().requires_grad_(True)
        amax_calls.clear()
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            y = m(xd)
        with amp.fp8_backward(recipe):
            y.sum().backward()
        outs[name] = (y.detach(), xd.grad.detach(), m.ln.weight.grad.detach(), m.wq.weight.grad.detach())
        if name == "fused":
            # the normalised activation arrives with its maxima: only the two weights and the two dy
            assert sorted(amax_calls) == sorted([(320, 256), (128, 256), (384, 320), (384, 128)])
        else:
            assert (4 * 96, 256) in amax_calls
    f, p = outs["fused"], outs["plain"]
    assert f[1].dtype == in_dtype
    assert max_rel_err(f[0], p[0]) <= 1e-2
    assert max_rel_err(f[1], p[1]) <= 2e-2
    assert max_rel_err(f[2], p[2]) <= 2e-2
    assert max_rel_err(f[3], p[3]) <= 1e-2


def test_fused_rmsnorm_equals_oracle_and_leaves_other_cases_alone(amp):
    from optimus_dl_amd.modules.fused import fuse_rmsnorm
    from optimus_dl_amd.modules.model.blocks import RMSNorm

    norm = RMSNorm(512, 1e-6).cuda()
    with torch.no_grad():
        norm.weight.copy_(torch.linspace(0.25, 2.0, 512))
    assert fuse_rmsnorm(norm) and not fuse_rmsnorm(norm)
    x = seeded_bf16((3, 40, 512), 3.0, 9)
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    with amp.fp8_autocast(torch.device("cuda"), recipe):
        y = norm(x.cuda())
        y32 = norm(x.float().cuda())                     # fp32 in, bf16 out under the bf16 autocast
    want, _ = O.c_rmsnorm(x, norm.weight.detach().cpu(), 1e-6)
    assert y.dtype == torch.bfloat16 and torch.equal(y.cpu().view(torch.int16), want.view(torch.int16))
    assert y32.dtype == torch.bfloat16 and torch.equal(y32.cpu().view(torch.int16), want.view(torch.int16))
    # no recipe: the module's own forward, dtype of the input
    y_plain = norm(x.float().cuda())
    assert y_plain.dtype == torch.float32
    # a recipe without the bf16 autocast around it and an fp32 input: own forward as well
    with recipe.autocast():
        assert norm(x.float().cuda()).dtype == torch.float32
        assert norm(x.cuda()).dtype == torch.bfloat16


@pytest.mark.parametrize("recipe_name", ["tensorwise", "delayed", "rowwise"])
def test_llama_block_with_fusions_trains_like_the_unfused_one(amp, recipe_name):
    from optimus_dl_amd.modules.model import Llama, LlamaConfig
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    def build(fuse):
        torch.manual_seed(0)
        m = Llama(LlamaConfig(vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=128, intermediate_size=256)).cuda()
        t = build_model_transform({"_name": "transformer_engine", "replace_norm": fuse, "fuse_swiglu": fuse})
        t.apply(m)
        return m, t

    ids = torch.randint(0, 256, (4, 33), generator=torch.Generator().manual_seed(2)).cuda()
    traces = {}
    for fuse in (True, False):
        m, t = build(fuse)
        assert (t.last_replacements.get("SwiGLU", 0) == 2) == fuse and (t.last_replacements["RMSNorm"] == 5) == fuse
        recipe = amp.FP8Recipe(recipe_type=recipe_name, amax_history_len=4)
        opt = torch.optim.AdamW(m.parameters(), lr=3e-3)
        trace = []
        for _ in range(6):
            opt.zero_grad(set_to_none=True)
            with amp.fp8_autocast(torch.device("cuda"), recipe):
                logits = m(ids[:, :-1])["logits"].float()
                loss = F.cross_entropy(logits.reshape(-1, 256), ids[:, 1:].reshape(-1))
            with amp.fp8_backward(recipe):
                loss.backward()
            opt.step()
            trace.append(loss.item())
        assert all(p.grad is not None for p in m.parameters())
        traces[fuse] = trace
    assert traces[True][-1] < traces[True][0] - 0.3, traces
    assert abs(traces[True][-1] - traces[False][-1]) < 0.15, traces


def test_bias_gradient_comes_out_of_the_amax_pass(amp, monkeypatch):
    from optimus_dl_amd import native
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    M, K, Nn = 320, 256, 768
    torch.manual_seed(0)
    lin = FP8Linear.from_linear(nn.Linear(K, Nn, bias=True).to("cuda", torch.bfloat16))
    x = seeded_bf16((M, K), 1.0, 1).cuda().requires_grad_(True)
    dy = seeded_bf16((M, Nn), 1e-2, 2)
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    amax_calls = count_calls(monkeypatch, native, "amax_parts")
    colsum_calls = count_calls(monkeypatch, native, "amax_parts_colsum")
    with recipe.autocast():
        y = lin(x)
    with recipe.backward():
        y.backward(dy.cuda())
    assert colsum_calls == [(M, Nn)] and (M, Nn) not in amax_calls
    want = dy.double().sum(0)
    got = lin.bias.grad.float().cpu().double()
    assert lin.bias.grad.dtype == torch.bfloat16
    assert ((got - want).abs() <= 2.0 ** -8 * want.abs() + 1e-6).all()           # one bf16 rounding of an fp32 sum
    # the codes are those of the plain route: same dx, dw as a bias-free twin fed the same tensors
    twin = FP8Linear.from_linear(nn.Linear(K, Nn, bias=False).to("cuda", torch.bfloat16))
    with torch.no_grad():
        twin.weight.copy_(lin.weight)
    x2 = x.detach().clone().requires_grad_(True)
    with recipe.autocast():
        y2 = twin(x2)
    with recipe.backward():
        y2.backward(dy.cuda())
    assert torch.equal(x.grad, x2.grad) and torch.equal(lin.weight.grad, twin.weight.grad)


@pytest.mark.parametrize("in_dtype", [torch.float32, torch.bfloat16])
def test_fused_layernorm_in_a_gpt2_block(amp, monkeypatch, in_dtype):
    """nn.LayerNorm -> Linear as in a GPT-2 block: the transform re-classes the norm, the Linear takes its maxima,
    outputs and gradients agree with the untouched norm."""
    from optimus_dl_amd import native
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    class Pre(nn.Module):
        def __init__(self):
            super().__init__()
            self.ln = nn.LayerNorm(256)
            self.c_fc = nn.Linear(256, 512)

        def forward(self, x):
            return self.c_fc(self.ln(x))

    torch.manual_seed(0)
    net = Pre().cuda()
    with torch.no_grad():
        net.ln.weight.copy_(torch.linspace(0.5, 1.5, 256))
        net.ln.bias.copy_(torch.linspace(-0.2, 0.2, 256))
    ref = Pre().cuda()
    ref.load_state_dict(net.state_dict())
    t = build_model_transform({"_name": "transformer_engine"})
    t.apply(net)
    assert t.last_replacements["LayerNorm"] == 1 and isinstance(net.ln, nn.LayerNorm)
    build_model_transform({"_name": "transformer_engine", "replace_norm": False}).apply(ref)
    x = (torch.randn(3, 128, 256, generator=torch.Generator().manual_seed(1)) * 2 + 0.3).to(in_dtype).cuda()
    dy = seeded_bf16((3, 128, 512), 1e-2, 2).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    amax_calls = count_calls(monkeypatch, native, "amax_parts")
    outs = {}
    for name, m in (("fused", net), ("plain", ref)):
        xd = x.clone().requires_grad_(True)
        amax_calls.clear()
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            y = m(xd)
        with amp.fp8_backward(recipe):
            y.backward(dy)
        outs[name] = (y.detach(), xd.grad.detach(), m.ln.weight.grad.detach(), m.ln.bias.grad.detach(), m.c_fc.weight.grad.detach())
        assert ((384, 256) in amax_calls) == (name == "plain")          # the normalised activation's own amax pass
    for a, b, tol in zip(outs["fused"], outs["plain"], (1e-2, 2e-2, 2e-2, 2e-2, 1e-2)):
        assert max_rel_err(a, b) <= tol
    assert outs["fused"][1].dtype == in_dtype


def test_gpt2_mlp_with_fused_gelu(amp, monkeypatch):
    """c_proj(gelu(c_fc(x))) with biases: the transform re-classes nn.GELU, c_proj takes the activation's maxima,
    c_fc's backward takes the gradient's, and the results agree with PyTorch's GELU."""
    from optimus_dl_amd import native
    from optimus_dl_amd.modules.model.blocks import GELUMLP
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    def build(fuse):
        torch.manual_seed(0)
        m = GELUMLP(256, 1024, bias=True).to("cuda", torch.bfloat16)
        t = build_model_transform({"_name": "transformer_engine", "fuse_gelu": fuse})
        t.apply(m)
        assert t.last_replacements.get("GELU", 0) == (1 if fuse else 0) and isinstance(m.gelu, nn.GELU)
        return m

    M = 384
    x = seeded_bf16((M, 256), 1.0, 1).cuda()
    dy = seeded_bf16((M, 256), 1e-2, 2).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    amax_calls = count_calls(monkeypatch, native, "amax_parts")
    colsum_calls = count_calls(monkeypatch, native, "amax_parts_colsum")
    fused = step(build(True), recipe, x, dy)
    # x and the two weights by amax_parts; h arrives with its maxima; both grad_outputs go through the amax + column-sum
    # pass because both Linears have a bias (for c_fc it runs for the column sums: the GELU backward left the maxima)
    assert sorted(amax_calls) == sorted([(M, 256), (1024, 256), (256, 1024)]) and colsum_calls == [(M, 256), (M, 1024)]
    amax_calls.clear(); colsum_calls.clear()
    plain = step(build(False), recipe, x, dy)
    assert (M, 1024) in amax_calls and (M, 1024) in colsum_calls
    for a, b in zip(fused, plain):
        assert max_rel_err(a, b) <= 1e-2


# ------------------------------------------------ activation checkpointing around the converted blocks
@pytest.mark.parametrize("fuse", [True, False])
def test_checkpointed_blocks_recompute_the_same_fp8_forward(amp, fuse):
    """The reference wraps blocks in torch.utils.checkpoint (its `activation_checkpoint` transform,
    model_transforms/checkpoint.py:45-81, non-reentrant by default) and runs backward inside the FP8
    backward context: the recomputation then finds the recipe, takes the FP8 path again, saves the same
    tensors, and with per-tensor current scaling reproduces the first forward bit for bit, so every gradient
    equals the one of the run without checkpointing."""
    from torch.utils.checkpoint import checkpoint

    from optimus_dl_amd.modules.model import Llama, LlamaConfig
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(0)
    m = Llama(LlamaConfig(vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=128, intermediate_size=256)).cuda()
    build_model_transform({"_name": "fp8_linear", "replace_norm": fuse, "fuse_swiglu": fuse}).apply(m)
    ids = torch.randint(0, 256, (4, 64), generator=torch.Generator().manual_seed(2)).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")

    def run(ckpt):
        for p in m.parameters():
            p.grad = None
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            x = m.embed(ids)
            for block in m.transformer.h:
                x = checkpoint(block, x, use_reentrant=False) if ckpt else block(x)
            logits = m.lm_head(m.transformer.ln_f(x)).float()
            loss = F.cross_entropy(logits.reshape(-1, 256), ids.reshape(-1))
        with amp.fp8_backward(recipe):
            loss.backward()
        assert recipe.shared_input is None and not recipe.producer_parts        # nothing is kept alive after the step
        return loss.detach(), [p.grad.detach().clone() for p in m.parameters()]

    calls_before = sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls"))
    loss0, grads0 = run(False)
    calls_plain = sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls")) - calls_before
    loss1, grads1 = run(True)
    calls_ckpt = sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls")) - calls_before - calls_plain
    # the Linears inside the blocks ran again on the FP8 path (the recomputation stops at a block's last saved tensor)
    assert calls_plain + 10 <= calls_ckpt <= 2 * calls_plain - 1
    assert torch.equal(loss0, loss1)
    for g0, g1 in zip(grads0, grads1):
        assert torch.equal(g0, g1)


@pytest.mark.parametrize("fuse", [True, False])
def test_a_graph_compiler_steps_around_the_fp8_modules(amp, fuse):
    """The reference can wrap the model in torch.compile (model_transforms/compile.py).  The FP8 modules call the
    native library and are marked so that the tracer leaves them alone: traced with the plain "eager" backend
    (no code generation) the model gives the same bits as without the tracer, forward and backward."""
    import torch._dynamo

    from optimus_dl_amd.modules.model import Llama, LlamaConfig
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(0)
    m = Llama(LlamaConfig(vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=128, intermediate_size=256)).cuda()
    build_model_transform({"_name": "fp8_linear", "replace_norm": fuse, "fuse_swiglu": fuse}).apply(m)
    ids = torch.randint(0, 256, (4, 64), generator=torch.Generator().manual_seed(2)).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")

    def run(model):
        for p in m.parameters():
            p.grad = None
        with amp.fp8_autocast(torch.device("cuda"), recipe):
            logits = model(ids)["logits"].float()
            loss = F.cross_entropy(logits.reshape(-1, 256), ids.reshape(-1))
        with amp.fp8_backward(recipe):
            loss.backward()
        return loss.detach(), [p.grad.detach().clone() for p in m.parameters()]

    before = sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls"))
    loss0, grads0 = run(m)
    plain_calls = sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls")) - before
    torch._dynamo.reset()
    compiled = torch.compile(m, backend="eager")
    loss1, grads1 = run(compiled)
    assert sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls")) - before == 2 * plain_calls
    assert torch.equal(loss0, loss1)
    for g0, g1 in zip(grads0, grads1):
        assert torch.equal(g0, g1)
    torch._dynamo.reset()


@pytest.mark.parametrize("fuse", [True, False])
def test_inference_mode_forward_equals_the_no_grad_forward(amp, fuse):
    """Tensors made under torch.inference_mode keep no version counter, which the hand-over caches key on:
    they must simply miss (every Linear quantises its own input) and the outputs stay the same bits."""
    from optimus_dl_amd.modules.model import Llama, LlamaConfig
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    torch.manual_seed(0)
    m = Llama(LlamaConfig(vocab_size=256, n_layer=2, n_head=4, n_kv_head=2, n_embd=128, intermediate_size=256)).cuda().eval()
    build_model_transform({"_name": "fp8_linear", "replace_norm": fuse, "fuse_swiglu": fuse}).apply(m)
    ids = torch.randint(0, 256, (4, 64), generator=torch.Generator().manual_seed(2)).cuda()
    recipe = amp.FP8Recipe(recipe_type="tensorwise")
    before = sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls"))
    with torch.no_grad(), amp.fp8_autocast(torch.device("cuda"), recipe):
        want = m(ids)["logits"]
    with torch.inference_mode(), amp.fp8_autocast(torch.device("cuda"), recipe):
        got = m(ids)["logits"]
    assert sum(mod.fp8_calls for mod in m.modules() if hasattr(mod, "fp8_calls")) - before == 2 * 15
    assert torch.equal(got, want)
