"""GPU parity at the full sizes of the benchmark configurations, through properties that do not need the
whole answer on the CPU:

  * a random sample of output rows x columns against the oracle's emulated matmul
    (the sample's operands are copied to the CPU; tolerance 1e-2 as for every GEMM);
  * every kernel variant that takes the shape produces the same bits (the accumulation
    order over K is the same in all of them), and C(a, b)^T == C(b, a) bit for bit;
  * doubling a scale doubles every output exactly (power of two);
  * casts: the transposed copy is the transpose of the row-major copy, a sample of rows
    matches the oracle bit for bit, amax equals the maximum of block maxima.

Inputs are drawn on the GPU (seeded) and are what the benchmark definition describes: N(0,1) activations,
N(0,0.02) weights, N(0,1e-3) gradients.
"""
import pytest
import torch

from oracle import oracle as O
from tests.helpers import assert_bytes_equal, assert_f32_bits_equal, max_rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def N():
    from optimus_dl_amd import native

    native.load()
    yield native
    native.gemm_set_variant(-1)


def draw(shape, std, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * std).bfloat16()


def quantise(N, x, fmt):
    amax, scale, scale_inv = N.amax_scale(x, fmt)
    q, q_t = N.cast_transpose(x, scale, fmt)
    return q, q_t, scale, scale_inv, amax


def sample_check(out, aq, bq, fa, fb, sa_inv, sb_inv, seed, what, rows=48, cols=640):
    """out[M,N] (GPU) against the oracle on a random rows x cols sample."""
    M, Nn = out.shape
    g = torch.Generator().manual_seed(seed)
    ri = torch.randperm(M, generator=g)[:rows].sort().values
    ci = torch.randperm(Nn, generator=g)[:cols].sort().values
    a_s, b_s = aq[ri.cuda()].cpu(), bq[ci.cuda()].cpu()
    sa = sa_inv.cpu() if sa_inv.numel() == 1 else sa_inv[ri.cuda()].cpu()
    sb = sb_inv.cpu() if sb_inv.numel() == 1 else sb_inv[ci.cuda()].cpu()
    ref = O.t_gemm_nt(a_s, b_s, fa, fb, sa, sb)
    got = out[ri.cuda()][:, ci.cuda()]
    err = max_rel_err(got, ref)
    assert err <= TOL, f"{what}: max rel err {err} on a {rows}x{cols} sample"


# (M, N, K) of the GEMMs that the benchmark configurations launch
CFG_SHAPES = [
    pytest.param(8192, 14336, 4096, id="cfg3-fwd-gate"),
    pytest.param(8192, 4096, 14336, id="cfg3-fwd-down"),
    pytest.param(14336, 4096, 8192, id="cfg3-wgrad-gate"),
    pytest.param(8192, 1024, 4096, id="cfg2-fwd-wk"),
    pytest.param(8192, 28672, 8192, id="cfg5-fwd-up"),
    pytest.param(8192, 8192, 28672, id="cfg5-fwd-down"),
]


@pytest.mark.parametrize("M,Nn,K", CFG_SHAPES)
def test_gemm_at_baseline_shapes(N, M, Nn, K):
    a = draw((M, K), 1e-3, 1)            # plays dY (E5M2) against a weight-like operand (E4M3)
    b = draw((Nn, K), 0.02, 2)
    aq, _, _, sa_inv, _ = quantise(N, a, O.E5M2)
    bq, _, _, sb_inv, _ = quantise(N, b, O.E4M3)
    del a, b
    N.gemm_set_variant(-1)
    out = N.gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv)
    sample_check(out, aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv, seed=M + Nn, what=f"auto {M}x{Nn}x{K}")
    # the same bits from every variant that keeps the K order (all tiled kernels do)
    names = N.gemm_variants()
    for v in range(2, len(names)):
        if "one tile per block" in names[v]:
            continue
        N.gemm_set_variant(v)
        other = N.gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv)
        assert torch.equal(out, other), f"variant {v} ({names[v]}) differs from the automatic choice"
    N.gemm_set_variant(-1)
    # operands swapped: the transpose, bit for bit
    swapped = N.gemm_nt(bq, aq, O.E4M3, O.E5M2, sb_inv, sa_inv)
    assert torch.equal(swapped.t(), out)
    # a scale doubled: every output doubled (exact in bf16 away from overflow)
    doubled = N.gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv * 2, sb_inv)
    assert torch.equal(doubled.float(), out.float() * 2)


def test_rowwise_gemm_at_config_4_shape_with_outlier_channels(N):
    M, Nn, K = 16384, 14336, 4096
    x = draw((M, K), 1.0, 3)
    g = torch.Generator().manual_seed(4)
    channels = torch.randperm(K, generator=g)[:4]
    x[:, channels.cuda()] *= 100.0
    w = draw((Nn, K), 0.02, 5)
    ax, aw = N.amax(x, O.SCALE_ROW), N.amax(w, O.SCALE_ROW)
    # per-row amax: torch on the GPU as an independent check of the reduction at this size
    assert torch.equal(ax, x.float().abs().amax(dim=1)) and torch.equal(aw, w.float().abs().amax(dim=1))
    sx, sx_inv = N.scale_from_amax(ax, O.E4M3)
    sw, sw_inv = N.scale_from_amax(aw, O.E4M3)
    xq, wq = N.cast(x, sx, O.E4M3, O.SCALE_ROW), N.cast(w, sw, O.E4M3, O.SCALE_ROW)
    rows = torch.tensor([0, 1, 4095, 8191, 16383])
    assert_bytes_equal(xq[rows.cuda()], O.t_cast(x[rows.cuda()].cpu(), sx[rows.cuda()].cpu(), O.E4M3, O.SCALE_ROW), "rowwise codes")
    out = N.gemm_nt(xq, wq, O.E4M3, O.E4M3, sx_inv, sw_inv)
    sample_check(out, xq, wq, O.E4M3, O.E4M3, sx_inv, sw_inv, seed=7, what="config 4 forward")
    # row isolation: scaling one row of X by 2^3 changes only that row's scale, no code, and only that output row
    x2 = x.clone()
    x2[123] *= 8.0
    ax2 = N.amax(x2, O.SCALE_ROW)
    sx2, sx2_inv = N.scale_from_amax(ax2, O.E4M3)
    xq2 = N.cast(x2, sx2, O.E4M3, O.SCALE_ROW)
    assert torch.equal(xq2, xq)
    assert sx2[123].item() == sx[123].item() / 8 and torch.equal(sx2[:123], sx[:123]) and torch.equal(sx2[124:], sx[124:])


def test_rowwise_backward_at_config_4_shape(N):
    """dgrad and wgrad of configuration 4 at its full size.  Each operand is scaled along its non-contracted axis
    from the bf16 source: dY per row (dgrad) and per column, transposed (wgrad), W per input channel, X per channel.
    Vectors of maxima against torch's reductions, sampled rows / columns of the codes bit for bit against the oracle's
    cast, sampled outputs against the oracle's emulated matmul, and the module's backward equal to the direct calls."""
    M, Nn, K = 16384, 14336, 4096
    x = draw((M, K), 1.0, 3)
    g = torch.Generator().manual_seed(4)
    channels = torch.randperm(K, generator=g)[:4]
    x[:, channels.cuda()] *= 100.0
    w = draw((Nn, K), 0.02, 5)
    dy = draw((M, Nn), 1e-3, 6)
    fb, ff = O.E5M2, O.E4M3

    def check_rowcol(t, fmt, what, seed):
        q, s_row_inv, q_t, s_col_inv, a_row, a_col = N.quantize_rowcol(t, fmt)
        assert torch.equal(a_row, t.float().abs().amax(dim=1)) and torch.equal(a_col, t.float().abs().amax(dim=0)), what
        s_row, s_col = O.t_scale(a_row.cpu(), fmt), O.t_scale(a_col.cpu(), fmt)
        assert_f32_bits_equal(s_row_inv, 1.0 / s_row, f"{what}: 1/scale per row")
        assert_f32_bits_equal(s_col_inv, 1.0 / s_col, f"{what}: 1/scale per column")
        gen = torch.Generator().manual_seed(seed)
        ri = torch.cat([torch.tensor([0, t.shape[0] - 1]), torch.randperm(t.shape[0], generator=gen)[:6]])
        ci = torch.cat([torch.tensor([0, t.shape[1] - 1]), torch.randperm(t.shape[1], generator=gen)[:6]])
        assert_bytes_equal(q[ri.cuda()], O.t_cast(t[ri.cuda()].cpu(), s_row[ri], fmt, O.SCALE_ROW), f"{what}: codes scaled per row")
        want_t = O.t_cast(t[:, ci.cuda()].cpu(), s_col[ci], fmt, O.SCALE_COL).t().contiguous()
        assert_bytes_equal(q_t[ci.cuda()], want_t, f"{what}: transposed codes scaled per column")
        return q, s_row_inv, q_t, s_col_inv

    gq, sg_inv, gq_t, sg_inv_t = check_rowcol(dy, fb, "dY", 21)
    _, _, wq_t, sw_inv_t = check_rowcol(w, ff, "W", 22)
    _, _, xq_t, sx_inv_t = check_rowcol(x, ff, "X", 23)
    # the outlier channels are isolated by the per-channel scales of X: every other channel keeps its own range
    plain = torch.ones(K, dtype=torch.bool)
    plain[channels] = False
    assert (1.0 / sx_inv_t.cpu()[plain]).min() > 20 * (1.0 / sx_inv_t.cpu()[channels]).max()
    N.gemm_set_variant(-1)
    dx = N.gemm_nt(gq, wq_t, fb, ff, sg_inv, sw_inv_t)                       # [M, K] = dY . W
    sample_check(dx, gq, wq_t, fb, ff, sg_inv, sw_inv_t, seed=31, what="config 4 dgrad")
    dw = N.gemm_nt(gq_t, xq_t, fb, ff, sg_inv_t, sx_inv_t)                   # [N, K] = dY^T . X
    sample_check(dw, gq_t, xq_t, fb, ff, sg_inv_t, sx_inv_t, seed=32, what="config 4 wgrad")
    del gq, gq_t, wq_t, xq_t
    # the module's backward under the rowwise recipe gives these very bits
    from optimus_dl_amd.modules.amp import create_fp8_recipe
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    lin = FP8Linear(K, Nn, bias=False, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    recipe = create_fp8_recipe("rowwise", "hybrid")
    xr = x.requires_grad_(True)
    with recipe.autocast():
        y = lin(xr)
    with recipe.backward():
        y.backward(dy)
    assert torch.equal(xr.grad, dx), "module dgrad differs from the direct calls"
    assert torch.equal(lin.weight.grad, dw), "module wgrad differs from the direct calls"


@pytest.mark.parametrize("shape,std,fmt", [((8192, 4096), 1.0, O.E4M3), ((14336, 4096), 0.02, O.E4M3),
                                           ((8192, 14336), 1e-3, O.E5M2), ((8192, 28672), 1e-3, O.E5M2)])
def test_quantisation_at_baseline_shapes(N, shape, std, fmt):
    x = draw(shape, std, 11)
    q, q_t, scale, scale_inv, amax = quantise(N, x, fmt)
    # amax: the maximum of block maxima (order does not matter for a max), and torch's own reduction
    blocks = torch.stack([N.amax(x[i:i + 1024]) for i in range(0, shape[0], 1024)])
    assert_f32_bits_equal(amax, blocks.max().reshape(1), "amax = max of block amaxes")
    assert_f32_bits_equal(amax, x.float().abs().max().reshape(1), "amax vs torch")
    want_scale = torch.tensor([O.c_scale(float(amax), fmt, 0, 1.0)])
    assert_f32_bits_equal(scale, want_scale, "scale")
    assert_f32_bits_equal(scale_inv, torch.tensor([O.c_scale_inv(float(want_scale))]), "1/scale")
    # transposed copy == transpose of the row-major copy; cast alone gives the same codes
    assert torch.equal(q_t, q.t().contiguous())
    assert torch.equal(N.cast(x, scale, fmt), q)
    # a sample of rows against the oracle, bit for bit
    rows = torch.tensor([0, 7, 1023, shape[0] // 2, shape[0] - 1])
    assert_bytes_equal(q[rows.cuda()], O.t_cast(x[rows.cuda()].cpu(), scale.cpu(), fmt), "codes of sampled rows")
    # idempotence: decoding (fp32) and re-quantising with the same scale gives the same codes
    again = N.cast((O.t_decode(q[rows.cuda()].cpu(), fmt) / scale.cpu()).cuda(), scale, fmt)
    assert_bytes_equal(again, q[rows.cuda()], "requantised codes")


def test_delayed_scaling_config_5_twenty_steps_at_full_size(N):
    """Llama-3-70B MLP shapes, history 16, 20 steps, input std 1.0 -> 1.5: after every step the
    histories and scales on the GPU equal the oracle's ring-buffer simulation fed with the amaxes
    of that step's tensors (torch reductions on the GPU supply them), bit for bit; the outputs of
    two steps are checked on a sample against the oracle's matmul with the STALE scales."""
    from optimus_dl_amd.modules import amp
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    M, K, F, H, STEPS = 8192, 8192, 28672, 16, 20
    recipe = amp.create_fp8_recipe("delayed", "hybrid", amax_history_len=H)
    up = FP8Linear(K, F, bias=False, device="cuda", dtype=torch.bfloat16)
    down = FP8Linear(F, K, bias=False, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        up.weight.copy_(draw((F, K), 0.01, 21))
        down.weight.copy_(draw((K, F), 0.01, 22))
    sim = {("up", "fwd"): O.DelayedState([O.E4M3] * 3, H), ("up", "bwd"): O.DelayedState([O.E5M2] * 2, H),
           ("down", "fwd"): O.DelayedState([O.E4M3] * 3, H), ("down", "bwd"): O.DelayedState([O.E5M2] * 2, H)}
    amax = lambda t: t.detach().float().abs().max().item()
    for step in range(STEPS):
        std = 1.0 + 0.5 * step / (STEPS - 1)
        x = draw((M, K), std, 100 + step).requires_grad_(True)
        dy = draw((M, K), 1e-3, 200 + step)
        stale_x, stale_w = sim[("up", "fwd")].scale[0], sim[("up", "fwd")].scale[1]
        with recipe.autocast():
            h = up(x)
            y = down(h)
        h.retain_grad()
        with recipe.backward():
            y.backward(dy)
        sim[("up", "fwd")].record(0, amax(x)); sim[("up", "fwd")].record(1, amax(up.weight))
        sim[("down", "fwd")].record(0, amax(h)); sim[("down", "fwd")].record(1, amax(down.weight))
        sim[("down", "bwd")].record(0, amax(dy)); sim[("up", "bwd")].record(0, amax(h.grad))
        for s in sim.values():
            s.update()
        for name, lin in (("up", up), ("down", down)):
            for direction, key in (("fwd", "scaling_fwd"), ("bwd", "scaling_bwd")):
                meta, want = lin.fp8_meta[key], sim[(name, direction)]
                assert_f32_bits_equal(meta.amax_history, torch.from_numpy(want.history), f"{name} {direction} history, step {step}")
                assert_f32_bits_equal(meta.scale, torch.from_numpy(want.scale), f"{name} {direction} scale, step {step}")
                assert_f32_bits_equal(meta.scale_inv, torch.from_numpy(want.scale_inv), f"{name} {direction} 1/scale, step {step}")
        if step in (1, STEPS - 1):
            # h = Q(x; stale scale) . Q(W_up; stale scale)^T on a sample
            sx, sw = torch.tensor([stale_x]), torch.tensor([stale_w])
            g = torch.Generator().manual_seed(step)
            ri, ci = torch.randperm(M, generator=g)[:32].sort().values, torch.randperm(F, generator=g)[:512].sort().values
            xq = O.t_cast(x.detach()[ri.cuda()].cpu(), sx, O.E4M3)
            wq = O.t_cast(up.weight.detach()[ci.cuda()].cpu(), sw, O.E4M3)
            ref = O.t_gemm_nt(xq, wq, O.E4M3, O.E4M3, 1.0 / sx, 1.0 / sw)
            err = max_rel_err(h.detach()[ri.cuda()][:, ci.cuda()], ref)
            assert err <= TOL, f"step {step}: h vs oracle with stale scales: {err}"
    # after 20 steps the 16-deep window has forgotten steps 0..3: the input scale is set by the last 16 amaxes only
    hist = up.fp8_meta["scaling_fwd"].amax_history[:, 0]
    assert int((hist > 0).sum()) == H - 1 and hist[0].item() == 0.0


def test_config_1_gpt2_up_projection_forward_against_the_cpu_path(N):
    """The one configuration the CPU emulation runs in full: X [4096, 768] ~N(0,1), W [3072, 768] ~N(0,0.02),
    per-tensor E4M3, bf16 out [4096, 3072].  Codes and scales bit for bit, the output within 1e-2."""
    from tests.helpers import seeded_bf16

    x, w = seeded_bf16((4096, 768), 1.0, 0), seeded_bf16((3072, 768), 0.02, 1)
    sx, sw = O.t_scale(O.t_amax(x), O.E4M3), O.t_scale(O.t_amax(w), O.E4M3)
    xq_ref, wq_ref = O.t_cast(x, sx, O.E4M3), O.t_cast(w, sw, O.E4M3)
    ref = O.t_gemm_nt(xq_ref, wq_ref, O.E4M3, O.E4M3, 1.0 / sx, 1.0 / sw)
    xq, _, ax, s_x, sxi = N.quantize_dynamic(x.cuda(), O.E4M3, want_transposed=False)
    wq, _, aw, s_w, swi = N.quantize_dynamic(w.cuda(), O.E4M3, want_transposed=False)
    assert_bytes_equal(xq, xq_ref, "x codes")
    assert_bytes_equal(wq, wq_ref, "w codes")
    assert_f32_bits_equal(torch.cat([s_x, s_w]), torch.cat([sx.reshape(1), sw.reshape(1)]), "scales")
    y = N.gemm_nt(xq, wq, O.E4M3, O.E4M3, sxi, swi)
    assert y.shape == (4096, 3072) and y.dtype == torch.bfloat16
    err = max_rel_err(y, ref)
    assert err <= TOL, f"config 1 forward: {err}"
    # and through the module, as a user would run it
    from optimus_dl_amd.modules import amp
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    lin = FP8Linear(768, 3072, bias=False, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
        with amp.create_fp8_recipe("tensorwise", "e4m3").autocast():
            y2 = lin(x.cuda().reshape(4, 1024, 768))
    assert torch.equal(y2.reshape(4096, 3072), y)


def test_config_2_attention_projections_forward_backward(N):
    """Wq, Wk, Wv, Wo of Llama-3-8B at M = 8192 through FP8Linear: the three projections that share X quantise
    it once; outputs and gradients on a sample against the oracle's matmul of the same codes."""
    from optimus_dl_amd import native
    from optimus_dl_amd.modules import amp
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    M, K = 8192, 4096
    recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
    x = draw((M, K), 1.0, 51).requires_grad_(True)
    outs = {}
    lins = {name: FP8Linear(K, n, bias=False, device="cuda", dtype=torch.bfloat16) for name, n in
            (("wq", 4096), ("wk", 1024), ("wv", 1024))}
    for i, lin in enumerate(lins.values()):
        with torch.no_grad():
            lin.weight.copy_(draw(tuple(lin.weight.shape), 0.02, 60 + i))
    with recipe.autocast():
        for name, lin in lins.items():
            outs[name] = lin(x)
    with recipe.backward():
        torch.autograd.backward(list(outs.values()), [draw(tuple(o.shape), 1e-3, 70 + i) for i, o in enumerate(outs.values())])
    xq, xq_t, _, sx, sxi = native.quantize_dynamic(x.detach(), O.E4M3)
    for name, lin in lins.items():
        wq, _, _, sw, swi = native.quantize_dynamic(lin.weight.detach(), O.E4M3, want_transposed=False)
        sample_check(outs[name].detach(), xq, wq, O.E4M3, O.E4M3, sxi, swi, seed=80, what=f"{name} forward", cols=256)
        assert lin.weight.grad is not None and lin.weight.grad.shape == lin.weight.shape
    assert x.grad is not None and torch.isfinite(x.grad.float()).all()
    # dW of wk against the oracle on a sample: dW = Q(dY)^T . Q(X)
    dy_k = draw((M, 1024), 1e-3, 71)
    gq, gq_t, _, sg, sgi = native.quantize_dynamic(dy_k, O.E5M2)
    sample_check(lins["wk"].weight.grad, gq_t, xq_t, O.E5M2, O.E4M3, sgi, sxi, seed=81, what="wk wgrad", cols=256)


# The transform swaps EVERY nn.Linear, the output head included (transformer_engine.py:501-513):
# vocabulary-sized N that is not a multiple of the big tiles (GPT-2 50304, Qwen3-0.6B 151936).
@pytest.mark.parametrize("M,K,V", [pytest.param(2048, 768, 50304, id="gpt2-lm_head"),
                                   pytest.param(1024, 1024, 151936, id="qwen3-0.6b-lm_head")])
def test_lm_head_shapes_forward_backward(N, M, K, V):
    from optimus_dl_amd.modules import amp as A
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    x, w, dy = draw((M, K), 1.0, 11), draw((V, K), 0.02, 12), draw((M, V), 1e-3, 13)
    lin = torch.nn.Linear(K, V, bias=False, device="cuda", dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    lin = FP8Linear.from_linear(lin)
    recipe = A.FP8Recipe(recipe_type="tensorwise")
    xd = x.clone().requires_grad_(True)
    with recipe.autocast():
        y = lin(xd)
    with recipe.backward():
        y.backward(dy)
    assert lin.fp8_calls == 1
    xq, xq_t, _, sx_inv, _ = quantise(N, x, O.E4M3)
    wq, wq_t, _, sw_inv, _ = quantise(N, w, O.E4M3)
    gq, gq_t, _, sg_inv, _ = quantise(N, dy, O.E5M2)
    sample_check(y.detach(), xq, wq, O.E4M3, O.E4M3, sx_inv, sw_inv, seed=V, what="lm_head fwd")
    sample_check(xd.grad, gq, wq_t, O.E5M2, O.E4M3, sg_inv, sw_inv, seed=V + 1, what="lm_head dgrad", cols=min(640, K))
    sample_check(lin.weight.grad, gq_t, xq_t, O.E5M2, O.E4M3, sg_inv, sx_inv, seed=V + 2, what="lm_head wgrad", cols=min(640, K))
    # the vocabulary ends half way through a 256-wide tile: the last 384 entries on their own
    tail = slice(V - 384, V)
    sample_check(y.detach()[:, tail].contiguous(), xq, wq[tail], O.E4M3, O.E4M3, sx_inv, sw_inv, seed=V + 3,
                 what="lm_head fwd, last columns", cols=384)
    sample_check(lin.weight.grad[tail], gq_t[tail], xq_t, O.E5M2, O.E4M3, sg_inv, sx_inv, seed=V + 4,
                 what="lm_head wgrad, last rows", cols=min(640, K))


def test_fused_producers_at_config_3_size(N):
    """SwiGLU forward / backward on the [8192, 14336] activations and RMSNorm on [8192, 4096]: a sample of
    rows against the oracle bit for bit (both are row-local), the partial maxima against the whole output."""
    M, H, C = 8192, 14336, 4096
    g, u, dh = draw((M, H), 1.5, 21), draw((M, H), 1.0, 22), draw((M, H), 1e-3, 23)
    h, parts = N.swiglu_amax_parts(g, u)
    dg, du, pg, pu = N.swiglu_bwd_amax_parts(dh, g, u)
    ri = torch.randperm(M, generator=torch.Generator().manual_seed(5))[:24].sort().values.cuda()
    gs, us, ds = g[ri].cpu(), u[ri].cpu(), dh[ri].cpu()
    assert torch.equal(h[ri].cpu().view(torch.int16), O.c_swiglu_fwd(gs, us).view(torch.int16))
    wg, wu = O.c_swiglu_bwd(ds, gs, us)
    assert torch.equal(dg[ri].cpu().view(torch.int16), wg.view(torch.int16))
    assert torch.equal(du[ri].cpu().view(torch.int16), wu.view(torch.int16))
    for t, p, what in ((h, parts, "h"), (dg, pg, "d_gate"), (du, pu, "d_up")):
        assert_f32_bits_equal(p.max().reshape(1), t.float().abs().max().reshape(1), f"partial maxima of {what}")
    # the cast fed by the producer's maxima equals the two-launch quantisation of the same tensor
    q, q_t, amax, scale, _ = N.cast_dynamic(h, parts, O.E4M3, 0)
    q2, q2_t, amax2, scale2, _ = N.quantize_dynamic(h, O.E4M3, 0)
    assert torch.equal(q, q2) and torch.equal(q_t, q2_t) and torch.equal(scale, scale2)
    del g, u, dh, h, dg, du, q, q_t, q2, q2_t
    for dtype in (torch.bfloat16, torch.float32):
        x = draw((M, C), 2.0, 31).to(dtype)
        w = torch.linspace(0.5, 1.5, C, device="cuda")
        y, rstd, parts = N.rmsnorm_amax_parts(x, w, 1e-5)
        dy = draw((M, C), 1e-2, 32)
        dx, dw = N.rmsnorm_bwd(dy, x, w, rstd)
        xs = x[ri].cpu()
        wy, wr = O.c_rmsnorm(xs, w.cpu(), 1e-5)
        assert torch.equal(y[ri].cpu().view(torch.int16), wy.view(torch.int16))
        assert_f32_bits_equal(rstd[ri], wr, "rstd")
        assert_f32_bits_equal(parts.max().reshape(1), y.float().abs().max().reshape(1), "partial maxima of y")
        wdx, _ = O.c_rmsnorm_bwd(dy[ri].cpu(), xs, w.cpu(), wr)
        if dtype == torch.bfloat16:
            assert torch.equal(dx[ri].cpu().view(torch.int16), wdx.view(torch.int16))
        else:
            assert_f32_bits_equal(dx[ri], wdx, "dx")
        want_dw = (dy.double() * (x.double() * rstd.double()[:, None])).sum(0)
        assert ((dw.double() - want_dw).abs().max() / want_dw.abs().max()).item() < 1e-5


@pytest.mark.parametrize("M,Nn,K,la,lb", [pytest.param(14336, 4096, 8192, 1, 1, id="cfg3-wgrad-gate"),
                                          pytest.param(8192, 4096, 14336, 0, 1, id="cfg3-dgrad-gate"),
                                          pytest.param(4096, 14336, 8192, 1, 1, id="cfg3-wgrad-down"),
                                          pytest.param(8192, 8192, 28672, 0, 1, id="cfg5-dgrad-up")])
def test_k_slow_layouts_at_baseline_shapes(N, M, Nn, K, la, lb):
    """dgrad / wgrad reading row-major codes (contraction index slow) against the same kernel on transposed copies."""
    a = draw((M, K), 1e-3, 41)
    b = draw((Nn, K), 1.0, 42)
    aq, aq_t, _, sa_inv, _ = quantise(N, a, O.E5M2)
    bq, bq_t, _, sb_inv, _ = quantise(N, b, O.E4M3)
    del a, b
    ref = N.gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv)
    out = N.gemm_layouts(aq_t if la else aq, bq_t if lb else bq, O.E5M2, O.E4M3, la, lb, sa_inv, sb_inv)
    assert torch.equal(out, ref)
    sample_check(out, aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv, seed=M + K, what=f"k-slow {M}x{Nn}x{K}")


def test_fp32_weight_gradient_at_the_baseline_shape(N):
    """wgrad of the gate projection (config 3) with fp32 output, dY read as stored: rounding it to bf16 gives the
    bf16 output of the same launch bit for bit, and a sample agrees with the oracle."""
    M, Nn, K = 14336, 4096, 8192
    aq, aq_t, _, sa_inv, _ = quantise(N, draw((M, K), 1e-3, 51), O.E5M2)
    bq, _, _, sb_inv, _ = quantise(N, draw((Nn, K), 1.0, 52), O.E4M3)
    out32 = N.gemm_layouts(aq_t, bq, O.E5M2, O.E4M3, N.K_SLOW, N.K_FAST, sa_inv, sb_inv, out_dtype=torch.float32)
    out16 = N.gemm_layouts(aq_t, bq, O.E5M2, O.E4M3, N.K_SLOW, N.K_FAST, sa_inv, sb_inv)
    assert out32.dtype == torch.float32 and torch.equal(out32.bfloat16(), out16)
    sample_check(out32, aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv, seed=7, what="fp32 wgrad 14336x4096x8192")


@pytest.mark.parametrize("M,Nn,K,kernel", [pytest.param(16384, 1024, 151936, "tiled", id="2.5GB-operand"),
                                           pytest.param(32768, 256, 151936, "generic", id="5GB-operand")])
def test_operands_beyond_the_32_bit_offset_limits(N, M, Nn, K, kernel):
    """The input gradient of a vocabulary-sized head at many tokens: dY codes of 2.5 GB (beyond the 2 GiB that the
    streaming and the pipelined kernel address: the tiled kernels take it) and of 5 GB (beyond 4 GiB: only the generic
    kernel, with 64-bit addressing, does).  The automatic choice must pick a kernel that can address the operand; a
    sample of the output against the oracle, the last rows included (highest addresses)."""
    g = torch.Generator(device="cuda").manual_seed(M + K)
    aq = torch.randint(0, 256, (M, K), generator=g, device="cuda", dtype=torch.uint8)
    aq[(aq & 0x7F) > 0x7B] = 0                          # no E5M2 Inf / NaN codes
    bq = torch.randint(0, 256, (Nn, K), generator=g, device="cuda", dtype=torch.uint8)
    bq[(bq & 0x7F) == 0x7F] = 0                         # no E4M3 NaN codes
    sa_inv, sb_inv = torch.tensor([2.0 ** -12], device="cuda"), torch.tensor([2.0 ** -6], device="cuda")
    assert N.gemm_split_count(M, Nn, K) == 1            # the K split rides on the streaming kernel: not for these
    out = N.gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv)
    sample_check(out, aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv, seed=K, what=f"{kernel} kernel, {M}x{Nn}x{K}", rows=24, cols=128)
    tail = out[M - 64:].contiguous()
    sample_check(tail, aq[M - 64:], bq, O.E5M2, O.E4M3, sa_inv, sb_inv, seed=K + 1, what=f"{kernel} kernel, last rows", rows=16, cols=128)


def test_quantisation_of_a_tensor_with_more_than_2_31_elements(N):
    """The logits gradient of a vocabulary-sized head at 16384 tokens: 2.49e9 elements (5 GB of bf16).  amax, cast and
    cast+transpose index with 64 bits: the maximum planted in the last row is found, rows from both ends of the tensor
    have the oracle's codes, and the transposed copy is the transpose."""
    M, V = 16384, 151936
    x = draw((M, V), 1e-3, 77)
    x[M - 1, V - 3] = -0.75                             # the maximum sits behind element 2^31
    parts = N.amax_parts(x)
    q, q_t, amax, scale, _ = N.cast_dynamic(x, parts, O.E5M2, 0, want_rowmajor=True, want_transposed=True)
    assert amax.item() == 0.75 and scale.item() == O.t_scale(torch.tensor([0.75]), O.E5M2).item()
    rows = torch.tensor([0, 1, 8191, 8192, M - 2, M - 1])
    want = O.t_cast(x[rows.cuda()].cpu(), scale.cpu(), O.E5M2)
    assert_bytes_equal(q[rows.cuda()], want, "codes of rows from both ends")
    assert_bytes_equal(q_t[:, rows.cuda()], want.t(), "the same rows in the transposed copy")
    cols = torch.tensor([0, 77, V - 1]).cuda()
    assert torch.equal(q_t[cols], q[:, cols].t())


# ------------------------------------------------------------------------------------------- block-scaled recipes
def _sampled_block_product(out, aq, asb, bq, bsb, fa, fb, seed, what, rows=48, cols=640):
    """out[M, N] against the emulated block-scaled product on a random rows x cols sample; asb / bsb are the scale bytes
    as [rows, K / 32]."""
    M, Nn = out.shape
    g = torch.Generator().manual_seed(seed)
    ri = torch.randperm(M, generator=g)[:rows].sort().values.cuda()
    ci = torch.randperm(Nn, generator=g)[:cols].sort().values.cuda()
    ref = O.t_mx_gemm_nt(aq[ri].cpu(), asb[ri].cpu(), bq[ci].cpu(), bsb[ci].cpu(), fa, fb)
    err = max_rel_err(out[ri][:, ci], ref)
    assert err <= TOL, f"{what}: max rel err {err} on a {rows}x{cols} sample"


@pytest.mark.parametrize("M,Nn,K", [pytest.param(8192, 14336, 4096, id="cfg3-fwd-gate"), pytest.param(8192, 4096, 14336, id="cfg3-dgrad-gate"),
                                    pytest.param(14336, 4096, 8192, id="cfg3-wgrad-gate")])
@pytest.mark.parametrize("recipe", ["mxfp8", "blockwise"])
def test_block_scaled_gemm_at_baseline_shapes(N, M, Nn, K, recipe):
    a = draw((M, K), 1e-3, 11)           # plays dY (E5M2) against a weight-like operand (E4M3)
    b = draw((Nn, K), 0.02, 12)
    if recipe == "mxfp8":
        aq, asc, _, _ = N.mx_cast(a, O.E5M2, True, False)
        bq, bsc, _, _ = N.mx_cast(b, O.E4M3, True, False)
    else:
        aq, asc, _, _ = N.block_cast(a, O.E5M2, 0, False, True, False)
        bq, bsc, _, _ = N.block_cast(b, O.E4M3, 0, True, True, False)
    # the casts themselves on sampled rows: bit-exact against the oracle (a row's blocks depend on that row only,
    # except for the 128 x 128 weight blocks, which are checked on whole row blocks)
    g = torch.Generator().manual_seed(M + K)
    ri = torch.randperm(M, generator=g)[:64].sort().values
    a_rows = a[ri.cuda()].cpu()
    asb = N.mx_scales_rowmajor(asc)
    if recipe == "mxfp8":
        wc, ws = O.c_mx_quantise(a_rows, O.E5M2)
        assert torch.equal(asb[ri.cuda()].cpu(), ws), "scale bytes of sampled rows"
    else:
        wc, ws = O.c_block_quantise(a_rows, 1, 128, O.E5M2, 0)
        assert torch.equal(asb[ri.cuda()].cpu(), O.block_scales_as_mx(ws, 1, 128)), "scale bytes of sampled rows"
        blk = int(torch.randint(0, Nn // 128, (1,), generator=g))
        wcb, wsb = O.c_block_quantise(b[128 * blk:128 * (blk + 1)].cpu(), 128, 128, O.E4M3, 0)
        assert torch.equal(bq[128 * blk:128 * (blk + 1)].cpu(), wcb), "codes of a sampled row of 128 x 128 weight blocks"
        assert torch.equal(N.mx_scales_rowmajor(bsc)[128 * blk:128 * (blk + 1)].cpu(), O.block_scales_as_mx(wsb, 128, 128))
    assert torch.equal(aq[ri.cuda()].cpu(), wc), "codes of sampled rows"
    del a, b
    out = N.mx_gemm_nt(aq, asc, bq, bsc, O.E5M2, O.E4M3)
    _sampled_block_product(out, aq, asb, bq, N.mx_scales_rowmajor(bsc), O.E5M2, O.E4M3, seed=M + Nn, what=f"{recipe} {M}x{Nn}x{K}")
    # operands swapped: the transpose, bit for bit (same kernel, same K order)
    swapped = N.mx_gemm_nt(bq, bsc, aq, asc, O.E4M3, O.E5M2)
    assert torch.equal(swapped.t(), out)
    # one more on every scale byte of A: every output doubled (exact in bf16 away from overflow)
    doubled = N.mx_gemm_nt(aq, asc + 1, bq, bsc, O.E5M2, O.E4M3)
    assert torch.equal(doubled.float(), out.float() * 2)


def test_fp32_source_quantisation_at_a_weight_shape(N):
    """fp32 master weights are the reference's usual AMP set-up: every cast also takes an fp32 source.  W of the up
    projection (4096 x 14336 as stored for the down projection's input side) with genuine fp32 mantissas: per-tensor
    codes in both layouts, MXFP8 codes and scale bytes, 128 x 128 block codes, against the oracle on samples and through
    the identities that hold at any size."""
    rows_n, cols_n = 4096, 14336
    g = torch.Generator(device="cuda").manual_seed(91)
    x = torch.randn((rows_n, cols_n), generator=g, device="cuda", dtype=torch.float32) * 0.02 + 3e-5
    assert not torch.equal(x.bfloat16().float(), x)                       # not representable in bf16: the fp32 path is what runs
    q, q_t, scale, scale_inv, amax = quantise(N, x, O.E4M3)
    assert_f32_bits_equal(amax, x.abs().max().reshape(1), "amax vs torch")
    assert_f32_bits_equal(scale, torch.tensor([O.c_scale(float(amax), O.E4M3, 0, 1.0)]), "scale")
    assert torch.equal(q_t, q.t().contiguous())
    assert torch.equal(N.cast(x, scale, O.E4M3), q)
    rows = torch.tensor([0, 5, 127, 128, rows_n // 2 + 1, rows_n - 1]).cuda()
    assert_bytes_equal(q[rows], O.t_cast(x[rows].cpu(), scale.cpu(), O.E4M3), "codes of sampled rows")
    # the partial maxima + cast route gives the same codes as amax -> scale -> cast
    q2, q2_t, _, scale2, _ = N.quantize_dynamic(x, O.E4M3)
    assert torch.equal(q2, q) and torch.equal(q2_t, q_t)
    assert_f32_bits_equal(scale2, scale, "scale of the dynamic route")
    # MXFP8, both shared-exponent rules: sampled rows (blocks along the columns) and sampled columns (blocks along the rows)
    for rule in (N.MX_FLOOR, N.MX_CEIL):
        mq, ms, mq_t, ms_t = N.mx_cast(x, O.E4M3, True, True, scale_rule=rule)
        wc, ws = O.t_mx_quantise(x[rows].cpu(), O.E4M3, rule)        # (the C oracle takes bf16; its torch twin any float)
        assert_bytes_equal(mq[rows], wc, f"mx codes of sampled rows, rule {rule}")
        assert_bytes_equal(N.mx_scales_rowmajor(ms)[rows], ws, f"mx scale bytes of sampled rows, rule {rule}")
        cols = torch.tensor([0, 3, 31, 32, 4097, cols_n - 1]).cuda()
        wct, wst = O.t_mx_quantise(x[:, cols].t().contiguous().cpu(), O.E4M3, rule)
        assert_bytes_equal(mq_t[cols], wct, f"mx codes of sampled columns, rule {rule}")
        assert_bytes_equal(N.mx_scales_rowmajor(ms_t)[cols], wst, f"mx scale bytes of sampled columns, rule {rule}")
    # 128 x 128 blocks (weights of the blockwise recipe): one set of scales serves both layouts
    bq, bs, bq_t, bs_t = N.block_cast(x, O.E4M3, 0, True, True, True)
    assert torch.equal(bq_t, bq.t().contiguous())
    strip = slice(rows_n - 128, rows_n)
    wc, ws = O.t_block_quantise(x[strip].cpu(), 128, 128, O.E4M3, 0)
    assert_bytes_equal(bq[strip], wc, "block codes of the last row of tiles")
    # 1 x 128 blocks (activations): a sampled strip of rows, and of columns for the transposed codes
    aq, as_, aq_t, as_t = N.block_cast(x, O.E4M3, 0, False, True, True)
    wc, ws = O.t_block_quantise(x[rows].cpu(), 1, 128, O.E4M3, 0)
    assert_bytes_equal(aq[rows], wc, "1 x 128 block codes of sampled rows")
    wct, wst = O.t_block_quantise(x[:, cols].t().contiguous().cpu(), 1, 128, O.E4M3, 0)
    assert_bytes_equal(aq_t[cols], wct, "128 x 1 block codes of sampled columns")


def test_config_2_grouped_projections_sum_their_data_gradients_in_the_gemms(N):
    """configs[1] as BASELINE writes it: ONE X for Wq, Wk, Wv.  The transform ties the three into a group: the outputs
    and weight gradients are the bits of the separate modules, and dX comes from ONE GEMM whose contraction runs through
    the three members' operands (one rounding), or, with that switched off, from GEMMs that add into it (a rounding per
    member); both stay within the roundings that autograd's bf16 sum of three rounded products makes."""
    import torch.nn as nn

    from optimus_dl_amd import native
    from optimus_dl_amd.modules import amp
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    class Projections(nn.Module):
        def __init__(self):
            super().__init__()
            self.wq, self.wk, self.wv = nn.Linear(4096, 4096, bias=False), nn.Linear(4096, 1024, bias=False), nn.Linear(4096, 1024, bias=False)

        def forward(self, x):
            return self.wq(x), self.wk(x), self.wv(x)

    M = 8192
    net = Projections().to("cuda", torch.bfloat16)
    with torch.no_grad():
        for i, p in enumerate(net.parameters()):
            p.copy_(draw(tuple(p.shape), 0.02, 100 + i))
    t = build_model_transform({"_name": "fp8_linear"})
    t.apply(net)
    assert t.sibling_groups == 1
    dys = [draw((M, n), 1e-3, 110 + i) for i, n in enumerate((4096, 1024, 1024))]
    results = {}
    for route in ("one gemm", "accumulate", "separate"):
        recipe = amp.create_fp8_recipe("tensorwise", "hybrid")
        recipe.fuse_dgrad_sum = route != "separate"
        recipe.fuse_dgrad_gemm = route == "one gemm"
        x = draw((M, 4096), 1.0, 120).requires_grad_(True)
        for p in net.parameters():
            p.grad = None
        calls, sums = [], []
        real, real_sum = native.gemm_nt, native.gemm_nt_sum
        native.gemm_nt = lambda *a, **k: (calls.append(bool(k.get("accumulate"))), real(*a, **k))[1]
        native.gemm_nt_sum = lambda *a, **k: (sums.append(len(a[0])), real_sum(*a, **k))[1]
        try:
            with recipe.autocast():
                ys = net(x)
            with recipe.backward():
                torch.autograd.backward(ys, dys)
        finally:
            native.gemm_nt, native.gemm_nt_sum = real, real_sum
        assert (sum(calls), sums) == {"one gemm": (0, [3]), "accumulate": (2, []), "separate": (0, [])}[route], (route, calls, sums)
        results[route] = ([y.detach() for y in ys], x.grad, [p.grad for p in net.parameters()])
    for route in ("one gemm", "accumulate"):
        for a, b in zip(results[route][0] + results[route][2], results["separate"][0] + results["separate"][2]):
            assert torch.equal(a, b)
    dx_s = results["separate"][1].float()
    for route in ("one gemm", "accumulate"):
        dx_f = results[route][1].float()
        assert torch.isfinite(dx_f).all()
        # the separate route rounds each product and each of the two sums to bf16 (up to 4 half-units of the largest term)
        bound = 4 * 2.0 ** -9 * dx_s.abs().max()
        assert float((dx_f - dx_s).abs().max()) <= float(bound), route
    # and against the oracle on a sample: dX = sum of Q(dY_i) . Q(W_i^T)^T with the codes the kernels made
    ri = torch.randperm(M, generator=torch.Generator().manual_seed(5))[:32].sort().values.cuda()
    ci = torch.randperm(4096, generator=torch.Generator().manual_seed(6))[:256].sort().values.cuda()
    ref = torch.zeros((32, 256))
    for dy, lin in zip(dys, (net.wq, net.wk, net.wv)):
        gq, _, _, _, sgi = native.quantize_dynamic(dy, O.E5M2, want_transposed=False)
        _, wq_t, _, _, swi = native.quantize_dynamic(lin.weight.detach(), O.E4M3)
        ref += O.t_gemm_nt(gq[ri].cpu(), wq_t[ci].cpu(), O.E5M2, O.E4M3, sgi.cpu(), swi.cpu(), want_f32=True)[1]
    for route in ("one gemm", "accumulate"):
        got = results[route][1][ri][:, ci].float().cpu()
        assert max_rel_err(got, ref) <= TOL, route
    # the one launch rounds the fp32 sum once: closer to it than a rounding per member
    err = {route: float((results[route][1][ri][:, ci].float().cpu() - ref).abs().max()) for route in ("one gemm", "accumulate")}
    assert err["one gemm"] <= err["accumulate"] * 1.05 + 1e-12, err


def test_gate_and_up_data_gradient_in_one_launch_at_config_3_size(N):
    """dX [8192, 4096] = dY_gate . W_gate + dY_up . W_up with contractions of 14336 each (configs[2] with gate and up fed
    one X): the one-launch route against a GEMM per pair adding into fp32 on the GPU (whole matrix) and against the
    oracle on sampled rows and columns; bf16 output = one rounding of the same fp32 values."""
    M, K, F = 8192, 4096, 14336
    gq, sg = [], []
    wq, sw = [], []
    for i in range(2):
        q, _, _, _, s_inv = N.quantize_dynamic(draw((M, F), 1e-3 * (3.0 ** i), 300 + i), O.E5M2, want_transposed=False)
        gq.append(q); sg.append(s_inv)
        _, q_t, _, _, s_inv = N.quantize_dynamic(draw((F, K), 0.02 / (2.0 ** i), 310 + i), O.E4M3)
        wq.append(q_t); sw.append(s_inv)
    one = N.gemm_nt_sum(gq, wq, O.E5M2, O.E4M3, sg, sw, out_dtype=torch.float32)
    N.gemm_set_variant(5)
    try:
        seq = N.gemm_nt_sum(gq, wq, O.E5M2, O.E4M3, sg, sw, out_dtype=torch.float32)
    finally:
        N.gemm_set_variant(-1)
    assert max_rel_err(one, seq) <= 2e-5
    assert torch.equal(N.gemm_nt_sum(gq, wq, O.E5M2, O.E4M3, sg, sw), one.bfloat16())
    ri = torch.randperm(M, generator=torch.Generator().manual_seed(7))[:48].sort().values.cuda()
    ci = torch.randperm(K, generator=torch.Generator().manual_seed(8))[:192].sort().values.cuda()
    ref = O.t_gemm_nt_sum([(gq[i][ri].cpu(), wq[i][ci].cpu(), sg[i].cpu(), sw[i].cpu()) for i in range(2)], O.E5M2, O.E4M3,
                          want_f32=True)[1]
    assert max_rel_err(one[ri][:, ci].cpu(), ref) <= 2e-5
