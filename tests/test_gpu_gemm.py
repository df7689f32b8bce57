"""GPU parity: FP8 MFMA GEMM vs the emulated-FP8 matmul of the oracle.

Tolerance (stated by the task): max|out - ref| / max|ref| <= 1e-2 on the bf16
output, ref = upcast codes to fp32, fp32 matmul, times the scale product, bf16.
Cases whose partial sums are all exactly representable must be bit-exact,
whatever order the hardware accumulates in.
"""
import pytest
import torch

from oracle import oracle as O
from tests.helpers import max_rel_err, seeded_bf16

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def N():
    from optimus_dl_amd import native

    native.load()
    yield native
    native.gemm_set_variant(-1)


def quantised(shape, fmt, std, seed):
    x = seeded_bf16(shape, std=std, seed=seed)
    s = O.t_scale(O.t_amax(x), fmt)
    return O.t_cast(x, s, fmt), (1.0 / s).float()


def variants(N):
    return list(range(len(N.gemm_variants())))


def test_variant_table(N):
    names = N.gemm_variants()
    assert len(names) >= 2 and "generic" in names[0]
    print("GEMM variants:", names)


@pytest.mark.parametrize("fmts", [(O.E4M3, O.E4M3), (O.E5M2, O.E4M3), (O.E4M3, O.E5M2), (O.E5M2, O.E5M2)])
def test_power_of_two_operands_are_bit_exact_every_variant(N, fmts):
    """Operands in {0, +-1, +-2, +-0.5}: every product and partial sum is exact in
    fp32, so the result must equal the oracle bit for bit in any summation order.
    A wrong lane->row map, a wrong output layout or a wrong format selector
    (e4m3 vs e5m2 decode the same byte differently) all break this."""
    fa, fb = fmts
    M, Nn, K = 320, 288, 512
    g = torch.Generator().manual_seed(5)
    vals = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, 4.0])
    av = vals[torch.randint(0, 8, (M, K), generator=g)]
    bv = vals[torch.randint(0, 8, (Nn, K), generator=g)]
    a = av.to(O.TORCH_FP8[fa]).view(torch.uint8)
    b = bv.to(O.TORCH_FP8[fb]).view(torch.uint8)
    sa, sb = torch.tensor([0.25]), torch.tensor([2.0])
    ref16, ref32 = O.t_gemm_nt(a, b, fa, fb, sa, sb, want_f32=True)
    assert torch.equal(ref32, (av @ bv.t()) * 0.5)                                 # the oracle itself is exact here
    for v in variants(N):
        N.gemm_set_variant(v)
        out32 = N.gemm_nt(a.cuda(), b.cuda(), fa, fb, sa.cuda(), sb.cuda(), out_dtype=torch.float32)
        assert torch.equal(out32.cpu(), ref32), f"variant {v} fp32 output differs: max diff {(out32.cpu() - ref32).abs().max()}"
        out16 = N.gemm_nt(a.cuda(), b.cuda(), fa, fb, sa.cuda(), sb.cuda())
        assert torch.equal(out16.cpu().view(torch.int16), ref16.view(torch.int16)), f"variant {v} bf16 output differs"
    N.gemm_set_variant(-1)


def test_one_hot_rows_pick_single_elements(N):
    """A = rows of an identity (as FP8 1.0) selects columns of B exactly."""
    K, M, Nn = 256, 256, 192
    a = torch.zeros((M, K))
    a[torch.arange(M), (torch.arange(M) * 7) % K] = 1.0
    bq, sb_inv = quantised((Nn, K), O.E4M3, 1.0, 3)
    aq = a.to(torch.float8_e4m3fn).view(torch.uint8)
    one = torch.ones(1)
    want = O.t_decode(bq, O.E4M3)[:, (torch.arange(M) * 7) % K].t().contiguous()
    for v in variants(N):
        N.gemm_set_variant(v)
        out = N.gemm_nt(aq.cuda(), bq.cuda(), O.E4M3, O.E4M3, one.cuda(), one.cuda(), out_dtype=torch.float32)
        assert torch.equal(out.cpu(), want), f"variant {v}"
    N.gemm_set_variant(-1)


SHAPES = [
    (256, 256, 128), (512, 768, 1024), (300, 200, 256), (1024, 1024, 4096), (64, 4096, 512),
    (33, 17, 128), (257, 255, 384), (128, 130, 64), (40, 24, 48), (1, 1, 16), (520, 1032, 2048),
]


@pytest.mark.parametrize("shape", SHAPES)
def test_random_gemm_within_tolerance_auto_variant(N, shape):
    M, Nn, K = shape
    aq, sa_inv = quantised((M, K), O.E5M2, 1e-3, 1)
    bq, sb_inv = quantised((Nn, K), O.E4M3, 0.02, 2)
    ref = O.t_gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv)
    out = N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_inv.cuda(), sb_inv.cuda())
    err = max_rel_err(out, ref)
    assert err <= TOL, f"{shape}: max rel err {err}"


@pytest.mark.parametrize("k_steps", [1, 2, 3, 4, 5, 6, 7, 9, 13])
def test_few_tile_outputs_at_every_pipeline_depth(N, k_steps):
    """Outputs of at most one 128 x 128 tile per compute unit take the four-stage form of the tiled kernel: every length
    of its prologue and tail (1 .. 3 K steps in flight, a trip count that is not a multiple of four), interior and
    ragged tiles, one-hot rows so that a misplaced stage shows as a wrong element rather than as noise."""
    M, Nn, K = 384, 200, 128 * k_steps
    aq, sa_inv = quantised((M, K), O.E5M2, 1e-3, 40 + k_steps)
    bq, sb_inv = quantised((Nn, K), O.E4M3, 0.02, 60 + k_steps)
    out = N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_inv.cuda(), sb_inv.cuda())
    assert max_rel_err(out, O.t_gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv)) <= TOL
    # A = rows that are zero except for the code of 1.0 at column (7 i) mod K: out[i, j] = B[j, (7 i) mod K] exactly
    one = torch.ones(1)
    a1 = torch.zeros((M, K), dtype=torch.uint8)
    cols = (7 * torch.arange(M)) % K
    a1[torch.arange(M), cols] = 0x38                                   # 1.0 in E4M3
    b1 = O.t_cast(seeded_bf16((Nn, K), 1.0, 80 + k_steps).float(), one, O.E4M3)
    got = N.gemm_nt(a1.cuda(), b1.cuda(), O.E4M3, O.E4M3, one.cuda(), one.cuda(), out_dtype=torch.float32).cpu()
    want = O.t_decode(b1, O.E4M3)[:, cols].t()
    assert torch.equal(got, want)


@pytest.mark.parametrize("shape", [(512, 512, 1024), (300, 520, 256), (256, 256, 128)])
def test_random_gemm_every_variant_vs_c_oracle(N, shape):
    """Against the plain-C oracle (sequential fp32 accumulation)."""
    M, Nn, K = shape
    aq, sa_inv = quantised((M, K), O.E4M3, 1.0, 4)
    bq, sb_inv = quantised((Nn, K), O.E4M3, 0.02, 5)
    ref = O.c_gemm_nt(aq, bq, O.E4M3, O.E4M3, sa_inv, sb_inv)
    for v in variants(N):
        N.gemm_set_variant(v)
        out = N.gemm_nt(aq.cuda(), bq.cuda(), O.E4M3, O.E4M3, sa_inv.cuda(), sb_inv.cuda())
        err = max_rel_err(out, ref)
        assert err <= TOL, f"variant {v} {shape}: max rel err {err}"
    N.gemm_set_variant(-1)


def test_rowwise_scales_and_bias_epilogue(N):
    M, Nn, K = 384, 320, 512
    x = seeded_bf16((M, K), seed=8)
    x[:, 5] *= 100.0                                                               # an outlier channel
    w = seeded_bf16((Nn, K), std=0.02, seed=9)
    sx = O.t_scale(O.t_amax(x, O.SCALE_ROW), O.E4M3)
    sw = O.t_scale(O.t_amax(w, O.SCALE_ROW), O.E4M3)
    xq, wq = O.t_cast(x, sx, O.E4M3, O.SCALE_ROW), O.t_cast(w, sw, O.E4M3, O.SCALE_ROW)
    bias = torch.randn(Nn)
    ref32 = O.t_gemm_nt(xq, wq, O.E4M3, O.E4M3, 1 / sx, 1 / sw, want_f32=True)[1]
    ref = (ref32 + bias).bfloat16()
    for v in variants(N):
        N.gemm_set_variant(v)
        out = N.gemm_nt(xq.cuda(), wq.cuda(), O.E4M3, O.E4M3, (1 / sx).cuda(), (1 / sw).cuda(), bias=bias.cuda())
        assert max_rel_err(out, ref) <= TOL, f"variant {v}"
    N.gemm_set_variant(-1)
    # rank-1 epilogue identity: scaling row i of the inverse scales by 2 doubles row i of the output exactly
    sa2 = (1 / sx).clone()
    sa2[7] *= 2
    o1 = N.gemm_nt(xq.cuda(), wq.cuda(), O.E4M3, O.E4M3, (1 / sx).cuda(), (1 / sw).cuda(), out_dtype=torch.float32)
    o2 = N.gemm_nt(xq.cuda(), wq.cuda(), O.E4M3, O.E4M3, sa2.cuda(), (1 / sw).cuda(), out_dtype=torch.float32)
    assert torch.equal(o2[7], o1[7] * 2) and torch.equal(o2[8], o1[8])


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("which", ["tensor", "rows+cols", "rows", "cols", "rows+cols+bias", "bias"])
@pytest.mark.parametrize("shape", [(768, 512, 1024), (384, 640, 512), (128, 128, 512), (384, 256, 640), (256, 512, 1152)])
def test_streaming_kernel_scale_vectors_and_bias(N, which, out_dtype, shape):
    """Whole-tile shapes with scale vectors and / or a bias go through the streaming kernel's folded
    epilogue (vectors staged in LDS): bit-identical to the pipelined kernel's staged epilogue, which
    evaluates the same expression acc * (sa * sb) + bias, and within tolerance of the oracle.
    M and N need only be multiples of 128: in the last tile row / column the waves that lie outside
    the matrix store nothing (the canary rows behind the output stay untouched).  K need only be a
    multiple of 128: an odd number of 128-byte steps is padded with a step of zeros (the reference
    kernel for those shapes is the tiled one, the pipelined kernel wants K % 256 == 0)."""
    M, Nn, K = shape
    x = seeded_bf16((M, K), seed=18)
    x[:, 5] *= 100.0
    w = seeded_bf16((Nn, K), std=0.02, seed=19)
    rows, cols, with_bias = "rows" in which, "cols" in which, "bias" in which
    sx = O.t_scale(O.t_amax(x, O.SCALE_ROW if rows else O.SCALE_TENSOR), O.E4M3)
    sw = O.t_scale(O.t_amax(w, O.SCALE_ROW if cols else O.SCALE_TENSOR), O.E4M3)
    xq = O.t_cast(x, sx, O.E4M3, O.SCALE_ROW if rows else O.SCALE_TENSOR)
    wq = O.t_cast(w, sw, O.E4M3, O.SCALE_ROW if cols else O.SCALE_TENSOR)
    sa_inv, sb_inv = (1 / sx).float().reshape(-1), (1 / sw).float().reshape(-1)
    bias = torch.randn(Nn, generator=torch.Generator().manual_seed(3)) if with_bias else None
    ref32 = O.t_gemm_nt(xq, wq, O.E4M3, O.E4M3, sa_inv, sb_inv, want_f32=True)[1]
    if with_bias:
        ref32 = ref32 + bias
    args = (xq.cuda(), wq.cuda(), O.E4M3, O.E4M3, sa_inv.cuda(), sb_inv.cuda())
    kw = dict(bias=bias.cuda() if with_bias else None, out_dtype=out_dtype)
    N.gemm_set_variant(5 if K % 256 == 0 else 2)
    pipe = N.gemm_nt(*args, **kw)
    N.gemm_set_variant(7)
    guarded = torch.full((M + 256, Nn), 7.0, dtype=out_dtype, device="cuda")      # 256 canary rows behind the output
    stream = N.gemm_nt(*args, out=guarded[:M], **kw)
    assert (guarded[M:] == 7.0).all(), "rows beyond M were written"
    N.gemm_set_variant(-1)
    auto = N.gemm_nt(*args, **kw)
    assert "streaming" in N.gemm_variants()[7]
    assert torch.equal(stream, pipe) and torch.equal(auto, pipe)
    # fp32 output: the outlier channel makes the sums cancel, and the MFMA adds its 64 products in its own order
    assert max_rel_err(stream, ref32.to(out_dtype)) <= (TOL if out_dtype == torch.bfloat16 else 1e-3)


def test_transpose_symmetry(N):
    """gemm(a, b)^T == gemm(b, a): same products, only the roles swap."""
    aq, sa = quantised((512, 1024), O.E4M3, 1.0, 1)
    bq, sb = quantised((768, 1024), O.E4M3, 1.0, 2)
    o1 = N.gemm_nt(aq.cuda(), bq.cuda(), O.E4M3, O.E4M3, sa.cuda(), sb.cuda(), out_dtype=torch.float32)
    o2 = N.gemm_nt(bq.cuda(), aq.cuda(), O.E4M3, O.E4M3, sb.cuda(), sa.cuda(), out_dtype=torch.float32)
    assert max_rel_err(o2.t(), o1) <= 1e-5


def test_gemm_refuses_bad_shapes(N):
    a = torch.zeros((32, 24), dtype=torch.uint8, device="cuda")                    # K % 16 != 0
    one = torch.ones(1, device="cuda")
    with pytest.raises(N.NativeError):
        N.gemm_nt(a, a, 0, 0, one, one)
    b = torch.zeros((32, 32), dtype=torch.uint8, device="cuda")
    with pytest.raises(N.NativeError):
        N.gemm_nt(b, b, 0, 0, torch.ones(5, device="cuda"), one)                   # scale vector of the wrong length
    with pytest.raises(N.NativeError):
        N.gemm_nt(b, torch.zeros((32, 48), dtype=torch.uint8, device="cuda"), 0, 0, one, one)


def test_linear_fwd_bwd_three_gemms_at_llama_mlp_slice(N):
    """One Linear (fwd, dgrad, wgrad) through the real kernels end to end at a
    slice of the Llama-3-8B MLP shape, against the oracle's Linear."""
    M, K, Nn = 1024, 4096, 1792
    x, w, dy = seeded_bf16((M, K), 1.0, 0), seeded_bf16((Nn, K), 0.02, 1), seeded_bf16((M, Nn), 1e-3, 2)
    ref = O.linear_fwd_bwd(x, w, dy)
    xd, wd, gd = x.cuda(), w.cuda(), dy.cuda()
    sx, sxi = N.scale_from_amax(N.amax(xd), O.E4M3)
    sw, swi = N.scale_from_amax(N.amax(wd), O.E4M3)
    sg, sgi = N.scale_from_amax(N.amax(gd), O.E5M2)
    xq, xqt = N.cast_transpose(xd, sx, O.E4M3)
    wq, wqt = N.cast_transpose(wd, sw, O.E4M3)
    gq, gqt = N.cast_transpose(gd, sg, O.E5M2)
    for name, got in (("xq", xq), ("wq", wq), ("gq", gq), ("xq_t", xqt), ("wq_t", wqt), ("gq_t", gqt)):
        assert torch.equal(got.cpu(), ref[name]), name
    for name, got in (("sx", sx), ("sw", sw), ("sg", sg)):
        assert torch.equal(got.cpu(), ref[name]), name
    y = N.gemm_nt(xq, wq, O.E4M3, O.E4M3, sxi, swi)
    dx = N.gemm_nt(gq, wqt, O.E5M2, O.E4M3, sgi, swi)
    dw = N.gemm_nt(gqt, xqt, O.E5M2, O.E4M3, sgi, sxi)
    for name, got in (("y", y), ("dx", dx), ("dw", dw)):
        err = max_rel_err(got, ref[name])
        assert err <= TOL, f"{name}: {err}"


# ------------------------------------------------ operands stored with the contraction index slow
@pytest.mark.parametrize("fmts", [(O.E4M3, O.E4M3), (O.E5M2, O.E4M3), (O.E4M3, O.E5M2), (O.E5M2, O.E5M2)])
@pytest.mark.parametrize("shape", [(256, 256, 512), (512, 768, 1024), (1024, 256, 2560)])
def test_k_slow_layouts_equal_the_transposed_copies_bit_for_bit(N, fmts, shape):
    M, Nn, K = shape
    fa, fb = fmts
    a, sa = quantised((M, K), fa, 1.0, 1)
    b, sb = quantised((Nn, K), fb, 0.05, 2)
    a, b, sa, sb = a.cuda(), b.cuda(), sa.cuda(), sb.cuda()
    a_t, b_t = a.t().contiguous(), b.t().contiguous()                 # [K, M], [K, N]
    ref = N.gemm_nt(a, b, fa, fb, sa, sb)
    assert max_rel_err(ref, O.t_gemm_nt(a.cpu(), b.cpu(), fa, fb, sa.cpu(), sb.cpu())) <= TOL
    for la, lb in ((N.K_FAST, N.K_FAST), (N.K_FAST, N.K_SLOW), (N.K_SLOW, N.K_FAST), (N.K_SLOW, N.K_SLOW)):
        out = N.gemm_layouts(a_t if la else a, b_t if lb else b, fa, fb, la, lb, sa, sb)
        assert torch.equal(out, ref), f"layouts {la}{lb} of {shape}"


@pytest.mark.parametrize("shape", [(256, 256, 512), (512, 768, 1024), (768, 512, 1536)])
def test_streaming_kernel_fp32_output(N, shape):
    """fp32 output of the streaming kernel (weight gradients of fp32 master weights), every layout:
    exact on power-of-two operands; on random ones bit-identical to the pipelined kernel (same order of
    accumulation), and rounding it to bf16 gives the kernel's own bf16 output (one rounding either way)."""
    M, Nn, K = shape
    g = torch.Generator().manual_seed(11)
    vals = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, 4.0])
    av, bv = vals[torch.randint(0, 8, (M, K), generator=g)], vals[torch.randint(0, 8, (Nn, K), generator=g)]
    a2 = av.to(O.TORCH_FP8[O.E5M2]).view(torch.uint8).cuda()
    b2 = bv.to(O.TORCH_FP8[O.E4M3]).view(torch.uint8).cuda()
    s1, s2 = torch.tensor([0.25]).cuda(), torch.tensor([2.0]).cuda()
    exact = (av @ bv.t()) * 0.5
    a, sa = quantised((M, K), O.E5M2, 1e-3, 3)
    b, sb = quantised((Nn, K), O.E4M3, 1.0, 4)
    a, b, sa, sb = a.cuda(), b.cuda(), sa.cuda(), sb.cuda()
    N.gemm_set_variant(5)                                              # software-pipelined kernel, staged epilogue
    ref32 = N.gemm_nt(a, b, O.E5M2, O.E4M3, sa, sb, out_dtype=torch.float32)
    N.gemm_set_variant(-1)
    ref32_cpu = O.t_gemm_nt(a.cpu(), b.cpu(), O.E5M2, O.E4M3, sa.cpu(), sb.cpu(), want_f32=True)[1]
    assert max_rel_err(ref32, ref32_cpu) <= 1e-4                       # fp32 sums in a different order (and the MFMA's own inside 64 products)
    for la, lb in ((N.K_FAST, N.K_FAST), (N.K_FAST, N.K_SLOW), (N.K_SLOW, N.K_FAST), (N.K_SLOW, N.K_SLOW)):
        lay = lambda t, l: t.t().contiguous() if l else t
        out = N.gemm_layouts(lay(a2, la), lay(b2, lb), O.E5M2, O.E4M3, la, lb, s1, s2, out_dtype=torch.float32)
        assert out.dtype == torch.float32 and torch.equal(out.cpu(), exact), f"layouts {la}{lb}: power-of-two case"
        out = N.gemm_layouts(lay(a, la), lay(b, lb), O.E5M2, O.E4M3, la, lb, sa, sb, out_dtype=torch.float32)
        assert torch.equal(out, ref32), f"layouts {la}{lb}: differs from the pipelined kernel"
        out16 = N.gemm_layouts(lay(a, la), lay(b, lb), O.E5M2, O.E4M3, la, lb, sa, sb)
        assert torch.equal(out.bfloat16(), out16), f"layouts {la}{lb}: bf16(fp32 output) != bf16 output"
    given = torch.full((M, Nn), 7.0, device="cuda")
    assert N.gemm_layouts(a, b, O.E5M2, O.E4M3, N.K_FAST, N.K_FAST, sa, sb, out=given) is given
    assert torch.equal(given, ref32)
    # the automatic choice of odl_fp8_gemm_nt takes the same kernel for fp32 output
    assert torch.equal(N.gemm_nt(a, b, O.E5M2, O.E4M3, sa, sb, out_dtype=torch.float32), ref32)


def test_k_slow_layouts_index_check_with_one_hot_operands(N):
    # A[m, k] = 1 at k = (7 m + 3) % K, B[n, k] = 2^(n % 5) at k = (5 n + 1) % K, stored K-slow:
    # C[m, n] is that power of two where the two columns coincide and 0 elsewhere, exactly
    M, Nn, K = 256, 512, 768
    a = torch.zeros((M, K)); b = torch.zeros((Nn, K))
    ka = (7 * torch.arange(M) + 3) % K
    kb = (5 * torch.arange(Nn) + 1) % K
    a[torch.arange(M), ka] = 1.0
    b[torch.arange(Nn), kb] = 2.0 ** (torch.arange(Nn) % 5).float()
    one = torch.ones(1)
    aq, bq = O.t_cast(a.bfloat16(), one, O.E4M3).cuda(), O.t_cast(b.bfloat16(), one, O.E4M3).cuda()
    want = ((ka[:, None] == kb[None, :]).float() * b.sum(1)[None, :]).bfloat16()
    out = N.gemm_layouts(aq.t().contiguous(), bq.t().contiguous(), O.E4M3, O.E4M3, N.K_SLOW, N.K_SLOW, one.cuda(), one.cuda())
    assert torch.equal(out.cpu(), want)


def test_k_slow_layouts_refusals(N):
    one = torch.ones(1, device="cuda")
    a = torch.zeros((256, 512), dtype=torch.uint8, device="cuda")
    with pytest.raises(N.NativeError, match="multiples of 256"):
        N.gemm_layouts(a[:128], a, O.E4M3, O.E4M3, N.K_FAST, N.K_FAST, one, one)
    with pytest.raises(N.NativeError, match="multiples of 256"):
        N.gemm_layouts(a[:, :256], a[:, :256], O.E4M3, O.E4M3, N.K_FAST, N.K_FAST, one, one)       # K = 256 < 512
    with pytest.raises(N.NativeError, match="contraction sizes differ"):
        N.gemm_layouts(a, a.t().contiguous(), O.E4M3, O.E4M3, N.K_FAST, N.K_FAST, one, one)
    assert not N.gemm_layouts_supported(256, 256, 256) and not N.gemm_layouts_supported(384, 256, 512)
    assert N.gemm_layouts_supported(256, 256, 512) and N.gemm_layouts_supported(256, 256, 512, torch.float32)
    assert not N.gemm_layouts_supported(256, 256, 512, torch.float16)
    with pytest.raises(N.NativeError, match="wrong shape / dtype"):
        N.gemm_layouts(a, a, O.E4M3, O.E4M3, N.K_FAST, N.K_FAST, one, one, out=torch.empty((256, 256), dtype=torch.float16, device="cuda"))


# ------------------------------------------------------------------ K cut into runs (few tiles, long contraction)
def _runs_ok(K, splits):
    steps = K // 128
    per = (-(-steps // splits) + 1) & ~1
    return per >= 4 and steps - (splits - 1) * per >= 4


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("splits", [2, 3, 4, 7])
@pytest.mark.parametrize("shape", [(256, 384, 4096), (128, 128, 2688), (384, 256, 5248)])
def test_split_k_equals_the_single_launch(N, shape, splits, out_dtype):
    """Power-of-two operands: every partial sum is exact, so the runs added up must equal the single
    launch (and the oracle) bit for bit, for every layout -- a run that starts at the wrong K offset, reads a
    neighbour's steps or misses the padding step of an odd run breaks this.  Random operands with scale
    vectors and a bias: within the GEMM tolerance of the oracle and close to the single launch."""
    M, Nn, K = shape
    if not _runs_ok(K, splits):
        one = torch.ones(1, device="cuda")
        z = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
        with pytest.raises(N.NativeError, match="shorter than 512"):
            N.gemm_splitk(z, torch.zeros((Nn, K), dtype=torch.uint8, device="cuda"), O.E4M3, O.E4M3, one, one, splits)
        return
    g = torch.Generator().manual_seed(21)
    vals = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, 4.0])
    av, bv = vals[torch.randint(0, 8, (M, K), generator=g)], vals[torch.randint(0, 8, (Nn, K), generator=g)]
    a2 = av.to(O.TORCH_FP8[O.E5M2]).view(torch.uint8).cuda()
    b2 = bv.to(O.TORCH_FP8[O.E4M3]).view(torch.uint8).cuda()
    s1, s2 = torch.tensor([0.25]).cuda(), torch.tensor([2.0]).cuda()
    exact = ((av @ bv.t()) * 0.5).to(out_dtype)
    layouts = [(N.K_FAST, N.K_FAST)]
    if M % 256 == 0 and Nn % 256 == 0:
        layouts += [(N.K_SLOW, N.K_FAST), (N.K_FAST, N.K_SLOW), (N.K_SLOW, N.K_SLOW)]
    for la, lb in layouts:
        lay = lambda t, l: t.t().contiguous() if l else t
        out = N.gemm_splitk(lay(a2, la), lay(b2, lb), O.E5M2, O.E4M3, s1, s2, splits, out_dtype=out_dtype, layout_a=la, layout_b=lb)
        assert torch.equal(out.cpu(), exact), f"layouts {la}{lb}"
    x = seeded_bf16((M, K), seed=28)
    w = seeded_bf16((Nn, K), std=0.02, seed=29)
    sx, sw = O.t_scale(O.t_amax(x, O.SCALE_ROW), O.E4M3), O.t_scale(O.t_amax(w, O.SCALE_ROW), O.E4M3)
    xq, wq = O.t_cast(x, sx, O.E4M3, O.SCALE_ROW), O.t_cast(w, sw, O.E4M3, O.SCALE_ROW)
    sa_inv, sb_inv = (1 / sx).float().reshape(-1), (1 / sw).float().reshape(-1)
    bias = torch.randn(Nn, generator=g)
    ref32 = O.t_gemm_nt(xq, wq, O.E4M3, O.E4M3, sa_inv, sb_inv, want_f32=True)[1] + bias
    args = (xq.cuda(), wq.cuda(), O.E4M3, O.E4M3, sa_inv.cuda(), sb_inv.cuda())
    out = N.gemm_splitk(*args, splits, bias=bias.cuda(), out_dtype=out_dtype)
    N.gemm_set_variant(7)                           # a forced variant is never split
    single = N.gemm_nt(*args, bias=bias.cuda(), out_dtype=out_dtype)
    N.gemm_set_variant(-1)
    assert max_rel_err(out, ref32.to(out_dtype)) <= (TOL if out_dtype == torch.bfloat16 else 1e-3)
    assert max_rel_err(out, single) <= (8e-3 if out_dtype == torch.bfloat16 else 1e-5)     # one bf16 ulp / fp32 sum order


def test_split_k_is_chosen_for_few_tiles_and_a_long_contraction(N, monkeypatch):
    assert N.gemm_split_count(8192, 14336, 4096) == 1          # 1792 tiles: nothing to gain
    assert N.gemm_split_count(8192, 1024, 4096) == 1           # 128 tiles, 32 steps: the reduction would cost the gain
    assert N.gemm_split_count(1024, 4096, 8192) == 1           # wgrad of a key / value projection: 128 x 128 tiles in one launch win
    assert N.gemm_split_count(1024, 1024, 16384) >= 8
    assert N.gemm_split_count(768, 768, 16384) >= 8            # wgrad of a small model's projection: 9 tiles
    assert N.gemm_split_count(8192, 1024, 151936) == 2         # dgrad of a vocabulary-sized head
    assert N.gemm_split_count(300, 512, 8192) == 1 and N.gemm_split_count(256, 256, 1024) == 1
    a, sa = quantised((768, 8192), O.E5M2, 1e-3, 31)
    b, sb = quantised((768, 8192), O.E4M3, 1.0, 32)
    a, b, sa, sb = a.cuda(), b.cuda(), sa.cuda(), sb.cuda()
    seen = []
    real = N._gemm_splitk
    monkeypatch.setattr(N, "_gemm_splitk", lambda *args: (seen.append(args[13]), real(*args))[1])
    out = N.gemm_nt(a, b, O.E5M2, O.E4M3, sa, sb)
    assert seen == [N.gemm_split_count(768, 768, 8192)] and seen[0] > 1
    assert max_rel_err(out, O.t_gemm_nt(a.cpu(), b.cpu(), O.E5M2, O.E4M3, sa.cpu(), sb.cpu())) <= TOL
    monkeypatch.setattr(N, "split_k", False)
    unsplit = N.gemm_nt(a, b, O.E5M2, O.E4M3, sa, sb)
    assert len(seen) == 1 and max_rel_err(out, unsplit) <= 8e-3


def test_split_k_entry_refuses_what_it_cannot_run(N):
    """Straight at the C entry point: a workspace that is too small, a null pointer, shapes off the 128 grid,
    an operand stored K-slow that does not fill whole tiles.  Nothing is launched in any of these cases."""
    L = N.load()
    M, Nn, K = 256, 384, 4096
    a = torch.zeros((M, K), dtype=torch.uint8, device="cuda")
    b = torch.zeros((Nn, K), dtype=torch.uint8, device="cuda")
    one = torch.ones(1, device="cuda")
    out = torch.full((M, Nn), 3.0, dtype=torch.bfloat16, device="cuda")
    ws = torch.empty((2, M, Nn), dtype=torch.float32, device="cuda")
    s = torch.cuda.current_stream().cuda_stream

    def call(M_=M, N_=Nn, K_=K, la=0, lb=0, splits=2, ws_bytes=ws.numel() * 4, ws_ptr=ws.data_ptr(), out_dtype=0):
        return L.odl_fp8_gemm_splitk(a.data_ptr(), b.data_ptr(), M_, N_, K_, 0, 0, la, lb, one.data_ptr(), 1, one.data_ptr(), 1,
                                     None, out.data_ptr(), out_dtype, 0, splits, ws_ptr, ws_bytes, s)

    assert call() == 0
    torch.cuda.synchronize()
    assert (out == 0).all()                                        # zero codes: the product is zero
    out.fill_(3.0)
    for kwargs, text in ((dict(ws_bytes=ws.numel() * 4 - 4), "workspace"), (dict(ws_ptr=None), "null pointer"),
                         (dict(M_=200), "multiples of 128"), (dict(K_=4100), "multiples of 128"),
                         (dict(M_=128, la=1), "256 for an operand stored K-slow"), (dict(splits=1), "splits"),
                         (dict(splits=65), "splits"), (dict(splits=9), "shorter than 512"), (dict(out_dtype=7), "out_dtype")):
        assert call(**kwargs) != 0, kwargs
        assert text in L.odl_fp8_last_error().decode(), (kwargs, L.odl_fp8_last_error().decode())
    torch.cuda.synchronize()
    assert (out == 3.0).all()                                      # nothing ran

@pytest.mark.parametrize("seed", range(48))
def test_seeded_random_shapes_through_the_automatic_choice(N, seed):
    """Shapes drawn on the grids the kernels distinguish (16, 128, 256), with and without scale vectors, bias and fp32
    output: whichever kernel the library picks (generic, tiled, pipelined, streaming, K runs), the result is the oracle's."""
    g = torch.Generator().manual_seed(1000 + seed)
    def draw(grids, hi):
        step = grids[int(torch.randint(0, len(grids), (1,), generator=g))]
        return step * int(torch.randint(1, hi // step + 1, (1,), generator=g))
    M, Nn = draw((16, 128, 256), 1024), draw((16, 128, 256), 1024)
    K = draw((16, 128, 256), 2048) if seed % 4 else 128 * int(torch.randint(16, 80, (1,), generator=g))   # every 4th: long contraction
    rows, cols, with_bias, f32 = (bool(int(torch.randint(0, 2, (1,), generator=g))) for _ in range(4))
    fa = O.E5M2 if seed % 3 == 0 else O.E4M3
    x = seeded_bf16((M, K), seed=2000 + seed)
    w = seeded_bf16((Nn, K), std=0.02, seed=3000 + seed)
    sx = O.t_scale(O.t_amax(x, O.SCALE_ROW if rows else O.SCALE_TENSOR), fa)
    sw = O.t_scale(O.t_amax(w, O.SCALE_ROW if cols else O.SCALE_TENSOR), O.E4M3)
    xq = O.t_cast(x, sx, fa, O.SCALE_ROW if rows else O.SCALE_TENSOR)
    wq = O.t_cast(w, sw, O.E4M3, O.SCALE_ROW if cols else O.SCALE_TENSOR)
    sa_inv, sb_inv = (1 / sx).float().reshape(-1), (1 / sw).float().reshape(-1)
    bias = torch.randn(Nn, generator=g) * 0.1 if with_bias else None
    ref32 = O.t_gemm_nt(xq, wq, fa, O.E4M3, sa_inv, sb_inv, want_f32=True)[1]
    if with_bias:
        ref32 = ref32 + bias
    out_dtype = torch.float32 if f32 else torch.bfloat16
    out = N.gemm_nt(xq.cuda(), wq.cuda(), fa, O.E4M3, sa_inv.cuda(), sb_inv.cuda(), bias=bias.cuda() if with_bias else None,
                    out_dtype=out_dtype)
    err = max_rel_err(out, ref32.to(out_dtype))
    assert err <= (1e-3 if f32 else TOL), f"{M}x{Nn}x{K} rows={rows} cols={cols} bias={with_bias} f32={f32}: {err}"


# ------------------------------------------------------------------ C = C + product
def _codes(value_by_col: dict, rows: int, K: int, fmt) -> torch.Tensor:
    x = torch.zeros((rows, K))
    for col, v in value_by_col.items():
        x[:, col] = v
    q = x.to(O.TORCH_FP8[fmt]).view(torch.uint8)
    assert torch.equal(O.t_decode(q, fmt), x), "test values must be exact in the format"
    return q


@pytest.mark.parametrize("variant", [-1, 0, 1, 2, 3, 4, 5, 6, 7])
def test_accumulate_rounds_once(N, variant):
    """C = C + product with ONE rounding, on every kernel that can be asked for (a forced streaming variant falls back,
    as the header says).  The product is exact (2^-8 + 2^-17); with C0 = 1 in bf16 the single rounding gives
    1 + 2^-7 where rounding the product first would give 1 (a tie to even)."""
    M, Nn, K = 512, 384, 512
    a = _codes({3: 2.0 ** -4, 200: 2.0 ** -9}, M, K, O.E4M3)
    b = _codes({3: 2.0 ** -4, 200: 2.0 ** -8}, Nn, K, O.E4M3)
    one = torch.ones(1)
    prod = O.t_gemm_nt(a, b, O.E4M3, O.E4M3, one, one, want_f32=True)[1]
    assert torch.all(prod == 2.0 ** -8 + 2.0 ** -17)
    N.gemm_set_variant(variant)
    try:
        c16 = torch.ones((M, Nn), dtype=torch.bfloat16, device="cuda")
        N.gemm_nt(a.cuda(), b.cuda(), O.E4M3, O.E4M3, one.cuda(), one.cuda(), out=c16, accumulate=True)
        assert torch.all(c16.float() == 1.0 + 2.0 ** -7), c16.float().unique()
        assert torch.equal(c16.cpu(), O.t_accumulate(torch.ones((M, Nn), dtype=torch.bfloat16), prod))
        c32 = torch.full((M, Nn), 2.0 ** 15, device="cuda")
        N.gemm_nt(a.cuda(), b.cuda(), O.E4M3, O.E4M3, one.cuda(), one.cuda(), out=c32, accumulate=True)
        assert torch.equal(c32.cpu(), O.t_accumulate(torch.full((M, Nn), 2.0 ** 15), prod))
        assert torch.all(c32 == 2.0 ** 15 + 2.0 ** -8)
    finally:
        N.gemm_set_variant(-1)


@pytest.mark.parametrize("shape", [(512, 768, 1024), (300, 200, 256), (257, 255, 384), (40, 24, 48), (1024, 512, 2048)])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_accumulate_random_every_variant(N, shape, out_dtype):
    """Random operands, scale vectors and a bias, interior and ragged tiles: out = out + product against the oracle's
    composition (product in fp32, bias, old C, one rounding) within the GEMM tolerance, and exactly equal to what the
    same kernel gives without the flag plus the old C where that sum needs no rounding (fp32 output, C0 = 0)."""
    M, Nn, K = shape
    aq, sa_inv = quantised((M, K), O.E5M2, 1e-3, 11)
    bq, sb_inv = quantised((Nn, K), O.E4M3, 0.02, 12)
    sa_vec = (sa_inv * torch.linspace(0.5, 2.0, M)).contiguous()
    bias = seeded_bf16((Nn,), 1e-5, 13).float()
    c0 = (seeded_bf16((M, Nn), 2e-5, 14).float()).to(out_dtype)
    prod = O.t_gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_vec, sb_inv, want_f32=True)[1]
    want = O.t_accumulate(c0, prod, bias)
    for v in [-1] + variants(N):
        N.gemm_set_variant(v)
        c = c0.cuda().clone()
        N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_vec.cuda(), sb_inv.cuda(), bias=bias.cuda(), out=c, accumulate=True)
        assert max_rel_err(c, want) <= TOL, f"variant {v} {shape} {out_dtype}"
        if out_dtype == torch.float32:
            z = torch.zeros((M, Nn), device="cuda")
            N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_vec.cuda(), sb_inv.cuda(), bias=bias.cuda(), out=z, accumulate=True)
            plain = N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_vec.cuda(), sb_inv.cuda(), bias=bias.cuda(), out_dtype=torch.float32)
            assert torch.equal(z, plain), f"variant {v}: adding into zeros must equal the plain product"
    N.gemm_set_variant(-1)


def test_accumulate_through_split_k_and_k_slow_layouts(N):
    """The routes that pass through the fp32 workspace: a split over K (few tiles, long contraction) and an operand
    stored K-slow (wgrad reading dY as stored), the latter also with a single run."""
    M, Nn, K = 768, 768, 16384
    aq, sa_inv = quantised((M, K), O.E5M2, 1e-3, 21)
    bq, sb_inv = quantised((Nn, K), O.E4M3, 1.0, 22)
    c0 = seeded_bf16((M, Nn), 1e-3, 23).float()
    prod = O.t_gemm_nt(aq, bq, O.E5M2, O.E4M3, sa_inv, sb_inv, want_f32=True)[1]
    want = O.t_accumulate(c0, prod)
    assert N.gemm_split_count(M, Nn, K) > 1
    c = c0.cuda().clone()
    N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_inv.cuda(), sb_inv.cuda(), out=c, accumulate=True)
    assert max_rel_err(c, want) <= 1e-4
    # K-slow A: the same product from a^T stored [K, M]
    for splits in (1, 4):
        c = c0.cuda().clone()
        N.gemm_splitk(aq.t().contiguous().cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_inv.cuda(), sb_inv.cuda(), splits,
                      layout_a=N.K_SLOW, out=c, accumulate=True)
        assert max_rel_err(c, want) <= 1e-4, splits
    c = c0.cuda().clone()
    N.gemm_layouts(aq.t().contiguous().cuda(), bq.cuda(), O.E5M2, O.E4M3, N.K_SLOW, N.K_FAST, sa_inv.cuda(), sb_inv.cuda(),
                   out=c, accumulate=True)
    assert max_rel_err(c, want) <= 1e-4
    with pytest.raises(N.NativeError):
        N.gemm_nt(aq.cuda(), bq.cuda(), O.E5M2, O.E4M3, sa_inv.cuda(), sb_inv.cuda(), accumulate=True)      # nothing to add into


# ---------------------------------------------------------------- sums of products in one launch (odl_fp8_gemm_nt_sum)
def _pow2_pairs(M, Nn, ks, seed):
    g = torch.Generator().manual_seed(seed)
    vals = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, 4.0])
    a = [vals[torch.randint(0, 8, (M, k), generator=g)].to(torch.float8_e5m2).view(torch.uint8) for k in ks]
    b = [vals[torch.randint(0, 8, (Nn, k), generator=g)].to(torch.float8_e4m3fn).view(torch.uint8) for k in ks]
    return a, b


@pytest.mark.parametrize("ks", [(512, 512), (1024, 512, 768), (512, 2048, 512, 1024)])
@pytest.mark.parametrize("variant", [-1, 2, 5])
def test_sum_of_products_power_of_two_is_bit_exact(N, ks, variant):
    """Power-of-two values and scales: every partial sum and every ratio of scale products is exact, so the one-launch
    route (accumulators carried from pair to pair, multiplied by the ratio in between) and the oracle must agree bit for
    bit, in fp32 and in bf16; so must the per-pair route (forced variants 2 and 5: a GEMM per pair adding into C) in
    fp32, and in bf16 with the oracle's composition of its one rounding per pair.
    M and N end in half a tile (384 = 256 + 128, 640 = 2 x 256 + 128).  A pair skipped or read twice, a ratio applied the
    wrong way round or to the wrong pair, or the wrong row pitch after a pair of another length all show."""
    M, Nn = 384, 640
    a, b = _pow2_pairs(M, Nn, ks, 31)
    scales = [(torch.tensor([2.0 ** (3 - 2 * i)]), torch.tensor([2.0 ** (i - 6)])) for i in range(len(ks))]
    ref16, ref32 = O.t_gemm_nt_sum([(x, y, p, q) for x, y, (p, q) in zip(a, b, scales)], O.E5M2, O.E4M3, want_f32=True)
    if variant >= 0:
        # a GEMM per pair rounds to the output type after every pair (the accumulate flag's definition)
        for i, (x, y, (p, q)) in enumerate(zip(a, b, scales)):
            part = O.t_gemm_nt(x, y, O.E5M2, O.E4M3, p, q, want_f32=True)[1]
            ref16 = part.bfloat16() if i == 0 else O.t_accumulate(ref16, part)
    dev = lambda ts: [t.cuda() for t in ts]
    N.gemm_set_variant(variant)
    try:
        for out_dtype, ref in ((torch.float32, ref32), (torch.bfloat16, ref16)):
            out = N.gemm_nt_sum(dev(a), dev(b), O.E5M2, O.E4M3, dev([p for p, _ in scales]), dev([q for _, q in scales]),
                                out_dtype=out_dtype)
            assert torch.equal(out.cpu(), ref), f"{out_dtype}: max diff {(out.cpu().float() - ref.float()).abs().max()}"
    finally:
        N.gemm_set_variant(-1)


@pytest.mark.parametrize("shape", [(512, 768, (1024, 512)), (1024, 1280, (512, 1536, 768)), (256, 256, (512, 512, 512, 512))])
def test_sum_of_products_random_operands_and_far_apart_scales(N, shape):
    """Quantised Gaussian operands whose scale products lie up to 2^20 apart between pairs: against the oracle within the
    GEMM tolerance in bf16 and within fp32 rounding of a few thousand additions in fp32; the per-pair route (a rounding
    to the output type per pair) agrees with the one-launch route within the GEMM tolerance too."""
    M, Nn, ks = shape
    pairs, dev_args = [], ([], [], [], [])
    for i, k in enumerate(ks):
        aq, sa_inv = quantised((M, k), O.E5M2, 1e-3 * 32.0 ** i, 40 + i)
        bq, sb_inv = quantised((Nn, k), O.E4M3, 0.02 * 32.0 ** i, 50 + i)
        pairs.append((aq, bq, sa_inv, sb_inv))
        for lst, t in zip(dev_args, (aq, bq, sa_inv, sb_inv)):
            lst.append(t.cuda())
    ref16, ref32 = O.t_gemm_nt_sum(pairs, O.E5M2, O.E4M3, want_f32=True)
    out32 = N.gemm_nt_sum(dev_args[0], dev_args[1], O.E5M2, O.E4M3, dev_args[2], dev_args[3], out_dtype=torch.float32)
    assert max_rel_err(out32, ref32) <= 2e-5
    out16 = N.gemm_nt_sum(dev_args[0], dev_args[1], O.E5M2, O.E4M3, dev_args[2], dev_args[3])
    assert max_rel_err(out16, ref16) <= TOL
    assert torch.equal(out16, out32.bfloat16())                     # one rounding of the same fp32 values
    N.gemm_set_variant(5)
    try:
        seq = N.gemm_nt_sum(dev_args[0], dev_args[1], O.E5M2, O.E4M3, dev_args[2], dev_args[3])
    finally:
        N.gemm_set_variant(-1)
    assert max_rel_err(seq, ref16) <= TOL


def test_sum_of_products_more_tiles_than_compute_units(N):
    """288 tiles: blocks walk on to a second tile, whose first pair follows a fold and not a rescale, with the loads of
    that pair requested while the last pair of the tile before was still being multiplied."""
    M, Nn, ks = 4096, 4608, (512, 1024)
    a, b = _pow2_pairs(M, Nn, ks, 61)
    scales = [(torch.tensor([0.5]), torch.tensor([0.25])), (torch.tensor([4.0]), torch.tensor([2.0 ** -7]))]
    ref = O.t_gemm_nt_sum([(x, y, p, q) for x, y, (p, q) in zip(a, b, scales)], O.E5M2, O.E4M3)
    out = N.gemm_nt_sum([t.cuda() for t in a], [t.cuda() for t in b], O.E5M2, O.E4M3, [p.cuda() for p, _ in scales],
                        [q.cuda() for _, q in scales])
    assert torch.equal(out.cpu(), ref)


def test_sum_of_products_shapes_outside_the_one_launch_route_and_errors(N):
    """A contraction that is no multiple of 256, an output that is no multiple of 128 and a single pair all go the
    per-pair way and still match the oracle; mismatched operands are refused before anything is launched."""
    for M, Nn, ks in ((512, 384, (384, 512)), (200, 136, (512, 1024)), (256, 256, (64,)), (256, 384, (512, 512, 512, 512, 512))):
        pairs, dev_args = [], ([], [], [], [])
        for i, k in enumerate(ks):
            aq, sa_inv = quantised((M, k), O.E5M2, 1e-3, 70 + i)
            bq, sb_inv = quantised((Nn, k), O.E4M3, 0.02, 80 + i)
            pairs.append((aq, bq, sa_inv, sb_inv))
            for lst, t in zip(dev_args, (aq, bq, sa_inv, sb_inv)):
                lst.append(t.cuda())
        ref = O.t_gemm_nt_sum(pairs, O.E5M2, O.E4M3)
        out = N.gemm_nt_sum(dev_args[0], dev_args[1], O.E5M2, O.E4M3, dev_args[2], dev_args[3])
        assert max_rel_err(out, ref) <= TOL, (M, Nn, ks)
    one = torch.ones(1, device="cuda")
    a = torch.zeros((256, 512), dtype=torch.uint8, device="cuda")
    with pytest.raises(N.NativeError):
        N.gemm_nt_sum([a, a], [a, a[:, :256].contiguous()], O.E5M2, O.E4M3, [one, one], [one, one])       # K differs inside a pair
    with pytest.raises(N.NativeError):
        N.gemm_nt_sum([a, a[:128]], [a, a], O.E5M2, O.E4M3, [one, one], [one, one])                        # M differs between pairs
    with pytest.raises(N.NativeError):
        N.gemm_nt_sum([a, a], [a, a], O.E5M2, O.E4M3, [one], [one, one])                                   # a scale missing
    with pytest.raises(N.NativeError):
        N.gemm_nt_sum([a] * 65, [a] * 65, O.E5M2, O.E4M3, [one] * 65, [one] * 65)                          # more pairs than the call takes


def test_sum_of_products_shape_sweep_against_the_per_pair_route(N):
    """Seeded sweep over pair counts, contraction lengths (equal and unequal, 512 .. 2304) and output shapes (whole and
    half tiles at either edge, one tile, more tiles than fit one round of a small grid): the one-launch route against a
    GEMM per pair adding into an fp32 C, which shares no code with it beyond the MFMA.  fp32 outputs, so the only
    differences are the order of fp32 additions and the ratio multiplications."""
    g = torch.Generator().manual_seed(77)
    lengths = [512, 768, 1024, 1280, 1536, 2304]
    shapes = [(128, 128), (256, 256), (384, 128), (128, 640), (640, 896), (1152, 256), (2176, 1408)]
    for case in range(21):
        M, Nn = shapes[case % len(shapes)]
        pairs = 2 + case % 3
        ks = [lengths[int(torch.randint(0, len(lengths), (1,), generator=g))] for _ in range(pairs)]
        a = [torch.randint(0, 256, (M, k), generator=g, dtype=torch.uint8) for k in ks]
        b = [torch.randint(0, 256, (Nn, k), generator=g, dtype=torch.uint8) for k in ks]
        for t in a:                                   # no NaN / Inf codes (e5m2: exponent 31; e4m3: 0x7f / 0xff)
            t[(t & 0x7C) == 0x7C] = 0x3C
        for t in b:
            t[(t & 0x7F) == 0x7F] = 0x38
        sa = [torch.rand(1, generator=g) * 2.0 ** float(torch.randint(-12, 4, (1,), generator=g)) + 2.0 ** -20 for _ in ks]
        sb = [torch.rand(1, generator=g) * 2.0 ** float(torch.randint(-12, 4, (1,), generator=g)) + 2.0 ** -20 for _ in ks]
        dev = lambda ts: [t.cuda() for t in ts]
        one = N.gemm_nt_sum(dev(a), dev(b), O.E5M2, O.E4M3, dev(sa), dev(sb), out_dtype=torch.float32)
        N.gemm_set_variant(2)
        try:
            seq = N.gemm_nt_sum(dev(a), dev(b), O.E5M2, O.E4M3, dev(sa), dev(sb), out_dtype=torch.float32)
        finally:
            N.gemm_set_variant(-1)
        assert torch.isfinite(one).all(), (case, M, Nn, ks)
        assert max_rel_err(one, seq) <= 2e-5, (case, M, Nn, ks, max_rel_err(one, seq))
        if case % 7 == 0:
            # uniformly drawn codes span the formats' whole range (products 2^-25 .. 2^24.6 side by side) and the sums cancel
            # heavily: the matrix instruction's adder keeps fewer bits below the largest product of its 64 than an fp32
            # sum does (both routes above share that), so against the oracle the bound is 1e-4 of the largest output,
            # still a hundredth of the GEMM tolerance and far below what a wrong pair, ratio or pitch would give
            ref = O.t_gemm_nt_sum(list(zip(a, b, sa, sb)), O.E5M2, O.E4M3, want_f32=True)[1]
            assert max_rel_err(one, ref) <= 1e-4, (case, M, Nn, ks)
