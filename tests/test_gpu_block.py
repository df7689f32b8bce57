"""GPU parity of the blockwise recipe (128-element and 128 x 128 blocks, power-of-two scales) against the CPU oracle.

Codes and scale bytes: bit-exact.  The products go through the block-scaled GEMM of the MXFP8 tests (a 128-block is four
32-blocks with the same scale byte) and are compared with the emulated product: max|err| / max|ref| <= 1e-2.
Every call goes through the C ABI.
"""
import pytest
import torch

from oracle import oracle as O
from tests.helpers import assert_bytes_equal, max_rel_err, seeded_bf16

pytestmark = pytest.mark.gpu

E4M3, E5M2 = O.E4M3, O.E5M2


@pytest.fixture(scope="module")
def N():
    from optimus_dl_amd import native

    native.load()
    return native


def _mixed(shape, seed):
    g = torch.Generator().manual_seed(seed)
    rows, cols = shape
    x = torch.randn(shape, generator=g)
    x = x * torch.exp2(torch.randint(-20, 20, (rows, 1), generator=g).float())
    x = x * torch.exp2(torch.randint(-6, 6, (1, cols), generator=g).float())
    x[torch.rand(shape, generator=g) < 0.05] = 0.0
    x[:128, :128] = 0.0                                    # a zero block in every sense
    x[rows - 1, cols - 1] = 3.0e38
    x[rows // 2, cols // 2] = -1.0e-38
    return x.bfloat16()


def _bytes(sc: torch.Tensor) -> torch.Tensor:
    """[K / 128, rows, 4] with four equal bytes -> [rows, K / 128]."""
    sc = sc.cpu()
    assert bool((sc == sc[:, :, :1]).all()), "the four bytes of a 128-block differ"
    return sc[:, :, 0].t().contiguous()


SHAPES = [(128, 128), (256, 128), (128, 384), (384, 512), (1024, 768), (2048, 256)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_block_cast_one_dimensional_blocks_bit_exact(N, shape, fmt, dtype):
    x = _mixed(shape, seed=shape[0] + 3 * shape[1] + fmt)
    for margin in (0, 1):
        out, sc, out_t, sc_t = N.block_cast(x.to(dtype).cuda(), fmt, margin, False, True, True)
        wc, ws = O.c_block_quantise(x, 1, 128, fmt, margin)
        assert_bytes_equal(_bytes(sc), ws, f"scale bytes {shape} fmt {fmt} margin {margin}")
        assert_bytes_equal(out, wc, f"codes {shape} fmt {fmt} margin {margin}")
        wct, wst = O.c_block_quantise(x.t().contiguous(), 1, 128, fmt, margin)
        assert_bytes_equal(_bytes(sc_t), wst, f"transposed scale bytes {shape}")
        assert_bytes_equal(out_t, wct, f"transposed codes {shape}")
    tc, ts = O.t_block_quantise(x, 1, 128, fmt, 1)
    assert_bytes_equal(out, tc, "codes (torch restatement)")
    assert_bytes_equal(_bytes(sc), ts, "scale bytes (torch restatement)")


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_block_cast_two_dimensional_blocks_bit_exact(N, shape, fmt, dtype):
    x = _mixed(shape, seed=shape[0] * 5 + shape[1] + fmt)
    out, sc, out_t, sc_t = N.block_cast(x.to(dtype).cuda(), fmt, 0, True, True, True)
    wc, ws = O.c_block_quantise(x, 128, 128, fmt, 0)                       # ws [R / 128, C / 128]
    assert_bytes_equal(out, wc, f"codes {shape}")
    assert_bytes_equal(out_t, wc.t().contiguous(), f"transposed codes {shape}: the same codes, transposed")
    assert_bytes_equal(_bytes(sc), ws.repeat_interleave(128, dim=0), f"scale bytes {shape}")
    assert_bytes_equal(_bytes(sc_t), ws.t().repeat_interleave(128, dim=0), f"transposed scale bytes {shape}")


@pytest.mark.parametrize("order", ["sorted", "shuffled"])
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_block_cast_every_bf16_pattern(N, fmt, order, dtype):
    """All 65536 bf16 bit patterns, sorted by magnitude (elements close to their block's amax) and shuffled (far below
    it; Inf and NaN scattered over the blocks), 1 x 128 blocks in both directions and 128 x 128 blocks."""
    from tests.test_gpu_mx import _every_bf16_pattern

    x = _every_bf16_pattern(order)                                        # [128, 512]
    out, sc, out_t, sc_t = N.block_cast(x.to(dtype).cuda(), fmt, 0, False, True, True)
    wc, ws = O.c_block_quantise(x, 1, 128, fmt, 0)
    assert_bytes_equal(_bytes(sc), ws, f"scale bytes, {order}")
    assert_bytes_equal(out, wc, f"codes, {order}")
    wct, wst = O.c_block_quantise(x.t().contiguous(), 1, 128, fmt, 0)
    assert_bytes_equal(_bytes(sc_t), wst, f"transposed scale bytes, {order}")
    assert_bytes_equal(out_t, wct, f"transposed codes, {order}")
    out, sc, out_t, sc_t = N.block_cast(x.to(dtype).cuda(), fmt, 0, True, True, True)
    wc, ws = O.c_block_quantise(x, 128, 128, fmt, 0)
    assert_bytes_equal(out, wc, f"codes, 128 x 128 blocks, {order}")
    assert_bytes_equal(out_t, wc.t().contiguous(), f"transposed codes, 128 x 128 blocks, {order}")
    assert_bytes_equal(_bytes(sc), ws.repeat_interleave(128, dim=0), f"scale bytes, 128 x 128 blocks, {order}")


def test_block_cast_single_layouts_and_specials(N):
    x = _mixed((256, 384), seed=7)
    x[5, 200] = float("inf")
    x[130, 3] = float("nan")
    xd = x.cuda()
    for two_d in (False, True):
        out, sc, out_t, sc_t = N.block_cast(xd, E4M3, 0, two_d, True, True)
        o1, s1, n1, n2 = N.block_cast(xd, E4M3, 0, two_d, True, False)
        assert n1 is None and n2 is None
        assert_bytes_equal(o1, out, "row-major only: codes")
        assert_bytes_equal(s1, sc, "row-major only: scales")
        n1, n2, o2, s2 = N.block_cast(xd, E4M3, 0, two_d, False, True)
        assert_bytes_equal(o2, out_t, "transposed only: codes")
        assert_bytes_equal(s2, sc_t, "transposed only: scales")
        br = 128 if two_d else 1
        wc, ws = O.c_block_quantise(x, br, 128, E4M3, 0)
        assert_bytes_equal(out, wc, f"codes with Inf / NaN, two_d {two_d}")
    with pytest.raises(N.NativeError, match="multiples of 128"):
        N.block_cast(torch.zeros((128, 192), dtype=torch.bfloat16, device="cuda"), E4M3)


def test_blockwise_gemm_through_the_block_scaled_kernels(N):
    """x in 1 x 128 blocks, w in 128 x 128 blocks, multiplied by odl_fp8_mx_gemm_nt: the tiled kernel (few tiles) and the
    streaming kernel (4096 x 4096)."""
    for (M, N_, K) in ((256, 384, 512), (4096, 4096, 1024)):
        a = seeded_bf16((M, K), 1.0, M)
        a[:, 5] *= 50.0
        b = seeded_bf16((N_, K), 0.02, N_)
        aq, asc, _, _ = N.block_cast(a.cuda(), E4M3, 0, False, True, False)
        bq, bsc, _, _ = N.block_cast(b.cuda(), E4M3, 0, True, True, False)
        got = N.mx_gemm_nt(aq, asc, bq, bsc, E4M3, E4M3).cpu()
        ac, asb = O.c_block_quantise(a, 1, 128, E4M3, 0)
        bc, bsb = O.c_block_quantise(b, 128, 128, E4M3, 0)
        ref = O.t_mx_gemm_nt(ac, O.block_scales_as_mx(asb, 1, 128), bc, O.block_scales_as_mx(bsb, 128, 128), E4M3, E4M3)
        assert max_rel_err(got.float(), ref.float()) <= 1e-2
        assert max_rel_err(got.float(), a.float() @ b.float().t()) <= 0.1


def _block_linear_reference(x, w, dy, fmt_fwd, fmt_bwd, margin=0):
    q = lambda t, br, f: (lambda c, s: (c, O.block_scales_as_mx(s, br, 128)))(*O.c_block_quantise(t, br, 128, f, margin))
    y = O.t_mx_gemm_nt(*q(x, 1, fmt_fwd), *q(w, 128, fmt_fwd), fmt_fwd, fmt_fwd)
    dx = O.t_mx_gemm_nt(*q(dy, 1, fmt_bwd), *q(w.t().contiguous(), 128, fmt_fwd), fmt_bwd, fmt_fwd)
    dw = O.t_mx_gemm_nt(*q(dy.t().contiguous(), 1, fmt_bwd), *q(x.t().contiguous(), 1, fmt_fwd), fmt_bwd, fmt_fwd)
    return {"y": y, "dx": dx, "dw": dw}


@pytest.mark.parametrize("fmt,margin", [("hybrid", 0), ("e4m3", 1)])
def test_blockwise_linear_matches_emulation(fmt, margin):
    from optimus_dl_amd.modules import amp
    from tests.test_gpu_linear import make_linear, run_step

    M, K, N_ = 512, 1024, 768
    x, w, dy = seeded_bf16((M, K), 1.0, 0), seeded_bf16((N_, K), 0.02, 1), seeded_bf16((M, N_), 1e-3, 2)
    x[:, 7] *= 64.0
    recipe = amp.create_fp8_recipe("blockwise", fmt, margin=margin)
    assert recipe.recipe.kind == "blockwise" and recipe.recipe_type == amp.Fp8RecipeType.BLOCKWISE
    lin = make_linear(w)
    y, dx, dw = run_step(lin, recipe, x, dy)
    assert lin.fp8_calls == 1
    fb = O.E5M2 if fmt == "hybrid" else O.E4M3
    ref = _block_linear_reference(x, w, dy, O.E4M3, fb, margin)
    for name, got in (("y", y), ("dx", dx), ("dw", dw)):
        err = max_rel_err(got, ref[name])
        assert err <= 1e-2, f"{name}: {err}"
    assert max_rel_err(y, x.float() @ w.float().t()) <= 0.1
    # sizes that are not multiples of 128 run as a plain Linear
    lin2 = make_linear(seeded_bf16((192, 256), 0.02, 1))
    with recipe.autocast():
        lin2(seeded_bf16((128, 256), 1.0, 2).cuda())
    assert lin2.fp8_calls == 0


def test_blockwise_round_trip_at_full_size(N):
    """Size-independent property at a model-sized shape: nothing saturates, so every element comes back within half a
    code spacing of its block's top binade: |x - dequant| <= 2^-4 * block amax (E4M3), in both layouts."""
    rows, cols = 8192, 4096
    x = seeded_bf16((rows, cols), 1.0, 5)
    out, sc, out_t, sc_t = N.block_cast(x.cuda(), E4M3, 0, False, True, True)
    deq = O.t_mx_dequantise(out.cpu(), O.block_scales_as_mx(_bytes(sc), 1, 128), E4M3)
    v = x.float().reshape(rows, cols // 128, 128)
    assert bool(((deq.reshape(rows, cols // 128, 128) - v).abs() <= v.abs().amax(dim=2, keepdim=True) * 2.0 ** -4).all())
    deq_t = O.t_mx_dequantise(out_t.cpu(), O.block_scales_as_mx(_bytes(sc_t), 1, 128), E4M3)
    vt = x.t().float().reshape(cols, rows // 128, 128)
    assert bool(((deq_t.reshape(cols, rows // 128, 128) - vt).abs() <= vt.abs().amax(dim=2, keepdim=True) * 2.0 ** -4).all())


@pytest.mark.parametrize("seed", range(12))
def test_seeded_random_block_scaled_linears_match_the_emulation(seed):
    """Random shapes (multiples of 128, so that both block-scaled recipes take them), recipe, format and data scale:
    forward, dgrad and wgrad of the module against the emulated block-scaled Linear."""
    import random

    from optimus_dl_amd.modules import amp
    from tests.test_gpu_linear import make_linear, run_step
    from tests.test_gpu_mx import _mx_linear_reference

    rng = random.Random(seed)
    M, K, N_ = (128 * rng.randint(1, 6) for _ in range(3))
    recipe_name, fmt = rng.choice(["mxfp8", "blockwise"]), rng.choice(["hybrid", "e4m3"])
    x = seeded_bf16((M, K), 10.0 ** rng.uniform(-2, 2), 3 * seed)
    w = seeded_bf16((N_, K), 10.0 ** rng.uniform(-3, 0), 3 * seed + 1)
    dy = seeded_bf16((M, N_), 10.0 ** rng.uniform(-5, 0), 3 * seed + 2)
    x[:, rng.randrange(K)] *= 30.0
    lin = make_linear(w)
    y, dx, dw = run_step(lin, amp.create_fp8_recipe(recipe_name, fmt), x, dy)
    assert lin.fp8_calls == 1
    fb = O.E5M2 if fmt == "hybrid" else O.E4M3
    ref = _mx_linear_reference(x, w, dy, O.E4M3, fb) if recipe_name == "mxfp8" else _block_linear_reference(x, w, dy, O.E4M3, fb)
    for name, got in (("y", y), ("dx", dx), ("dw", dw)):
        err = max_rel_err(got, ref[name])
        assert err <= 1e-2, f"seed {seed} {recipe_name} {fmt} {M}x{K}x{N_} {name}: {err}"
