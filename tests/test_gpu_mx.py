"""GPU parity of the MXFP8 kernels (32-element blocks, E8M0 scale bytes) against the CPU oracle.

Codes and scale bytes must be bit-exact (C restatement and the independent torch restatement).  The block-scaled
matmul is compared with the emulated one (exact dequantisation, fp32 matmul): max|err| / max|ref| <= 1e-2 on the bf16
output, the bar of the FP8 GEMMs, and element by element on the fp32 output against what the matrix instruction's
internal adder can lose.
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
    """Gaussian values whose magnitude changes by powers of two from block to block and row to row, so that the scale
    bytes cover a wide range, plus zeros, an all-zero block and a few large outliers."""
    g = torch.Generator().manual_seed(seed)
    rows, cols = shape
    x = torch.randn(shape, generator=g)
    x = x * torch.exp2(torch.randint(-20, 20, (rows, 1), generator=g).float())
    x = x * torch.exp2(torch.randint(-6, 6, (1, cols), generator=g).float())
    x[torch.rand(shape, generator=g) < 0.05] = 0.0
    if rows >= 32 and cols >= 32:
        x[:32, :32] = 0.0                                   # a zero block in both directions
        x[rows - 1, cols - 1] = 3.0e38
        x[rows // 2, cols // 2] = -1.0e-38
    return x.bfloat16()


def N_mod():
    from optimus_dl_amd import native

    return native


CAST_SHAPES = [(32, 32), (128, 64), (64, 96), (160, 224), (256, 1024), (1024, 768), (96, 4096), (2016, 160)]


def _kstep(scales: torch.Tensor) -> torch.Tensor:
    """Row-major scale bytes [rows, blocks] -> the K-step-major layout [blocks / 4, rows, 4]."""
    rows, blocks = scales.shape
    return scales.reshape(rows, blocks // 4, 4).permute(1, 0, 2).contiguous()


@pytest.mark.parametrize("shape", CAST_SHAPES)
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_mx_cast_round_up_rule_bit_exact(N, shape, fmt, dtype):
    """The shared exponent rounded up (ODL_MX_SCALE_CEIL): codes and scale bytes of both layouts against the C oracle and
    its torch restatement, on data with block maxima on and around the 1.75 boundary where the two rules part."""
    x = _mixed(shape, seed=shape[0] * 5 + shape[1] + fmt).float()
    rows, cols = shape
    x[0, 0], x[0, 1:32] = 1.75 * 2.0 ** 3, 0.0                      # exactly fp8_max after scaling: no bump
    x[rows - 1, cols - 32], x[rows - 1, cols - 31:] = -1.7578125 * 2.0 ** -4, 0.0      # the next bf16 above: bump
    x = x.bfloat16()
    out, sc, out_t, sc_t = N.mx_cast(x.to(dtype).cuda(), fmt, want_rowmajor=True, want_transposed=True, scale_rule=N.MX_CEIL)
    sc, sc_t = N.mx_scales_rowmajor(sc), N.mx_scales_rowmajor(sc_t)
    wc, ws = O.c_mx_quantise(x, fmt, O.MX_CEIL)
    assert_bytes_equal(sc, ws, f"scale bytes {shape} fmt {fmt}")
    assert_bytes_equal(out, wc, f"codes {shape} fmt {fmt}")
    tc, ts = O.t_mx_quantise(x, fmt, O.MX_CEIL)
    assert_bytes_equal(sc, ts, f"scale bytes (torch restatement) {shape}")
    assert_bytes_equal(out, tc, f"codes (torch restatement) {shape}")
    wct, wst = O.c_mx_quantise(x.t().contiguous(), fmt, O.MX_CEIL)
    assert_bytes_equal(sc_t, wst, f"transposed scale bytes {shape} fmt {fmt}")
    assert_bytes_equal(out_t, wct, f"transposed codes {shape} fmt {fmt}")
    floor_sc = N.mx_scales_rowmajor(N.mx_cast(x.to(dtype).cuda(), fmt, scale_rule=N.MX_FLOOR)[1])
    assert int(sc[0, 0]) == int(floor_sc[0, 0]) and int(sc[rows - 1, -1]) == int(floor_sc[rows - 1, -1]) + 1


@pytest.mark.parametrize("shape", CAST_SHAPES)
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_mx_cast_both_layouts_bit_exact(N, shape, fmt, dtype):
    x = _mixed(shape, seed=shape[0] * 7 + shape[1] + fmt)
    out, sc, out_t, sc_t = N.mx_cast(x.to(dtype).cuda(), fmt, want_rowmajor=True, want_transposed=True)
    # by default the scales are K-step-major wherever the blocked axis is a multiple of 128
    assert sc.dim() == (3 if shape[1] % 128 == 0 else 2) and sc_t.dim() == (3 if shape[0] % 128 == 0 else 2)
    if sc.dim() == 3:
        assert_bytes_equal(sc, _kstep(O.c_mx_quantise(x, fmt)[1]), f"K-step-major scale bytes {shape}")
    sc, sc_t = N.mx_scales_rowmajor(sc), N.mx_scales_rowmajor(sc_t)
    wc, ws = O.c_mx_quantise(x, fmt)
    assert_bytes_equal(sc, ws, f"scale bytes {shape} fmt {fmt}")
    assert_bytes_equal(out, wc, f"codes {shape} fmt {fmt}")
    tc, ts = O.t_mx_quantise(x, fmt)
    assert_bytes_equal(sc, ts, f"scale bytes (torch restatement) {shape}")
    assert_bytes_equal(out, tc, f"codes (torch restatement) {shape}")
    wct, wst = O.c_mx_quantise(x.t().contiguous(), fmt)
    assert_bytes_equal(sc_t, wst, f"transposed scale bytes {shape} fmt {fmt}")
    assert_bytes_equal(out_t, wct, f"transposed codes {shape} fmt {fmt}")


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
def test_mx_cast_single_layouts_match_the_pair(N, fmt):
    x = _mixed((384, 320), seed=5).cuda()
    out, sc, out_t, sc_t = N.mx_cast(x, fmt, True, True)
    # the same bytes in the other storage order when the row-major layout is asked for explicitly
    r = N.mx_cast(x, fmt, True, True, layout=N.MX_ROWMAJOR)
    assert r[1].dim() == 2 and r[3].dim() == 2
    assert_bytes_equal(r[1], N.mx_scales_rowmajor(sc), "explicit row-major scales")
    assert_bytes_equal(r[3], N.mx_scales_rowmajor(sc_t), "explicit row-major transposed scales")
    assert_bytes_equal(r[0], out, "codes do not depend on the scale layout")
    o1, s1, n1, n2 = N.mx_cast(x, fmt, True, False)
    assert n1 is None and n2 is None
    assert_bytes_equal(o1, out, "row-major only: codes")
    assert_bytes_equal(s1, sc, "row-major only: scales")
    n1, n2, o2, s2 = N.mx_cast(x, fmt, False, True)
    assert n1 is None and n2 is None
    assert_bytes_equal(o2, out_t, "transposed only: codes")
    assert_bytes_equal(s2, sc_t, "transposed only: scales")


def test_mx_cast_row_major_accepts_any_row_count(N):
    x = _mixed((45, 64), seed=9)
    out, sc, _, _ = N.mx_cast(x.cuda(), E4M3, True, False)
    wc, ws = O.c_mx_quantise(x, E4M3)
    assert_bytes_equal(out, wc, "codes, 45 rows")
    assert_bytes_equal(sc, ws, "scales, 45 rows")


def test_mx_cast_specials(N):
    x = torch.zeros((64, 64), dtype=torch.bfloat16)
    x[0, 0] = float("inf")
    x[1, 40] = float("nan")
    x[2, :32] = torch.tensor(2.0 ** -130).bfloat16()         # bf16 subnormals: scale byte at the lower clamp
    x[3, 0] = 448.0
    x[3, 1] = 260.0
    x[40, 5] = -float("inf")
    for fmt in (E4M3, E5M2):
        out, sc, out_t, sc_t = N.mx_cast(x.cuda(), fmt, True, True)
        sc, sc_t = N.mx_scales_rowmajor(sc), N.mx_scales_rowmajor(sc_t)
        wc, ws = O.c_mx_quantise(x, fmt)
        assert_bytes_equal(sc, ws, f"special scale bytes fmt {fmt}")
        assert_bytes_equal(out, wc, f"special codes fmt {fmt}")
        wct, wst = O.c_mx_quantise(x.t().contiguous(), fmt)
        assert_bytes_equal(sc_t, wst, f"special transposed scale bytes fmt {fmt}")
        assert_bytes_equal(out_t, wct, f"special transposed codes fmt {fmt}")
        assert int(sc[0, 0]) == 255 and int(sc[1, 1]) == 255 and int(sc[5, 0]) == 0


def _every_bf16_pattern(order: str) -> torch.Tensor:
    """All 65536 bf16 bit patterns as a [128, 512] matrix: sorted by magnitude (the neighbours that share a block are
    close to its amax, where the conversion saturates) or shuffled (most elements far below the block amax: subnormal
    codes, underflow to zero; about one block in eight holds an Inf or a NaN)."""
    import numpy as np

    pats = np.arange(65536, dtype=np.uint32)
    if order == "sorted":
        pats = pats[np.argsort(pats & 0x7fff, kind="stable")]
    else:
        pats = pats[np.random.default_rng(1).permutation(65536)]
    return torch.from_numpy(pats.astype(np.uint16).view(np.int16).copy()).view(torch.bfloat16).reshape(128, 512)


@pytest.mark.parametrize("order", ["sorted", "shuffled"])
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_mx_cast_every_bf16_pattern(N, fmt, order, dtype):
    x = _every_bf16_pattern(order)
    out, sc, out_t, sc_t = N.mx_cast(x.to(dtype).cuda(), fmt, want_rowmajor=True, want_transposed=True)
    sc, sc_t = N.mx_scales_rowmajor(sc), N.mx_scales_rowmajor(sc_t)
    wc, ws = O.c_mx_quantise(x, fmt)
    assert_bytes_equal(sc, ws, f"scale bytes, {order}")
    assert_bytes_equal(out, wc, f"codes, {order}")
    wct, wst = O.c_mx_quantise(x.t().contiguous(), fmt)
    assert_bytes_equal(sc_t, wst, f"transposed scale bytes, {order}")
    assert_bytes_equal(out_t, wct, f"transposed codes, {order}")


@pytest.mark.parametrize("fmt", [E4M3, E5M2])
def test_mx_cast_fp32_inputs_around_every_rounding_midpoint(N, fmt):
    """fp32 inputs on, one ulp below and one ulp above every midpoint between neighbouring FP8 values (a tie goes to
    the even code, one fp32 ulp decides the others) and around the largest value (saturation), at several shared
    exponents.  Every block holds 31 of them and an anchor just below the next binade that fixes the block's scale."""
    top = 0x7E if fmt == E4M3 else 0x7B                                  # code of the largest finite value
    vals = O.t_decode(torch.arange(0, top + 1, dtype=torch.uint8), fmt).double()
    step_up = vals[-1] - vals[-2]
    mids = torch.cat([(vals[:-1] + vals[1:]) / 2, (vals[-1] + step_up / 2).reshape(1)]).float()
    assert bool((mids.double() == torch.cat([(vals[:-1] + vals[1:]) / 2, (vals[-1] + step_up / 2).reshape(1)])).all())
    inf = torch.tensor(float("inf"))
    cands = torch.cat([torch.nextafter(mids, -inf), mids, torch.nextafter(mids, inf)])
    cands = torch.cat([cands, -cands])
    pad = (-cands.numel()) % 31
    cands = torch.cat([cands, cands[:pad]]).reshape(-1, 31)
    emax = O.MX_EMAX[fmt]
    blocks = []
    for se in (-30, -3, 0, 11, 40):
        anchor = torch.full((cands.shape[0], 1), 1.984375 * 2.0 ** emax)
        blk = torch.cat([cands[:, :7], anchor, cands[:, 7:]], dim=1)
        blocks.append(torch.ldexp(blk, torch.tensor(se)))
    x = torch.cat(blocks)                                                # [blocks, 32] fp32
    x = torch.cat([x, x[: (-x.shape[0]) % 64]])                          # a row count the transposed call accepts
    want_codes, want_scales = O.t_mx_quantise(x, fmt)
    assert sorted(set(int(b) for b in want_scales.flatten())) == [127 + se for se in (-30, -3, 0, 11, 40)]
    out, sc, _, _ = N.mx_cast(x.cuda(), fmt, want_rowmajor=True, want_transposed=False)
    assert_bytes_equal(N.mx_scales_rowmajor(sc), want_scales, "scale bytes")
    assert_bytes_equal(out, want_codes, "codes of fp32 inputs around the midpoints")
    # the other direction: the same blocks run down the columns of the transposed matrix
    _, _, out_t, sc_t = N.mx_cast(x.t().contiguous().cuda(), fmt, want_rowmajor=False, want_transposed=True)
    assert_bytes_equal(N.mx_scales_rowmajor(sc_t), want_scales, "scale bytes, blocks down the columns")
    assert_bytes_equal(out_t, want_codes, "codes, blocks down the columns")
    # ties really are among the inputs and go to the even code
    tie = torch.ldexp(mids[5], torch.tensor(0)).item()
    row = torch.tensor([tie] + [1.984375 * 2.0 ** emax] + [0.0] * 30).reshape(1, 32)
    code = int(O.t_mx_quantise(row, fmt)[0][0, 0])
    assert code % 2 == 0 and code in (5, 6)


def test_mx_cast_rejects_bad_shapes(N):
    with pytest.raises(N.NativeError, match="multiple of 32"):
        N.mx_cast(torch.zeros((32, 48), dtype=torch.bfloat16, device="cuda"), E4M3, True, False)
    with pytest.raises(N.NativeError, match="multiple of 32"):
        N.mx_cast(torch.zeros((48, 64), dtype=torch.bfloat16, device="cuda"), E4M3, False, True)
    with pytest.raises(N.NativeError, match="multiple of 128"):
        N.mx_cast(torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda"), E4M3, True, False, layout=N.MX_KSTEP)
    out = N.mx_cast(torch.zeros((0, 64), dtype=torch.bfloat16, device="cuda"), E4M3, True, True)
    assert out[0].shape == (0, 64) and out[2].shape == (64, 0)


# ------------------------------------------------------------------------------------------------ GEMM
def _operands(M, N_, K, fa, fb, seed):
    a = _mixed((M, K), seed)
    b = _mixed((N_, K), seed + 1)
    # keep the products inside fp32 / bf16 range: the outliers of _mixed are for the cast tests
    a = a.float().clamp(-1e4, 1e4).bfloat16()
    b = b.float().clamp(-1e4, 1e4).bfloat16()
    ac, asc = O.c_mx_quantise(a, fa)
    bc, bsc = O.c_mx_quantise(b, fb)
    return ac, asc, bc, bsc


def _assert_within_hardware_sum(got32, ac, asc, bc, bsc, fa, fb, bias=None):
    """Element by element against the exact (float64) block-scaled dot product.  The FP8 MFMA adds the 8 products of two
    consecutive operand dwords in an adder aligned to the largest of them that keeps 13 bits below it (measured: a
    product 2^-14 of the largest in its group of 8 is dropped, 2^-13 is kept; between groups the sum is fp32), so
    |error| <= 7 * 2^-14 * sum|a||b| plus fp32 rounding; 2^-10 * sum|a||b| is the bar here."""
    A, B = O.t_mx_dequantise(ac, asc, fa).double(), O.t_mx_dequantise(bc, bsc, fb).double()
    exact, absdot = A @ B.t(), A.abs() @ B.abs().t()
    if bias is not None:
        exact, absdot = exact + bias.double(), absdot + bias.double().abs()
    err = (got32.double() - exact).abs()
    worst = float((err / absdot.clamp_min(1e-30)).max())
    assert bool((err <= absdot * 2.0 ** -10 + 1e-30).all()), worst      # 1e-30: results below the fp32 range become 0


GEMM_SHAPES = [
    (32, 32, 32), (32, 32, 96), (64, 96, 160), (100, 72, 224), (7, 13, 64), (16, 24, 256),   # plain kernel (K % 128 != 0 or tiny)
    (128, 128, 128), (256, 256, 512), (384, 640, 1024), (200, 136, 256), (130, 70, 384),  # 128 x 128 tiles, edges
    (4096, 4096, 256), (4100, 4232, 128),                                                # 256 x 256 tiles, interior and edges
    (4096, 4096, 512), (4224, 4480, 640), (3968, 4352, 1152),      # K-step-major: the streaming kernel, also with half tiles at the edges and an odd number of K steps
]


# every format pair at the small shapes; the large ones once, one of them also with E5M2 gradients
GEMM_CASES = [(shape, fmts) for shape in GEMM_SHAPES for fmts in ((E4M3, E4M3), (E5M2, E4M3), (E4M3, E5M2))
              if shape[0] * shape[1] <= 4096 * 1024 or fmts == (E4M3, E4M3) or (shape == (4224, 4480, 640) and fmts == (E5M2, E4M3))]


@pytest.mark.parametrize("shape,fmts", GEMM_CASES)
def test_mx_gemm_matches_emulation(N, shape, fmts):
    M, N_, K = shape
    fa, fb = fmts
    ac, asc, bc, bsc = _operands(M, N_, K, fa, fb, seed=M + N_ + K)
    ref_bf16, ref_f32 = O.t_mx_gemm_nt(ac, asc, bc, bsc, fa, fb, want_f32=True)
    # every scale layout the shape allows: row-major always, K-step-major when K is a multiple of 128
    for kstep in ((False, True) if K % 128 == 0 else (False,)):
        sa_d, sb_d = (_kstep(asc).cuda(), _kstep(bsc).cuda()) if kstep else (asc.cuda(), bsc.cuda())
        got32 = N.mx_gemm_nt(ac.cuda(), sa_d, bc.cuda(), sb_d, fa, fb, out_dtype=torch.float32).cpu()
        assert got32.shape == (M, N_)
        _assert_within_hardware_sum(got32, ac, asc, bc, bsc, fa, fb)
        got = N.mx_gemm_nt(ac.cuda(), sa_d, bc.cuda(), sb_d, fa, fb).cpu()
        assert max_rel_err(got.float(), ref_bf16.float()) <= 1e-2
        assert torch.equal(got, got32.bfloat16())


@pytest.mark.parametrize("k_steps", [1, 2, 3, 4, 5, 6, 7, 9, 13])
def test_mx_gemm_few_tile_outputs_at_every_pipeline_depth(N, k_steps):
    """The four-stage form of the tiled kernel (outputs of at most one 128 x 128 tile per compute unit): every length of
    its prologue and tail, with scale bytes that differ from K step to K step so that a scale dword that arrives with
    the wrong stage shows."""
    M, N_, K = 384, 200, 128 * k_steps
    ac, asc, bc, bsc = _operands(M, N_, K, E5M2, E4M3, seed=500 + k_steps)
    ref_bf16, _ = O.t_mx_gemm_nt(ac, asc, bc, bsc, E5M2, E4M3, want_f32=True)
    assert len(set(int(b) for b in asc[0])) > 1 or k_steps == 1
    for sa_d, sb_d in ((asc.cuda(), bsc.cuda()), (_kstep(asc).cuda(), _kstep(bsc).cuda())):
        got32 = N.mx_gemm_nt(ac.cuda(), sa_d, bc.cuda(), sb_d, E5M2, E4M3, out_dtype=torch.float32).cpu()
        _assert_within_hardware_sum(got32, ac, asc, bc, bsc, E5M2, E4M3)
        got = N.mx_gemm_nt(ac.cuda(), sa_d, bc.cuda(), sb_d, E5M2, E4M3).cpu()
        assert max_rel_err(got.float(), ref_bf16.float()) <= 1e-2


def test_mx_gemm_small_case_against_the_c_oracle_and_bias(N):
    M, N_, K = 48, 40, 96
    ac, asc, bc, bsc = _operands(M, N_, K, E4M3, E4M3, seed=3)
    bias = torch.randn(N_)
    c_bf16, c_f32 = O.c_mx_gemm_nt(ac, asc, bc, bsc, E4M3, E4M3, bias)
    got = N.mx_gemm_nt(ac.cuda(), asc.cuda(), bc.cuda(), bsc.cuda(), E4M3, E4M3, bias=bias.cuda(), out_dtype=torch.float32).cpu()
    assert max_rel_err(got, c_f32) <= 2e-3
    _assert_within_hardware_sum(got, ac, asc, bc, bsc, E4M3, E4M3, bias)
    M, N_, K = 256, 384, 256
    ac, asc, bc, bsc = _operands(M, N_, K, E4M3, E4M3, seed=4)
    bias = torch.randn(N_)
    got = N.mx_gemm_nt(ac.cuda(), asc.cuda(), bc.cuda(), bsc.cuda(), E4M3, E4M3, bias=bias.cuda(), out_dtype=torch.float32).cpu()
    _assert_within_hardware_sum(got, ac, asc, bc, bsc, E4M3, E4M3, bias)
    gotb = N.mx_gemm_nt(ac.cuda(), asc.cuda(), bc.cuda(), bsc.cuda(), E4M3, E4M3, bias=bias.cuda()).cpu()
    assert torch.equal(gotb, got.bfloat16())


def test_mx_gemm_streaming_kernel_with_bias_and_repeated_launches(N):
    """K-step-major scales at a shape the streaming kernel takes: bias, fp32 and bf16 outputs, and the same launch three
    times (a persistent kernel that leaves LDS or descriptors in a bad state shows on the second one)."""
    M, N_, K = 4096, 4096, 768
    ac, asc, bc, bsc = _operands(M, N_, K, E5M2, E4M3, seed=17)
    bias = torch.randn(N_)
    dev = [t.cuda() for t in (ac, _kstep(asc), bc, _kstep(bsc))]
    first = None
    for _ in range(3):
        got = N.mx_gemm_nt(dev[0], dev[1], dev[2], dev[3], E5M2, E4M3, bias=bias.cuda(), out_dtype=torch.float32)
        first = got if first is None else first
        assert torch.equal(got, first)
    _assert_within_hardware_sum(first.cpu(), ac, asc, bc, bsc, E5M2, E4M3, bias)
    gotb = N.mx_gemm_nt(dev[0], dev[1], dev[2], dev[3], E5M2, E4M3, bias=bias.cuda())
    assert torch.equal(gotb, first.bfloat16())
    # and the row-major route (LDS-tiled kernel) sums the same blocks in another order: close, not equal
    rm = N.mx_gemm_nt(dev[0], asc.cuda(), dev[2], bsc.cuda(), E5M2, E4M3, bias=bias.cuda(), out_dtype=torch.float32)
    assert max_rel_err(rm.cpu(), first.cpu()) <= 1e-3


def test_mx_gemm_block_scales_act_per_block(N):
    """Raising one scale byte of A by 1 doubles exactly that block's contribution: with every other block zeroed the
    output doubles bit for bit; and a NaN scale byte poisons its row only."""
    M, N_, K = 128, 128, 256
    ac, asc, bc, bsc = _operands(M, N_, K, E4M3, E4M3, seed=11)
    keep = torch.zeros_like(ac)
    keep[:, 64:96] = ac[:, 64:96]
    base = N.mx_gemm_nt(keep.cuda(), asc.cuda(), bc.cuda(), bsc.cuda(), E4M3, E4M3, out_dtype=torch.float32).cpu()
    asc2 = asc.clone()
    asc2[:, 2] = (asc2[:, 2].int() + 1).clamp(max=254).to(torch.uint8)
    grown = asc2[:, 2] != asc[:, 2]
    twice = N.mx_gemm_nt(keep.cuda(), asc2.cuda(), bc.cuda(), bsc.cuda(), E4M3, E4M3, out_dtype=torch.float32).cpu()
    assert torch.equal(twice[grown], 2 * base[grown])
    asc3 = asc.clone()
    asc3[5, 7] = 255
    out = N.mx_gemm_nt(ac.cuda(), asc3.cuda(), bc.cuda(), bsc.cuda(), E4M3, E4M3, out_dtype=torch.float32).cpu()
    assert bool(torch.isnan(out[5]).all()) and not bool(torch.isnan(out[:5]).any()) and not bool(torch.isnan(out[6:]).any())


def test_mx_round_trip_error_bound_at_full_size(N):
    """Size-independent property at a model-sized shape: |x - dequant(quant(x))| <= 2^-3 * block amax for E4M3 (the
    scaled amax lies in [256, 512): up to 448 the spacing is 32, above it the value saturates, at most 64 away), in
    both layouts."""
    rows, cols = 4096, 4096
    x = seeded_bf16((rows, cols), std=1.0, seed=21)
    out, sc, out_t, sc_t = N.mx_cast(x.cuda(), E4M3, True, True)
    sc, sc_t = N.mx_scales_rowmajor(sc), N.mx_scales_rowmajor(sc_t)
    deq = O.t_mx_dequantise(out.cpu(), sc.cpu(), E4M3)
    v = x.float().reshape(rows, cols // 32, 32)
    amax = v.abs().amax(dim=2, keepdim=True)
    err = (deq.reshape(rows, cols // 32, 32) - v).abs()
    assert bool((err <= amax * 2.0 ** -3).all())
    deq_t = O.t_mx_dequantise(out_t.cpu(), sc_t.cpu(), E4M3)
    vt = x.t().float().reshape(cols, rows // 32, 32)
    amax_t = vt.abs().amax(dim=2, keepdim=True)
    assert bool(((deq_t.reshape(cols, rows // 32, 32) - vt).abs() <= amax_t * 2.0 ** -3).all())


# ------------------------------------------------------------------------------------------------ the Linear
def _mx_linear_reference(x, w, dy, fmt_fwd, fmt_bwd, bias=None, rule=O.MX_CEIL):
    """The three GEMMs of a Linear under MXFP8, emulated: every operand quantised along the axis its GEMM contracts, the
    shared exponents by `rule` (the recipe's default is the round-up rule)."""
    q = lambda t, fmt: O.c_mx_quantise(t, fmt, rule)
    y = O.t_mx_gemm_nt(*q(x, fmt_fwd), *q(w, fmt_fwd), fmt_fwd, fmt_fwd, bias=bias)
    gq, gs = q(dy, fmt_bwd)
    wtq, wts = q(w.t().contiguous(), fmt_fwd)
    dx = O.t_mx_gemm_nt(gq, gs, wtq, wts, fmt_bwd, fmt_fwd)
    gtq, gts = q(dy.t().contiguous(), fmt_bwd)
    xtq, xts = q(x.t().contiguous(), fmt_fwd)
    dw = O.t_mx_gemm_nt(gtq, gts, xtq, xts, fmt_bwd, fmt_fwd)
    return {"y": y, "dx": dx, "dw": dw}


@pytest.mark.parametrize("fmt", ["hybrid", "e4m3"])
@pytest.mark.parametrize("shape", [(512, 1024, 768), (96, 160, 224)])
def test_mxfp8_linear_matches_emulation(fmt, shape):
    from optimus_dl_amd.modules import amp
    from tests.test_gpu_linear import make_linear, run_step

    M, K, N_ = shape
    x, w, dy = seeded_bf16((M, K), 1.0, 0), seeded_bf16((N_, K), 0.02, 1), seeded_bf16((M, N_), 1e-3, 2)
    x[:, 7] *= 64.0                                           # an outlier channel: block scales isolate it
    recipe = amp.create_fp8_recipe("mxfp8", fmt)
    assert recipe.recipe.kind == "mxfp8" and recipe.recipe_type == amp.Fp8RecipeType.MXFP8
    lin = make_linear(w)
    y, dx, dw = run_step(lin, recipe, x, dy)
    assert lin.fp8_calls == 1
    fb = O.E5M2 if fmt == "hybrid" else O.E4M3
    ref = _mx_linear_reference(x, w, dy, O.E4M3, fb)
    for name, got in (("y", y), ("dx", dx), ("dw", dw)):
        assert got.dtype == torch.bfloat16
        err = max_rel_err(got, ref[name])
        assert err <= 1e-2, f"{name}: {err}"
    # and it is a Linear: near the bf16 product
    want = x.float() @ w.float().t()
    assert max_rel_err(y, want) <= 0.1
    # the same under the specification's floor rule, which lets a block amax in the top eighth of its binade saturate (up
    # to 12.5 % off on that element, which the outlier channel makes visible)
    floor = amp.create_fp8_recipe("mxfp8", fmt, mx_scale_rule="floor")
    assert floor.recipe.mx_scale_rule == N_mod().MX_FLOOR and recipe.recipe.mx_scale_rule == N_mod().MX_CEIL
    lin2 = make_linear(w)
    y2, dx2, dw2 = run_step(lin2, floor, x, dy)
    ref2 = _mx_linear_reference(x, w, dy, O.E4M3, fb, rule=O.MX_FLOOR)
    for name, got in (("y", y2), ("dx", dx2), ("dw", dw2)):
        assert max_rel_err(got, ref2[name]) <= 1e-2, name
    assert max_rel_err(y2, want) <= 0.2
    assert not torch.equal(y, y2)


def test_mxfp8_linear_bias_fp32_weights_and_weight_cache():
    from optimus_dl_amd.modules import amp
    from tests.test_gpu_linear import make_linear

    B, S, K, N_ = 2, 64, 256, 512
    x = seeded_bf16((B * S, K), 1.0, 3)
    # fp32 master weights whose values bf16 holds exactly, so that the oracle (bf16 input) quantises the same numbers
    w32 = (torch.randn(N_, K, generator=torch.Generator().manual_seed(4)) * 0.02).bfloat16().float()
    bias = torch.randn(N_, generator=torch.Generator().manual_seed(5)) * 0.1
    dy = seeded_bf16((B * S, N_), 1e-2, 6)
    recipe = amp.create_fp8_recipe("mxfp8", "hybrid")
    lin = make_linear(w32, bias, dtype=torch.float32)
    xd = x.cuda().reshape(B, S, K).requires_grad_(True)
    with amp.fp8_autocast(torch.device("cuda"), recipe, dtype=torch.bfloat16):
        y = lin(xd)
    assert y.shape == (B, S, N_) and y.dtype == torch.bfloat16
    with amp.fp8_backward(recipe):
        y.backward(dy.cuda().reshape(B, S, N_))
    ref = _mx_linear_reference(x, w32.bfloat16(), dy, O.E4M3, O.E5M2, bias=bias)
    assert max_rel_err(y.reshape(B * S, N_), ref["y"]) <= 1e-2
    assert max_rel_err(xd.grad.reshape(B * S, K), ref["dx"]) <= 1e-2
    assert lin.weight.grad.dtype == torch.float32 and max_rel_err(lin.weight.grad, ref["dw"]) <= 1e-2
    want_db = dy.float().sum(dim=0)
    assert max_rel_err(lin.bias.grad, want_db) <= 1e-3
    # the weight's codes are kept while the Parameter is unchanged, and made again after an update
    first = lin._wcache_rowwise["mx"][1]
    with recipe.autocast():
        lin(xd.detach())
    assert lin._wcache_rowwise["mx"][1] is first
    with torch.no_grad():
        lin.weight.mul_(2.0)
    with recipe.autocast():
        y2 = lin(xd.detach())
    assert lin._wcache_rowwise["mx"][1] is not first
    assert max_rel_err(y2.reshape(B * S, N_) - bias.cuda().bfloat16(), 2 * (ref["y"].cuda() - bias.cuda().bfloat16())) <= 3e-2


def test_mxfp8_linear_falls_back_for_sizes_that_are_not_multiples_of_32():
    from optimus_dl_amd.modules import amp
    from tests.test_gpu_linear import make_linear

    recipe = amp.create_fp8_recipe("mxfp8", "hybrid")
    lin = make_linear(seeded_bf16((48, 64), 0.02, 1))             # 48 outputs
    with recipe.autocast():
        y = lin(seeded_bf16((32, 64), 1.0, 2).cuda())
    assert lin.fp8_calls == 0 and y.shape == (32, 48)
    lin2 = make_linear(seeded_bf16((64, 64), 0.02, 1))
    with recipe.autocast():
        lin2(seeded_bf16((48, 64), 1.0, 3).cuda())                # 48 tokens
    assert lin2.fp8_calls == 0
    with recipe.autocast():
        lin2(seeded_bf16((64, 64), 1.0, 3).cuda())
    assert lin2.fp8_calls == 1


def test_mxfp8_shared_input_is_quantised_once():
    from optimus_dl_amd.modules import amp
    from optimus_dl_amd import native
    from tests.test_gpu_linear import make_linear

    recipe = amp.create_fp8_recipe("mxfp8", "hybrid")
    a, b = make_linear(seeded_bf16((64, 128), 0.02, 1)), make_linear(seeded_bf16((96, 128), 0.02, 2))
    x = seeded_bf16((32, 128), 1.0, 3).cuda().requires_grad_(True)
    calls = []
    real = native.mx_cast
    native.mx_cast = lambda t, *a_, **k_: (calls.append(tuple(t.shape)), real(t, *a_, **k_))[1]
    try:
        with recipe.autocast():
            ya, yb = a(x), b(x)
    finally:
        native.mx_cast = real
    assert calls.count((32, 128)) == 1 and len(calls) == 3, calls   # x once, each weight once
    with recipe.backward():
        (ya.sum() + yb.sum()).backward()
    assert x.grad is not None and a.weight.grad is not None and b.weight.grad is not None


@pytest.mark.parametrize("shape", [(768, 768, 16384), (2304, 768, 16384), (1024, 1024, 16384)])
def test_mx_gemm_split_over_k_matches_the_single_launch(N, shape):
    """Weight-gradient shapes of small models: few output tiles, a long contraction.  The wrapper cuts K into runs
    (odl_fp8_mx_gemm_splitk); the result is the emulated product, and equal to a single launch up to fp32 rounding of
    the partial sums."""
    M, N_, K = shape
    a = seeded_bf16((M, K), 1e-3, 31)
    b = seeded_bf16((N_, K), 1.0, 32)
    aq, asc, _, _ = N.mx_cast(a.cuda(), E5M2, True, False)
    bq, bsc, _, _ = N.mx_cast(b.cuda(), E4M3, True, False)
    assert N.gemm_split_count(M, N_, K) > 1, "the shape is meant to be split"
    bias = torch.randn(N_).cuda()
    real = N.load().odl_fp8_mx_gemm_splitk
    got = N.mx_gemm_nt(aq, asc, bq, bsc, E5M2, E4M3, bias=bias, out_dtype=torch.float32)
    N.split_k = False
    try:
        single = N.mx_gemm_nt(aq, asc, bq, bsc, E5M2, E4M3, bias=bias, out_dtype=torch.float32)
    finally:
        N.split_k = True
    assert max_rel_err(got.cpu(), single.cpu()) <= 1e-5
    ref = O.t_mx_gemm_nt(aq.cpu(), N.mx_scales_rowmajor(asc).cpu(), bq.cpu(), N.mx_scales_rowmajor(bsc).cpu(), E5M2, E4M3,
                         bias=bias.cpu(), want_f32=True)[1]
    assert max_rel_err(got.cpu(), ref) <= 1e-3
    gotb = N.mx_gemm_nt(aq, asc, bq, bsc, E5M2, E4M3, bias=bias)
    assert torch.equal(gotb, got.bfloat16())
    # called directly with a workspace that is too small: refused
    ws = torch.empty(16, dtype=torch.float32, device="cuda")
    out = torch.empty((M, N_), dtype=torch.float32, device="cuda")
    rc = real(aq.data_ptr(), asc.data_ptr(), bq.data_ptr(), bsc.data_ptr(), M, N_, K, E5M2, E4M3, None, out.data_ptr(), 1, 0, 4,
              ws.data_ptr(), 64, None)
    assert rc != 0
