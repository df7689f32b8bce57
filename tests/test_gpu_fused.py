"""GPU parity: SwiGLU forward / backward and RMSNorm producers vs the CPU oracle, bit for bit,
through the C ABI; their partial maxima fed to the dynamic cast give the codes the plain
two-launch quantisation gives."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import assert_bytes_equal, assert_f32_bits_equal, seeded_bf16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def N():
    from optimus_dl_amd import native

    native.load()
    return native


def all_bf16() -> torch.Tensor:
    bits = np.arange(65536, dtype=np.uint16)
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def assert_bf16_equal(got: torch.Tensor, want: torch.Tensor, what: str):
    """Same bits, except that any NaN matches any NaN."""
    got, want = got.cpu().contiguous(), want.cpu().contiguous()
    assert got.shape == want.shape and got.dtype == want.dtype == torch.bfloat16, (what, got.shape, want.shape)
    nan_g, nan_w = torch.isnan(got), torch.isnan(want)
    ok = (got.view(torch.int16) == want.view(torch.int16)) | (nan_g & nan_w)
    if not bool(ok.all()):
        bad = (~ok).nonzero()
        first = [(tuple(i.tolist()), float(got[tuple(i)]), float(want[tuple(i)])) for i in bad[:6]]
        raise AssertionError(f"{what}: {bad.shape[0]} of {got.numel()} values differ; first (index, got, want): {first}")


def parts_max(parts: torch.Tensor) -> torch.Tensor:
    p = parts.cpu()
    return torch.tensor(float("nan")) if bool(torch.isnan(p).any()) else p.max()


# ---------------------------------------------------------------------- SwiGLU
def test_swiglu_forward_every_gate_pattern(N):
    g = all_bf16().reshape(256, 256)
    for seed, std in ((0, 1.0), (1, 30.0)):
        u = seeded_bf16((256, 256), std, seed)
        h, parts = N.swiglu_amax_parts(g.cuda(), u.cuda())
        assert_bf16_equal(h, O.c_swiglu_fwd(g, u), f"swiglu fwd, all gate patterns, up std {std}")
        assert torch.isnan(parts_max(parts))                      # NaN gates are among the inputs


@pytest.mark.parametrize("shape", [(16, 24), (1, 8), (1000, 8), (257, 96), (3, 5, 64), (2048, 1408)])
def test_swiglu_forward_bit_exact_and_parts(N, shape):
    g, u = seeded_bf16(shape, 1.5, 11), seeded_bf16(shape, 1.0, 12)
    h, parts = N.swiglu_amax_parts(g.cuda(), u.cuda())
    want = O.c_swiglu_fwd(g, u)
    assert_bf16_equal(h, want, f"swiglu fwd {shape}")
    assert_f32_bits_equal(parts_max(parts).reshape(1), want.float().abs().max().reshape(1), f"swiglu fwd parts {shape}")
    assert parts.numel() == N.AMAX_PARTS


@pytest.mark.parametrize("shape", [(16, 24), (1, 8), (1000, 8), (257, 96), (1024, 1408)])
def test_swiglu_backward_bit_exact_and_parts(N, shape):
    g, u, dh = seeded_bf16(shape, 1.5, 21), seeded_bf16(shape, 1.0, 22), seeded_bf16(shape, 1e-3, 23)
    dg, du, pg, pu = N.swiglu_bwd_amax_parts(dh.cuda(), g.cuda(), u.cuda())
    wg, wu = O.c_swiglu_bwd(dh, g, u)
    assert_bf16_equal(dg, wg, f"swiglu bwd d_gate {shape}")
    assert_bf16_equal(du, wu, f"swiglu bwd d_up {shape}")
    assert_f32_bits_equal(parts_max(pg).reshape(1), wg.float().abs().max().reshape(1), "d_gate parts")
    assert_f32_bits_equal(parts_max(pu).reshape(1), wu.float().abs().max().reshape(1), "d_up parts")


def test_swiglu_backward_every_gate_pattern(N):
    g = all_bf16().reshape(256, 256)
    u, dh = seeded_bf16((256, 256), 2.0, 3), seeded_bf16((256, 256), 0.01, 4)
    dg, du, _, _ = N.swiglu_bwd_amax_parts(dh.cuda(), g.cuda(), u.cuda())
    wg, wu = O.c_swiglu_bwd(dh, g, u)
    assert_bf16_equal(dg, wg, "swiglu bwd d_gate, all gate patterns")
    assert_bf16_equal(du, wu, "swiglu bwd d_up, all gate patterns")


def test_swiglu_special_values(N):
    g = torch.tensor([0.0, -0.0, 3.0, -3.0, 90.0, -90.0, float("inf"), float("-inf")], dtype=torch.bfloat16)
    u = torch.tensor([5.0, 5.0, 0.0, -0.0, 2.0, 2.0, 1.0, 1.0], dtype=torch.bfloat16)
    h, parts = N.swiglu_amax_parts(g.cuda(), u.cuda())
    assert_bf16_equal(h, O.c_swiglu_fwd(g, u), "swiglu specials")
    assert torch.isnan(parts_max(parts))                          # -inf * 0 is NaN, as in eager arithmetic
    z = torch.zeros((4, 8), dtype=torch.bfloat16)
    h, parts = N.swiglu_amax_parts(z.cuda(), z.cuda())
    assert float(h.abs().max()) == 0.0 and float(parts.max()) == 0.0
    e = torch.empty((0, 8), dtype=torch.bfloat16).cuda()
    h, parts = N.swiglu_amax_parts(e, e)
    assert h.numel() == 0 and float(parts.abs().max()) == 0.0


def test_swiglu_refusals(N):
    a = torch.zeros((3, 5), dtype=torch.bfloat16).cuda()
    with pytest.raises(N.NativeError, match="multiple of 8"):
        N.swiglu_amax_parts(a, a)
    with pytest.raises(N.NativeError, match="bf16"):
        N.swiglu_amax_parts(a.float(), a.float())
    with pytest.raises(N.NativeError, match="differ"):
        N.swiglu_amax_parts(torch.zeros((2, 8), dtype=torch.bfloat16).cuda(), torch.zeros((4, 8), dtype=torch.bfloat16).cuda())
    with pytest.raises(N.NativeError, match="GPU only"):
        N.swiglu_amax_parts(torch.zeros((2, 8), dtype=torch.bfloat16), torch.zeros((2, 8), dtype=torch.bfloat16))


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_swiglu_parts_feed_the_dynamic_cast(N, fmt):
    shape = (512, 384)
    g, u = seeded_bf16(shape, 2.0, 31), seeded_bf16(shape, 1.0, 32)
    h, parts = N.swiglu_amax_parts(g.cuda(), u.cuda())
    q, q_t, amax, scale, scale_inv = N.cast_dynamic(h, parts, fmt, 0)
    q2, q2_t, amax2, scale2, scale_inv2 = N.quantize_dynamic(h, fmt, 0)
    assert_bytes_equal(q, q2, "codes with producer parts")
    assert_bytes_equal(q_t, q2_t, "transposed codes with producer parts")
    assert_f32_bits_equal(torch.cat([amax, scale, scale_inv]), torch.cat([amax2, scale2, scale_inv2]), "amax/scale")
    want_h = O.c_swiglu_fwd(g, u)
    s = O.c_scale(float(want_h.float().abs().max()), fmt)
    assert_bytes_equal(q, O.c_cast(want_h, s, fmt), "codes vs oracle")


# --------------------------------------------------------------------- RMSNorm
# many rows only for the narrow-row kernels: the oracle is a scalar loop
@pytest.mark.parametrize("rows,cols", [(r, c) for c in (8, 64, 96, 128, 256, 264, 520, 1024, 4096, 8192)
                                       for r in (1, 37, 70001) if r < 1000 or c <= 264])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_bit_exact(N, rows, cols, dtype):
    gen = torch.Generator().manual_seed(rows * 100003 + cols)
    x = (torch.randn((rows, cols), generator=gen) * 2.5).to(dtype)
    w = (torch.randn(cols, generator=gen) * 0.3 + 1.0)
    eps = 1e-5
    y, rstd, parts = N.rmsnorm_amax_parts(x.cuda(), w.cuda(), eps)
    wy, wr = O.c_rmsnorm(x, w, eps)
    assert_f32_bits_equal(rstd, wr, f"rmsnorm rstd {rows}x{cols} {dtype}")
    assert_bf16_equal(y, wy, f"rmsnorm y {rows}x{cols} {dtype}")
    assert_f32_bits_equal(parts_max(parts).reshape(1), wy.float().abs().max().reshape(1), "rmsnorm parts")


def test_rmsnorm_many_rows_and_leading_dims(N):
    x = seeded_bf16((4, 700, 256), 1.0, 9)                        # 2800 rows: more than one trip per wave
    w = torch.linspace(0.5, 1.5, 256)
    y, rstd, parts = N.rmsnorm_amax_parts(x.cuda(), w.cuda(), 1e-6)
    wy, wr = O.c_rmsnorm(x, w, 1e-6)
    assert y.shape == x.shape and rstd.shape == x.shape[:-1]
    assert_bf16_equal(y, wy, "rmsnorm 3-D")
    assert_f32_bits_equal(rstd, wr, "rmsnorm 3-D rstd")
    q, _, amax, _, _ = N.cast_dynamic(y.reshape(-1, 256), parts, O.E4M3, 0, want_transposed=False)
    q2, _, amax2, _, _ = N.quantize_dynamic(y.reshape(-1, 256), O.E4M3, 0, want_transposed=False)
    assert_bytes_equal(q, q2, "rmsnorm parts feed the cast")
    assert_f32_bits_equal(amax, amax2, "rmsnorm amax")


def test_rmsnorm_exact_case_and_refusals(N):
    rows, cols = 6, 136
    sign = torch.where(torch.arange(cols) % 3 == 0, -1.0, 1.0)
    x = torch.stack([sign * 2.0 ** r for r in range(rows)]).bfloat16()
    w = torch.arange(1, cols + 1, dtype=torch.float32) / 8.0
    y, rstd, _ = N.rmsnorm_amax_parts(x.cuda(), w.cuda(), 0.0)
    assert torch.equal(rstd.cpu(), torch.tensor([2.0 ** -r for r in range(rows)]))
    assert torch.equal(y.cpu(), (sign * w).bfloat16().expand(rows, cols))
    with pytest.raises(N.NativeError, match="multiple of 8"):
        N.rmsnorm_amax_parts(torch.zeros((4, 12), dtype=torch.bfloat16).cuda(), torch.ones(12).cuda(), 1e-5)
    with pytest.raises(N.NativeError, match="8192"):
        N.rmsnorm_amax_parts(torch.zeros((1, 32768), dtype=torch.bfloat16).cuda(), torch.ones(32768).cuda(), 1e-5)
    with pytest.raises(N.NativeError, match="weight"):
        N.rmsnorm_amax_parts(torch.zeros((4, 16), dtype=torch.bfloat16).cuda(), torch.ones(8).cuda(), 1e-5)


@pytest.mark.parametrize("rows,cols", [(1, 8), (37, 8), (2100, 8), (1, 64), (37, 64), (2100, 64), (1, 520), (37, 520), (2100, 520),
                                       (1, 4096), (37, 4096), (1, 8192), (37, 8192),
                                       (37, 96), (2100, 128), (9000, 128), (5000, 256), (2100, 512)])   # several rows per wave
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_backward(N, rows, cols, dtype):
    gen = torch.Generator().manual_seed(rows * 7 + cols)
    x = (torch.randn((rows, cols), generator=gen) * 2.0).to(dtype)
    w = torch.randn(cols, generator=gen) * 0.3 + 1.0
    dy = (torch.randn((rows, cols), generator=gen) * 1e-2).bfloat16()
    _, rstd = O.c_rmsnorm(x, w, 1e-5)
    dx, dw = N.rmsnorm_bwd(dy.cuda(), x.cuda(), w.cuda(), rstd.cuda())
    wdx, wdw = O.c_rmsnorm_bwd(dy, x, w, rstd)
    if dtype == torch.bfloat16:
        assert_bf16_equal(dx, wdx, f"rmsnorm dx {rows}x{cols}")                  # bit for bit
    else:
        assert_f32_bits_equal(dx, wdx, f"rmsnorm dx fp32 {rows}x{cols}")
    # d_weight: fp32 partial sums in a fixed order on the device, double in the oracle: 1e-5 of the largest entry
    err = (dw.cpu().double() - wdw.double()).abs().max().item()
    assert err <= 1e-5 * max(wdw.abs().max().item(), 1e-30), (err, wdw.abs().max().item())
    dx2, dw2 = N.rmsnorm_bwd(dy.cuda(), x.cuda(), w.cuda(), rstd.cuda())
    assert torch.equal(dw, dw2) and torch.equal(dx.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                                                dx2.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))


# ------------------------------------------------- partial maxima + column sums (bias gradient)
@pytest.mark.parametrize("shape", [(1, 8), (33, 256), (1000, 264), (4096, 768), (777, 3072), (64, 14336)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_amax_parts_colsum(N, shape, dtype):
    x = seeded_bf16(shape, 1e-2, sum(shape)).to(dtype)
    x[shape[0] // 2, shape[1] // 3] = -3.5
    parts, colsum = N.amax_parts_colsum(x.cuda())
    assert_f32_bits_equal(parts_max(parts).reshape(1), x.float().abs().max().reshape(1), f"colsum parts {shape}")
    assert_f32_bits_equal(parts_max(parts).reshape(1), parts_max(N.amax_parts(x.cuda())).reshape(1), "same maximum as amax_parts")
    want = x.double().sum(0)
    # fp32 partial sums in a fixed order against a double-precision sum: 1e-5 of sum |x| per column
    bound = 1e-5 * x.double().abs().sum(0) + 1e-30
    assert bool(((colsum.cpu().double() - want).abs() <= bound).all())
    _, again = N.amax_parts_colsum(x.cuda())
    assert torch.equal(colsum, again)                               # reproducible


def colsum_in_kernel_order(x):
    """The column sums as the kernel forms them, one fp32 addition at a time: per slab of rows, 32 row-lanes each add
    rows ty, ty + 32, ... in order; the row-lanes are added in order; 16 groups add every 16th slab in order; the
    groups are added in order."""
    rows, cols = x.shape
    cpl = 8 if x.dtype == torch.bfloat16 else 4
    col_blocks = -(-cols // (32 * cpl))
    slabs = 512 // col_blocks
    rpb = -(-(-(-rows // slabs)) // 32) * 32
    slabs = -(-rows // rpb)
    xf = x.float()
    slab_sums = []
    for s in range(slabs):
        part = xf[s * rpb:min(rows, (s + 1) * rpb)]
        pad = (-part.shape[0]) % 32
        if pad:
            part = torch.cat([part, torch.zeros((pad, cols))])           # acc + 0.0 == acc
        part = part.reshape(-1, 32, cols)
        acc = torch.zeros((32, cols))
        for it in range(part.shape[0]):
            acc = acc + part[it]
        t = acc[0]
        for y in range(1, 32):
            t = t + acc[y]
        slab_sums.append(t)
    groups = []
    for g in range(16):
        a = torch.zeros(cols)
        for b in range(g, slabs, 16):
            a = a + slab_sums[b]
        groups.append(a)
    t = groups[0]
    for g in range(1, 16):
        t = t + groups[g]
    return t


@pytest.mark.parametrize("shape", [(33, 256), (1000, 264), (4096, 768), (2000, 3072)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_amax_parts_colsum_adds_in_the_documented_order(N, shape, dtype):
    """The sum is not just reproducible: it is this sequence of fp32 additions, restated here one addition at a time."""
    x = seeded_bf16(shape, 1.0, 7 + sum(shape)).to(dtype)
    if dtype == torch.float32:
        x = x * 1.00390625 + 3e-4                                        # mantissas that do not fit bf16
    want = colsum_in_kernel_order(x)
    for _ in range(3):
        _, colsum = N.amax_parts_colsum(x.cuda())
        assert_f32_bits_equal(colsum, want, f"colsum order {shape} {dtype}")


def test_amax_parts_colsum_exact_and_refusals(N):
    # integers: every partial sum is exact, so the result is too, whatever the order
    rows, cols = 515, 264
    x = (torch.arange(rows * cols).reshape(rows, cols) % 7 - 3).bfloat16()
    _, colsum = N.amax_parts_colsum(x.cuda())
    assert torch.equal(colsum.cpu(), x.float().sum(0))
    z = torch.zeros((16, 16), dtype=torch.bfloat16)
    z[3, 4] = float("nan")
    parts, colsum = N.amax_parts_colsum(z.cuda())
    assert torch.isnan(parts_max(parts)) and torch.isnan(colsum[4]) and colsum[5].item() == 0.0
    with pytest.raises(N.NativeError, match="multiple of"):
        N.amax_parts_colsum(torch.zeros((4, 12), dtype=torch.bfloat16).cuda())
    assert not N.colsum_supported(torch.zeros((4, 12), dtype=torch.bfloat16).cuda())
    assert not N.colsum_supported(torch.zeros((0, 16), dtype=torch.bfloat16).cuda())
    assert N.colsum_supported(torch.zeros((4, 16), dtype=torch.bfloat16).cuda())


# ------------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("rows,cols", [(1, 8), (37, 64), (2100, 64), (37, 520), (300, 768), (37, 1600), (37, 4096),
                                       (37, 96), (9000, 128), (2100, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_bias", [True, False])
def test_layernorm_forward_and_backward(N, rows, cols, dtype, with_bias):
    gen = torch.Generator().manual_seed(rows * 13 + cols)
    x = (torch.randn((rows, cols), generator=gen) * 2.0 + 0.5).to(dtype)
    w = torch.randn(cols, generator=gen) * 0.3 + 1.0
    b = torch.randn(cols, generator=gen) * 0.2 if with_bias else None
    dy = (torch.randn((rows, cols), generator=gen) * 1e-2).bfloat16()
    y, mean, rstd, parts = N.layernorm_amax_parts(x.cuda(), w.cuda(), None if b is None else b.cuda(), 1e-5)
    wy, wm, wr = O.c_layernorm(x, w, b, 1e-5)
    assert_f32_bits_equal(mean, wm, f"layernorm mean {rows}x{cols}")
    assert_f32_bits_equal(rstd, wr, f"layernorm rstd {rows}x{cols}")
    assert_bf16_equal(y, wy, f"layernorm y {rows}x{cols} {dtype}")
    assert_f32_bits_equal(parts_max(parts).reshape(1), wy.float().abs().max().reshape(1), "layernorm parts")
    dx, dw, db = N.layernorm_bwd(dy.cuda(), x.cuda(), w.cuda(), mean, rstd)
    wdx, wdw, wdb = O.c_layernorm_bwd(dy, x, w, wm, wr)
    if dtype == torch.bfloat16:
        assert_bf16_equal(dx, wdx, f"layernorm dx {rows}x{cols}")
    else:
        assert_f32_bits_equal(dx, wdx, f"layernorm dx fp32 {rows}x{cols}")
    for got, want, what in ((dw, wdw, "d_weight"), (db, wdb, "d_bias")):
        err = (got.cpu().double() - want.double()).abs().max().item()
        assert err <= 1e-5 * max(want.abs().max().item(), 1e-30), (what, err)


def test_layernorm_refusals(N):
    with pytest.raises(N.NativeError, match="multiple of 8"):
        N.layernorm_amax_parts(torch.zeros((4, 12), dtype=torch.bfloat16).cuda(), torch.ones(12).cuda(), None, 1e-5)
    with pytest.raises(N.NativeError, match="4096"):
        N.layernorm_amax_parts(torch.zeros((1, 8192), dtype=torch.bfloat16).cuda(), torch.ones(8192).cuda(), None, 1e-5)


# ------------------------------------------------------------------ committed golden vectors
def _golden(name):
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as fh:
        return json.load(fh)


def _bf16_from_hex(hexes, shape=None):
    a = np.array([int(h, 16) for h in hexes], dtype=np.uint16)
    t = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return t if shape is None else t.reshape(shape)


def _f32_from_hex(hexes):
    return torch.from_numpy(np.array([int(h, 16) for h in hexes], dtype=np.uint32).view(np.float32).copy())


def test_kernels_against_golden_swiglu_vectors(N):
    """tests/golden/swiglu_bf16.json holds what torch's CPU bf16 silu / multiply / autograd give."""
    doc = _golden("swiglu_bf16.json")
    g, u, dh = (_bf16_from_hex(doc[k]) for k in ("gate_bf16_hex", "up_bf16_hex", "dh_bf16_hex"))
    n8 = g.numel() // 8 * 8
    g, u, dh = g[:n8].reshape(-1, 8), u[:n8].reshape(-1, 8), dh[:n8].reshape(-1, 8)
    h, _ = N.swiglu_amax_parts(g.cuda(), u.cuda())
    assert_bf16_equal(h, _bf16_from_hex(doc["h_bf16_hex"])[:n8].reshape(-1, 8), "h vs golden")
    s, _ = N.swiglu_amax_parts(g.cuda(), torch.ones_like(g).cuda())
    assert_bf16_equal(s, _bf16_from_hex(doc["silu_bf16_hex"])[:n8].reshape(-1, 8), "silu vs golden")
    dg, du, _, _ = N.swiglu_bwd_amax_parts(dh.cuda(), g.cuda(), u.cuda())
    assert_bf16_equal(du, _bf16_from_hex(doc["d_up_bf16_hex"])[:n8].reshape(-1, 8), "d_up vs golden")
    want = _bf16_from_hex(doc["d_gate_bf16_hex"])[:n8].reshape(-1, 8)
    d = (dg.cpu().view(torch.int16).int() - want.view(torch.int16).int()).abs()
    assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 0.02


def test_kernels_against_golden_norm_vectors(N):
    """tests/golden/norm_rows.json holds float64 closed forms rounded once: within one bf16 unit."""
    for case in _golden("norm_rows.json")["cases"]:
        shape = (case["rows"], case["cols"])
        x = _bf16_from_hex(case["x_hex"], shape) if case["dtype"] == "bf16" else _f32_from_hex(case["x_hex"]).reshape(shape)
        w, b = _f32_from_hex(case["weight_f32_hex"]), _f32_from_hex(case["bias_f32_hex"])
        y, rstd, _ = N.rmsnorm_amax_parts(x.cuda(), w.cuda(), case["eps"])
        assert torch.allclose(rstd.cpu(), _f32_from_hex(case["rms_rstd_f32_hex"]), rtol=1e-6, atol=0)
        d = (y.cpu().view(torch.int16).int() - _bf16_from_hex(case["rms_y_bf16_hex"], shape).view(torch.int16).int()).abs()
        assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 0.01
        y, mean, rstd, _ = N.layernorm_amax_parts(x.cuda(), w.cuda(), b.cuda(), case["eps"])
        assert torch.allclose(mean.cpu(), _f32_from_hex(case["ln_mean_f32_hex"]), rtol=1e-5, atol=1e-6)
        assert torch.allclose(rstd.cpu(), _f32_from_hex(case["ln_rstd_f32_hex"]), rtol=1e-6, atol=0)
        d = (y.cpu().view(torch.int16).int() - _bf16_from_hex(case["ln_y_bf16_hex"], shape).view(torch.int16).int()).abs()
        assert int(d.max()) <= 1 and float((d > 0).float().mean()) < 0.01


# ------------------------------------------------------------------------ GELU
def test_gelu_forward_every_bf16_input(N):
    x = all_bf16().reshape(256, 256)
    y, parts = N.gelu_amax_parts(x.cuda())
    assert_bf16_equal(y, O.c_gelu_fwd(x), "gelu, every bf16 input")
    assert torch.isnan(parts_max(parts))
    fin = torch.where(torch.isfinite(x.float()), x, torch.zeros_like(x))
    y, parts = N.gelu_amax_parts(fin.cuda())
    assert_f32_bits_equal(parts_max(parts).reshape(1), O.c_gelu_fwd(fin).float().abs().max().reshape(1), "gelu parts")


@pytest.mark.parametrize("dy_std", [1.0, 1e-3])
def test_gelu_backward_every_bf16_input(N, dy_std):
    x = all_bf16().reshape(256, 256)
    dy = seeded_bf16((256, 256), dy_std, 17)
    dx, parts = N.gelu_bwd_amax_parts(dy.cuda(), x.cuda())
    assert_bf16_equal(dx, O.c_gelu_bwd(dy, x), "gelu backward, every bf16 input")


@pytest.mark.parametrize("shape", [(16, 24), (1, 8), (1000, 8), (4, 96, 768), (2048, 3072)])
def test_gelu_shapes_and_parts(N, shape):
    x, dy = seeded_bf16(shape, 1.5, 41), seeded_bf16(shape, 1e-2, 42)
    y, parts = N.gelu_amax_parts(x.cuda())
    want = O.c_gelu_fwd(x)
    assert_bf16_equal(y, want, f"gelu {shape}")
    assert_f32_bits_equal(parts_max(parts).reshape(1), want.float().abs().max().reshape(1), "gelu parts")
    dx, parts = N.gelu_bwd_amax_parts(dy.cuda(), x.cuda())
    wdx = O.c_gelu_bwd(dy, x)
    assert_bf16_equal(dx, wdx, f"gelu bwd {shape}")
    assert_f32_bits_equal(parts_max(parts).reshape(1), wdx.float().abs().max().reshape(1), "gelu bwd parts")
    with pytest.raises(N.NativeError, match="multiple of 8"):
        N.gelu_amax_parts(torch.zeros((3, 5), dtype=torch.bfloat16).cuda())


def test_producers_take_empty_inputs(N):
    """Zero rows: empty outputs, all-zero partial maxima, zero weight / bias gradients, no launch fault."""
    e = torch.empty((0, 64), dtype=torch.bfloat16, device="cuda")
    w = torch.ones(64, device="cuda")
    none = torch.empty(0, device="cuda")
    for out in (N.swiglu_amax_parts(e, e), N.swiglu_bwd_amax_parts(e, e, e), N.rmsnorm_amax_parts(e, w, 1e-5),
                N.rmsnorm_bwd(e, e, w, none), N.layernorm_amax_parts(e, w, None, 1e-5), N.layernorm_bwd(e, e, w, none, none),
                N.gelu_amax_parts(e), N.gelu_bwd_amax_parts(e, e)):
        torch.cuda.synchronize()
        for t in out if isinstance(out, tuple) else (out,):
            assert t.numel() == 0 or float(t.abs().max()) == 0.0
