"""GPU parity: amax / scale / cast / cast+transpose kernels vs the CPU oracle.

Integer / byte results must be bit-exact.  Every call goes through the C ABI.
"""
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


SHAPES = [(128, 64), (256, 256), (1024, 768), (16, 16), (48, 80), (1000, 200), (7, 13), (1, 1), (3, 4096), (513, 1032)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_amax_all_modes_bit_exact(N, shape, dtype):
    x = seeded_bf16(shape, std=3.0, seed=sum(shape))
    x[shape[0] // 2, shape[1] // 3] = -77.5                         # a lone outlier, negative on purpose
    xd = x.to(dtype).cuda()
    for mode in (O.SCALE_TENSOR, O.SCALE_ROW, O.SCALE_COL):
        got = N.amax(xd, mode)
        assert_f32_bits_equal(got, O.t_amax(x, mode), f"amax mode {mode} {shape} {dtype}")
        assert_f32_bits_equal(got, O.c_amax(x, mode), f"amax(C oracle) mode {mode} {shape}")


def test_amax_accumulate_and_specials(N):
    x = seeded_bf16((64, 128), seed=1)
    y = seeded_bf16((64, 128), std=5.0, seed=2)
    for mode in (O.SCALE_TENSOR, O.SCALE_ROW, O.SCALE_COL):
        acc = N.amax(x.cuda(), mode)
        N.amax(y.cuda(), mode, out=acc, accumulate=True)
        assert_f32_bits_equal(acc, torch.maximum(O.t_amax(x, mode), O.t_amax(y, mode)), f"accumulate mode {mode}")
    z = torch.zeros((32, 64), dtype=torch.bfloat16)
    z[3, 5] = -0.0
    assert float(N.amax(z.cuda())[0]) == 0.0
    z[4, 7] = float("nan")
    assert torch.isnan(N.amax(z.cuda())).all()
    r = N.amax(z.cuda(), O.SCALE_ROW).cpu()
    assert torch.isnan(r[4]) and float(r[3]) == 0.0
    z[4, 7] = float("inf")
    assert torch.isinf(N.amax(z.cuda())).all()
    assert N.amax(torch.empty((0, 16), dtype=torch.bfloat16).cuda(), O.SCALE_COL).abs().sum().item() == 0.0


def test_amax_unaligned_view(N):
    flat = seeded_bf16((1, 5000), seed=6).cuda()
    view = flat[0, 3:4003].reshape(1, 4000)
    assert view.data_ptr() % 16 != 0
    assert_f32_bits_equal(N.amax(view), O.t_amax(view.cpu()), "unaligned amax")
    assert_f32_bits_equal(N.amax(view, O.SCALE_ROW), O.t_amax(view.cpu(), O.SCALE_ROW), "unaligned row amax")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_amax_scale_in_one_launch_equals_the_two_step_route(N, fmt):
    """One call after another on the same stream: the shared workspace must come back to zero
    every time, whatever the grid size of the call before."""
    cases = [((8192, 4096), 1.0, torch.bfloat16), ((16, 16), 0.02, torch.bfloat16), ((1000, 200), 3.0, torch.float32),
             ((7, 13), 1e-3, torch.bfloat16), ((4096, 1024), 50.0, torch.bfloat16), ((1, 8), 1.0, torch.float32)]
    for margin in (0, 2):
        for i, (shape, std, dtype) in enumerate(cases):
            x = seeded_bf16(shape, std=std, seed=10 + i)
            xd = x.to(dtype).cuda()
            amax, scale, scale_inv = N.amax_scale(xd, fmt, margin)
            want_amax = O.t_amax(x)
            want_scale = np.float32(O.c_scale(float(want_amax), fmt, margin, 1.0))
            assert_f32_bits_equal(amax, want_amax, f"fused amax {shape}")
            assert_f32_bits_equal(scale, torch.tensor([want_scale]), f"fused scale {shape}")
            assert_f32_bits_equal(scale_inv, torch.tensor([np.float32(O.c_scale_inv(want_scale))]), f"fused 1/scale {shape}")
            two_a = N.amax(xd)
            two_s, two_si = N.scale_from_amax(two_a, fmt, margin)
            assert_f32_bits_equal(torch.cat([amax, scale, scale_inv]), torch.cat([two_a, two_s, two_si]).cpu(), "fused vs two-step")
    # specials: all zero -> scale 1; NaN propagates into amax and falls back to scale 1; unaligned and empty inputs
    z = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    amax, scale, scale_inv = N.amax_scale(z, fmt)
    assert amax.item() == 0.0 and scale.item() == 1.0 and scale_inv.item() == 1.0
    z[3, 5] = float("nan")
    amax, scale, _ = N.amax_scale(z, fmt)
    assert torch.isnan(amax).item() and scale.item() == 1.0
    flat = seeded_bf16((1, 5000), seed=6).cuda()
    view = flat[0, 3:4003].reshape(1, 4000)
    amax, scale, _ = N.amax_scale(view, fmt)
    assert_f32_bits_equal(amax, O.t_amax(view.cpu()), "fused amax, unaligned")
    amax, scale, _ = N.amax_scale(torch.empty((0, 16), dtype=torch.bfloat16, device="cuda"), fmt)
    assert amax.item() == 0.0 and scale.item() == 1.0
    # and the workspace really is zero again
    assert all(int(w.abs().sum()) == 0 for w in N._workspaces.values())


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_two_launch_dynamic_quantisation_equals_the_step_by_step_route(N, fmt):
    """amax_parts + cast_dynamic against amax -> scale_from_amax -> cast / cast_transpose (and the oracle):
    same codes, same amax, scale and 1/scale, for shapes on the fast and on the element-at-a-time routes."""
    cases = [((8192, 4096), 1.0, torch.bfloat16), ((256, 128), 0.02, torch.bfloat16), ((1000, 48), 3.0, torch.float32),
             ((33, 20), 1e-3, torch.bfloat16), ((16, 16), 5.0, torch.float32), ((5, 3), 1.0, torch.bfloat16),
             ((2048, 14336), 1e-3, torch.bfloat16)]
    for margin in (0, 1):
        for i, (shape, std, dtype) in enumerate(cases):
            x = seeded_bf16(shape, std=std, seed=70 + i)
            xd = x.to(dtype).cuda()
            q, q_t, amax, scale, scale_inv = N.quantize_dynamic(xd, fmt, margin)
            a2 = N.amax(xd)
            s2, si2 = N.scale_from_amax(a2, fmt, margin)
            q2, q2_t = N.cast_transpose(xd, s2, fmt)
            assert_f32_bits_equal(torch.cat([amax, scale, scale_inv]), torch.cat([a2, s2, si2]).cpu(), f"dynamic numbers {shape}")
            assert_bytes_equal(q, q2, f"dynamic codes {shape}")
            assert_bytes_equal(q_t, q2_t, f"dynamic transposed codes {shape}")
            assert_f32_bits_equal(amax, O.t_amax(x), f"amax vs oracle {shape}")
            if shape[0] * shape[1] <= 1 << 20:
                assert_bytes_equal(q, O.t_cast(x, scale.cpu(), fmt), f"codes vs oracle {shape}")
            only_q, none_t, *_ = N.quantize_dynamic(xd, fmt, margin, want_transposed=False)
            none_q, only_t, *_ = N.quantize_dynamic(xd, fmt, margin, want_rowmajor=False)
            assert none_t is None and none_q is None
            assert_bytes_equal(only_q, q2, "row-major only")
            assert_bytes_equal(only_t, q2_t, "transposed only")
    # specials: zeros -> scale 1; NaN -> amax NaN, scale 1, code 0x7F; empty; unaligned view
    z = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    q, _, amax, scale, _ = N.quantize_dynamic(z, fmt)
    assert amax.item() == 0.0 and scale.item() == 1.0 and int(q.max()) == 0
    z[3, 5] = float("nan")
    q, _, amax, scale, _ = N.quantize_dynamic(z, fmt)
    assert torch.isnan(amax).item() and scale.item() == 1.0 and int(q[3, 5]) == 0x7F
    q, q_t, amax, scale, _ = N.quantize_dynamic(torch.empty((0, 16), dtype=torch.bfloat16, device="cuda"), fmt)
    assert q.shape == (0, 16) and q_t.shape == (16, 0)
    flat = seeded_bf16((1, 5000), seed=6).cuda()
    view = flat[0, 3:4003].reshape(40, 100)
    q, q_t, amax, scale, _ = N.quantize_dynamic(view, fmt)
    assert_f32_bits_equal(amax, O.t_amax(view.cpu()), "unaligned amax")
    assert_bytes_equal(q, O.t_cast(view.cpu(), scale.cpu(), fmt), "unaligned codes")
    assert torch.equal(q_t, q.t().contiguous())


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_scale_from_amax_bit_exact(N, fmt):
    rng = np.random.default_rng(0)
    a = np.concatenate([
        np.abs(rng.normal(0, 1, 5000)).astype(np.float32) * 5,
        (2.0 ** rng.uniform(-140, 127, 5000)).astype(np.float32),
        np.array([0.0, -1.0, np.inf, np.nan, 1e-45, 3e-39, 448.0, 57344.0, 3.4e38, 1.0], dtype=np.float32),
        torch.randn(2000).abs().bfloat16().float().numpy(),
    ])
    for margin in (0, 1, 3):
        s, si = N.scale_from_amax(torch.from_numpy(a).cuda(), fmt, margin)
        want = np.array([O.c_scale(v, fmt, margin, 1.0) for v in a], dtype=np.float32)
        want_inv = np.array([O.c_scale_inv(v) for v in want], dtype=np.float32)
        assert_f32_bits_equal(s, torch.from_numpy(want), f"scale fmt {fmt} margin {margin}")
        assert_f32_bits_equal(si, torch.from_numpy(want_inv), f"scale_inv fmt {fmt} margin {margin}")
        if margin == 0:
            assert_f32_bits_equal(s, O.t_scale(torch.from_numpy(a), fmt), "scale vs torch rule")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_cast_every_bf16_pattern_times_many_scales(N, fmt):
    """All 65536 bf16 inputs x 256 scales: exercises RNE ties, subnormals, the
    clamp, NaN/Inf and signed zeros of the hardware conversion."""
    allbits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    rng = np.random.default_rng(3)
    scales = np.concatenate([
        np.array([1.0, 0.5, 2.0, 448.0, 57344.0, 3.4028235e38, 1e-30, 2.0 ** -20, 2.0 ** 20, 0.3333333], dtype=np.float32),
        (O.FP8_MAX[fmt] / np.abs(rng.normal(0, 2, 123)).astype(np.float32)).astype(np.float32),
        (2.0 ** rng.uniform(-30, 30, 123)).astype(np.float32),
    ])
    x = allbits.reshape(1, 65536).expand(len(scales), 65536).contiguous()       # row r uses scale r
    s = torch.from_numpy(scales)
    got = N.cast(x.cuda(), s.cuda(), fmt, O.SCALE_ROW)
    assert_bytes_equal(got, O.c_cast(x, s, fmt, O.SCALE_ROW), f"cast exhaustive fmt {fmt} (C oracle)")
    assert_bytes_equal(got, O.t_cast(x, s, fmt, O.SCALE_ROW), f"cast exhaustive fmt {fmt} (torch CPU)")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("mode", [O.SCALE_TENSOR, O.SCALE_ROW, O.SCALE_COL])
@pytest.mark.parametrize("shape", [(256, 128), (128, 4096), (1000, 48), (64, 16), (33, 20), (5, 3)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_cast_and_cast_transpose_match_oracle(N, fmt, mode, shape, dtype):
    x = seeded_bf16(shape, std=1.0, seed=shape[0] * 7 + shape[1])
    x[0, 0] = float("nan")
    x[-1, -1] = float("-inf")
    x[shape[0] // 2, 0] = 300.0
    am = O.t_amax(torch.nan_to_num(x, nan=0.0, posinf=0.0, neginf=0.0), mode)
    s = O.t_scale(am, fmt) * (1.7 if mode == O.SCALE_TENSOR else 1.0)              # >1: makes the clamp fire
    xd = x.to(dtype).cuda()
    want = O.t_cast(x, s, fmt, mode)
    got = N.cast(xd, s.cuda(), fmt, mode)
    assert_bytes_equal(got, want, f"cast {shape} mode {mode} fmt {fmt} {dtype}")
    q, qt = N.cast_transpose(xd, s.cuda(), fmt, mode)
    assert_bytes_equal(q, want, f"cast_transpose row-major {shape} mode {mode}")
    assert_bytes_equal(qt, want.t().contiguous(), f"cast_transpose transposed {shape} mode {mode}")
    q2, qt2 = N.cast_transpose(xd, s.cuda(), fmt, mode, want_rowmajor=False)
    assert q2 is None
    assert_bytes_equal(qt2, want.t().contiguous(), f"cast_transpose only-T {shape} mode {mode}")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_cast_with_fused_amax_for_delayed_scaling(N, fmt):
    x = seeded_bf16((512, 384), std=2.0, seed=11)
    stale = torch.tensor([O.FP8_MAX[fmt] / 3.0])                                   # smaller amax than the data: clamps
    for fn in ("cast", "cast_transpose"):
        slot = torch.zeros(1, device="cuda")
        if fn == "cast":
            q = N.cast(x.cuda(), stale.cuda(), fmt, amax_out=slot)
        else:
            q, qt = N.cast_transpose(x.cuda(), stale.cuda(), fmt, amax_out=slot)
            assert_bytes_equal(qt, O.t_cast(x, stale, fmt).t().contiguous(), "fused-amax transposed codes")
        assert_bytes_equal(q, O.t_cast(x, stale, fmt), f"{fn} with fused amax codes")
        assert_f32_bits_equal(slot, O.t_amax(x), f"{fn} fused amax")
        # a second tensor folds into the same slot (max), as microbatches do
        y = seeded_bf16((512, 384), std=0.5, seed=12)
        N.cast(y.cuda(), stale.cuda(), fmt, amax_out=slot)
        assert_f32_bits_equal(slot, torch.maximum(O.t_amax(x), O.t_amax(y)), "amax slot folds")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("shape", [(512, 384), (2048, 1536), (48, 40), (17, 16)])
def test_cast_delayed_codes_partial_maxima_and_inverse_scale(N, fmt, shape):
    """The one-launch cast of the delayed recipe: codes as odl_fp8_cast / _cast_transpose with the same scale (the oracle's
    cast), the maximum of the recorded partial maxima equal to the tensor's amax, 1/scale by IEEE division; a second cast
    into the same strip accumulates; nothing is recorded without a strip.  (48, 40) and (17, 16) take the
    element-at-a-time route (rows not a multiple of 16 / columns not of 16)."""
    x = seeded_bf16(shape, std=2.0, seed=11)
    stale = torch.tensor([O.FP8_MAX[fmt] / 3.0])                                   # smaller amax than the data: clamps
    want = O.t_cast(x, stale, fmt)
    inv = torch.tensor([np.float32(1.0) / np.float32(stale.item())])
    for rm, t in ((True, False), (True, True), (False, True)):
        parts = torch.zeros(N.AMAX_PARTS, device="cuda")
        q, qt, s_inv = N.cast_delayed(x.cuda(), stale.cuda(), fmt, amax_parts=parts, want_rowmajor=rm, want_transposed=t)
        assert (q is None) == (not rm) and (qt is None) == (not t)
        if rm:
            assert_bytes_equal(q, want, f"row-major codes {shape}")
        if t:
            assert_bytes_equal(qt, want.t().contiguous(), f"transposed codes {shape}")
        assert_f32_bits_equal(s_inv, inv, "inverse scale")
        assert_f32_bits_equal(parts.max().reshape(1), O.t_amax(x), "maximum of the partial maxima")
        y = seeded_bf16(shape, std=0.5, seed=12)
        y[0, 0] = 300.0
        N.cast_delayed(y.cuda(), stale.cuda(), fmt, amax_parts=parts, want_rowmajor=rm, want_transposed=t)
        assert_f32_bits_equal(parts.max().reshape(1), torch.tensor([300.0]), "a second cast accumulates")
    q, _, s_inv = N.cast_delayed(x.cuda(), stale.cuda(), fmt)                        # eval mode: nothing recorded
    assert_bytes_equal(q, want, "codes without a strip")
    assert_f32_bits_equal(s_inv, inv, "inverse scale without a strip")
    # fp32 source
    q, qt, _ = N.cast_delayed(x.float().cuda(), stale.cuda(), fmt, want_transposed=True)
    assert_bytes_equal(q, want, "fp32 source")
    assert_bytes_equal(qt, want.t().contiguous(), "fp32 source, transposed")


def test_cast_delayed_spreads_the_maxima_of_a_large_tensor(N):
    """8192 x 4096: 4096 tiles of the cast+transpose kernel fold into 512 words; the amax sits in the very last tile."""
    x = seeded_bf16((8192, 4096), seed=3).cuda()
    x[8191, 4095] = 123.0
    s = torch.tensor([2.0], device="cuda")
    for t in (False, True):
        parts = torch.zeros(N.AMAX_PARTS, device="cuda")
        q, qt, _ = N.cast_delayed(x, s, O.E4M3, amax_parts=parts, want_transposed=t)
        assert parts.max().item() == 123.0 and (parts > 0).sum().item() > 64
        assert torch.equal(q, N.cast(x, s, O.E4M3))
        if t:
            assert torch.equal(qt, q.t().contiguous())


def test_cast_transpose_large_matches_cast_then_transpose(N):
    """Size-independent property at a full benchmark shape: out_t == out^T bytewise."""
    x = seeded_bf16((8192, 4096), seed=0).cuda()
    am = N.amax(x)
    s, _ = N.scale_from_amax(am, O.E4M3)
    q, qt = N.cast_transpose(x, s, O.E4M3)
    assert torch.equal(qt, q.t().contiguous())
    assert torch.equal(q, N.cast(x, s, O.E4M3))
    # against torch CPU on a slab (the whole tensor would take seconds, a slab pins the same code path)
    want = O.t_cast(x[:512].cpu(), s.cpu(), O.E4M3)
    assert_bytes_equal(q[:512], want, "large cast slab")


def test_delayed_update_matches_oracle(N):
    H, R = 16, 5
    fmts = [O.E4M3, O.E4M3, O.E4M3, O.E5M2, O.E5M2]
    rng = np.random.default_rng(7)
    hist = np.zeros((H, R), dtype=np.float32)
    scale = np.ones(R, dtype=np.float32)
    inv = np.ones(R, dtype=np.float32)
    dh, ds, di = torch.from_numpy(hist.copy()).cuda(), torch.from_numpy(scale.copy()).cuda(), torch.from_numpy(inv.copy()).cuda()
    dfm = torch.tensor(fmts, dtype=torch.int32).cuda()
    for algo_name, algo in (("max", 0), ("most_recent", 1)):
        for step in range(40):
            new = np.abs(rng.normal(0, 1 + step * 0.1, R)).astype(np.float32)
            if step == 5:
                new[1] = 0.0
            if step == 9:
                new[2] = np.inf
            if step == 13:
                new[4] = np.nan
            hist[0] = new
            dh[0] = torch.from_numpy(new).cuda()
            O.c_delayed_update(hist, scale, inv, fmts, margin=1, algo=algo_name)
            N.delayed_update(dh, ds, di, dfm, margin=1, algo=algo)
            assert_f32_bits_equal(dh, torch.from_numpy(hist), f"history step {step} {algo_name}")
            assert_f32_bits_equal(ds, torch.from_numpy(scale), f"scale step {step} {algo_name}")
            assert_f32_bits_equal(di, torch.from_numpy(inv), f"scale_inv step {step} {algo_name}")

@pytest.mark.parametrize("H,R", [(1, 3), (2, 17), (15, 16), (16, 40), (17, 5), (33, 1), (64, 33), (1024, 21)])
@pytest.mark.parametrize("algo_name,algo", [("max", 0), ("most_recent", 1)])
def test_delayed_update_every_history_length_with_partial_maxima(N, H, R, algo_name, algo):
    """History lengths around the 16 lanes that share a role (one row per lane, several, a ragged last segment, the
    reference's default of 1024), role counts around the 16 roles of a block, the step's amax arriving as partial maxima
    (folded into row 0 and cleared) or directly in row 0, against the oracle value for value."""
    rng = np.random.default_rng(H * 131 + R)
    fmts = [int(f) for f in rng.integers(0, 2, R)]
    hist = np.abs(rng.normal(0, 1, (H, R))).astype(np.float32)                      # a full window to start with
    hist[0] = 0
    scale, inv = np.ones(R, dtype=np.float32), np.ones(R, dtype=np.float32)
    dh, ds, di = torch.from_numpy(hist.copy()).cuda(), torch.from_numpy(scale.copy()).cuda(), torch.from_numpy(inv.copy()).cuda()
    dfm = torch.tensor(fmts, dtype=torch.int32).cuda()
    parts = torch.zeros((R, N.AMAX_PARTS), device="cuda")
    for step in range(H + 3 if H <= 64 else 6):
        new = np.abs(rng.normal(0, 1 + step * 0.1, R)).astype(np.float32)
        if step == 2:
            new[0] = 0.0
        direct = np.where(rng.random(R) < 0.5, new, 0).astype(np.float32)            # some roles in row 0, some as partials
        dh[0] = torch.from_numpy(direct).cuda()
        where = torch.from_numpy(rng.integers(0, N.AMAX_PARTS, R)).cuda()
        parts[torch.arange(R, device="cuda"), where] = torch.from_numpy(new).cuda()
        parts[:, 7] = torch.maximum(parts[:, 7], torch.from_numpy(new * 0.5).cuda())  # a smaller entry elsewhere in the strip
        hist[0] = new
        O.c_delayed_update(hist, scale, inv, fmts, margin=0, algo=algo_name)
        N.delayed_update(dh, ds, di, dfm, margin=0, algo=algo, amax_parts=parts)
        assert_f32_bits_equal(dh, torch.from_numpy(hist), f"history step {step}")
        assert_f32_bits_equal(ds, torch.from_numpy(scale), f"scale step {step}")
        assert_f32_bits_equal(di, torch.from_numpy(inv), f"scale_inv step {step}")
        assert not parts.any(), "the partial maxima are cleared"



def test_bad_arguments_are_refused(N):
    x = seeded_bf16((16, 16)).cuda()
    with pytest.raises(N.NativeError):
        N.cast(x, torch.ones(3, device="cuda"), O.E4M3)                            # wrong scale count
    with pytest.raises(N.NativeError):
        N.cast(x.cpu(), torch.ones(1), O.E4M3)                                     # CPU tensor
    with pytest.raises(N.NativeError):
        N.amax(x.half())                                                           # unsupported dtype
    with pytest.raises(N.NativeError):
        N._check(N.load().odl_fp8_cast(x.data_ptr(), 0, 16, 16, torch.ones(1, device="cuda").data_ptr(), 0, 9,
                                       x.data_ptr(), None, None), "bad fmt")


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_rowwise_pair_in_two_passes_equals_the_four_pass_route(N, fmt):
    """amax_rowcol + cast_rowcol against amax(ROW), amax(COL), scale_from_amax, cast(ROW), cast_transpose(COL)
    and the oracle: same amaxes, same inverse scales, same codes; outlier channels included."""
    cases = [((1024, 512), torch.bfloat16), ((256, 128), torch.bfloat16), ((4096, 4096), torch.bfloat16),
             ((144, 72), torch.float32), ((1000, 48), torch.bfloat16), ((33, 20), torch.bfloat16), ((16, 8), torch.float32)]
    for i, (shape, dtype) in enumerate(cases):
        x = seeded_bf16(shape, std=1.0, seed=120 + i)
        x[:, 3 % shape[1]] *= 100.0                                   # an outlier channel
        x[5 % shape[0]] *= 0.01                                       # and a quiet row
        xd = x.to(dtype).cuda()
        for margin in (0, 1):
            q, s_row_inv, q_t, s_col_inv, a_row, a_col = N.quantize_rowcol(xd, fmt, margin)
            ar, ac = N.amax(xd, O.SCALE_ROW), N.amax(xd, O.SCALE_COL)
            assert_f32_bits_equal(a_row, ar, f"row amax {shape}")
            assert_f32_bits_equal(a_col, ac, f"col amax {shape}")
            assert_f32_bits_equal(a_row, O.t_amax(x, O.SCALE_ROW), f"row amax vs oracle {shape}")
            assert_f32_bits_equal(a_col, O.t_amax(x, O.SCALE_COL), f"col amax vs oracle {shape}")
            sr, sri = N.scale_from_amax(ar, fmt, margin)
            sc, sci = N.scale_from_amax(ac, fmt, margin)
            assert_f32_bits_equal(s_row_inv, sri, f"1/row scale {shape}")
            assert_f32_bits_equal(s_col_inv, sci, f"1/col scale {shape}")
            assert_bytes_equal(q, N.cast(xd, sr, fmt, O.SCALE_ROW), f"row-scaled codes {shape}")
            assert_bytes_equal(q_t, N.cast_transpose(xd, sc, fmt, O.SCALE_COL, want_rowmajor=False)[1], f"col-scaled codes {shape}")
            if margin == 0:
                assert_bytes_equal(q, O.t_cast(x, sr.cpu(), fmt, O.SCALE_ROW), f"row-scaled codes vs oracle {shape}")
                assert_bytes_equal(q_t, O.t_cast(x, sc.cpu(), fmt, O.SCALE_COL).t().contiguous(), f"col-scaled codes vs oracle {shape}")


def _golden(name):
    import json
    import os

    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", name)) as fh:
        return json.load(fh)


def _f32(hexes):
    return np.array([int(h, 16) for h in hexes], dtype=np.uint32).view(np.float32)


@pytest.mark.parametrize("name,fmt", [("e4m3", O.E4M3), ("e5m2", O.E5M2)])
def test_kernels_against_the_committed_golden_vectors(N, name, fmt):
    """tests/golden/*.json: edge inputs (every tie between neighbouring codes, one ulp to either side,
    overflow, NaN, Inf, subnormals), scale rule specials, a 20-step delayed-scaling sequence."""
    doc = _golden("fp8_encode_edges.json")[name]
    x = _f32(doc["x_f32_hex"])
    want = torch.tensor(doc["code_saturating"], dtype=torch.uint8)
    n = (len(x) // 16) * 16                                              # a multiple of 16 takes the vector kernel
    one = torch.ones(1, device="cuda")
    xs = torch.from_numpy(x.copy())
    assert_bytes_equal(N.cast(xs[:n].reshape(1, n).cuda(), one, fmt).reshape(-1), want[:n], "golden edges, vector kernel")
    assert_bytes_equal(N.cast(xs.reshape(1, -1).cuda(), one, fmt).reshape(-1), want, "golden edges, element kernel")
    assert_bytes_equal(N.cast_transpose(xs[:n].reshape(n // 8, 8).cuda(), one, fmt)[1].t().reshape(-1), want[:n], "golden edges, cast+transpose")

    doc = _golden("scale_from_amax.json")
    amax = torch.from_numpy(_f32(doc["amax_f32_hex"]).copy()).cuda()
    for case in doc["cases"]:
        if case["fmt"] != name:
            continue
        s, si = N.scale_from_amax(amax, fmt, case["margin"])
        assert_f32_bits_equal(s, torch.from_numpy(_f32(case["scale_f32_hex"]).copy()), f"golden scales margin {case['margin']}")
        assert_f32_bits_equal(si, torch.from_numpy(_f32(case["scale_inv_f32_hex"]).copy()), "golden inverse scales")

    doc = _golden("delayed_scaling_sequence.json")
    H, amaxes = doc["H"], _f32(doc["amax_f32_hex"])
    for case in doc["cases"]:
        if case["fmt"] != name:
            continue
        hist = torch.zeros((H, 1), device="cuda")
        scale, scale_inv = torch.ones(1, device="cuda"), torch.ones(1, device="cuda")
        fmts = torch.tensor([fmt], dtype=torch.int32, device="cuda")
        used, after = _f32(case["scale_used_f32_hex"]), _f32(case["scale_after_f32_hex"])
        for t, a in enumerate(amaxes):
            assert_f32_bits_equal(scale, torch.tensor([used[t]]), f"scale used at step {t}")
            hist[0, 0] = max(hist[0, 0].item(), float(a))
            N.delayed_update(hist, scale, scale_inv, fmts, 0, N.AMAX_MAX if case["algo"] == "max" else N.AMAX_MOST_RECENT)
            assert_f32_bits_equal(scale, torch.tensor([after[t]]), f"scale after step {t}")
        assert_f32_bits_equal(hist[:, 0], torch.from_numpy(_f32(case["final_history_f32_hex"]).copy()), "final history")
