"""Pins the oracle's amax / scale / cast / cast+transpose / GEMM / delayed-scaling
functions (CPU only).  Each is anchored on something other than its own formula:
closed forms evaluated by numpy/torch, byte identities, float64 brute force,
special cases whose result is exact, and hand-worked sequences."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import seeded_bf16


# ------------------------------------------------------------------------ amax
@pytest.mark.parametrize("shape", [(7, 13), (64, 128), (1, 1)])
def test_amax_three_modes_vs_numpy(shape):
    x = seeded_bf16(shape, 2.0, 1)
    x[0, 0] = -9.5
    ref = np.abs(x.float().numpy())
    assert O.c_amax(x, O.SCALE_TENSOR).item() == ref.max()
    assert np.array_equal(O.c_amax(x, O.SCALE_ROW).numpy(), ref.max(axis=1))
    assert np.array_equal(O.c_amax(x, O.SCALE_COL).numpy(), ref.max(axis=0))
    for mode in (O.SCALE_TENSOR, O.SCALE_ROW, O.SCALE_COL):
        assert torch.equal(O.t_amax(x, mode), O.c_amax(x, mode))


def test_amax_nan_and_zero():
    z = torch.zeros((4, 4), dtype=torch.bfloat16)
    assert O.c_amax(z).item() == 0.0
    z[1, 2] = float("nan")
    assert np.isnan(O.c_amax(z).item()) and np.isnan(O.t_amax(z).item())
    r = O.c_amax(z, O.SCALE_ROW).numpy()
    assert np.isnan(r[1]) and r[0] == 0.0


# ----------------------------------------------------------------------- scale
@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_scale_is_ieee_fp32_division(fmt):
    rng = np.random.default_rng(0)
    amax = np.concatenate([np.abs(rng.normal(0, 3, 20000)), 2.0 ** rng.uniform(-100, 100, 5000)]).astype(np.float32)
    amax = amax[amax > 0]
    got = np.array([O.c_scale(a, fmt) for a in amax], dtype=np.float32)
    # correctly rounded quotient via float64 (2p+2 bits: double rounding is innocuous)
    want = (np.float64(O.FP8_MAX[fmt]) / amax.astype(np.float64)).astype(np.float32)
    want = np.where(np.isinf(want), np.float32(O.FLT_MAX), want)
    assert np.array_equal(got, want)
    assert np.array_equal(O.t_scale(torch.from_numpy(amax), fmt).numpy(), want)


def test_scale_guards_margin_and_inverse():
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        assert O.c_scale(bad, O.E4M3, 0, 1.0) == 1.0
        assert O.c_scale(bad, O.E4M3, 0, 7.5) == 7.5          # delayed scaling keeps the previous scale
    assert O.c_scale(1e-42, O.E4M3) == O.FLT_MAX               # quotient overflows
    assert O.c_scale(2.0, O.E4M3) == 224.0 and O.c_scale(2.0, O.E5M2) == 28672.0
    assert O.c_scale(2.0, O.E4M3, margin=3) == 28.0            # each unit of margin halves the scale
    assert O.c_scale_inv(224.0) == np.float32(1.0) / np.float32(224.0)
    t = O.t_scale(torch.tensor([0.0, 2.0, float("nan")]), O.E4M3, margin=3, fallback=torch.tensor([5.0, 5.0, 6.0]))
    assert t.tolist() == [5.0, 28.0, 6.0]


# ------------------------------------------------------------------------ cast
@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
@pytest.mark.parametrize("mode", [O.SCALE_TENSOR, O.SCALE_ROW, O.SCALE_COL])
def test_cast_c_equals_torch_and_transpose_identity(fmt, mode):
    x = seeded_bf16((48, 40), 1.0, 2)
    x[0, 0], x[1, 1], x[2, 2], x[3, 3] = float("nan"), float("inf"), -float("inf"), -0.0
    n = {O.SCALE_TENSOR: 1, O.SCALE_ROW: 48, O.SCALE_COL: 40}[mode]
    s = torch.rand(n, generator=torch.Generator().manual_seed(3)) * 600 + 1.0      # large: the clamp fires
    c = O.c_cast(x, s, fmt, mode)
    t = O.t_cast(x, s, fmt, mode)
    assert torch.equal(c, t)
    q, qt = O.c_cast_transpose(x, s, fmt, mode)
    assert torch.equal(q, c) and torch.equal(qt, c.t().contiguous())
    top = 0x7E if fmt == O.E4M3 else 0x7B
    assert int(c[1, 1]) == top and int(c[2, 2]) == (top | 0x80)                    # Inf saturates after the clamp
    assert int(c[0, 0]) & 0x7F == 0x7F and int(c[3, 3]) == 0x80                    # NaN code, signed zero


def test_cast_rowwise_is_per_tensor_applied_to_each_row():
    x = seeded_bf16((6, 32), 1.0, 4)
    s = O.t_scale(O.t_amax(x, O.SCALE_ROW), O.E4M3)
    whole = O.c_cast(x, s, O.E4M3, O.SCALE_ROW)
    for r in range(6):
        assert torch.equal(whole[r:r + 1], O.c_cast(x[r:r + 1], s[r:r + 1], O.E4M3, O.SCALE_TENSOR))
    # scaling a row by 2^k changes only that row's scale, and none of its codes
    x2 = x.clone()
    x2[2] = (x2[2].float() * 16).bfloat16()
    s2 = O.t_scale(O.t_amax(x2, O.SCALE_ROW), O.E4M3)
    assert s2[2] == s[2] / 16 and torch.equal(s2[[0, 1, 3, 4, 5]], s[[0, 1, 3, 4, 5]])
    assert torch.equal(O.c_cast(x2, s2, O.E4M3, O.SCALE_ROW), whole)


def test_dynamic_scaling_never_needs_the_clamp_but_stale_scales_do():
    x = seeded_bf16((256, 256), 1.0, 5)
    s = O.t_scale(O.t_amax(x), O.E4M3)
    unclamped = (x.float() * s).to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(O.c_cast(x, s, O.E4M3), unclamped)
    stale = s * 4
    clamped = O.c_cast(x, stale, O.E4M3)
    assert (clamped & 0x7F).max() == 0x7E and ((x.float() * stale).to(torch.float8_e4m3fn).view(torch.uint8) & 0x7F).max() == 0x7F


# ------------------------------------------------------------------------ GEMM
def test_gemm_tiny_vs_float64_brute_force():
    rng = np.random.default_rng(6)
    M, N, K = 5, 7, 16
    a = torch.from_numpy(rng.integers(0, 256, (M, K)).astype(np.uint8))
    b = torch.from_numpy(rng.integers(0, 256, (N, K)).astype(np.uint8))
    a[(a & 0x7F) == 0x7F] = 0x10                                                   # no NaN codes (e4m3)
    b[(b & 0x7C) == 0x7C] = 0x10                                                   # no Inf/NaN codes (e5m2)
    da = O.c_decode(a.numpy(), O.E4M3).astype(np.float64)
    db = O.c_decode(b.numpy(), O.E5M2).astype(np.float64)
    sa, sb = np.float32(0.37), np.float32(1.9)
    want = (da @ db.T) * float(np.float32(sa * sb))
    got16, got32 = O.c_gemm_nt(a, b, O.E4M3, O.E5M2, [sa], [sb], want_f32=True)
    np.testing.assert_allclose(got32.numpy(), want, rtol=2e-6, atol=1e-30)
    assert torch.equal(got16, got32.bfloat16())
    t16, t32 = O.t_gemm_nt(a, b, O.E4M3, O.E5M2, [sa], [sb], want_f32=True)
    np.testing.assert_allclose(t32.numpy(), want, rtol=2e-6, atol=1e-30)


def test_gemm_exact_cases_and_epilogue():
    # one-hot A picks single columns of B: no rounding anywhere
    K, N = 32, 8
    b = torch.from_numpy(np.random.default_rng(7).integers(1, 0x70, (N, K)).astype(np.uint8))
    a = torch.zeros((K, K))
    a[torch.arange(K), torch.arange(K)] = 1.0
    aq = a.to(torch.float8_e4m3fn).view(torch.uint8)
    out32 = O.c_gemm_nt(aq, b, O.E4M3, O.E4M3, [1.0], [1.0], want_f32=True)[1]
    assert np.array_equal(out32.numpy(), O.c_decode(b.numpy(), O.E4M3).T)
    # rank-1 epilogue: per-row and per-column inverse scales
    sa = torch.tensor([2.0 ** (i % 5) for i in range(K)])
    sb = torch.tensor([2.0 ** -(j % 3) for j in range(N)])
    out_v = O.c_gemm_nt(aq, b, O.E4M3, O.E4M3, sa, sb, want_f32=True)[1]
    assert torch.equal(out_v, out32 * sa[:, None] * sb[None, :])
    assert torch.equal(O.t_gemm_nt(aq, b, O.E4M3, O.E4M3, sa, sb, want_f32=True)[1], out_v)
    # transpose symmetry
    o1 = O.c_gemm_nt(b, aq, O.E4M3, O.E4M3, [1.0], [1.0], want_f32=True)[1]
    assert torch.equal(o1, out32.t())


def test_gemm_matches_torch_scaled_mm_on_cpu():
    x, w = seeded_bf16((32, 64), 1.0, 8), seeded_bf16((16, 64), 0.02, 9)
    sx, sw = O.t_scale(O.t_amax(x), O.E4M3), O.t_scale(O.t_amax(w), O.E4M3)
    xq, wq = O.t_cast(x, sx, O.E4M3), O.t_cast(w, sw, O.E4M3)
    try:
        ref = torch._scaled_mm(xq.view(torch.float8_e4m3fn), wq.view(torch.float8_e4m3fn).t(),
                               scale_a=(1 / sx).float().reshape(()), scale_b=(1 / sw).float().reshape(()),
                               out_dtype=torch.bfloat16)
    except Exception as e:  # pragma: no cover - depends on the torch build
        pytest.skip(f"torch._scaled_mm not usable on this CPU build: {e}")
    got = O.t_gemm_nt(xq, wq, O.E4M3, O.E4M3, 1 / sx, 1 / sw)
    assert (got.float() - ref.float()).abs().max() <= 2 * ref.float().abs().max() * 2 ** -8


def test_linear_grads_equal_autograd_of_the_dequantised_operands():
    x, w, dy = seeded_bf16((64, 48), 1.0, 1), seeded_bf16((32, 48), 0.02, 2), seeded_bf16((64, 32), 1e-3, 3)
    r = O.linear_fwd_bwd(x, w, dy)
    xd = (O.t_decode(r["xq"], O.E4M3) / r["sx"]).requires_grad_(True)
    wd = (O.t_decode(r["wq"], O.E4M3) / r["sw"]).requires_grad_(True)
    gd = O.t_decode(r["gq"], O.E5M2) / r["sg"]
    (xd @ wd.t()).backward(gd)
    np.testing.assert_allclose(r["dx"].float().numpy(), xd.grad.numpy(), rtol=1e-2, atol=1e-9)
    np.testing.assert_allclose(r["dw"].float().numpy(), wd.grad.numpy(), rtol=1e-2, atol=1e-9)
    assert torch.equal(r["xq_t"], r["xq"].t().contiguous()) and torch.equal(r["gq_t"], r["gq"].t().contiguous())


def test_rowwise_linear_isolates_an_outlier_token_but_not_an_outlier_channel():
    x, w, dy = seeded_bf16((32, 64), 1.0, 1), seeded_bf16((16, 64), 0.02, 2), seeded_bf16((32, 16), 1e-3, 3)
    base = O.linear_fwd_bwd(x, w, dy, rowwise=True)
    x2 = x.clone()
    x2[3] = (x2[3].float() * 64).bfloat16()
    r2 = O.linear_fwd_bwd(x2, w, dy, rowwise=True)
    assert torch.equal(r2["xq"], base["xq"])                                       # codes untouched
    assert torch.equal(r2["y"][3].float(), base["y"][3].float() * 64) and torch.equal(r2["y"][4], base["y"][4])
    exact = x.float() @ w.float().t()
    assert (base["y"].float() - exact).abs().max() / exact.abs().max() < 0.08


# -------------------------------------------------------------- delayed scaling
def test_delayed_update_hand_worked_sequence():
    H = 3
    hist = np.zeros((H, 1), dtype=np.float32)
    scale, inv = np.ones(1, dtype=np.float32), np.ones(1, dtype=np.float32)
    used = []
    for amax in [4.0, 2.0, 1.0, 0.5, 0.25, 0.0, 0.0, 0.0]:
        used.append(float(scale[0]))
        hist[0, 0] = amax
        O.c_delayed_update(hist, scale, inv, [O.E4M3], margin=0, algo="max")
        assert hist[0, 0] == 0.0                                                    # row 0 is cleared for the next step
    # scale used at step t = 448 / max(amax_{t-3..t-1}); step 0 uses 1; an all-zero window keeps the last scale
    assert used == [1.0, 112.0, 112.0, 112.0, 224.0, 448.0, 896.0, 1792.0]
    assert scale[0] == 1792.0 and inv[0] == np.float32(1.0) / np.float32(1792.0)


def test_delayed_update_most_recent_margin_and_bad_values():
    hist = np.zeros((4, 2), dtype=np.float32)
    scale, inv = np.ones(2, dtype=np.float32), np.ones(2, dtype=np.float32)
    for amax in ([8.0, 1.0], [2.0, 4.0]):
        hist[0] = amax
        O.c_delayed_update(hist, scale, inv, [O.E4M3, O.E5M2], margin=1, algo="most_recent")
    assert scale.tolist() == [448.0 / 2.0 / 2.0, 57344.0 / 4.0 / 2.0]             # newest amax only, halved by the margin
    before = scale.copy()
    hist[0] = [np.nan, np.inf]
    O.c_delayed_update(hist, scale, inv, [O.E4M3, O.E5M2], margin=1, algo="most_recent")
    assert np.array_equal(scale, before)                                           # non-finite amax: scale kept


def test_python_delayed_state_equals_c_oracle():
    rng = np.random.default_rng(11)
    H, R = 16, 5
    fmts = [O.E4M3, O.E4M3, O.E4M3, O.E5M2, O.E5M2]
    for algo in ("max", "most_recent"):
        st = O.DelayedState(fmts, H, margin=2, algo=algo)
        hist = np.zeros((H, R), dtype=np.float32)
        scale, inv = np.ones(R, dtype=np.float32), np.ones(R, dtype=np.float32)
        for step in range(40):
            new = np.abs(rng.normal(0, 1 + 0.05 * step, R)).astype(np.float32)
            if step % 7 == 3:
                new[step % R] = 0.0
            for r in range(R):
                st.record(r, new[r])
            hist[0] = new
            st.update()
            O.c_delayed_update(hist, scale, inv, fmts, margin=2, algo=algo)
            assert np.array_equal(st.history, hist) and np.array_equal(st.scale, scale) and np.array_equal(st.scale_inv, inv)


def test_sum_of_products_equals_one_product_over_joined_operands():
    """With one scale pair for all, the sum over operand pairs is the product of the operands joined along the
    contraction; on power-of-two values every partial sum is exact, so the two must agree bit for bit.  A pair dropped,
    counted twice or scaled by another pair's scales breaks it."""
    g = torch.Generator().manual_seed(3)
    vals = torch.tensor([0.0, 1.0, -1.0, 2.0, -2.0, 0.5, -0.5, 4.0])
    ks = (64, 32, 96)
    a = [vals[torch.randint(0, 8, (24, k), generator=g)].to(torch.float8_e5m2).view(torch.uint8) for k in ks]
    b = [vals[torch.randint(0, 8, (40, k), generator=g)].to(torch.float8_e4m3fn).view(torch.uint8) for k in ks]
    sa, sb = torch.tensor([0.5]), torch.tensor([0.125])
    joined = O.t_gemm_nt(torch.cat(a, 1), torch.cat(b, 1), O.E5M2, O.E4M3, sa, sb, want_f32=True)[1]
    got16, got32 = O.t_gemm_nt_sum([(x, y, sa, sb) for x, y in zip(a, b)], O.E5M2, O.E4M3, want_f32=True)
    assert torch.equal(got32, joined) and torch.equal(got16, joined.bfloat16())
    # a scale of its own per pair: linear in each
    scales = [(torch.tensor([2.0 ** -i]), torch.tensor([2.0 ** i * 0.25])) for i in range(3)]
    want = sum(O.t_gemm_nt(x, y, O.E5M2, O.E4M3, p, q, want_f32=True)[1] for x, y, (p, q) in zip(a, b, scales))
    got = O.t_gemm_nt_sum([(x, y, p, q) for x, y, (p, q) in zip(a, b, scales)], O.E5M2, O.E4M3, want_f32=True)[1]
    assert torch.equal(got, want) and torch.equal(got, joined * 0.25 / 0.0625)
