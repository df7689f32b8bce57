"""Pins the oracle's SwiGLU and RMSNorm functions (CPU only).  The kernels are later required to
equal these functions bit for bit, so what is checked here is that the fixed arithmetic IS the
mathematical function and IS what eager PyTorch computes, by means other than retyping it:
float64 evaluation over every bf16 input, torch's own bf16 silu / multiply / autograd, closed
forms with exact results, and index-revealing special cases."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O
from tests.helpers import seeded_bf16


def all_bf16() -> torch.Tensor:
    bits = np.arange(65536, dtype=np.uint16)
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def ulp_distance(a: torch.Tensor, b: torch.Tensor) -> np.ndarray:
    """Distance in bf16 units between same-signed finite values (bit patterns are monotone)."""
    ab = a.contiguous().view(torch.int16).numpy().astype(np.int32)
    bb = b.contiguous().view(torch.int16).numpy().astype(np.int32)
    same_zero = (a.float().numpy() == 0) & (b.float().numpy() == 0)
    return np.where(same_zero, 0, np.abs(ab - bb))


# --------------------------------------------------------------------- sigmoid
def test_sigmoid_every_bf16_input_against_float64():
    g = all_bf16().float().numpy()
    got = np.array([O.c_sigmoid(float(v)) for v in g], dtype=np.float64)
    finite = np.isfinite(g)
    with np.errstate(over="ignore"):
        want = 1.0 / (1.0 + np.exp(-g[finite].astype(np.float64)))
    inside = g[finite] >= -80.0
    with np.errstate(invalid="ignore", divide="ignore"):
        rel = np.abs(got[finite] - want) / want
    assert rel[inside].max() < 2.0 ** -22                         # about two units of fp32
    # below -80 the function is defined as 0; the exact value there is under 2e-35
    assert np.all(got[finite][~inside] == 0.0) and want[~inside].max() < 2e-35
    assert np.all(np.isnan(got[np.isnan(g)]))
    assert O.c_sigmoid(float("inf")) == 1.0 and O.c_sigmoid(float("-inf")) == 0.0


def test_sigmoid_exact_points_and_symmetry():
    assert O.c_sigmoid(0.0) == 0.5
    assert O.c_sigmoid(100.0) == 1.0 and O.c_sigmoid(-100.0) == 0.0
    # sigmoid(g) + sigmoid(-g) = 1 up to rounding; monotone non-decreasing over the bf16 grid
    g = all_bf16().float().numpy()
    g = np.sort(g[np.isfinite(g)])
    s = np.array([O.c_sigmoid(float(v)) for v in g], dtype=np.float64)
    assert np.all(np.diff(s) >= 0)
    pos = g[(g > 0) & (g < 60)]
    sp = np.array([O.c_sigmoid(float(v)) + O.c_sigmoid(float(-v)) for v in pos])
    assert np.abs(sp - 1.0).max() < 3e-7


# ---------------------------------------------------------------------- SwiGLU
def test_silu_every_bf16_input_equals_torch():
    g = all_bf16()
    got = O.c_swiglu_fwd(g, torch.ones_like(g))                   # up = 1: h is silu(g) itself
    want = F.silu(g)
    nan = torch.isnan(want)
    assert torch.equal(torch.isnan(got), nan)
    keep = ~nan & (g.float() >= -80.0)
    assert torch.equal(got[keep].view(torch.int16), want[keep].view(torch.int16))
    low = ~nan & (g.float() < -80.0)                              # defined as -0 there; torch leaves < 1e-32
    assert torch.all(got[low].float() == 0) and want[low].float().abs().max() < 1e-32


@pytest.mark.parametrize("std_g,std_u,seed", [(1.0, 1.0, 0), (4.0, 0.5, 1), (0.05, 20.0, 2)])
def test_swiglu_forward_equals_torch_eager_bf16(std_g, std_u, seed):
    g, u = seeded_bf16((257, 96), std_g, seed), seeded_bf16((257, 96), std_u, seed + 100)
    got = O.c_swiglu_fwd(g, u)
    want = F.silu(g) * u
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_swiglu_forward_special_values():
    g = torch.tensor([0.0, -0.0, 3.0, -3.0, 90.0, -90.0, float("inf"), float("nan"), 2.0], dtype=torch.bfloat16)
    u = torch.tensor([5.0, 5.0, 0.0, -0.0, 2.0, 2.0, 1.0, 1.0, float("nan")], dtype=torch.bfloat16)
    h = O.c_swiglu_fwd(g, u).float()
    assert h[0] == 0 and h[1] == 0 and h[2] == 0 and h[3] == 0
    assert h[4] == 180.0                                         # sigmoid(90) is exactly 1
    assert h[5] == 0.0
    assert h[6] == float("inf") and torch.isnan(h[7]) and torch.isnan(h[8])


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_swiglu_backward_against_torch_autograd_bf16(seed):
    shape = (193, 128)
    g, u = seeded_bf16(shape, 1.5, seed), seeded_bf16(shape, 1.0, seed + 10)
    dh = seeded_bf16(shape, 1e-3, seed + 20)
    ga, ua = g.clone().requires_grad_(True), u.clone().requires_grad_(True)
    (F.silu(ga) * ua).backward(dh)
    dg, du = O.c_swiglu_bwd(dh, g, u)
    # d_up = dh * silu(g): the same two roundings as autograd -> identical
    assert torch.equal(du.view(torch.int16), ua.grad.view(torch.int16))
    # d_gate: autograd multiplies (grad * sig) * (1 + g (1 - sig)), here grad * (sig * (...)):
    # the products differ in the last fp32 bit now and then, which can move a bf16 rounding by one unit
    d = ulp_distance(dg, ga.grad)
    assert d.max() <= 1
    assert (d > 0).mean() < 0.01
    # and against float64: within one bf16 unit of the exact derivative of the bf16 intermediate
    g64, u64, d64 = g.double(), u.double(), dh.double()
    sig = torch.sigmoid(g64)
    exact = (dh.float() * u.float()).bfloat16().double() * sig * (1 + g64 * (1 - sig))
    assert ulp_distance(dg, exact.float().bfloat16()).max() <= 1
    del d64, u64


def test_swiglu_backward_zero_and_saturated():
    g = torch.tensor([0.0, 50.0, -50.0, 1.0], dtype=torch.bfloat16)
    u = torch.tensor([2.0, 3.0, 3.0, 0.0], dtype=torch.bfloat16)
    dh = torch.tensor([1.0, 1.0, 1.0, 0.0], dtype=torch.bfloat16)
    dg, du = O.c_swiglu_bwd(dh, g, u)
    assert dg[0].item() == 1.0                                   # silu'(0) = 1/2, times dh * u = 2
    assert dg[1].item() == 3.0 and du[1].item() == 50.0          # silu(g) = g, silu' = 1 for large g
    assert abs(dg[2].item()) < 1e-18 and abs(du[2].item()) < 1e-18
    assert dg[3].item() == 0.0 and du[3].item() == 0.0


# --------------------------------------------------------------------- RMSNorm
@pytest.mark.parametrize("cols", [8, 64, 520, 4096])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_against_float64_closed_form(cols, dtype):
    rows, eps = 9, 1e-5
    g = torch.Generator().manual_seed(cols)
    x = (torch.randn((rows, cols), generator=g) * 3.0).to(dtype)
    w = torch.randn(cols, generator=g) * 0.5 + 1.0
    y, rstd = O.c_rmsnorm(x, w, eps)
    x64 = x.double()
    rstd64 = 1.0 / torch.sqrt((x64 * x64).mean(-1) + eps)
    assert ((rstd.double() - rstd64).abs() / rstd64).max() < 1e-6
    want = (x64 * rstd64[:, None] * w.double()).float().bfloat16()
    d = ulp_distance(y, want)
    assert d.max() <= 1 and (d > 0).mean() < 0.01
    # the reference module's own expression, evaluated by torch in fp32 (layer_norms.py:86-119)
    xf = x.float()
    ref = ((xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)) * w).bfloat16()
    d = ulp_distance(y, ref)
    assert d.max() <= 1 and (d > 0).mean() < 0.01


def test_rmsnorm_exact_case_reveals_indexing():
    # every element of row r is +-2^r: the mean of squares is 4^r exactly, rstd = 2^-r exactly
    # (eps = 0), so y[r, c] = +-weight[c] rounded to bf16, whatever the summation order
    rows, cols = 6, 136
    sign = torch.where(torch.arange(cols) % 3 == 0, -1.0, 1.0)
    x = torch.stack([sign * 2.0 ** r for r in range(rows)]).bfloat16()
    w = torch.arange(1, cols + 1, dtype=torch.float32) / 8.0
    y, rstd = O.c_rmsnorm(x, w, 0.0)
    assert torch.equal(rstd, torch.tensor([2.0 ** -r for r in range(rows)]))
    assert torch.equal(y, (sign * w).bfloat16().expand(rows, cols))


def test_rmsnorm_summation_order_is_the_documented_one():
    # numpy restatement of the stated order (64 lanes, chunks of 8 dealt round-robin, xor butterfly)
    rows, cols, eps = 3, 1032, 1e-6
    x = seeded_bf16((rows, cols), 2.0, 5)
    _, rstd = O.c_rmsnorm(x, torch.ones(cols), eps)
    xf = x.float().numpy()
    for r in range(rows):
        acc = np.zeros(64, dtype=np.float32)
        chunks = xf[r].reshape(-1, 8)
        for lane in range(64):
            a = np.float64(0.0)
            s = np.float32(0.0)
            for c in range(lane, chunks.shape[0], 64):
                for v in chunks[c]:
                    # fma: the product of two bf16 values is exact in float64, so is product + fp32 sum
                    a = np.float64(v) * np.float64(v) + np.float64(s)
                    s = np.float32(a)
            acc[lane] = s
        off = 32
        while off:
            acc = (acc + acc[np.arange(64) ^ off]).astype(np.float32)
            off //= 2
        mean = np.float32(acc[0] / np.float32(cols))
        want = np.float32(1.0) / np.sqrt(np.float32(mean + np.float32(eps)), dtype=np.float32)
        assert rstd[r].item() == want


@pytest.mark.parametrize("cols", [8, 520, 2048])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rmsnorm_backward_against_torch_autograd(cols, dtype):
    rows, eps = 21, 1e-5
    g = torch.Generator().manual_seed(cols + 7)
    x = (torch.randn((rows, cols), generator=g) * 2.0).to(dtype)
    w = torch.randn(cols, generator=g) * 0.5 + 1.0
    dy = (torch.randn((rows, cols), generator=g) * 1e-2).bfloat16()
    _, rstd = O.c_rmsnorm(x, w, eps)
    dx, dw = O.c_rmsnorm_bwd(dy, x, w, rstd)
    # autograd through the reference module's expression (layer_norms.py:86-119), in float64
    xa = x.double().requires_grad_(True)
    wa = w.double().requires_grad_(True)
    y = (xa * torch.rsqrt(xa.pow(2).mean(-1, keepdim=True) + eps)) * wa
    y.backward(dy.double())
    assert dx.dtype == dtype
    scale = xa.grad.abs().max().item()
    tol = 2.0 ** -8 if dtype == torch.bfloat16 else 1e-5             # half a bf16 unit at the top of the range / fp32 noise
    assert (dx.double() - xa.grad).abs().max().item() <= tol * scale
    assert ((dw.double() - wa.grad).abs() / wa.grad.abs().max()).max().item() < 1e-5


def test_rmsnorm_backward_exact_case():
    # x[r, :] = +-2^r, weight = 1, eps = 0: xh = +-1, rstd = 2^-r.  With dy = xh * 2^-3 the projection
    # removes everything: t = dy, c = mean(dy * xh) = 2^-3, dx = rstd * (dy - xh * 2^-3) = 0 exactly;
    # d_weight[col] = sum_r dy * xh = rows * 2^-3
    rows, cols = 5, 64
    sign = torch.where(torch.arange(cols) % 2 == 0, -1.0, 1.0)
    x = torch.stack([sign * 2.0 ** r for r in range(rows)]).bfloat16()
    w = torch.ones(cols)
    _, rstd = O.c_rmsnorm(x, w, 0.0)
    dy = (sign * 0.125).bfloat16().expand(rows, cols).contiguous()
    dx, dw = O.c_rmsnorm_bwd(dy, x, w, rstd)
    assert torch.all(dx.float() == 0)
    assert torch.equal(dw, torch.full((cols,), rows * 0.125))
    # a gradient along one column only: dx[r, k] = rstd * (w_k dy - xh_k * xh_k w_k dy / cols) for that column
    dy = torch.zeros((rows, cols), dtype=torch.bfloat16)
    dy[:, 3] = 1.0
    dx, dw = O.c_rmsnorm_bwd(dy, x, w, rstd)
    want3 = torch.tensor([2.0 ** -r * (1 - 1 / cols) for r in range(rows)]).bfloat16()
    assert torch.equal(dx[:, 3], want3)
    assert torch.equal(dw, torch.nn.functional.one_hot(torch.tensor(3), cols).float() * rows * sign[3])


# ------------------------------------------------------------------- LayerNorm
@pytest.mark.parametrize("cols", [8, 520, 768, 4096])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_bias", [True, False])
def test_layernorm_against_float64_and_torch(cols, dtype, with_bias):
    rows, eps = 11, 1e-5
    g = torch.Generator().manual_seed(cols + 3)
    x = (torch.randn((rows, cols), generator=g) * 2.0 + 0.7).to(dtype)
    w = torch.randn(cols, generator=g) * 0.5 + 1.0
    b = torch.randn(cols, generator=g) * 0.2 if with_bias else None
    y, mean, rstd = O.c_layernorm(x, w, b, eps)
    x64 = x.double()
    mean64 = x64.mean(-1)
    rstd64 = 1.0 / torch.sqrt(x64.var(-1, unbiased=False) + eps)
    assert (mean.double() - mean64).abs().max() < 1e-6 and ((rstd.double() - rstd64).abs() / rstd64).max() < 1e-6
    want = (x64 - mean64[:, None]) * rstd64[:, None] * w.double() + (0 if b is None else b.double())
    d = ulp_distance(y, want.float().bfloat16())
    assert d.max() <= 1 and (d > 0).mean() < 0.01
    ref = F.layer_norm(x.float(), (cols,), w, b, eps).bfloat16()            # the routine the reference module calls
    d = ulp_distance(y, ref)
    assert d.max() <= 1 and (d > 0).mean() < 0.01


def test_layernorm_exact_case_reveals_indexing():
    # row r holds +-2^r in equal numbers: mean 0, variance 4^r, rstd 2^-r (eps = 0): y = +-weight + bias exactly
    rows, cols = 5, 144
    sign = torch.where(torch.arange(cols) % 2 == 0, -1.0, 1.0)
    x = torch.stack([sign * 2.0 ** r for r in range(rows)]).bfloat16()
    w = torch.arange(1, cols + 1, dtype=torch.float32) / 16.0
    b = torch.arange(cols, dtype=torch.float32) / 4.0
    y, mean, rstd = O.c_layernorm(x, w, b, 0.0)
    assert torch.equal(mean, torch.zeros(rows)) and torch.equal(rstd, torch.tensor([2.0 ** -r for r in range(rows)]))
    assert torch.equal(y, (sign * w + b).bfloat16().expand(rows, cols))
    # a constant shift changes nothing but the mean
    y2, mean2, _ = O.c_layernorm((x.float() + 8.0).bfloat16()[:3], w, b, 0.0)
    assert torch.equal(mean2, torch.full((3,), 8.0)) and torch.equal(y2, y[:3])


@pytest.mark.parametrize("cols", [8, 520, 768])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_layernorm_backward_against_torch_autograd(cols, dtype):
    rows, eps = 19, 1e-5
    g = torch.Generator().manual_seed(cols + 11)
    x = (torch.randn((rows, cols), generator=g) * 2.0 - 0.3).to(dtype)
    w = torch.randn(cols, generator=g) * 0.5 + 1.0
    b = torch.randn(cols, generator=g) * 0.1
    dy = (torch.randn((rows, cols), generator=g) * 1e-2).bfloat16()
    _, mean, rstd = O.c_layernorm(x, w, b, eps)
    dx, dw, db = O.c_layernorm_bwd(dy, x, w, mean, rstd)
    xa, wa, ba = x.double().requires_grad_(True), w.double().requires_grad_(True), b.double().requires_grad_(True)
    F.layer_norm(xa, (cols,), wa, ba, eps).backward(dy.double())
    scale = xa.grad.abs().max().item()
    tol = 2.0 ** -8 if dtype == torch.bfloat16 else 1e-5
    assert dx.dtype == dtype and (dx.double() - xa.grad).abs().max().item() <= tol * scale
    assert ((dw.double() - wa.grad).abs() / wa.grad.abs().max()).max().item() < 1e-5
    assert ((db.double() - ba.grad).abs() / ba.grad.abs().max()).max().item() < 1e-5


# ------------------------------------------------------------------------ GELU
def test_gelu_every_bf16_input_against_torch_and_float64():
    x = all_bf16()
    with np.errstate(invalid="ignore"):
        xs = x.float().numpy().astype(np.float64)
    y = O.c_gelu_fwd(x)
    finite = np.isfinite(xs)
    # float64 closed form with scipy's erfc: the oracle is its value rounded to float, then to bf16
    from scipy.special import erfc

    with np.errstate(over="ignore", invalid="ignore"):
        exact = xs[finite] * 0.5 * erfc(-xs[finite] / np.sqrt(2.0))
    want = torch.from_numpy(exact.astype(np.float32)).bfloat16()
    assert torch.equal(y[torch.from_numpy(finite)].view(torch.int16), want.view(torch.int16))
    # torch's own F.gelu (1 + erf evaluated in float): identical wherever that formula is accurate and neither
    # side is in the denormal / overflow range; below -3 torch loses the tail: absolute comparison there
    t = F.gelu(x)
    ys, ts = y.float().numpy(), t.float().numpy()
    core = finite & (xs >= -3.0) & (np.abs(xs) < 1e38) & (np.abs(ys) >= 1.2e-38)
    assert core.sum() > 48000
    assert np.array_equal(y.view(torch.int16).numpy()[core], t.view(torch.int16).numpy()[core])
    tail = finite & (xs < -3.0)
    assert np.abs(ys[tail] - ts[tail]).max() < 2e-5
    assert np.isnan(ys[np.isnan(xs)]).all() and ys[xs == np.inf][0] == np.inf


def test_gelu_backward_against_torch_autograd():
    x = all_bf16()
    keep = torch.isfinite(x.float())
    xk = x[keep]
    for scale in (1.0, -0.0078125, 3.0):
        dy = torch.full_like(xk, scale)
        xa = xk.clone().requires_grad_(True)
        F.gelu(xa).backward(dy)
        dx = O.c_gelu_bwd(dy, xk)
        xs = xk.float().numpy()
        core = (xs >= -3.0) & (np.abs(xs) < 1e38)
        d = ulp_distance(dx, xa.grad)
        assert d[core].max() <= 1 and (d[core] > 0).mean() < 0.01
        assert np.abs(dx.float().numpy() - xa.grad.float().numpy())[~core & np.isfinite(xa.grad.float().numpy())].max() < 4e-5 * abs(scale) + 1e-30
    # closed-form spot values: gelu'(0) = 1/2, gelu'(large) = 1, gelu'(-large) = 0
    pts = torch.tensor([0.0, 20.0, -20.0], dtype=torch.bfloat16)
    assert O.c_gelu_bwd(torch.ones_like(pts), pts).tolist() == [0.5, 1.0, 0.0]
