"""CPU oracle for the FP8 Linear path (TEST INFRASTRUCTURE ONLY).

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module.  It offers the same operations twice:

* ``c_*``  : thin ctypes wrappers over the plain-C restatement in
  ``fp8_oracle.c`` (scalar loops; every rounding step is spelled out).
* ``t_*``  : the same definitions written with torch CPU library routines
  (``Tensor.to(torch.float8_*)``, fp32 ``@``).  They are fast enough for the
  medium-sized parity cases and serve as the CPU baseline that is timed.

The reference repository contains no FP8 arithmetic (it forwards to a
third-party CUDA library at
optimus_dl/modules/model_transforms/transformer_engine.py:97-108 and
optimus_dl/modules/amp/fp8.py:254-306); both families follow the definitions in
the header of ``fp8_oracle.c`` and are cross-checked against each other, against
the 8-bit format definitions and against brute force in ``tests/``.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

E4M3, E5M2 = 0, 1
SCALE_TENSOR, SCALE_ROW, SCALE_COL = 0, 1, 2
FP8_MAX = {E4M3: 448.0, E5M2: 57344.0}
TORCH_FP8 = {E4M3: torch.float8_e4m3fn, E5M2: torch.float8_e5m2}
FLT_MAX = float(np.finfo(np.float32).max)

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libfp8_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile fp8_oracle.c with the Makefile beside it (gcc only)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.oracle_f32_to_e4m3.argtypes = [f32]
        L.oracle_f32_to_e4m3.restype = ctypes.c_uint8
        L.oracle_f32_to_e5m2.argtypes = [f32]
        L.oracle_f32_to_e5m2.restype = ctypes.c_uint8
        L.oracle_encode_f32.argtypes = [vp, i64, i32, vp]
        L.oracle_decode.argtypes = [vp, i64, i32, vp]
        L.oracle_amax_bf16.argtypes = [vp, i64, i64, i32, vp]
        L.oracle_scale.argtypes = [f32, i32, i32, f32]
        L.oracle_scale.restype = f32
        L.oracle_scale_inv.argtypes = [f32]
        L.oracle_scale_inv.restype = f32
        L.oracle_cast_bf16.argtypes = [vp, i64, i64, vp, i32, i32, vp]
        L.oracle_cast_transpose_bf16.argtypes = [vp, i64, i64, vp, i32, i32, vp, vp]
        L.oracle_gemm_nt.argtypes = [vp, vp, i64, i64, i64, i32, i32, vp, i64, vp, i64, vp, vp]
        L.oracle_delayed_update.argtypes = [vp, i64, i64, vp, vp, vp, i32, i32]
        L.oracle_mx_quantise_bf16.argtypes = [vp, i64, i64, i32, i32, vp, vp]
        L.oracle_mx_gemm_nt.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32, vp, vp, vp]
        L.oracle_block_quantise_bf16.argtypes = [vp, i64, i64, i64, i64, i32, i32, vp, vp]
        L.oracle_sigmoid.argtypes = [f32]
        L.oracle_sigmoid.restype = f32
        L.oracle_swiglu_fwd.argtypes = [vp, vp, i64, vp]
        L.oracle_swiglu_bwd.argtypes = [vp, vp, vp, i64, vp, vp]
        L.oracle_rmsnorm.argtypes = [vp, i32, vp, i64, i64, f32, vp, vp]
        L.oracle_rmsnorm_bwd.argtypes = [vp, vp, i32, vp, vp, i64, i64, vp, vp]
        L.oracle_gelu_fwd.argtypes = [vp, i64, vp]
        L.oracle_gelu_bwd.argtypes = [vp, vp, i64, vp]
        L.oracle_layernorm.argtypes = [vp, i32, vp, vp, i64, i64, f32, vp, vp, vp]
        L.oracle_layernorm_bwd.argtypes = [vp, vp, i32, vp, vp, vp, i64, i64, vp, vp, vp]
        _lib = L
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


def _bf16_bits(x: torch.Tensor) -> np.ndarray:
    assert x.dtype == torch.bfloat16 and x.device.type == "cpu"
    return np.ascontiguousarray(x.contiguous().view(torch.int16).numpy().view(np.uint16))


def _as_f32(s) -> np.ndarray:
    if isinstance(s, torch.Tensor):
        s = s.detach().cpu().float().numpy()
    return np.ascontiguousarray(np.asarray(s, dtype=np.float32).reshape(-1))


# --------------------------------------------------------------------- C family
def c_encode(x_f32: np.ndarray, fmt: int) -> np.ndarray:
    x = np.ascontiguousarray(x_f32, dtype=np.float32).reshape(-1)
    out = np.empty(x.size, dtype=np.uint8)
    lib().oracle_encode_f32(_p(x), x.size, fmt, _p(out))
    return out.reshape(np.shape(x_f32))


def c_decode(codes: np.ndarray, fmt: int) -> np.ndarray:
    c = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
    out = np.empty(c.size, dtype=np.float32)
    lib().oracle_decode(_p(c), c.size, fmt, _p(out))
    return out.reshape(np.shape(codes))


def c_amax(x: torch.Tensor, mode: int = SCALE_TENSOR) -> torch.Tensor:
    rows, cols = x.shape
    bits = _bf16_bits(x)
    n = 1 if mode == SCALE_TENSOR else (rows if mode == SCALE_ROW else cols)
    out = np.empty(n, dtype=np.float32)
    lib().oracle_amax_bf16(_p(bits), rows, cols, mode, _p(out))
    return torch.from_numpy(out)


def c_scale(amax: float, fmt: int, margin: int = 0, fallback: float = 1.0) -> float:
    return float(lib().oracle_scale(float(amax), fmt, margin, float(fallback)))


def c_scale_inv(scale: float) -> float:
    return float(lib().oracle_scale_inv(float(scale)))


def c_cast(x: torch.Tensor, scale, fmt: int, mode: int = SCALE_TENSOR) -> torch.Tensor:
    rows, cols = x.shape
    bits, s = _bf16_bits(x), _as_f32(scale)
    assert s.size == (1 if mode == SCALE_TENSOR else (rows if mode == SCALE_ROW else cols))
    out = np.empty((rows, cols), dtype=np.uint8)
    lib().oracle_cast_bf16(_p(bits), rows, cols, _p(s), mode, fmt, _p(out))
    return torch.from_numpy(out)


def c_cast_transpose(x: torch.Tensor, scale, fmt: int, mode: int = SCALE_TENSOR):
    rows, cols = x.shape
    bits, s = _bf16_bits(x), _as_f32(scale)
    out = np.empty((rows, cols), dtype=np.uint8)
    out_t = np.empty((cols, rows), dtype=np.uint8)
    lib().oracle_cast_transpose_bf16(_p(bits), rows, cols, _p(s), mode, fmt, _p(out), _p(out_t))
    return torch.from_numpy(out), torch.from_numpy(out_t)


def c_gemm_nt(a: torch.Tensor, b: torch.Tensor, fmt_a: int, fmt_b: int, sa_inv, sb_inv, want_f32: bool = False):
    """a[M,K], b[N,K] uint8 codes -> bf16 [M,N] (and the unrounded fp32 when asked)."""
    M, K = a.shape
    N, K2 = b.shape
    assert K == K2
    an = np.ascontiguousarray(a.numpy(), dtype=np.uint8)
    bn = np.ascontiguousarray(b.numpy(), dtype=np.uint8)
    sa, sb = _as_f32(sa_inv), _as_f32(sb_inv)
    assert sa.size in (1, M) and sb.size in (1, N)
    c16 = np.empty((M, N), dtype=np.uint16)
    c32 = np.empty((M, N), dtype=np.float32) if want_f32 else None
    lib().oracle_gemm_nt(_p(an), _p(bn), M, N, K, fmt_a, fmt_b, _p(sa), sa.size, _p(sb), sb.size,
                         _p(c16), _p(c32) if want_f32 else None)
    out = torch.from_numpy(c16.view(np.int16)).view(torch.bfloat16)
    return (out, torch.from_numpy(c32)) if want_f32 else out


def c_delayed_update(history: np.ndarray, scale: np.ndarray, scale_inv: np.ndarray, fmts, margin: int, algo: str):
    """In-place update of history[H,R], scale[R], scale_inv[R] (fp32 numpy arrays)."""
    H, R = history.shape
    assert history.dtype == np.float32 and history.flags.c_contiguous
    f = np.ascontiguousarray(np.asarray(fmts, dtype=np.int32))
    lib().oracle_delayed_update(_p(history), H, R, _p(scale), _p(scale_inv), _p(f), margin,
                                0 if algo == "max" else 1)


# ----------------------------------------------------------------- torch family
def _from_bf16_bits(bits: np.ndarray, shape) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16).copy()).view(torch.bfloat16).reshape(shape)


def c_sigmoid(g: float) -> float:
    return float(lib().oracle_sigmoid(float(g)))


def c_swiglu_fwd(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """h = silu(gate) * up with the roundings of eager bf16 arithmetic (bf16 tensors in and out)."""
    g, u = _bf16_bits(gate), _bf16_bits(up)
    h = np.empty_like(g)
    lib().oracle_swiglu_fwd(_p(g), _p(u), g.size, _p(h))
    return _from_bf16_bits(h, gate.shape)


def c_swiglu_bwd(dh: torch.Tensor, gate: torch.Tensor, up: torch.Tensor):
    d, g, u = _bf16_bits(dh), _bf16_bits(gate), _bf16_bits(up)
    dg, du = np.empty_like(g), np.empty_like(g)
    lib().oracle_swiglu_bwd(_p(d), _p(g), _p(u), g.size, _p(dg), _p(du))
    return _from_bf16_bits(dg, gate.shape), _from_bf16_bits(du, gate.shape)


def c_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """-> (y bf16, rstd fp32[rows]); x bf16 or fp32, normalised over the last axis."""
    cols = x.shape[-1]
    rows = x.numel() // cols
    if x.dtype == torch.bfloat16:
        xs, src = _bf16_bits(x), 0
    else:
        xs, src = np.ascontiguousarray(x.detach().float().cpu().numpy()).reshape(-1), 1
    w = np.ascontiguousarray(weight.detach().float().cpu().numpy())
    y = np.empty(rows * cols, dtype=np.uint16)
    rstd = np.empty(rows, dtype=np.float32)
    lib().oracle_rmsnorm(_p(xs), src, _p(w), rows, cols, float(eps), _p(y), _p(rstd))
    return _from_bf16_bits(y, x.shape), torch.from_numpy(rstd).reshape(x.shape[:-1])


def c_rmsnorm_bwd(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, rstd: torch.Tensor):
    """-> (dx in the dtype of x, d_weight fp32); dy bf16."""
    cols = x.shape[-1]
    rows = x.numel() // cols
    d = _bf16_bits(dy)
    if x.dtype == torch.bfloat16:
        xs, src, dx = _bf16_bits(x), 0, np.empty(rows * cols, dtype=np.uint16)
    else:
        xs, src, dx = np.ascontiguousarray(x.detach().float().cpu().numpy()).reshape(-1), 1, np.empty(rows * cols, dtype=np.float32)
    w = np.ascontiguousarray(weight.detach().float().cpu().numpy())
    rs = np.ascontiguousarray(rstd.detach().float().cpu().numpy().reshape(-1))
    dw = np.empty(cols, dtype=np.float32)
    lib().oracle_rmsnorm_bwd(_p(d), _p(xs), src, _p(w), _p(rs), rows, cols, _p(dx), _p(dw))
    dx_t = _from_bf16_bits(dx, x.shape) if src == 0 else torch.from_numpy(dx).reshape(x.shape)
    return dx_t, torch.from_numpy(dw)


def _src_array(x: torch.Tensor):
    if x.dtype == torch.bfloat16:
        return _bf16_bits(x), 0
    return np.ascontiguousarray(x.detach().float().cpu().numpy()).reshape(-1), 1


def c_layernorm(x: torch.Tensor, weight: torch.Tensor, bias, eps: float):
    """-> (y bf16, mean fp32, rstd fp32); x bf16 or fp32, normalised over the last axis; bias may be None."""
    cols = x.shape[-1]
    rows = x.numel() // cols
    xs, src = _src_array(x)
    w = np.ascontiguousarray(weight.detach().float().cpu().numpy())
    b = None if bias is None else np.ascontiguousarray(bias.detach().float().cpu().numpy())
    y = np.empty(rows * cols, dtype=np.uint16)
    mean, rstd = np.empty(rows, dtype=np.float32), np.empty(rows, dtype=np.float32)
    lib().oracle_layernorm(_p(xs), src, _p(w), None if b is None else _p(b), rows, cols, float(eps), _p(y), _p(mean), _p(rstd))
    lead = x.shape[:-1]
    return _from_bf16_bits(y, x.shape), torch.from_numpy(mean).reshape(lead), torch.from_numpy(rstd).reshape(lead)


def c_layernorm_bwd(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, mean: torch.Tensor, rstd: torch.Tensor):
    """-> (dx in the dtype of x, d_weight fp32, d_bias fp32); dy bf16."""
    cols = x.shape[-1]
    rows = x.numel() // cols
    d = _bf16_bits(dy)
    xs, src = _src_array(x)
    dx = np.empty(rows * cols, dtype=np.uint16 if src == 0 else np.float32)
    w = np.ascontiguousarray(weight.detach().float().cpu().numpy())
    mu = np.ascontiguousarray(mean.detach().float().cpu().numpy().reshape(-1))
    rs = np.ascontiguousarray(rstd.detach().float().cpu().numpy().reshape(-1))
    dw, db = np.empty(cols, dtype=np.float32), np.empty(cols, dtype=np.float32)
    lib().oracle_layernorm_bwd(_p(d), _p(xs), src, _p(w), _p(mu), _p(rs), rows, cols, _p(dx), _p(dw), _p(db))
    dx_t = _from_bf16_bits(dx, x.shape) if src == 0 else torch.from_numpy(dx).reshape(x.shape)
    return dx_t, torch.from_numpy(dw), torch.from_numpy(db)


def c_gelu_fwd(x: torch.Tensor) -> torch.Tensor:
    xs = _bf16_bits(x)
    y = np.empty_like(xs)
    lib().oracle_gelu_fwd(_p(xs), xs.size, _p(y))
    return _from_bf16_bits(y, x.shape)


def c_gelu_bwd(dy: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    d, xs = _bf16_bits(dy), _bf16_bits(x)
    dx = np.empty_like(xs)
    lib().oracle_gelu_bwd(_p(d), _p(xs), xs.size, _p(dx))
    return _from_bf16_bits(dx, x.shape)


def t_amax(x: torch.Tensor, mode: int = SCALE_TENSOR) -> torch.Tensor:
    a = x.abs()
    if mode == SCALE_TENSOR:
        return a.amax().float().reshape(1)
    return a.amax(dim=1 if mode == SCALE_ROW else 0).float()


def t_scale(amax: torch.Tensor, fmt: int, margin: int = 0, fallback=1.0) -> torch.Tensor:
    """Vectorised fp32 scale rule; `fallback` may be a scalar or a tensor like amax."""
    amax = amax.float()
    s = torch.tensor(FP8_MAX[fmt], dtype=torch.float32) / amax
    if margin:
        s = torch.ldexp(s, torch.tensor(-margin))
    s = torch.where(torch.isinf(s), torch.tensor(FLT_MAX), s)
    ok = torch.isfinite(amax) & (amax > 0)
    fb = fallback if isinstance(fallback, torch.Tensor) else torch.tensor(float(fallback))
    return torch.where(ok, s, fb.float())


def t_cast(x: torch.Tensor, scale, fmt: int, mode: int = SCALE_TENSOR) -> torch.Tensor:
    s = torch.as_tensor(scale, dtype=torch.float32)
    if mode == SCALE_ROW:
        s = s.reshape(-1, 1)
    elif mode == SCALE_COL:
        s = s.reshape(1, -1)
    m = FP8_MAX[fmt]
    return (x.float() * s).clamp(-m, m).to(TORCH_FP8[fmt]).view(torch.uint8)


def t_cast_transpose(x, scale, fmt, mode=SCALE_TENSOR):
    q = t_cast(x, scale, fmt, mode)
    return q, q.t().contiguous()


def t_decode(codes: torch.Tensor, fmt: int) -> torch.Tensor:
    return codes.view(TORCH_FP8[fmt]).float()


def t_gemm_nt(a, b, fmt_a, fmt_b, sa_inv, sb_inv, want_f32: bool = False):
    """Emulated FP8 matmul: upcast, fp32 matmul, scale product, bf16."""
    acc = t_decode(a, fmt_a) @ t_decode(b, fmt_b).t()
    sa = torch.as_tensor(sa_inv, dtype=torch.float32).reshape(-1, 1)
    sb = torch.as_tensor(sb_inv, dtype=torch.float32).reshape(1, -1)
    out = acc * (sa * sb)
    return (out.bfloat16(), out) if want_f32 else out.bfloat16()


def t_accumulate(c_old: torch.Tensor, product_f32: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """C = C + product as the GEMMs' accumulate flag defines it (include/odl_fp8.h, odl_fp8_gemm_nt): the UNROUNDED fp32
    product (what c_gemm_nt / t_gemm_nt return with want_f32), plus the fp32 bias, plus the old C widened to fp32, each
    addition rounded to fp32, then ONE rounding to C's type.  The backend's GEMM has the same flag (the reference
    accumulates microbatch gradients, optimus_dl/recipe/train/mixins/execution/iteration_mixin.py:332)."""
    v = product_f32.float()
    if bias is not None:
        v = v + bias.float().reshape(1, -1)
    return (v + c_old.float()).to(c_old.dtype)


def t_gemm_nt_sum(pairs, fmt_a, fmt_b, want_f32: bool = False):
    """sum_s (a_s . b_s^T) * (sa_s * sb_s) over pairs (a_s, b_s, sa_inv_s, sb_inv_s): the data gradient of Linears that are
    fed one tensor (the reference's wq / wk / wv, optimus_dl/modules/model/blocks/attention.py:317-319, and w1 / w2,
    optimus_dl/modules/model/blocks/mlp.py:76-78, whose per-Linear data gradients autograd adds up).  Every scaled
    product in fp32 (t_gemm_nt), added in pair order in fp32, ONE rounding to bf16."""
    total = None
    for a, b, sa_inv, sb_inv in pairs:
        part = t_gemm_nt(a, b, fmt_a, fmt_b, sa_inv, sb_inv, want_f32=True)[1]
        total = part if total is None else total + part
    return (total.bfloat16(), total) if want_f32 else total.bfloat16()


# -------------------------------------------------- the Linear, end to end (torch)
def linear_fwd_bwd(x, w, dy, fmt_fwd=E4M3, fmt_bwd=E5M2, rowwise=False, scales=None):
    """One FP8 Linear forward + backward on CPU with dynamic scaling.

    x[M,K], w[N,K], dy[M,N] bf16.  Returns dict with y, dx, dw (bf16) and the
    quantised operands / scales used.  `scales` = (sx, sw, sg) overrides the
    dynamic per-tensor scales (delayed scaling feeds stale ones).
    """
    out = {}
    if not rowwise:
        if scales is None:
            sx = t_scale(t_amax(x), fmt_fwd)
            sw = t_scale(t_amax(w), fmt_fwd)
            sg = t_scale(t_amax(dy), fmt_bwd)
        else:
            sx, sw, sg = (torch.as_tensor(s, dtype=torch.float32).reshape(1) for s in scales)
        xq, xq_t = t_cast_transpose(x, sx, fmt_fwd)
        wq, wq_t = t_cast_transpose(w, sw, fmt_fwd)
        gq, gq_t = t_cast_transpose(dy, sg, fmt_bwd)
        out["y"] = t_gemm_nt(xq, wq, fmt_fwd, fmt_fwd, 1.0 / sx, 1.0 / sw)
        out["dx"] = t_gemm_nt(gq, wq_t, fmt_bwd, fmt_fwd, 1.0 / sg, 1.0 / sw)
        out["dw"] = t_gemm_nt(gq_t, xq_t, fmt_bwd, fmt_fwd, 1.0 / sg, 1.0 / sx)
        out.update(xq=xq, wq=wq, gq=gq, xq_t=xq_t, wq_t=wq_t, gq_t=gq_t, sx=sx, sw=sw, sg=sg)
        return out
    # rowwise: every operand is scaled along its non-contracted axis, from the bf16 source
    sx_r = t_scale(t_amax(x, SCALE_ROW), fmt_fwd)
    sw_r = t_scale(t_amax(w, SCALE_ROW), fmt_fwd)
    xq = t_cast(x, sx_r, fmt_fwd, SCALE_ROW)
    wq = t_cast(w, sw_r, fmt_fwd, SCALE_ROW)
    out["y"] = t_gemm_nt(xq, wq, fmt_fwd, fmt_fwd, 1.0 / sx_r, 1.0 / sw_r)
    sg_r = t_scale(t_amax(dy, SCALE_ROW), fmt_bwd)
    sw_c = t_scale(t_amax(w, SCALE_COL), fmt_fwd)
    gq = t_cast(dy, sg_r, fmt_bwd, SCALE_ROW)
    wq_t = t_cast(w, sw_c, fmt_fwd, SCALE_COL).t().contiguous()
    out["dx"] = t_gemm_nt(gq, wq_t, fmt_bwd, fmt_fwd, 1.0 / sg_r, 1.0 / sw_c)
    sg_c = t_scale(t_amax(dy, SCALE_COL), fmt_bwd)
    sx_c = t_scale(t_amax(x, SCALE_COL), fmt_fwd)
    gq_t = t_cast(dy, sg_c, fmt_bwd, SCALE_COL).t().contiguous()
    xq_t = t_cast(x, sx_c, fmt_fwd, SCALE_COL).t().contiguous()
    out["dw"] = t_gemm_nt(gq_t, xq_t, fmt_bwd, fmt_fwd, 1.0 / sg_c, 1.0 / sx_c)
    out.update(xq=xq, wq=wq, gq=gq, xq_t=xq_t, wq_t=wq_t, gq_t=gq_t,
               sx=sx_r, sw=sw_r, sg=sg_r, sx_c=sx_c, sw_c=sw_c, sg_c=sg_c)
    return out


class DelayedState:
    """Pure-Python delayed-scaling bookkeeping (ring of H amaxes per role)."""

    def __init__(self, fmts, history_len: int, margin: int = 0, algo: str = "max"):
        self.fmts = list(fmts)
        self.H, self.R = history_len, len(self.fmts)
        self.margin, self.algo = margin, algo
        self.history = np.zeros((self.H, self.R), dtype=np.float32)
        self.scale = np.ones(self.R, dtype=np.float32)
        self.scale_inv = np.ones(self.R, dtype=np.float32)

    def record(self, role: int, amax: float):
        self.history[0, role] = max(self.history[0, role], np.float32(amax))

    def update(self):
        for r in range(self.R):
            col = self.history[:, r]
            a = col.max() if self.algo == "max" else col[0]
            if np.isnan(col).any() and self.algo == "max":
                a = np.float32("nan")
            self.history[:, r] = np.roll(col, -1)
            self.history[0, r] = 0.0
            if np.isfinite(a) and a > 0:
                s = np.float32(FP8_MAX[self.fmts[r]]) / np.float32(a)
                s = np.float32(np.ldexp(s, -self.margin))
                if np.isinf(s):
                    s = np.float32(FLT_MAX)
                self.scale[r] = s
            self.scale_inv[r] = np.float32(1.0) / self.scale[r]


# ------------------------------------------------------------------------ MXFP8
MX_BLOCK = 32
MX_EMAX = {E4M3: 8, E5M2: 15}
MX_FLOOR, MX_CEIL = 0, 1       # shared exponent: floor(log2 amax) - emax (OCP MX v1.0) / ceil(log2(amax / fp8_max))


def c_mx_quantise(x: torch.Tensor, fmt: int, rule: int = MX_FLOOR):
    """MXFP8 of a bf16 matrix, blocks of 32 along the last axis -> (codes uint8 [R, C], scale bytes uint8 [R, C/32])."""
    rows, cols = x.shape
    assert cols % MX_BLOCK == 0
    xb = _bf16_bits(x)
    codes, scales = np.empty((rows, cols), dtype=np.uint8), np.empty((rows, cols // MX_BLOCK), dtype=np.uint8)
    lib().oracle_mx_quantise_bf16(_p(xb), rows, cols, fmt, rule, _p(codes), _p(scales))
    return torch.from_numpy(codes), torch.from_numpy(scales)


def t_mx_quantise(x: torch.Tensor, fmt: int, rule: int = MX_FLOOR):
    """The same conversion with torch routines (frexp for floor(log2), exact power-of-two scaling, the CPU float8 cast).
    MX_CEIL: the exponent of the smallest power of two p with amax / p <= fp8_max, found by comparing amax with
    fp8_max * 2^k for the two candidates k (both products are exact)."""
    rows, cols = x.shape
    v = x.float().reshape(rows, cols // MX_BLOCK, MX_BLOCK)
    amax = v.abs().amax(dim=2)
    _, e = torch.frexp(amax)                                   # amax = m * 2^e with 0.5 <= m < 1: floor(log2) = e - 1
    se = e - 1 - MX_EMAX[fmt]
    if rule == MX_CEIL:
        fits = amax.double() <= torch.ldexp(torch.full_like(amax, FP8_MAX[fmt]).double(), se)
        se = torch.where(fits, se, se + 1)
    se = se.clamp(-127, 127)
    bad = ~torch.isfinite(amax)
    se = torch.where((amax == 0) | bad, torch.full_like(se, -127), se)
    scaled = torch.ldexp(v, (-se).unsqueeze(2).expand_as(v).to(torch.int32))
    scaled = torch.where(bad.unsqueeze(2), v, scaled)          # such a block keeps its values (scale byte 0xFF)
    m = FP8_MAX[fmt]
    codes = scaled.clamp(-m, m).to(TORCH_FP8[fmt]).view(torch.uint8).reshape(rows, cols)
    scales = torch.where(bad, torch.full_like(se, 255), se + 127).to(torch.uint8)
    return codes, scales


def t_mx_dequantise(codes: torch.Tensor, scales: torch.Tensor, fmt: int) -> torch.Tensor:
    rows, cols = codes.shape
    v = t_decode(codes, fmt).reshape(rows, cols // MX_BLOCK, MX_BLOCK)
    out = torch.ldexp(v, (scales.to(torch.int32) - 127).unsqueeze(2).expand_as(v))
    out = torch.where((scales == 255).unsqueeze(2), torch.full_like(out, float("nan")), out)
    return out.reshape(rows, cols)


def t_mx_gemm_nt(a, sa, b, sb, fmt_a, fmt_b, bias=None, want_f32: bool = False):
    """Emulated MXFP8 matmul: dequantise both operands (exact in fp32), fp32 matmul, optional bias, bf16."""
    out = t_mx_dequantise(a, sa, fmt_a) @ t_mx_dequantise(b, sb, fmt_b).t()
    if bias is not None:
        out = out + bias.float()
    return (out.bfloat16(), out) if want_f32 else out.bfloat16()


def c_mx_gemm_nt(a, sa, b, sb, fmt_a, fmt_b, bias=None):
    M, K = a.shape
    N = b.shape[0]
    arrs = [np.ascontiguousarray(t.numpy()) for t in (a, sa, b, sb)]
    out_bf16, out_f32 = np.empty((M, N), dtype=np.uint16), np.empty((M, N), dtype=np.float32)
    bias_np = None if bias is None else np.ascontiguousarray(bias.float().numpy())
    lib().oracle_mx_gemm_nt(_p(arrs[0]), _p(arrs[1]), _p(arrs[2]), _p(arrs[3]), M, N, K, fmt_a, fmt_b,
                            _p(bias_np) if bias_np is not None else None, _p(out_bf16), _p(out_f32))
    return torch.from_numpy(out_bf16.view(np.int16)).view(torch.bfloat16), torch.from_numpy(out_f32)


# ------------------------------------------------------------------------------------------------ blockwise recipe
def c_block_quantise(x: torch.Tensor, block_r: int, block_c: int, fmt: int, margin: int = 0):
    """Blockwise quantisation of a bf16 matrix (power-of-two scale per block of block_r x block_c elements) ->
    (codes uint8 [R, C], E8M0 bytes of the inverse scales uint8 [R / block_r, C / block_c])."""
    rows, cols = x.shape
    assert rows % block_r == 0 and cols % block_c == 0
    xb = _bf16_bits(x)
    codes = np.empty((rows, cols), dtype=np.uint8)
    sb = np.empty((rows // block_r, cols // block_c), dtype=np.uint8)
    lib().oracle_block_quantise_bf16(_p(xb), rows, cols, block_r, block_c, fmt, margin, _p(codes), _p(sb))
    return torch.from_numpy(codes), torch.from_numpy(sb)


def t_block_quantise(x: torch.Tensor, block_r: int, block_c: int, fmt: int, margin: int = 0):
    """The same with torch routines: the per-tensor scale rule on every block's amax, frexp for the power of two below
    it, exact power-of-two scaling, the CPU float8 cast."""
    rows, cols = x.shape
    v = x.float().reshape(rows // block_r, block_r, cols // block_c, block_c)
    amax = v.abs().amax(dim=(1, 3))
    s = t_scale(amax, fmt, margin, 1.0)
    _, e = torch.frexp(s)                                       # s = m * 2^e, 0.5 <= m < 1: the power of two below is 2^(e-1)
    e = (e - 1).clamp(min=-126)
    scaled = torch.ldexp(v, e[:, None, :, None].expand_as(v).to(torch.int32))
    m = FP8_MAX[fmt]
    codes = scaled.clamp(-m, m).to(TORCH_FP8[fmt]).view(torch.uint8).reshape(rows, cols)
    return codes, (127 - e).to(torch.uint8)


def block_scales_as_mx(scale_bytes: torch.Tensor, block_r: int, block_c: int) -> torch.Tensor:
    """Block scale bytes [R / block_r, C / block_c] spread out to one byte per row and 32 columns ([R, C / 32]): the
    layout of the MXFP8 functions above, which then dequantise and multiply blockwise tensors as well."""
    return scale_bytes.repeat_interleave(block_r, dim=0).repeat_interleave(block_c // MX_BLOCK, dim=1).contiguous()
