#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (run from the repository root:
``python tests/golden/make_golden.py``).

Nothing here uses the oracle or the GPU kernels: the vectors come from the OCP FP8 format
definitions, from torch's CPU routines (``Tensor.to(torch.float8_*)``, ``F.silu``, bf16 multiply and
autograd), from float64 closed forms and from numpy float32 arithmetic, so that they pin the oracle (tests/test_golden_vectors.py) and, through it and
directly, the kernels.  The files are small JSON documents; floats are stored as the hex of
their IEEE bit patterns so that nothing depends on decimal printing.
"""
import json
import math
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
FMT = {"e4m3": (torch.float8_e4m3fn, 448.0, 4, 3, 7, True), "e5m2": (torch.float8_e5m2, 57344.0, 5, 2, 15, False)}


def f32_hex(a):
    return [f"{int(v):08x}" for v in np.asarray(a, dtype=np.float32).view(np.uint32).ravel()]


def definition_table(ebits, mbits, bias, fn):
    """decode value of codes 0..255 straight from the bit layout"""
    vals = []
    for c in range(128):
        e, m = c >> mbits, c & ((1 << mbits) - 1)
        if fn and c == 0x7F:
            v = math.nan
        elif not fn and e == (1 << ebits) - 1:
            v = math.inf if m == 0 else math.nan
        elif e == 0:
            v = m / (1 << mbits) * 2.0 ** (1 - bias)
        else:
            v = (1 + m / (1 << mbits)) * 2.0 ** (e - bias)
        vals.append(v)
    return np.array(vals + [-v for v in vals], dtype=np.float32)


def decode_tables():
    out = {}
    for name, (dt, fmax, eb, mb, bias, fn) in FMT.items():
        table = definition_table(eb, mb, bias, fn)
        lib = torch.arange(256, dtype=torch.uint8).view(dt).float().numpy()
        same = (table.view(np.uint32) == lib.view(np.uint32)) | (np.isnan(table) & np.isnan(lib))
        assert same.all(), f"{name}: torch decodes differently from the format definition"
        out[name] = {"max": fmax, "decode_f32_hex": f32_hex(table)}
    return out


def edge_inputs(name):
    dt, fmax, eb, mb, bias, fn = FMT[name]
    table = definition_table(eb, mb, bias, fn)
    finite = np.sort(np.unique(table[np.isfinite(table) & (table >= 0)]))
    xs = [0.0, -0.0, math.inf, -math.inf, math.nan, fmax, -fmax, np.nextafter(np.float32(fmax), np.float32(np.inf)),
          fmax * 1.03125, fmax * 1.04, fmax * 2, 1e30, -1e30, 1e-30, -1e-30, float(finite[1]) / 2, float(finite[1]) * 0.75,
          float(finite[1]) * 0.5000001, float(finite[1]) * 1.5, float(finite[1]) * 2.5]
    # every midpoint between neighbouring values (the tie cases) and one float32 ulp to either side
    for a, b in zip(finite[:-1], finite[1:]):
        mid = np.float32((np.float64(a) + np.float64(b)) / 2)
        xs += [float(mid), float(np.nextafter(mid, np.float32(0))), float(np.nextafter(mid, np.float32(np.inf)))]
    rng = np.random.default_rng(20240611)
    xs += list((rng.standard_normal(96) * fmax / 3).astype(np.float32))
    xs += list((2.0 ** rng.uniform(-20, 18, 64) * rng.choice([-1, 1], 64)).astype(np.float32))
    return np.array(xs, dtype=np.float32)


def encode_vectors():
    out = {}
    for name, (dt, fmax, *_rest) in FMT.items():
        x = edge_inputs(name)
        t = torch.from_numpy(x.copy())
        plain = t.to(dt).view(torch.uint8).numpy()                               # torch's own rule: no saturation
        sat = t.clamp(-fmax, fmax).to(dt).view(torch.uint8).numpy()             # clamp, then convert: the kernels' rule
        nan = np.isnan(x)
        sat = np.where(nan, np.where(np.signbit(x), 0xFF, 0x7F), sat).astype(np.uint8)   # NaN -> 0x7F | sign in both formats
        out[name] = {"x_f32_hex": f32_hex(x), "code_torch": [int(v) for v in plain], "code_saturating": [int(v) for v in sat]}
    return out


def scale_vectors():
    rng = np.random.default_rng(7)
    amax = np.concatenate([
        np.array([0.0, -1.0, np.inf, np.nan, 1e-45, 3e-39, 1e-38, 448.0, 57344.0, 3.4e38, 1.0, 0.5, 3.0, 1e-3], dtype=np.float32),
        np.abs(rng.standard_normal(40)).astype(np.float32) * 5,
        (2.0 ** rng.uniform(-140, 127, 40)).astype(np.float32),
    ])
    out = {"amax_f32_hex": f32_hex(amax), "cases": []}
    flt_max = np.float32(np.finfo(np.float32).max)
    for name, (_, fmax, *_rest) in FMT.items():
        for margin in (0, 1, 3):
            with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
                s = np.float32(fmax) / amax                                      # IEEE float32 division
                s = np.ldexp(s, -margin).astype(np.float32)
            s = np.where(np.isinf(s), flt_max, s)
            s = np.where((amax > 0) & np.isfinite(amax), s, np.float32(1.0)).astype(np.float32)
            inv = (np.float32(1.0) / s).astype(np.float32)
            out["cases"].append({"fmt": name, "margin": margin, "scale_f32_hex": f32_hex(s), "scale_inv_f32_hex": f32_hex(inv)})
    return out


def delayed_sequence():
    """History 16, 20 steps, one role per format, amax drifting upwards with one step of zeros and one NaN-free spike:
    scale used at step t, and the history after the update of step t, by a plain list-based simulation."""
    H, steps = 16, 20
    rng = np.random.default_rng(11)
    amaxes = (np.linspace(1.0, 1.5, steps) * (3.5 + 0.1 * rng.standard_normal(steps))).astype(np.float32)
    amaxes[6] = 0.0
    amaxes[9] *= 4
    out = {"H": H, "amax_f32_hex": f32_hex(amaxes), "cases": []}
    for name, (_, fmax, *_rest) in FMT.items():
        for algo in ("max", "most_recent"):
            hist = [np.float32(0.0)] * H
            scale = np.float32(1.0)
            used, after = [], []
            for a in amaxes:
                used.append(scale)                       # the cast of this step uses the scale from before
                hist[0] = max(hist[0], a)
                pick = max(hist) if algo == "max" else hist[0]
                hist = hist[1:] + hist[:1]               # roll by -1
                hist[0] = np.float32(0.0)
                if pick > 0 and np.isfinite(pick):
                    s = np.float32(fmax) / np.float32(pick)
                    scale = np.float32(np.finfo(np.float32).max) if np.isinf(s) else np.float32(s)
                after.append(scale)
            out["cases"].append({"fmt": name, "algo": algo, "scale_used_f32_hex": f32_hex(used), "scale_after_f32_hex": f32_hex(after),
                                 "final_history_f32_hex": f32_hex(hist)})
    return out


def bf16_hex(t):
    return [f"{int(v) & 0xffff:04x}" for v in t.contiguous().view(torch.int16).flatten().tolist()]


def swiglu_vectors():
    """silu(gate) * up and its gradients as torch computes them in bf16 on the CPU (F.silu, tensor multiply, autograd).
    Gates: every 37th bf16 pattern above -80 (finite), the exact points 0 / +-1 / saturation, and Gaussian draws."""
    import torch.nn.functional as F

    bits = torch.arange(0, 65536, 37, dtype=torch.int32)
    gates = bits.to(torch.int16).view(torch.bfloat16)
    gates = gates[torch.isfinite(gates.float()) & (gates.float() >= -80.0)]
    gen = torch.Generator().manual_seed(5)
    extra = torch.cat([torch.tensor([0.0, -0.0, 1.0, -1.0, 30.0, -30.0, 79.5, -79.5, 100.0]),
                       torch.randn(600, generator=gen) * 2.0]).bfloat16()
    g = torch.cat([gates, extra])
    u = (torch.randn(g.numel(), generator=gen) * 1.5).bfloat16()
    dh = (torch.randn(g.numel(), generator=gen) * 1e-2).bfloat16()
    ga, ua = g.clone().requires_grad_(True), u.clone().requires_grad_(True)
    h = F.silu(ga) * ua
    h.backward(dh)
    return {"gate_bf16_hex": bf16_hex(g), "up_bf16_hex": bf16_hex(u), "dh_bf16_hex": bf16_hex(dh),
            "silu_bf16_hex": bf16_hex(F.silu(g)), "h_bf16_hex": bf16_hex(h.detach()),
            "d_up_bf16_hex": bf16_hex(ua.grad), "d_gate_bf16_hex": bf16_hex(ga.grad),
            "note": "d_gate is torch's association (grad * sig) * (1 + g (1 - sig)); the library's differs: within one bf16 unit"}


def norm_vectors():
    """RMSNorm and LayerNorm rows with outputs from float64 closed forms, rounded once to bf16 (y) / float32 (statistics)."""
    gen = torch.Generator().manual_seed(9)
    out = {"cases": []}
    for cols, dtype in ((8, "bf16"), (264, "bf16"), (768, "f32")):
        rows = 3
        x = torch.randn((rows, cols), generator=gen) * 2.5 + 0.4
        x = x.bfloat16() if dtype == "bf16" else x
        w = torch.randn(cols, generator=gen) * 0.4 + 1.0
        b = torch.randn(cols, generator=gen) * 0.2
        eps = 1e-5
        x64 = x.double()
        rstd_rms = 1.0 / torch.sqrt((x64 * x64).mean(-1) + eps)
        y_rms = (x64 * rstd_rms[:, None] * w.double()).float().bfloat16()
        mean = x64.mean(-1)
        rstd_ln = 1.0 / torch.sqrt(x64.var(-1, unbiased=False) + eps)
        y_ln = ((x64 - mean[:, None]) * rstd_ln[:, None] * w.double() + b.double()).float().bfloat16()
        out["cases"].append({
            "rows": rows, "cols": cols, "dtype": dtype, "eps": eps,
            "x_hex": bf16_hex(x) if dtype == "bf16" else f32_hex(x.numpy()),
            "weight_f32_hex": f32_hex(w.numpy()), "bias_f32_hex": f32_hex(b.numpy()),
            "rms_rstd_f32_hex": f32_hex(rstd_rms.float().numpy()), "rms_y_bf16_hex": bf16_hex(y_rms),
            "ln_mean_f32_hex": f32_hex(mean.float().numpy()), "ln_rstd_f32_hex": f32_hex(rstd_ln.float().numpy()),
            "ln_y_bf16_hex": bf16_hex(y_ln)})
    return out


def main():
    docs = {"fp8_decode_tables.json": decode_tables(), "fp8_encode_edges.json": encode_vectors(),
            "scale_from_amax.json": scale_vectors(), "delayed_scaling_sequence.json": delayed_sequence(),
            "swiglu_bf16.json": swiglu_vectors(), "norm_rows.json": norm_vectors()}
    for name, doc in docs.items():
        with open(os.path.join(HERE, name), "w") as fh:
            json.dump(doc, fh, separators=(",", ":"))
            fh.write("\n")
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
