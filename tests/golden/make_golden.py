#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (run from the repository root:
``python tests/golden/make_golden.py``).

Nothing here uses the oracle or the GPU kernels: the vectors come from the OCP FP8 format
definitions, from torch's CPU conversion ``Tensor.to(torch.float8_*)`` and from numpy float32
arithmetic, so that they pin the oracle (tests/test_golden_vectors.py) and, through it and
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


def main():
    docs = {"fp8_decode_tables.json": decode_tables(), "fp8_encode_edges.json": encode_vectors(),
            "scale_from_amax.json": scale_vectors(), "delayed_scaling_sequence.json": delayed_sequence()}
    for name, doc in docs.items():
        with open(os.path.join(HERE, name), "w") as fh:
            json.dump(doc, fh, separators=(",", ":"))
            fh.write("\n")
        print(name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
