"""The oracle against the committed golden vectors (tests/golden/*.json).

The vectors were produced by tests/golden/make_golden.py from the format definitions, torch's CPU
float8 conversion and numpy float32 arithmetic, none of which is the oracle.  The GPU kernels meet
the same files in tests/test_gpu_quant.py.
"""
import json
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FMT = {"e4m3": O.E4M3, "e5m2": O.E5M2}


def load(name):
    with open(os.path.join(GOLDEN, name)) as fh:
        return json.load(fh)


def f32(hexes):
    return np.array([int(h, 16) for h in hexes], dtype=np.uint32).view(np.float32)


def same_bits(a, b):
    a, b = np.asarray(a, dtype=np.float32), np.asarray(b, dtype=np.float32)
    return ((a.view(np.uint32) == b.view(np.uint32)) | (np.isnan(a) & np.isnan(b))).all()


@pytest.mark.parametrize("name", ["e4m3", "e5m2"])
def test_decode_tables(name):
    doc = load("fp8_decode_tables.json")[name]
    table = f32(doc["decode_f32_hex"])
    assert len(table) == 256 and doc["max"] == O.FP8_MAX[FMT[name]]
    assert same_bits(O.c_decode(np.arange(256, dtype=np.uint8), FMT[name]), table)
    assert same_bits(O.t_decode(torch.arange(256, dtype=torch.uint8), FMT[name]).numpy(), table)


@pytest.mark.parametrize("name", ["e4m3", "e5m2"])
def test_encode_edge_vectors(name):
    doc = load("fp8_encode_edges.json")[name]
    x = f32(doc["x_f32_hex"])
    plain, sat = np.array(doc["code_torch"], dtype=np.uint8), np.array(doc["code_saturating"], dtype=np.uint8)
    assert len(x) > 300
    table = f32(load("fp8_decode_tables.json")[name]["decode_f32_hex"])
    finite_out = ~np.isnan(table[plain])
    got = O.c_encode(x, FMT[name])                       # the plain-C encoder follows torch: no saturation
    assert np.array_equal(got[finite_out], plain[finite_out])
    assert np.isnan(table[got[~finite_out]]).all()       # NaN results: any NaN code
    # clamp-then-convert, as the cast kernels do it (torch twin of the oracle; NaN inputs keep a NaN code)
    t = O.t_cast(torch.from_numpy(x.copy()).reshape(1, -1), 1.0, FMT[name]).numpy().ravel()
    not_nan = ~np.isnan(x)
    assert np.array_equal(t[not_nan], sat[not_nan])
    assert np.isnan(table[t[~not_nan]]).all()
    # the C cast takes bf16 input: the vectors that are bf16 values must agree there too
    xb = torch.from_numpy(x.copy()).bfloat16()
    exact = (xb.float().numpy().view(np.uint32) == x.view(np.uint32)) & not_nan
    c = O.c_cast(xb.reshape(1, -1), 1.0, FMT[name]).numpy().ravel()
    assert exact.sum() > 100 and np.array_equal(c[exact], sat[exact])


def test_scale_vectors():
    doc = load("scale_from_amax.json")
    amax = f32(doc["amax_f32_hex"])
    for case in doc["cases"]:
        fmt, margin = FMT[case["fmt"]], case["margin"]
        want, want_inv = f32(case["scale_f32_hex"]), f32(case["scale_inv_f32_hex"])
        got = np.array([O.c_scale(a, fmt, margin, 1.0) for a in amax], dtype=np.float32)
        assert same_bits(got, want), (case["fmt"], margin)
        assert same_bits(np.array([O.c_scale_inv(s) for s in got], dtype=np.float32), want_inv)
        assert same_bits(O.t_scale(torch.from_numpy(amax.copy()), fmt, margin).numpy(), want)


def test_delayed_scaling_sequence():
    doc = load("delayed_scaling_sequence.json")
    H, amaxes = doc["H"], f32(doc["amax_f32_hex"])
    for case in doc["cases"]:
        fmt, algo = FMT[case["fmt"]], case["algo"]
        used, after = f32(case["scale_used_f32_hex"]), f32(case["scale_after_f32_hex"])
        py = O.DelayedState([fmt], H, algo=algo)
        hist = np.zeros((H, 1), dtype=np.float32)
        scale, scale_inv = np.ones(1, dtype=np.float32), np.ones(1, dtype=np.float32)
        for t, a in enumerate(amaxes):
            assert same_bits(py.scale, used[t:t + 1]) and same_bits(scale, used[t:t + 1]), (case, t)
            py.record(0, float(a))
            py.update()
            hist[0, 0] = max(hist[0, 0], a)
            O.c_delayed_update(hist, scale, scale_inv, [fmt], 0, algo)
            assert same_bits(py.scale, after[t:t + 1]) and same_bits(scale, after[t:t + 1]), (case, t)
        assert same_bits(hist[:, 0], f32(case["final_history_f32_hex"]))
        assert same_bits(py.history[:, 0], f32(case["final_history_f32_hex"]))


# ----------------------------------------------------------------- producers: SwiGLU, RMSNorm, LayerNorm
def bf16(hexes, shape=None):
    a = np.array([int(h, 16) for h in hexes], dtype=np.uint16)
    t = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
    return t if shape is None else t.reshape(shape)


def bf16_units_apart(a: torch.Tensor, b: torch.Tensor) -> np.ndarray:
    ai = a.contiguous().view(torch.int16).numpy().astype(np.int32)
    bi = b.contiguous().view(torch.int16).numpy().astype(np.int32)
    return np.abs(ai - bi)


def test_swiglu_vectors_from_torch_bf16():
    doc = load("swiglu_bf16.json")
    g, u, dh = bf16(doc["gate_bf16_hex"]), bf16(doc["up_bf16_hex"]), bf16(doc["dh_bf16_hex"])
    assert g.numel() > 1500
    ones = torch.ones_like(g)
    assert torch.equal(O.c_swiglu_fwd(g, ones).view(torch.int16), bf16(doc["silu_bf16_hex"]).view(torch.int16))
    assert torch.equal(O.c_swiglu_fwd(g, u).view(torch.int16), bf16(doc["h_bf16_hex"]).view(torch.int16))
    dg, du = O.c_swiglu_bwd(dh, g, u)
    assert torch.equal(du.view(torch.int16), bf16(doc["d_up_bf16_hex"]).view(torch.int16))
    d = bf16_units_apart(dg, bf16(doc["d_gate_bf16_hex"]))
    assert d.max() <= 1 and (d > 0).mean() < 0.02                  # torch associates the product differently


def norm_case_tensors(case):
    shape = (case["rows"], case["cols"])
    x = bf16(case["x_hex"], shape) if case["dtype"] == "bf16" else torch.from_numpy(f32(case["x_hex"]).copy()).reshape(shape)
    w = torch.from_numpy(f32(case["weight_f32_hex"]).copy())
    b = torch.from_numpy(f32(case["bias_f32_hex"]).copy())
    return x, w, b


def test_norm_vectors_from_float64_closed_forms():
    for case in load("norm_rows.json")["cases"]:
        x, w, b = norm_case_tensors(case)
        shape = tuple(x.shape)
        y, rstd = O.c_rmsnorm(x, w, case["eps"])
        assert np.allclose(rstd.numpy(), f32(case["rms_rstd_f32_hex"]), rtol=1e-6, atol=0)
        d = bf16_units_apart(y, bf16(case["rms_y_bf16_hex"], shape))
        assert d.max() <= 1 and (d > 0).mean() < 0.01
        y, mean, rstd = O.c_layernorm(x, w, b, case["eps"])
        assert np.allclose(mean.numpy(), f32(case["ln_mean_f32_hex"]), rtol=1e-5, atol=1e-6)
        assert np.allclose(rstd.numpy(), f32(case["ln_rstd_f32_hex"]), rtol=1e-6, atol=0)
        d = bf16_units_apart(y, bf16(case["ln_y_bf16_hex"], shape))
        assert d.max() <= 1 and (d > 0).mean() < 0.01
