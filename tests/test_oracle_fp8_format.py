"""Pins the oracle's 8-bit float encode/decode.

Three independent anchors, so that a wrong bias, a wrong tie rule or a wrong
special-value code fails at least one:
  1. the format definition (decode tables written here from the OCP layout),
  2. brute force: the encoded value must be the nearest table entry in float64,
     ties to the even code,
  3. the library routine: torch CPU Tensor.to(float8_*).
"""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O


def definition_table(ebits, mbits, bias, fn):
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
    return np.array(vals + [-v for v in vals], dtype=np.float64)


TABLES = {O.E4M3: definition_table(4, 3, 7, True), O.E5M2: definition_table(5, 2, 15, False)}


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_decode_matches_definition_and_torch(fmt):
    codes = np.arange(256, dtype=np.uint8)
    got = O.c_decode(codes, fmt).astype(np.float64)
    want = TABLES[fmt]
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(got[ok], want[ok])
    assert np.array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
    tt = O.t_decode(torch.from_numpy(codes), fmt).numpy().astype(np.float64)
    assert np.array_equal(tt[ok], want[ok])
    # published extremes
    assert want[0x7E if fmt == O.E4M3 else 0x7B] == O.FP8_MAX[fmt]
    assert want[1] == (2.0 ** -9 if fmt == O.E4M3 else 2.0 ** -16)


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_encode_roundtrips_every_finite_code(fmt):
    codes = np.arange(256, dtype=np.uint8)
    vals = O.c_decode(codes, fmt)
    finite = np.isfinite(vals)
    back = O.c_encode(vals[finite], fmt)
    assert np.array_equal(back, codes[finite])


def brute_force_encode(x64, fmt):
    """Nearest finite table value, ties to even code; beyond the overflow
    threshold the non-saturating special (NaN code for e4m3fn, Inf for e5m2)."""
    table = TABLES[fmt][:128]
    top = 0x7E if fmt == O.E4M3 else 0x7B
    mags = table[: top + 1]
    step_top = mags[top] - mags[top - 1]
    out = np.empty(x64.shape, dtype=np.uint8)
    ax = np.abs(x64)
    d = np.abs(ax[:, None] - mags[None, :])
    best = d.min(axis=1)
    for i in range(x64.size):
        cand = np.nonzero(d[i] == best[i])[0]
        c = int(cand[0]) if cand.size == 1 else int([k for k in cand if k % 2 == 0][0])
        # values at or past the midpoint to the (absent) next binade value overflow
        if ax[i] > mags[top] + step_top / 2 or (ax[i] == mags[top] + step_top / 2 and top % 2 == 1):
            c = top + 1
        out[i] = c | (0x80 if np.signbit(x64[i]) else 0)
    return out


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_encode_is_nearest_even_by_brute_force(fmt):
    rng = np.random.default_rng(0)
    top = O.FP8_MAX[fmt]
    xs = [rng.normal(0, 1, 4000), rng.uniform(-top * 1.2, top * 1.2, 4000),
          rng.uniform(-1, 1, 2000) * (2.0 ** -8 if fmt == O.E4M3 else 2.0 ** -15)]
    # every midpoint between neighbouring codes, and its fp32 neighbours
    t = TABLES[fmt][: (0x7F if fmt == O.E4M3 else 0x7C)]
    mid = ((t[:-1] + t[1:]) / 2).astype(np.float32)
    xs += [mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)), -mid]
    x = np.concatenate(xs).astype(np.float32)
    x = x[np.isfinite(x)]
    got = O.c_encode(x, fmt)
    want = brute_force_encode(x.astype(np.float64), fmt)
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, (x[bad[:5]], got[bad[:5]], want[bad[:5]])


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_encode_matches_torch_cpu_cast(fmt):
    # all 65536 bf16 patterns as the high half, with several low halves, plus a
    # stride over the whole fp32 space
    hi = np.arange(65536, dtype=np.uint32) << 16
    parts = [hi, hi | 0x8000, hi | 0x7FFF, hi | 0x8001, hi | 0x1234]
    parts.append(np.arange(0, 2 ** 32, 4099, dtype=np.uint64).astype(np.uint32))
    bits = np.concatenate(parts)
    x = bits.view(np.float32)
    got = O.c_encode(x, fmt)
    want = torch.from_numpy(x.copy()).to(O.TORCH_FP8[fmt]).view(torch.uint8).numpy()
    bad = np.nonzero(got != want)[0]
    assert bad.size == 0, [(hex(bits[i]), got[i], want[i]) for i in bad[:8]]


def test_special_values_documented_for_torch_cpu():
    f = np.float32
    e4 = lambda v: int(O.c_encode(np.array([v], dtype=f), O.E4M3)[0])
    e5 = lambda v: int(O.c_encode(np.array([v], dtype=f), O.E5M2)[0])
    assert [e4(v) for v in (17, 19, 21, 23)] == [int(O.c_encode(np.array([w], dtype=f), O.E4M3)[0]) for w in (16, 20, 20, 24)]
    assert e4(448) == 0x7E and e4(464) == 0x7E and e4(465) == 0x7F and e4(-500) == 0xFF
    assert e4(2.0 ** -9) == 0x01 and e4(2.0 ** -10) == 0x00 and e4(1.5 * 2.0 ** -10) == 0x01
    assert e4(0.0) == 0x00 and e4(-0.0) == 0x80 and e4(np.inf) == 0x7F and e4(np.nan) & 0x7F == 0x7F
    assert e5(57344) == 0x7B and e5(61439) == 0x7B and e5(61440) == 0x7C and e5(1e6) == 0x7C
    assert e5(-np.inf) == 0xFC and e5(2.0 ** -16) == 0x01 and e5(2.0 ** -17) == 0x00
    assert e5(1.5 * 2.0 ** -17) == 0x01 and e5(2.0 ** -14) == 0x04 and e5(1.25 * 2.0 ** -15) == 0x02


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_encode_monotone_and_sign_symmetric(fmt):
    x = np.sort(np.random.default_rng(1).uniform(-O.FP8_MAX[fmt], O.FP8_MAX[fmt], 20000).astype(np.float32))
    v = O.c_decode(O.c_encode(x, fmt), fmt)
    assert np.all(np.diff(v) >= 0)
    assert np.array_equal(O.c_encode(-x, fmt), O.c_encode(x, fmt) ^ 0x80)
