"""Pins of the MXFP8 oracle (oracle_mx_quantise_bf16, oracle_mx_gemm_nt): the OCP MX v1.0 conversion formula, restated
independently, hand-worked blocks, and the invariances the formula implies."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import assert_bytes_equal, seeded_bf16


def bf16(vals):
    return torch.tensor(vals, dtype=torch.float32).bfloat16()


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_hand_worked_blocks(fmt):
    emax = O.MX_EMAX[fmt]
    row = torch.zeros(1, 128, dtype=torch.bfloat16)
    row[0, :32] = bf16([1.0] + [0.5] * 31)                        # amax 1 = 2^0: shared exponent -emax
    row[0, 32:64] = bf16([-3.0, 1.5] + [0.0] * 30)                 # amax 3: floor(log2) = 1
    row[0, 64:96] = 0                                              # zeros: byte 0
    row[0, 96:128] = bf16([2.0 ** -20] * 32)
    codes, scales = O.c_mx_quantise(row, fmt)
    assert scales.tolist() == [[127 - emax, 128 - emax, 0, 107 - emax]]
    dec = O.t_decode(codes, fmt)
    # the largest element of a block lands in the top binade [2^emax, 2^(emax+1)) (or saturates at the format's maximum)
    assert dec[0, 0].item() == 2.0 ** emax and dec[0, 1].item() == 2.0 ** (emax - 1)
    assert dec[0, 32].item() == -min(3.0 * 2.0 ** (emax - 1), O.FP8_MAX[fmt]) and dec[0, 33].item() == 1.5 * 2.0 ** (emax - 1)
    assert not dec[0, 64:96].any() and (dec[0, 96:128] == 2.0 ** emax).all()
    # and the dequantised values are the inputs again (all of them representable here)
    assert torch.equal(O.t_mx_dequantise(codes, scales, fmt), row.float())
    # the one place where the conversion saturates: a block maximum above the format's largest value 1.75 x 2^emax after scaling
    top = torch.zeros(1, 32, dtype=torch.bfloat16)
    top[0, 0], top[0, 1] = 1.9375, 1.0
    codes, scales = O.c_mx_quantise(top, fmt)
    back = O.t_mx_dequantise(codes, scales, fmt)
    assert scales.tolist() == [[127 - emax]] and back[0, 0].item() == 1.75 and back[0, 1].item() == 1.0


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_c_and_torch_restatements_agree_and_follow_the_formula(fmt):
    x = seeded_bf16((64, 256), 1.0, 5)
    x[3, 40] = 3.0e38
    x[5, :32] = 0
    x[7, 100] = float("inf")
    x[9, 7] = float("nan")
    x[11, 64:96] = (x[11, 64:96].float() * 2.0 ** -120).bfloat16()  # tiny block: the shared exponent reaches its lower clamp region
    x[13, 96:128] = (x[13, 96:128].float() * 2.0 ** -130).bfloat16()  # bf16 subnormals
    cc, cs = O.c_mx_quantise(x, fmt)
    tc, ts = O.t_mx_quantise(x, fmt)
    assert_bytes_equal(cs, ts, "scale bytes, C vs torch")
    assert_bytes_equal(cc, tc, "codes, C vs torch")
    # the formula, block by block, in float64
    v = x.double().reshape(64, 8, 32)
    amax = v.abs().amax(dim=2)
    ok = torch.isfinite(amax) & (amax > 0)
    want = torch.where(ok, (torch.floor(torch.log2(torch.where(ok, amax, torch.ones_like(amax)))) - O.MX_EMAX[fmt]).clamp(-127, 127) + 127,
                       torch.where(amax == 0, torch.zeros_like(amax), torch.full_like(amax, 255)))
    assert torch.equal(cs.double(), want)
    assert cs[7, 3] == 255 and cs[9, 0] == 255 and cs[5, 0] == 0
    assert cc[9, 7] & 0x7f == 0x7f                                 # the NaN stays a NaN code


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_invariances_of_the_block_scale(fmt):
    x = seeded_bf16((32, 128), 3.0, 6)
    codes, scales = O.c_mx_quantise(x, fmt)
    # a power of two applied to one block moves only that block's scale byte, no code
    y = x.clone()
    y[:, 32:64] = (y[:, 32:64].float() * 2.0 ** 5).bfloat16()
    c2, s2 = O.c_mx_quantise(y, fmt)
    assert torch.equal(c2, codes) and torch.equal(s2[:, 1].int(), scales[:, 1].int() + 5)
    assert torch.equal(s2[:, [0, 2, 3]], scales[:, [0, 2, 3]])
    # sign symmetry, and blocks do not see each other
    c3, s3 = O.c_mx_quantise((-x.float()).bfloat16(), fmt)
    assert torch.equal(c3 ^ 0x80, codes) and torch.equal(s3, scales)
    c4, s4 = O.c_mx_quantise(x[:, 64:96].contiguous(), fmt)
    assert torch.equal(c4, codes[:, 64:96]) and torch.equal(s4[:, 0], scales[:, 2])
    # relative error of the round trip: half a unit of the element format at the block's top binade
    back = O.t_mx_dequantise(codes, scales, fmt)
    amax = x.float().reshape(32, 4, 32).abs().amax(dim=2, keepdim=True).expand(32, 4, 32).reshape(32, 128)
    mbits = 3 if fmt == O.E4M3 else 2
    assert ((back - x.float()).abs() <= amax * 2.0 ** -mbits).all()


def test_mx_gemm_c_vs_torch_vs_float64():
    fa, fb = O.E5M2, O.E4M3
    a, b = seeded_bf16((24, 256), 1e-3, 7), seeded_bf16((40, 256), 0.02, 8)
    a[:, 64:96] = (a[:, 64:96].float() * 300).bfloat16()           # blocks of very different magnitude
    (ac, asc), (bc, bsc) = O.c_mx_quantise(a, fa), O.c_mx_quantise(b, fb)
    bias = torch.linspace(-1, 1, 40) * 1e-3
    c_bf16, c_f32 = O.c_mx_gemm_nt(ac, asc, bc, bsc, fa, fb, bias)
    t_bf16, t_f32 = O.t_mx_gemm_nt(ac, asc, bc, bsc, fa, fb, bias, want_f32=True)
    ref = O.t_mx_dequantise(ac, asc, fa).double() @ O.t_mx_dequantise(bc, bsc, fb).double().t() + bias.double()
    for got in (c_f32, t_f32):
        assert ((got.double() - ref).abs().max() / ref.abs().max()).item() < 1e-6
    assert ((c_bf16.float() - t_bf16.float()).abs().max() / ref.abs().max()).item() < 1e-2
    # exact case: codes that are powers of two, scales that differ per block: every term is representable, any order gives the same sum
    one_hot = torch.zeros(4, 64, dtype=torch.bfloat16)
    one_hot[0, 3], one_hot[1, 40], one_hot[2, 0], one_hot[3, 63] = 2.0, 0.25, -8.0, 1.0
    w = torch.zeros(2, 64, dtype=torch.bfloat16)
    w[0, :] = 1.0
    w[1, 32:] = -0.5
    (oc, osc), (wc, wsc) = O.c_mx_quantise(one_hot, O.E4M3), O.c_mx_quantise(w, O.E4M3)
    _, exact = O.c_mx_gemm_nt(oc, osc, wc, wsc, O.E4M3, O.E4M3)
    assert exact.tolist() == [[2.0, 0.0], [0.25, -0.125], [-8.0, 0.0], [1.0, -0.5]]
    # a NaN scale byte poisons the row
    asc2 = asc.clone()
    asc2[2, 1] = 255
    _, poisoned = O.c_mx_gemm_nt(ac, asc2, bc, bsc, fa, fb)
    assert torch.isnan(poisoned[2]).all() and not torch.isnan(poisoned[3]).any()


# ------------------------------------------------------------------ the round-up rule of the shared exponent (MX_CEIL)
@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_round_up_rule_hand_worked(fmt):
    """amax = m * 2^e: the shared exponent is e - emax for m <= 1.75 (as under the floor rule) and one more for m > 1.75,
    where the floor rule saturates.  fp8_max = 1.75 * 2^emax, so 1.75 itself still fits exactly."""
    emax = O.MX_EMAX[fmt]
    row = torch.zeros(1, 128, dtype=torch.bfloat16)
    row[0, :32] = bf16([1.75] + [1.0] * 31)                       # exactly fp8_max after scaling by 2^emax: no bump
    row[0, 32:64] = bf16([1.7578125, 1.0] + [0.0] * 30)           # the next bf16 above 1.75: one more
    row[0, 64:96] = bf16([-1.9375, 0.5] + [0.0] * 30)
    row[0, 96:128] = bf16([3.0] + [0.0] * 31)                     # 1.5 * 2^1
    codes, scales = O.c_mx_quantise(row, fmt, O.MX_CEIL)
    assert scales.tolist() == [[127 - emax, 128 - emax, 128 - emax, 128 - emax]]
    floor_scales = O.c_mx_quantise(row, fmt, O.MX_FLOOR)[1]
    assert floor_scales.tolist() == [[127 - emax, 127 - emax, 127 - emax, 128 - emax]]
    back = O.t_mx_dequantise(codes, scales, fmt)
    # nothing saturated: 1.9375 is rounded like any other value (to 2.0, the nearest code one binade up), not clamped
    assert back[0, 0].item() == 1.75 and back[0, 64].item() == -2.0 and back[0, 65].item() == 0.5
    assert O.t_mx_dequantise(*O.c_mx_quantise(row, fmt, O.MX_FLOOR), fmt)[0, 64].item() == -1.75         # the floor rule did


@pytest.mark.parametrize("fmt", [O.E4M3, O.E5M2])
def test_round_up_rule_c_vs_torch_vs_float64(fmt):
    """C and torch restatements agree byte for byte; the scale is 2^ceil(log2(amax / fp8_max)) evaluated in float64
    (the quotient of an 8-bit-mantissa amax and 1.75 * 2^emax, and log2 of a value that is a power of two exactly when
    the quotient is, so ceil is safe); no element of a finite block saturates: |element| * 2^-shared <= fp8_max; and
    the two rules differ exactly in the blocks whose amax has a mantissa above 1.75."""
    x = seeded_bf16((96, 512), 1.0, 15)
    x[3, 40] = 3.0e38
    x[5, :32] = 0
    x[7, 100] = float("inf")
    x[9, 7] = float("nan")
    x[11, 64:96] = (x[11, 64:96].float() * 2.0 ** -120).bfloat16()
    x[13, 96:128] = (x[13, 96:128].float() * 2.0 ** -130).bfloat16()
    x[15, 128] = 1.75 * 2.0 ** 5                                   # a block maximum exactly on the boundary
    x[15, 129:160] = 0.0
    cc, cs = O.c_mx_quantise(x, fmt, O.MX_CEIL)
    tc, ts = O.t_mx_quantise(x, fmt, O.MX_CEIL)
    assert_bytes_equal(cs, ts, "scale bytes, C vs torch")
    assert_bytes_equal(cc, tc, "codes, C vs torch")
    v = x.double().reshape(96, 16, 32)
    amax = v.abs().amax(dim=2)
    ok = torch.isfinite(amax) & (amax > 0)
    q = torch.where(ok, amax, torch.ones_like(amax)) / O.FP8_MAX[fmt]
    want = torch.where(ok, torch.ceil(torch.log2(q)).clamp(-127, 127) + 127,
                       torch.where(amax == 0, torch.zeros_like(amax), torch.full_like(amax, 255)))
    assert torch.equal(cs.double(), want)
    shared = cs.double() - 127
    fits = (v.abs() <= (O.FP8_MAX[fmt] * torch.exp2(shared)).unsqueeze(2)) | ~ok.unsqueeze(2) | (shared == -127).unsqueeze(2)
    assert bool(fits.all()), "an element would saturate under the round-up rule"
    fs = O.c_mx_quantise(x, fmt, O.MX_FLOOR)[1]
    mant = amax / torch.exp2(torch.floor(torch.log2(torch.where(ok, amax, torch.ones_like(amax)))))
    bumped = ok & (mant > 1.75) & (fs < 254) & (fs > 0)
    assert torch.equal((cs.int() - fs.int())[ok], bumped[ok].int())
    # error of the largest element of a block: at most half a unit of a 3-bit (E4M3) / 2-bit (E5M2) mantissa, never 12.5 %
    back = O.t_mx_dequantise(cc, cs, fmt).double().reshape(96, 16, 32)
    top = v.abs() == amax.unsqueeze(2)
    rel = ((back - v).abs() / amax.unsqueeze(2).clamp_min(1e-300))[top & ok.unsqueeze(2) & (shared > -127).unsqueeze(2)]
    assert rel.max().item() <= (2.0 ** -4 if fmt == O.E4M3 else 2.0 ** -3)
