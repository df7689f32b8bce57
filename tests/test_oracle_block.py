"""Pins of the blockwise oracle (oracle_block_quantise_bf16): "the per-tensor rule on every block, scale rounded down to
a power of two", restated independently with torch routines and with Python's math on single blocks, hand-worked
blocks, and the invariances the rule implies.  A wrong block shape, a scale rounded up instead of down, a byte off by
one or a transposed block index fails one of them."""
import math

import numpy as np
import pytest
import torch

from oracle import oracle as O
from tests.helpers import assert_bytes_equal, seeded_bf16

E4M3, E5M2 = O.E4M3, O.E5M2


def _mixed(shape, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    x = x * torch.exp2(torch.randint(-12, 12, (shape[0], 1), generator=g).float())
    x = x * torch.exp2(torch.randint(-5, 5, (1, shape[1]), generator=g).float())
    x[torch.rand(shape, generator=g) < 0.05] = 0.0
    return x.bfloat16()


@pytest.mark.parametrize("blocks", [(1, 128), (128, 1), (128, 128), (2, 4)])
@pytest.mark.parametrize("fmt", [E4M3, E5M2])
@pytest.mark.parametrize("margin", [0, 2])
def test_c_and_torch_restatements_agree(blocks, fmt, margin):
    br, bc = blocks
    x = _mixed((256, 384), seed=br * 7 + bc + fmt + margin)
    cc, cs = O.c_block_quantise(x, br, bc, fmt, margin)
    tc, ts = O.t_block_quantise(x, br, bc, fmt, margin)
    assert_bytes_equal(cs, ts, f"scale bytes {blocks}")
    assert_bytes_equal(cc, tc, f"codes {blocks}")


def test_every_block_is_the_per_tensor_cast_with_the_power_of_two_below_its_scale():
    x = _mixed((8, 512), seed=3)
    codes, sb = O.c_block_quantise(x, 1, 128, E4M3, 0)
    for r in range(8):
        for b in range(4):
            blk = x[r:r + 1, 128 * b:128 * (b + 1)]
            s = O.c_scale(float(blk.abs().max()), E4M3, 0, 1.0)            # the per-tensor rule on this block
            m, e = math.frexp(s)
            p = math.ldexp(1.0, e - 1)                                     # largest power of two <= s
            assert p <= s < 2 * p
            assert_bytes_equal(codes[r:r + 1, 128 * b:128 * (b + 1)], O.c_cast(blk, p, E4M3), f"block {r},{b}")
            assert int(sb[r, b]) == 127 - (e - 1)


def test_hand_worked_blocks():
    x = torch.zeros((1, 256), dtype=torch.bfloat16)
    x[0, 5] = 3.0                    # 448 / 3 = 149.3 -> scale 128 = 2^7 -> byte 120; 3 * 128 = 384
    x[0, 6] = -0.75                  # -96
    x[0, 128 + 1] = 448.0            # scale exactly 1 -> byte 127
    x[0, 128 + 2] = 0.0078125        # 2^-7: below half of E4M3's smallest subnormal step?  2^-9 is the smallest: 2^-7 is kept
    codes, sb = O.c_block_quantise(x, 1, 128, E4M3, 0)
    assert sb.tolist() == [[120, 127]]
    dec = O.t_decode(codes, E4M3)
    assert float(dec[0, 5]) == 384.0 and float(dec[0, 6]) == -96.0 and float(dec[0, 129]) == 448.0 and float(dec[0, 130]) == 2.0 ** -7
    # E5M2: 57344 / 3 = 19114.7 -> 2^14 -> byte 113
    codes, sb = O.c_block_quantise(x[:, :128], 1, 128, E5M2, 0)
    assert sb.tolist() == [[113]] and float(O.t_decode(codes, E5M2)[0, 5]) == 3.0 * 2 ** 14
    # margin 1 halves the scale: byte + 1
    _, sb1 = O.c_block_quantise(x[:, :128], 1, 128, E4M3, 1)
    assert sb1.tolist() == [[121]]


def test_nothing_saturates_and_the_scaled_amax_uses_the_top_binade():
    x = _mixed((128, 512), seed=9)
    for fmt, fmax in ((E4M3, 448.0), (E5M2, 57344.0)):
        codes, sb = O.c_block_quantise(x, 1, 128, fmt, 0)
        amax = x.float().reshape(128, 4, 128).abs().amax(dim=2)
        scaled = torch.ldexp(amax, (127 - sb.int()))
        live = amax > 0
        assert bool((scaled[live] <= fmax).all()) and bool((scaled[live] > fmax / 2).all())
        # round trip: within half a spacing of the top binade, relative to the block amax: 2^-4 (E4M3), 2^-3 (E5M2)
        deq = O.t_mx_dequantise(codes, O.block_scales_as_mx(sb, 1, 128), fmt).reshape(128, 4, 128)
        err = (deq - x.float().reshape(128, 4, 128)).abs()
        assert bool((err <= amax.unsqueeze(2) * (2.0 ** -4 if fmt == E4M3 else 2.0 ** -3)).all())


def test_two_dimensional_blocks_and_block_index_order():
    """A 128 x 128 block takes its scale from all of its rows; blocks are indexed [row block, column block]."""
    x = torch.full((256, 384), 0.5, dtype=torch.bfloat16)
    x[130, 5] = 100.0                # block (1, 0)
    x[3, 300] = 0.001                # block (0, 2): does not raise its amax
    codes, sb = O.c_block_quantise(x, 128, 128, E4M3, 0)
    assert sb.shape == (2, 3)
    want_small = 127 - 9             # 448 / 0.5 = 896 -> 512 = 2^9
    want_big = 127 - 2               # 448 / 100 = 4.48 -> 4
    assert sb.tolist() == [[want_small] * 3, [want_big, want_small, want_small]]
    assert float(O.t_decode(codes, E4M3)[255, 127]) == 2.0 and float(O.t_decode(codes, E4M3)[0, 0]) == 256.0


def test_specials_and_power_of_two_invariance():
    x = _mixed((4, 256), seed=11)
    x[0, 3] = float("inf")
    x[1, 200] = float("nan")
    x[2, :128] = 0.0
    codes, sb = O.c_block_quantise(x, 1, 128, E4M3, 0)
    assert int(sb[0, 0]) == 127 and int(sb[1, 1]) == 127 and int(sb[2, 0]) == 127
    assert int(codes[0, 3]) == 0x7E and int(codes[1, 200]) & 0x7F == 0x7F and int(codes[2, 5]) == 0
    y = _mixed((4, 256), seed=12)
    c0, s0 = O.c_block_quantise(y, 1, 128, E4M3, 0)
    z = y.clone()
    z[:, 128:] = (z[:, 128:].float() * 8.0).bfloat16()
    c1, s1 = O.c_block_quantise(z, 1, 128, E4M3, 0)
    assert_bytes_equal(c1, c0, "codes under a power-of-two change of one block")
    assert torch.equal(s1[:, 0], s0[:, 0]) and torch.equal(s1[:, 1].int(), s0[:, 1].int() + 3)


def test_blockwise_tensors_multiply_through_the_mx_emulation():
    a, b = _mixed((64, 256), seed=20), _mixed((128, 256), seed=21)
    ac, asb = O.c_block_quantise(a, 1, 128, E4M3, 0)
    bc, bsb = O.c_block_quantise(b, 128, 128, E4M3, 0)
    got = O.t_mx_gemm_nt(ac, O.block_scales_as_mx(asb, 1, 128), bc, O.block_scales_as_mx(bsb, 128, 128), E4M3, E4M3, want_f32=True)[1]
    want = a.float() @ b.float().t()
    assert float((got - want).abs().max() / want.abs().max()) < 0.1          # it is the product, to FP8 accuracy
    # exact on data every block represents exactly
    a2 = torch.randint(-8, 9, (64, 256)).float().bfloat16()
    b2 = torch.randint(-8, 9, (128, 256)).float().bfloat16()
    ac, asb = O.c_block_quantise(a2, 1, 128, E4M3, 0)
    bc, bsb = O.c_block_quantise(b2, 128, 128, E4M3, 0)
    got = O.t_mx_gemm_nt(ac, O.block_scales_as_mx(asb, 1, 128), bc, O.block_scales_as_mx(bsb, 128, 128), E4M3, E4M3, want_f32=True)[1]
    assert torch.equal(got, a2.float() @ b2.float().t())
