"""The entry point that allocates nothing (odl_fp8_cast_dynamic_noalloc) against the two calls it
stands for (odl_fp8_amax_parts + odl_fp8_cast_dynamic with a caller-owned buffer), through the C ABI.

Bit-exact: codes, transposed codes and {amax, scale, 1/scale}.  Two calls in a row share the GPU's one
static array, the second on a smaller input: whatever the first call left there must not leak into the
second.  Collected last on purpose (file name): it must pass alone in a fresh process and after every
other test.
"""
import ctypes

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


def reference_route(N, x, fmt, margin, want_rm, want_t):
    parts = N.amax_parts(x)
    return N.cast_dynamic(x, parts, fmt, margin, want_rowmajor=want_rm, want_transposed=want_t)


def noalloc_route(N, x, fmt, margin, want_rm, want_t, bufs):
    """Every output lives in `bufs`, allocated before the call; the call itself must not allocate."""
    rows, cols = x.shape
    out = bufs["out"][: rows * cols].view(rows, cols) if want_rm else None
    out_t = bufs["out_t"][: rows * cols].view(cols, rows) if want_t else None
    dyn = bufs["dyn"]
    before = torch.cuda.memory_stats()["allocation.all.allocated"]
    N.cast_dynamic_noalloc(x, fmt, margin, out, out_t, dyn)
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == before, "the wrapper allocated device memory"
    return out, out_t, dyn


@pytest.mark.parametrize("fmt,margin", [(0, 0), (1, 2)])
def test_noalloc_equals_the_two_call_route_twice_in_a_row(N, fmt, margin):
    big = seeded_bf16((2048, 1536), 3.0, 700).cuda()                 # amax sits in a late block's partial
    big[1999, 1500] = 77.0
    small = seeded_bf16((256, 128), 0.02, 701).cuda()                # fewer blocks than `big`: stale partials would win
    bufs = {"out": torch.empty(big.numel(), dtype=torch.uint8, device="cuda"),
            "out_t": torch.empty(big.numel(), dtype=torch.uint8, device="cuda"),
            "dyn": torch.empty(3, dtype=torch.float32, device="cuda")}
    for x, what in ((big, "first call"), (small, "second call, smaller input")):
        want_q, want_qt, w_amax, w_scale, w_inv = reference_route(N, x, fmt, margin, True, True)
        got_q, got_qt, dyn = noalloc_route(N, x, fmt, margin, True, True, bufs)
        torch.cuda.synchronize()
        assert_bytes_equal(got_q, want_q, f"{what}: row-major codes")
        assert_bytes_equal(got_qt, want_qt, f"{what}: transposed codes")
        assert_f32_bits_equal(dyn, torch.cat([w_amax, w_scale, w_inv]), f"{what}: amax / scale / 1/scale")
        # and against the oracle, so that both routes cannot be wrong together
        amax = O.t_amax(x.cpu())
        assert float(dyn[0]) == float(amax)
        assert_bytes_equal(got_q, O.t_cast(x.cpu(), O.t_scale(amax, fmt, margin), fmt), f"{what}: codes vs oracle")
    # only one of the outputs; fp32 source; a pointer that is not 16-byte aligned (element-at-a-time route)
    x32 = seeded_bf16((512, 256), 1.0, 702).float().cuda()
    for x, rm, t in ((x32, True, False), (x32, False, True), (small.flatten()[1:1 + 64 * 48].view(64, 48), True, True)):
        want = reference_route(N, x, fmt, margin, rm, t)
        got_q, got_qt, dyn = noalloc_route(N, x, fmt, margin, rm, t, bufs)
        torch.cuda.synchronize()
        if rm:
            assert_bytes_equal(got_q, want[0], "row-major codes")
        if t:
            assert_bytes_equal(got_qt, want[1], "transposed codes")
        assert_f32_bits_equal(dyn, torch.cat(want[2:]), "amax / scale / 1/scale")


def test_noalloc_refuses_what_it_cannot_take(N):
    L = N.load()
    x = torch.zeros((16, 16), dtype=torch.bfloat16, device="cuda")
    out = torch.empty((16, 16), dtype=torch.uint8, device="cuda")
    dyn = torch.empty(3, dtype=torch.float32, device="cuda")
    too_many = 1 << 16                                                # 2^16 x 2^16 = 2^32 elements > ODL_FP8_NOALLOC_MAX_ELEMS
    rc = L.odl_fp8_cast_dynamic_noalloc(x.data_ptr(), N.DT_BF16, too_many, too_many, N.E4M3, 0, out.data_ptr(), None, dyn.data_ptr(), None)
    assert rc == 2 and b"exceed the limit" in L.odl_fp8_last_error()
    assert L.odl_fp8_cast_dynamic_noalloc(x.data_ptr(), N.DT_BF16, 16, 16, N.E4M3, 0, None, None, dyn.data_ptr(), None) == 1
    assert L.odl_fp8_cast_dynamic_noalloc(x.data_ptr(), N.DT_BF16, 16, 16, N.E4M3, 0, out.data_ptr(), None, None, None) == 1
    assert L.odl_fp8_cast_dynamic_noalloc(x.data_ptr(), 7, 16, 16, N.E4M3, 0, out.data_ptr(), None, dyn.data_ptr(), None) == 1
    # an empty tensor: nothing is cast, the three numbers are those of amax 0 (scale 1)
    rc = L.odl_fp8_cast_dynamic_noalloc(None, N.DT_BF16, 0, 16, N.E4M3, 0, None, None, dyn.data_ptr(), ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert rc == 0 and dyn.tolist() == [0.0, 1.0, 1.0]
