"""CPU-side checks of the native boundary: the library loads and exports every
symbol that include/odl_fp8.h declares (no compute calls: there is no GPU here)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "odl_fp8.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(odl_fp8_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for must in ("odl_fp8_amax", "odl_fp8_cast", "odl_fp8_cast_transpose", "odl_fp8_gemm_nt",
                 "odl_fp8_scale_from_amax", "odl_fp8_delayed_update"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    from optimus_dl_amd import native

    if not native.is_built():
        pytest.skip("libodl_fp8.so not built here (run `python -m optimus_dl_amd.build`)")
    lib = native.load()
    for sym in declared_symbols():
        assert hasattr(lib, sym), f"{sym} is declared in include/odl_fp8.h but not exported"
    assert sorted(native.EXPORTS) == declared_symbols()
    assert lib.odl_fp8_abi_version() == native.ABI_VERSION
    assert lib.odl_fp8_gemm_num_variants() >= 2
    assert b"generic" in lib.odl_fp8_gemm_variant_name(0)


def torch_equal(a, b):
    import torch

    return torch.equal(a, b)


def test_multi_tensor_planner_counts_work_and_refuses_bad_tables():
    """odl_fp8_multi_plan is host code: blocks of the amax pass (one per 64 KB, at most 512 per tensor), tiles of the
    cast (128 x 64), and the checks on shapes and pointers."""
    import numpy as np

    from optimus_dl_amd import native

    if not native.is_built():
        pytest.skip("library not built")
    table = np.zeros((3, 9), dtype=np.int64)       # x, out, out_t, parts, dyn_out, scale, rows, cols, {src_dtype, reserved}
    table[0] = (4096, 8192, 16384, 32768, 64, 0, 1024, 1024, native.DT_BF16)           # 2 MB: 32 blocks, 8 x 16 tiles
    table[1] = (4096, 8192, 16384, 32768, 64, 0, 3072, 1024, native.DT_F32)            # 12 MB: 192 blocks, 24 x 16 tiles
    table[2] = (4096, 8192, 16384, 32768, 64, 0, 16384, 16384, native.DT_BF16)         # 512 MB: capped at 512 blocks
    amax, cast = native.MultiTensorPlan.plan_work(table, 0), native.MultiTensorPlan.plan_work(table, 1)
    assert amax.shape == (32 + 192 + 512, 2) and cast.shape == (128 + 384 + 128 * 256, 2)
    assert amax[:32, 0].eq(0).all() and amax[:32, 1].tolist() == list(range(32)) and amax[32, :].tolist() == [1, 0]
    assert cast[-1].tolist() == [2, 128 * 256 - 1]
    for col, bad in ((6, 1000), (7, 1020), (8, 5), (0, 0), (2, 16392), (1, 8196), (3, 0)):
        t = table.copy()
        t[1, col] = bad
        with pytest.raises(native.NativeError, match="odl_fp8_multi_plan"):
            native.MultiTensorPlan.plan_work(t, 0)
    with pytest.raises(native.NativeError, match="needs `scale`"):                      # the delayed phase reads *scale
        native.MultiTensorPlan.plan_work(table, 2)
    table[:, 5] = 128
    assert torch_equal(native.MultiTensorPlan.plan_work(table, 2), cast)
    assert native.load().odl_fp8_multi_plan(None, 0, 0, None, 0) == 0
    assert native.load().odl_fp8_multi_plan(table.ctypes.data, 3, 7, None, 0) == -1


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from optimus_dl_amd import native

    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(native.NativeError, match="no fallback"):
        native.load()


def test_cpu_tensors_are_refused_not_emulated():
    import torch

    from optimus_dl_amd import native

    if not native.is_built():
        pytest.skip("library not built")
    with pytest.raises(native.NativeError):
        native.amax(torch.zeros((4, 4), dtype=torch.bfloat16))


def test_build_rejects_asm_that_reads_a_scalar_too_soon_after_a_vector_write():
    from optimus_dl_amd.build import check_asm_hazards

    bad = """
	v_readlane_b32 s0, v180, 14
	;;#ASMSTART
	buffer_store_dwordx4 v[60:63], v0, s[16:19], s0 offen
	;;#ASMEND
"""
    good = bad.replace("\tbuffer_store", "\ts_nop 4\n\tbuffer_store")
    other_register = bad.replace("s_readlane", "s_readlane").replace("v_readlane_b32 s0", "v_readlane_b32 s7")
    in_descriptor = bad.replace("v_readlane_b32 s0", "v_readlane_b32 s18")
    assert len(check_asm_hazards(bad, "x.s")) == 1
    assert check_asm_hazards(good, "x.s") == []
    assert check_asm_hazards(other_register, "x.s") == []
    assert len(check_asm_hazards(in_descriptor, "x.s")) == 1
    # instructions the compiler emitted itself are its own business
    assert check_asm_hazards("\tv_readlane_b32 s0, v1, 2\n\tbuffer_load_dword v1, v0, s[16:19], s0 offen\n", "x.s") == []


def test_build_rejects_scaled_conversions_that_run_before_the_saturation_mode_is_set():
    from optimus_dl_amd.build import check_saturating_conversions

    mode = "\ts_setreg_imm32_b32 hwreg(HW_REG_MODE, 23, 1), 1\n"
    cvt = "\tv_cvt_scalef32_pk_fp8_bf16 v3, v1, s2\n"
    assert check_saturating_conversions("_Z1kv:\n" + mode + "\tv_mov_b32 v0, 0\n" + cvt, "x.s") == []
    assert len(check_saturating_conversions("_Z1kv:\n" + cvt + mode, "x.s")) == 1
    # the mode belongs to the wave that set it: the next function starts without it
    assert len(check_saturating_conversions("_Z1kv:\n" + mode + cvt + "_Z1lv:\n" + cvt + cvt, "x.s")) == 1
    assert check_saturating_conversions("_Z1kv:\n\tv_cvt_pk_fp8_f32 v3, v1, v2\n", "x.s") == []


def test_split_count_is_a_host_side_decision_with_the_documented_shape_rules():
    """odl_fp8_gemm_split_count launches nothing; without a GPU it plans for 256 compute units."""
    from optimus_dl_amd import native

    if not native.is_built():
        pytest.skip("library not built")
    raw = native.load().odl_fp8_gemm_split_count
    count = lambda M, N, K, k_slow=0: raw(M, N, K, k_slow)
    assert count(8192, 14336, 4096) == 1                    # enough tiles: one launch
    assert count(8192, 1024, 4096) == 1                     # 128 tiles, short contraction
    assert count(1024, 4096, 8192) == 1 and count(1024, 4096, 8192, 1) >= 2      # no 128 x 128 alternative for K-slow operands
    for M, N, K in ((768, 768, 16384), (2304, 768, 16384), (1024, 1024, 16384), (8192, 1024, 151936), (8192, 768, 50304)):
        s = count(M, N, K)
        assert 2 <= s <= 16
        assert ((M + 255) // 256) * ((N + 255) // 256) * s <= 256             # the runs fit the chip at once
        steps, per = K // 128, ((-(-(K // 128) // s)) + 1) & ~1
        assert per >= 8 and steps - (s - 1) * per >= 4                        # no run shorter than 512
    for M, N, K in ((300, 512, 8192), (768, 768, 1024), (768, 776, 16384), (768, 768, 16400), (0, 768, 16384)):
        assert count(M, N, K) == 1                          # not multiples of 128, or too short to split


def test_block_scaled_entry_points_refuse_bad_arguments_before_touching_a_device():
    """Argument and shape checks of the MXFP8 / blockwise entry points are host code that runs before any HIP call: they
    answer with an error code and a message here, where no GPU exists."""
    from optimus_dl_amd import native

    if not native.is_built():
        pytest.skip("library not built")
    L = native.load()
    err = lambda: L.odl_fp8_last_error().decode()
    p = 4096                                                     # any aligned non-null address: it is never dereferenced
    # cast: negative shape, unknown format, scale bytes without codes, blocked axis not a multiple of 32 / of 128
    assert L.odl_fp8_mx_cast(p, 0, -1, 64, 0, p, p, 0, None, None, 0, 0, None) != 0 and "negative" in err()
    assert L.odl_fp8_mx_cast(p, 0, 64, 64, 7, p, p, 0, None, None, 0, 0, None) != 0 and "fmt" in err()
    assert L.odl_fp8_mx_cast(p, 0, 64, 64, 0, p, None, 0, None, None, 0, 0, None) != 0 and "go together" in err()
    assert L.odl_fp8_mx_cast(p, 0, 64, 48, 0, p, p, 0, None, None, 0, 0, None) != 0 and "multiple of 32" in err()
    assert L.odl_fp8_mx_cast(p, 0, 64, 64, 0, p, p, 1, None, None, 0, 0, None) != 0 and "multiple of 128" in err()
    assert L.odl_fp8_mx_cast(p, 0, 0, 64, 0, None, None, 0, None, None, 0, 0, None) == 0        # nothing to do
    assert L.odl_fp8_mx_cast(p, 0, 64, 64, 0, p, p, 0, None, None, 0, 2, None) != 0 and "scale_rule" in err()
    # GEMM: K not a multiple of 32, unknown layout, K-step-major scales with K % 128 != 0, misaligned operand
    assert L.odl_fp8_mx_gemm_nt(p, p, p, p, 0, 64, 64, 48, 0, 0, None, p, 0, 0, None) != 0 and "multiple of 32" in err()
    assert L.odl_fp8_mx_gemm_nt(p, p, p, p, 5, 64, 64, 64, 0, 0, None, p, 0, 0, None) != 0 and "scales_layout" in err()
    assert L.odl_fp8_mx_gemm_nt(p, p, p, p, 1, 64, 64, 64, 0, 0, None, p, 0, 0, None) != 0 and "128" in err()
    assert L.odl_fp8_mx_gemm_nt(p + 8, p, p, p, 0, 64, 64, 64, 0, 0, None, p, 0, 0, None) != 0 and "aligned" in err()
    assert L.odl_fp8_mx_gemm_nt(p, p, p, p, 0, 0, 64, 64, 0, 0, None, p, 0, 0, None) == 0           # empty output
    # split over K: too few steps per run, workspace too small
    assert L.odl_fp8_mx_gemm_splitk(p, p, p, p, 256, 256, 1024, 0, 0, None, p, 0, 0, 4, p, 1 << 30, None) != 0 and "shorter than 512" in err()
    assert L.odl_fp8_mx_gemm_splitk(p, p, p, p, 256, 256, 8192, 0, 0, None, p, 0, 0, 4, p, 64, None) != 0 and "workspace" in err()
    # blockwise cast: sizes must be multiples of 128, margin in range
    assert L.odl_fp8_block_cast(p, 0, 128, 192, 0, 0, 0, p, p, None, None, None) != 0 and "multiples of 128" in err()
    assert L.odl_fp8_block_cast(p, 0, 128, 128, 0, 1000, 0, p, p, None, None, None) != 0 and "margin" in err()
