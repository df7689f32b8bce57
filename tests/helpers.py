"""Shared helpers for the GPU parity tests."""
import torch


def seeded_bf16(shape, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).bfloat16()


def assert_bytes_equal(got: torch.Tensor, want: torch.Tensor, what: str):
    got, want = got.cpu(), want.cpu()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if not torch.equal(got, want):
        bad = (got != want).nonzero()
        first = bad[:8].tolist()
        detail = [(idx, int(got[tuple(idx)]), int(want[tuple(idx)])) for idx in first]
        raise AssertionError(f"{what}: {bad.shape[0]} of {got.numel()} bytes differ; first (index, got, want): {detail}")


def assert_f32_bits_equal(got: torch.Tensor, want: torch.Tensor, what: str):
    got, want = got.cpu().float().contiguous(), want.cpu().float().contiguous()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    gb, wb = got.view(torch.int32), want.view(torch.int32)
    both_nan = torch.isnan(got) & torch.isnan(want)
    ok = (gb == wb) | both_nan
    if not bool(ok.all()):
        bad = (~ok).nonzero()[:8].flatten().tolist()
        raise AssertionError(f"{what}: fp32 bits differ at {bad}: got {got.flatten()[bad].tolist()} want {want.flatten()[bad].tolist()}")


def max_rel_err(out: torch.Tensor, ref: torch.Tensor) -> float:
    """max|out - ref| / max|ref| over the whole output (the GEMM parity metric)."""
    out, ref = out.float().cpu(), ref.float().cpu()
    denom = ref.abs().max().item()
    return (out - ref).abs().max().item() / (denom if denom > 0 else 1.0)
