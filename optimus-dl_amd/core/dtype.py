"""String <-> torch dtype tables, including the FP8 spellings the AMP config accepts.

Counterpart of optimus_dl/core/dtype.py (str_to_dtype :10, is_fp8_dtype :101,
get_fp8_format_from_dtype :119); the alias sets are the ones pinned by the
reference's tests/optim/test_fp8.py:36-97.
"""

from __future__ import annotations

import torch

_PLAIN = {
    torch.float32: ("float32", "fp32", "float"),
    torch.float16: ("float16", "fp16", "half"),
    torch.bfloat16: ("bfloat16", "bf16"),
    torch.float64: ("float64", "fp64", "double"),
    torch.int8: ("int8", "i8"),
    torch.int16: ("int16", "i16"),
    torch.int32: ("int32", "i32"),
    torch.int64: ("int64", "i64"),
    torch.uint8: ("uint8", "u8"),
    torch.bool: ("bool",),
    torch.complex64: ("complex64", "c64"),
    torch.complex128: ("complex128", "c128"),
}
# every way the configs spell the two OCP FP8 types
_FP8 = {
    torch.float8_e4m3fn: ("float8_e4m3fn", "fp8_e4m3fn", "e4m3fn", "e4m3", "float8_e4m3", "fp8_e4m3"),
    torch.float8_e5m2: ("float8_e5m2", "fp8_e5m2", "e5m2fn", "e5m2", "float8_e5m2fn", "fp8_e5m2fn"),
}
_FORMAT_NAME = {torch.float8_e4m3fn: "e4m3fn", torch.float8_e5m2: "e5m2"}

_TABLE: dict[str, torch.dtype] = {}
for _dtype, _names in {**_PLAIN, **_FP8}.items():
    for _n in _names:
        _TABLE[_n] = _dtype
        _TABLE["torch." + _n] = _dtype


def str_to_dtype(dtype_str: str | torch.dtype) -> torch.dtype:
    if isinstance(dtype_str, torch.dtype):
        return dtype_str
    try:
        return _TABLE[dtype_str]
    except KeyError:
        raise ValueError(f"Unsupported dtype string: {dtype_str}, supported: {sorted(_TABLE)}") from None


def is_fp8_dtype(dtype: torch.dtype) -> bool:
    return dtype in _FP8


def get_fp8_format_from_dtype(dtype: torch.dtype) -> str | None:
    return _FORMAT_NAME.get(dtype)
