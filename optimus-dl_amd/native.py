"""ctypes binding of ``libodl_fp8.so`` (the C ABI declared in include/odl_fp8.h).

The library is the product: there is no eager / CPU fallback behind these
functions.  If the shared object is missing or a call is refused, the caller
gets an exception.

Tensors are passed as raw device pointers together with torch's current HIP
stream, so every kernel is ordered with the surrounding torch work and nothing
synchronises with the host.
"""

from __future__ import annotations

import ctypes
import os
import threading

import numpy as np
import torch

E4M3, E5M2 = 0, 1
SCALE_TENSOR, SCALE_ROW, SCALE_COL = 0, 1, 2
DT_BF16, DT_F32 = 0, 1
AMAX_MAX, AMAX_MOST_RECENT = 0, 1
FP8_MAX = {E4M3: 448.0, E5M2: 57344.0}
TORCH_FP8 = {E4M3: torch.float8_e4m3fn, E5M2: torch.float8_e5m2}
ABI_VERSION = 16
AMAX_PARTS = 512                       # ODL_FP8_AMAX_PARTS

_HERE = os.path.dirname(os.path.abspath(__file__))
# ODL_FP8_LIB names another build of the same library (e.g. one made for an experiment)
LIB_PATH = os.environ.get("ODL_FP8_LIB") or os.path.join(_HERE, "libodl_fp8.so")

EXPORTS = (
    "odl_fp8_abi_version",
    "odl_fp8_last_error",
    "odl_fp8_init_device",
    "odl_fp8_amax",
    "odl_fp8_scale_from_amax",
    "odl_fp8_amax_scale",
    "odl_fp8_amax_parts",
    "odl_fp8_cast_dynamic",
    "odl_fp8_cast_dynamic_noalloc",
    "odl_fp8_multi_plan",
    "odl_fp8_multi_amax_parts",
    "odl_fp8_multi_cast_dynamic",
    "odl_fp8_multi_cast_delayed",
    "odl_fp8_amax_parts_colsum",
    "odl_fp8_swiglu_amax_parts",
    "odl_fp8_swiglu_bwd_amax_parts",
    "odl_fp8_rmsnorm_amax_parts",
    "odl_fp8_rmsnorm_bwd",
    "odl_fp8_layernorm_amax_parts",
    "odl_fp8_layernorm_bwd",
    "odl_fp8_gelu_table",
    "odl_fp8_gelu_amax_parts",
    "odl_fp8_gelu_bwd_amax_parts",
    "odl_fp8_amax_rowcol",
    "odl_fp8_cast_rowcol",
    "odl_fp8_cast",
    "odl_fp8_cast_transpose",
    "odl_fp8_cast_delayed",
    "odl_fp8_gemm_nt",
    "odl_fp8_gemm_nt_sum",
    "odl_fp8_gemm_layouts",
    "odl_fp8_gemm_split_count",
    "odl_fp8_gemm_splitk",
    "odl_fp8_delayed_update",
    "odl_fp8_gemm_num_variants",
    "odl_fp8_gemm_variant_name",
    "odl_fp8_gemm_set_variant",
    "odl_fp8_gemm_set_clock_probe",
    "odl_fp8_mx_cast",
    "odl_fp8_mx_gemm_nt",
    "odl_fp8_block_cast",
    "odl_fp8_mx_gemm_splitk",
)

_lib = None
_lock = threading.Lock()


class NativeError(RuntimeError):
    """Raised when the native library is missing or refuses a call."""


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def load() -> ctypes.CDLL:
    """Load the library once (torch is imported first so that its HIP runtime,
    which has the same SONAME, is the one the library binds to)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not is_built():
            raise NativeError(
                f"{LIB_PATH} is missing: build it with `python -m optimus_dl_amd.build` "
                "(hipcc, gfx950). There is no fallback path."
            )
        L = ctypes.CDLL(LIB_PATH)
        vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
        L.odl_fp8_abi_version.restype = i32
        L.odl_fp8_last_error.restype = ctypes.c_char_p
        L.odl_fp8_amax.argtypes = [vp, i32, i64, i64, i32, vp, i32, vp]
        L.odl_fp8_scale_from_amax.argtypes = [vp, i64, i32, i32, vp, vp, vp]
        L.odl_fp8_amax_scale.argtypes = [vp, i32, i64, i64, i32, i32, vp, vp, vp, vp, vp]
        L.odl_fp8_amax_parts.argtypes = [vp, i32, i64, i64, vp, vp]
        L.odl_fp8_cast_dynamic.argtypes = [vp, i32, i64, i64, vp, i32, i32, vp, vp, vp, vp]
        L.odl_fp8_cast_dynamic_noalloc.argtypes = [vp, i32, i64, i64, i32, i32, vp, vp, vp, vp]
        L.odl_fp8_multi_plan.argtypes = [vp, i64, i32, vp, i64]
        L.odl_fp8_multi_plan.restype = ctypes.c_int64
        L.odl_fp8_multi_amax_parts.argtypes = [vp, vp, i64, vp]
        L.odl_fp8_multi_cast_dynamic.argtypes = [vp, vp, i64, i32, i32, vp]
        L.odl_fp8_multi_cast_delayed.argtypes = [vp, vp, i64, i32, vp]
        L.odl_fp8_amax_parts_colsum.argtypes = [vp, i32, i64, i64, vp, vp, vp, vp]
        L.odl_fp8_swiglu_amax_parts.argtypes = [vp, vp, i64, i64, vp, vp, vp]
        L.odl_fp8_swiglu_bwd_amax_parts.argtypes = [vp, vp, vp, i64, i64, vp, vp, vp, vp, vp]
        L.odl_fp8_rmsnorm_amax_parts.argtypes = [vp, i32, vp, i64, i64, ctypes.c_float, vp, vp, vp, vp]
        L.odl_fp8_rmsnorm_bwd.argtypes = [vp, vp, i32, vp, vp, i64, i64, vp, vp, vp, vp]
        L.odl_fp8_layernorm_amax_parts.argtypes = [vp, i32, vp, vp, i64, i64, ctypes.c_float, vp, vp, vp, vp, vp]
        L.odl_fp8_gelu_table.argtypes = [vp, vp]
        L.odl_fp8_gelu_amax_parts.argtypes = [vp, i64, i64, vp, vp, vp, vp]
        L.odl_fp8_gelu_bwd_amax_parts.argtypes = [vp, vp, i64, i64, vp, vp, vp, vp]
        L.odl_fp8_layernorm_bwd.argtypes = [vp, vp, i32, vp, vp, vp, i64, i64, vp, vp, vp, vp, vp]
        L.odl_fp8_amax_rowcol.argtypes = [vp, i32, i64, i64, vp, vp, vp]
        L.odl_fp8_cast_rowcol.argtypes = [vp, i32, i64, i64, vp, vp, i32, i32, vp, vp, vp, vp, vp, vp, vp]
        L.odl_fp8_cast.argtypes = [vp, i32, i64, i64, vp, i32, i32, vp, vp, vp]
        L.odl_fp8_cast_transpose.argtypes = [vp, i32, i64, i64, vp, i32, i32, vp, vp, vp, vp]
        L.odl_fp8_cast_delayed.argtypes = [vp, i32, i64, i64, vp, i32, vp, vp, vp, vp, vp]
        L.odl_fp8_gemm_nt.argtypes = [vp, vp, i64, i64, i64, i32, i32, vp, i64, vp, i64, vp, i32, vp, i32, i32, vp]
        L.odl_fp8_gemm_nt_sum.argtypes = [i32, vp, vp, vp, i64, i64, i32, i32, vp, vp, vp, i32, vp]
        L.odl_fp8_gemm_layouts.argtypes = [vp, vp, i64, i64, i64, i32, i32, i32, i32, vp, vp, vp, i32, vp]
        L.odl_fp8_gemm_split_count.argtypes = [i64, i64, i64, i32]
        L.odl_fp8_gemm_split_count.restype = i32
        L.odl_fp8_gemm_splitk.argtypes = [vp, vp, i64, i64, i64, i32, i32, i32, i32, vp, i64, vp, i64, vp, vp, i32, i32, i32, vp, i64, vp]
        L.odl_fp8_delayed_update.argtypes = [vp, i64, i64, i64, vp, vp, vp, i32, i32, vp, vp]
        L.odl_fp8_gemm_num_variants.restype = i32
        L.odl_fp8_gemm_variant_name.argtypes = [i32]
        L.odl_fp8_gemm_variant_name.restype = ctypes.c_char_p
        L.odl_fp8_gemm_set_variant.argtypes = [i32]
        L.odl_fp8_gemm_set_clock_probe.argtypes = [vp, i32]
        L.odl_fp8_mx_cast.argtypes = [vp, i32, i64, i64, i32, vp, vp, i32, vp, vp, i32, i32, vp]
        L.odl_fp8_mx_gemm_nt.argtypes = [vp, vp, vp, vp, i32, i64, i64, i64, i32, i32, vp, vp, i32, i32, vp]
        L.odl_fp8_block_cast.argtypes = [vp, i32, i64, i64, i32, i32, i32, vp, vp, vp, vp, vp]
        L.odl_fp8_mx_gemm_splitk.argtypes = [vp, vp, vp, vp, i64, i64, i64, i32, i32, vp, vp, i32, i32, i32, vp, i64, vp]
        for name in EXPORTS:
            getattr(L, name)  # AttributeError here = the library does not match the header
        if L.odl_fp8_abi_version() != ABI_VERSION:
            raise NativeError(f"{LIB_PATH}: ABI {L.odl_fp8_abi_version()} != expected {ABI_VERSION}; rebuild")
        _lib = L
    return _lib


_devices_ready: set[int] = set()


def init_device(device: "torch.device | int | None" = None) -> None:
    """Per-device set-up of the library (``odl_fp8_init_device``), once per device and process.  The wrappers whose
    kernels need it (:func:`cast_dynamic_noalloc`, the block-scaled GEMMs) call it themselves; it has to happen outside
    of HIP stream capture, so a caller that captures graphs and has not used those wrappers before calls this first
    (``FP8Recipe`` does, when it is built)."""
    if device is None:
        index = torch.cuda.current_device()
    elif isinstance(device, int):
        index = device
    else:
        index = device.index if device.index is not None else torch.cuda.current_device()
    if index in _devices_ready:
        return
    if torch.cuda.is_current_stream_capturing():
        raise NativeError(f"cuda:{index} has not been set up for the FP8 library yet and the current stream is being captured: "
                          "call optimus_dl_amd.native.init_device() once before the capture")
    with torch.cuda.device(index):
        _check(load().odl_fp8_init_device(), "odl_fp8_init_device")
    _devices_ready.add(index)


def _check(status: int, what: str) -> None:
    if status != 0:
        msg = load().odl_fp8_last_error().decode(errors="replace")
        raise NativeError(f"{what} refused (status {status}): {msg}")


# the handle of the current stream without building a torch.cuda.Stream object around it: that constructor and the
# device look-ups on its way cost 10 us a call, 0.4 ms over the 40 launches of a small step
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _src_dtype(x: torch.Tensor) -> int:
    if x.dtype == torch.bfloat16:
        return DT_BF16
    if x.dtype == torch.float32:
        return DT_F32
    raise NativeError(f"source dtype {x.dtype} is not supported (bf16 or fp32)")


def _as_2d(x: torch.Tensor) -> torch.Tensor:
    if not x.is_cuda:
        raise NativeError("the FP8 kernels run on the GPU only; got a tensor on " + str(x.device))
    if x.dim() != 2:
        raise NativeError(f"expected a 2-D tensor, got shape {tuple(x.shape)}")
    return x if x.is_contiguous() else x.contiguous()


def _f32_dev(t: torch.Tensor, n: int, what: str) -> torch.Tensor:
    if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() == n):
        raise NativeError(f"{what}: need a contiguous fp32 CUDA tensor with {n} element(s), got "
                          f"{t.dtype} {tuple(t.shape)} on {t.device}")
    return t


def _n_scales(mode: int, rows: int, cols: int) -> int:
    return 1 if mode == SCALE_TENSOR else (rows if mode == SCALE_ROW else cols)


# ------------------------------------------------------------------ operations
def amax(x: torch.Tensor, mode: int = SCALE_TENSOR, out: torch.Tensor | None = None,
         accumulate: bool = False) -> torch.Tensor:
    x = _as_2d(x)
    rows, cols = x.shape
    n = _n_scales(mode, rows, cols)
    if out is None:
        if accumulate:
            raise NativeError("amax(accumulate=True) needs an `out` tensor to fold into")
        out = torch.empty(n, dtype=torch.float32, device=x.device)
    _f32_dev(out, n, "amax out")
    _check(load().odl_fp8_amax(x.data_ptr(), _src_dtype(x), rows, cols, mode, out.data_ptr(), int(accumulate), _stream()),
           "odl_fp8_amax")
    return out


_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device, stream: int) -> torch.Tensor:
    """Two zeroed words per (device, stream): calls on one stream are ordered, and every
    call leaves the words zero for the next one."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), stream)
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.zeros(2, dtype=torch.int32, device=device)
        _workspaces[key] = ws
    return ws


def amax_scale(x: torch.Tensor, fmt: int, margin: int = 0):
    """Per-tensor amax, scale and 1/scale in one launch -> (amax, scale, scale_inv), each fp32[1]."""
    x = _as_2d(x)
    rows, cols = x.shape
    out = torch.empty(3, dtype=torch.float32, device=x.device)
    stream = _stream()
    ws = _workspace(x.device, stream)
    base = out.data_ptr()
    _check(load().odl_fp8_amax_scale(x.data_ptr(), _src_dtype(x), rows, cols, fmt, margin, base, base + 4, base + 8,
                                     ws.data_ptr(), stream), "odl_fp8_amax_scale")
    return out[0:1], out[1:2], out[2:3]


def amax_parts(x: torch.Tensor) -> torch.Tensor:
    """AMAX_PARTS partial maxima of |x| (no atomics); input of :func:`cast_dynamic`.  The kernel
    writes every entry, so the buffer is a fresh allocation per call: callers on several threads
    cannot get each other's partials."""
    x = _as_2d(x)
    rows, cols = x.shape
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_amax_parts(x.data_ptr(), _src_dtype(x), rows, cols, parts.data_ptr(), _stream()), "odl_fp8_amax_parts")
    return parts


COLSUM_WORKSPACE = 512 * 256


def colsum_supported(x: torch.Tensor) -> bool:
    """Shapes :func:`amax_parts_colsum` takes (others: amax_parts and a separate sum)."""
    if x.dim() != 2 or x.numel() == 0 or x.dtype not in (torch.bfloat16, torch.float32):
        return False
    cpl = 8 if x.dtype == torch.bfloat16 else 4
    return x.shape[1] % cpl == 0 and x.shape[1] <= AMAX_PARTS * 32 * cpl and x.is_contiguous() and x.data_ptr() % 16 == 0


def amax_parts_colsum(x: torch.Tensor):
    """Partial maxima of |x| and the fp32 column sums of x in one pass.  -> (parts, colsum[cols])."""
    x = _as_2d(x)
    rows, cols = x.shape
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=x.device)
    colsum = torch.empty(cols, dtype=torch.float32, device=x.device)
    ws = torch.empty(COLSUM_WORKSPACE, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_amax_parts_colsum(x.data_ptr(), _src_dtype(x), rows, cols, parts.data_ptr(), colsum.data_ptr(),
                                            ws.data_ptr(), _stream()), "odl_fp8_amax_parts_colsum")
    return parts, colsum


def _codes_out(t: torch.Tensor, shape: tuple, device, what: str) -> torch.Tensor:
    if t.dtype != torch.uint8 or tuple(t.shape) != tuple(shape) or not t.is_contiguous() or t.device != device:
        raise NativeError(f"{what}: a contiguous uint8 tensor {tuple(shape)} on {device} expected, got {t.dtype} {tuple(t.shape)} on {t.device}")
    return t


def cast_dynamic(x: torch.Tensor, parts: torch.Tensor, fmt: int, margin: int = 0, want_rowmajor: bool = True,
                 want_transposed: bool = True, out_t: torch.Tensor | None = None):
    """Cast with the per-tensor scale derived inside the kernel from the partial maxima.  out_t: where the transposed
    codes go (a [cols, rows] uint8 tensor of the caller's, e.g. a run of rows of a larger buffer that holds the codes of
    several tensors); implies want_transposed.
    -> (q or None, q_t or None, amax, scale, scale_inv); the last three are fp32[1]."""
    want_transposed = want_transposed or out_t is not None
    if not (want_rowmajor or want_transposed):
        raise NativeError("cast_dynamic: nothing to produce")
    x = _as_2d(x)
    rows, cols = x.shape
    _f32_dev(parts, AMAX_PARTS, "cast_dynamic parts")
    q = torch.empty((rows, cols), dtype=torch.uint8, device=x.device) if want_rowmajor else None
    if out_t is not None:
        q_t = _codes_out(out_t, (cols, rows), x.device, "cast_dynamic out_t")
    else:
        q_t = torch.empty((cols, rows), dtype=torch.uint8, device=x.device) if want_transposed else None
    dyn = torch.empty(3, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_cast_dynamic(x.data_ptr(), _src_dtype(x), rows, cols, parts.data_ptr(), fmt, margin,
                                       q.data_ptr() if q is not None else None, q_t.data_ptr() if q_t is not None else None,
                                       dyn.data_ptr(), _stream()), "odl_fp8_cast_dynamic")
    return q, q_t, dyn[0:1], dyn[1:2], dyn[2:3]


NOALLOC_MAX_ELEMS = 1 << 31            # ODL_FP8_NOALLOC_MAX_ELEMS


def cast_dynamic_noalloc(x: torch.Tensor, fmt: int, margin: int, out: torch.Tensor | None, out_t: torch.Tensor | None,
                         dyn_out: torch.Tensor) -> None:
    """Current scaling of ``x`` into buffers the CALLER owns, through the entry point that allocates
    nothing: the partial maxima pass through the library's per-GPU static array instead of a workspace.
    Neither this wrapper nor the library allocates; calls that may overlap on one GPU race on that array.
    out [rows, cols] / out_t [cols, rows] uint8 (either may be None), dyn_out fp32[3] = {amax, scale, 1/scale}."""
    if not (x.is_cuda and x.dim() == 2 and x.is_contiguous()):
        raise NativeError("cast_dynamic_noalloc: x must be a contiguous 2-D CUDA tensor (no copy is made here)")
    rows, cols = x.shape
    for t, shape, what in ((out, (rows, cols), "out"), (out_t, (cols, rows), "out_t")):
        if t is not None and not (t.is_cuda and t.dtype == torch.uint8 and t.is_contiguous() and tuple(t.shape) == shape):
            raise NativeError(f"cast_dynamic_noalloc: {what} must be a contiguous uint8 CUDA tensor of shape {shape}")
    _f32_dev(dyn_out, 3, "cast_dynamic_noalloc dyn_out")
    init_device(x.device)
    _check(load().odl_fp8_cast_dynamic_noalloc(x.data_ptr(), _src_dtype(x), rows, cols, fmt, margin,
                                               out.data_ptr() if out is not None else None,
                                               out_t.data_ptr() if out_t is not None else None, dyn_out.data_ptr(), _stream()),
           "odl_fp8_cast_dynamic_noalloc")


class MultiTensorPlan:
    """Many tensors quantised per launch.  Current scaling (``scales`` None): ``odl_fp8_multi_amax_parts`` +
    ``odl_fp8_multi_cast_dynamic``, two launches.  Delayed scaling (``scales`` and ``parts`` given, one 1-element scale
    and one AMAX_PARTS strip per tensor, e.g. views into a scaling arena): ``odl_fp8_multi_cast_delayed``, one launch
    that casts with the scales in force and folds the maxima into the strips.

    Built once from the source tensors: allocates every output (codes, transposed codes, {amax, scale, 1/scale} per
    tensor, and the partial maxima for current scaling), the table that describes them and the work lists, all on the
    tensors' device.  :meth:`run` allocates nothing and writes the same buffers every time.  Sources must be 2-D,
    contiguous, bf16 or fp32, rows a multiple of 16 and columns of 8 (``eligible``).  The plan holds ADDRESSES:
    ``stale()`` tells whether a source (or a scale / strip) moved."""

    MT_AMAX, MT_CAST, MT_CAST_DELAYED = 0, 1, 2

    @staticmethod
    def eligible(x: torch.Tensor) -> bool:
        return (x.is_cuda and x.dim() == 2 and x.is_contiguous() and x.dtype in (torch.bfloat16, torch.float32)
                and x.shape[0] > 0 and x.shape[0] % 16 == 0 and x.shape[1] > 0 and x.shape[1] % 8 == 0 and x.data_ptr() % 16 == 0)

    def __init__(self, sources: list[torch.Tensor], fmt: int, margin: int = 0, scales: list[torch.Tensor] | None = None,
                 parts: list[torch.Tensor] | None = None):
        if not sources:
            raise NativeError("MultiTensorPlan: no tensors")
        for x in sources:
            if not self.eligible(x):
                raise NativeError(f"MultiTensorPlan: a {x.dtype} tensor of shape {tuple(x.shape)} on {x.device} cannot take the "
                                  "multi-tensor route (2-D contiguous bf16 / fp32 on the GPU, rows % 16 == 0, cols % 8 == 0)")
        dev = sources[0].device
        if any(x.device != dev for x in sources):
            raise NativeError("MultiTensorPlan: tensors on different devices")
        self.delayed = scales is not None
        n = len(sources)
        if self.delayed:
            if parts is None or len(scales) != n or len(parts) != n:
                raise NativeError("MultiTensorPlan: delayed scaling needs one scale and one strip of partial maxima per tensor")
            for sc, pt in zip(scales, parts):
                _f32_dev(sc, 1, "MultiTensorPlan scale")
                _f32_dev(pt, AMAX_PARTS, "MultiTensorPlan partial maxima")
            self.scales, self.parts = list(scales), list(parts)
        else:
            self.scales = None
            strips = torch.zeros((n, AMAX_PARTS), dtype=torch.float32, device=dev)
            self.parts = [strips[i] for i in range(n)]
        self.sources, self.fmt, self.margin, self.device = list(sources), fmt, margin, dev
        self.codes = [torch.empty(tuple(x.shape), dtype=torch.uint8, device=dev) for x in sources]
        self.codes_t = [torch.empty((x.shape[1], x.shape[0]), dtype=torch.uint8, device=dev) for x in sources]
        self.dyn = torch.zeros((n, 3), dtype=torch.float32, device=dev)          # rows {amax, scale, 1/scale}
        self._ptrs = self._addresses()
        # odl_fp8_mt_tensor: six pointers, rows, cols, {src_dtype, reserved} = 9 x 8 bytes
        table = np.zeros((n, 9), dtype=np.int64)
        for i, x in enumerate(sources):
            table[i] = (x.data_ptr(), self.codes[i].data_ptr(), self.codes_t[i].data_ptr(), self.parts[i].data_ptr(),
                        self.dyn[i].data_ptr(), self.scales[i].data_ptr() if self.delayed else 0, x.shape[0], x.shape[1], _src_dtype(x))
        phases = (self.MT_CAST_DELAYED,) if self.delayed else (self.MT_AMAX, self.MT_CAST)
        self._work = [self.plan_work(table, phase).to(dev) for phase in phases]
        self._table = torch.from_numpy(table).to(dev)

    def _addresses(self) -> list[int]:
        extra = (self.scales + self.parts) if self.delayed else []
        return [t.data_ptr() for t in self.sources + extra]

    @staticmethod
    def plan_work(table: "np.ndarray", phase: int) -> torch.Tensor:
        """The work list of one phase for a host copy of the table ([n, 9] int64), as a [count, 2] int32 CPU tensor."""
        L = load()
        n = table.shape[0]
        count = L.odl_fp8_multi_plan(table.ctypes.data, n, phase, None, 0)
        if count < 0:
            raise NativeError(f"odl_fp8_multi_plan: {L.odl_fp8_last_error().decode()}")
        work = torch.empty((count, 2), dtype=torch.int32)
        if L.odl_fp8_multi_plan(table.ctypes.data, n, phase, work.data_ptr(), count) != count:
            raise NativeError(f"odl_fp8_multi_plan: {L.odl_fp8_last_error().decode()}")
        return work

    def stale(self) -> bool:
        return self._addresses() != self._ptrs

    def run(self) -> None:
        L, stream = load(), _stream()
        if self.delayed:
            (w_cast,) = self._work
            _check(L.odl_fp8_multi_cast_delayed(self._table.data_ptr(), w_cast.data_ptr(), w_cast.shape[0], self.fmt, stream),
                   "odl_fp8_multi_cast_delayed")
            return
        w_amax, w_cast = self._work
        _check(L.odl_fp8_multi_amax_parts(self._table.data_ptr(), w_amax.data_ptr(), w_amax.shape[0], stream), "odl_fp8_multi_amax_parts")
        _check(L.odl_fp8_multi_cast_dynamic(self._table.data_ptr(), w_cast.data_ptr(), w_cast.shape[0], self.fmt, self.margin, stream),
               "odl_fp8_multi_cast_dynamic")


def quantize_dynamic(x: torch.Tensor, fmt: int, margin: int = 0, want_rowmajor: bool = True, want_transposed: bool = True,
                     parts: torch.Tensor | None = None, out_t: torch.Tensor | None = None):
    """Current scaling of one tensor in two launches: partial maxima, then a cast that derives the
    scale itself.  parts: the partial maxima, when the kernel that produced x already delivered
    them (one launch then).  -> (q or None, q_t or None, amax, scale, scale_inv)."""
    return cast_dynamic(x, amax_parts(x) if parts is None else parts, fmt, margin, want_rowmajor, want_transposed, out_t=out_t)


def _bf16_dense(t: torch.Tensor, what: str) -> torch.Tensor:
    if not t.is_cuda:
        raise NativeError(f"{what}: the kernels run on the GPU only; got a tensor on {t.device}")
    if t.dtype != torch.bfloat16:
        raise NativeError(f"{what}: bf16 expected, got {t.dtype}")
    if not t.is_contiguous():
        t = t.contiguous()
    if t.data_ptr() % 16:
        t = t.clone(memory_format=torch.contiguous_format)
    return t


def swiglu_amax_parts(gate: torch.Tensor, up: torch.Tensor):
    """h = silu(gate) * up as eager bf16 arithmetic leaves it, and the partial maxima of |h| for
    :func:`cast_dynamic`.  -> (h, parts)."""
    gate, up = _bf16_dense(gate, "swiglu gate"), _bf16_dense(up, "swiglu up")
    if gate.shape != up.shape:
        raise NativeError(f"swiglu: gate {tuple(gate.shape)} and up {tuple(up.shape)} differ")
    cols = gate.shape[-1] if gate.dim() else 1
    rows = gate.numel() // max(cols, 1)
    h = torch.empty_like(gate)
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=gate.device)
    _check(load().odl_fp8_swiglu_amax_parts(gate.data_ptr(), up.data_ptr(), rows, cols, h.data_ptr(), parts.data_ptr(), _stream()),
           "odl_fp8_swiglu_amax_parts")
    return h, parts


def swiglu_bwd_amax_parts(dh: torch.Tensor, gate: torch.Tensor, up: torch.Tensor):
    """Gradients of silu(gate) * up for grad_output dh, with their partial maxima.
    -> (d_gate, d_up, parts_d_gate, parts_d_up)."""
    dh, gate, up = _bf16_dense(dh, "swiglu dh"), _bf16_dense(gate, "swiglu gate"), _bf16_dense(up, "swiglu up")
    if not (dh.shape == gate.shape == up.shape):
        raise NativeError(f"swiglu backward: shapes {tuple(dh.shape)}, {tuple(gate.shape)}, {tuple(up.shape)} differ")
    cols = gate.shape[-1] if gate.dim() else 1
    rows = gate.numel() // max(cols, 1)
    dgate, dup = torch.empty_like(gate), torch.empty_like(up)
    parts = torch.empty(2 * AMAX_PARTS, dtype=torch.float32, device=gate.device)
    pg, pu = parts[:AMAX_PARTS], parts[AMAX_PARTS:]
    _check(load().odl_fp8_swiglu_bwd_amax_parts(dh.data_ptr(), gate.data_ptr(), up.data_ptr(), rows, cols, dgate.data_ptr(),
                                                dup.data_ptr(), pg.data_ptr(), pu.data_ptr(), _stream()),
           "odl_fp8_swiglu_bwd_amax_parts")
    return dgate, dup, pg, pu


def rmsnorm_amax_parts(x: torch.Tensor, weight: torch.Tensor, eps: float):
    """y = bf16(x * rsqrt(mean(x^2, -1) + eps) * weight) over the last axis, the per-row
    1/rms, and the partial maxima of |y|.  x: bf16 or fp32.  -> (y bf16, rstd fp32, parts)."""
    if not x.is_cuda:
        raise NativeError(f"rmsnorm: the kernels run on the GPU only; got a tensor on {x.device}")
    src = _src_dtype(x)
    x = _dense_16(x)
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    w = _f32_vector(weight, cols, x.device, "rmsnorm weight")
    y = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    rstd = torch.empty(x.shape[:-1], dtype=torch.float32, device=x.device)
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_rmsnorm_amax_parts(x.data_ptr(), src, w.data_ptr(), rows, cols, float(eps), y.data_ptr(), rstd.data_ptr(),
                                             parts.data_ptr(), _stream()), "odl_fp8_rmsnorm_amax_parts")
    return y, rstd, parts


RMSNORM_BWD_SLABS = 512


def rmsnorm_bwd(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, rstd: torch.Tensor):
    """Gradients of :func:`rmsnorm_amax_parts`'s y for grad_output dy (bf16).
    -> (dx in the dtype of x, d_weight fp32[cols])."""
    dy = _bf16_dense(dy, "rmsnorm dy")
    src = _src_dtype(x)
    x = _dense_16(x)
    if dy.shape != x.shape:
        raise NativeError(f"rmsnorm backward: dy {tuple(dy.shape)} and x {tuple(x.shape)} differ")
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    w = _f32_vector(weight, cols, x.device, "rmsnorm weight")
    rstd = rstd.contiguous()
    _f32_dev(rstd.reshape(-1), rows, "rmsnorm backward rstd")
    dx = torch.empty_like(x)
    dw = torch.empty(cols, dtype=torch.float32, device=x.device)
    ws = torch.empty(RMSNORM_BWD_SLABS * cols, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_rmsnorm_bwd(dy.data_ptr(), x.data_ptr(), src, w.data_ptr(), rstd.data_ptr(), rows, cols, dx.data_ptr(),
                                      dw.data_ptr(), ws.data_ptr(), _stream()), "odl_fp8_rmsnorm_bwd")
    return dx, dw


def _f32_vector(t: torch.Tensor | None, n: int, device, what: str) -> torch.Tensor | None:
    if t is None:
        return None
    v = t.detach()
    if v.dtype != torch.float32:
        v = v.float()
    if not v.is_contiguous():
        v = v.contiguous()
    if v.data_ptr() % 16:
        v = v.clone()
    if v.numel() != n or v.device != device:
        raise NativeError(f"{what}: {v.numel()} elements on {v.device}, expected {n} on {device}")
    return v


def _dense_16(x: torch.Tensor) -> torch.Tensor:
    if not x.is_contiguous():
        x = x.contiguous()
    if x.data_ptr() % 16:
        x = x.clone(memory_format=torch.contiguous_format)
    return x


def layernorm_amax_parts(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, eps: float):
    """y = bf16(layer_norm(x) * weight + bias) over the last axis, per-row mean and 1/std, and the
    partial maxima of |y|.  x: bf16 or fp32.  -> (y bf16, mean fp32, rstd fp32, parts)."""
    if not x.is_cuda:
        raise NativeError(f"layernorm: the kernels run on the GPU only; got a tensor on {x.device}")
    src = _src_dtype(x)
    x = _dense_16(x)
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    w = _f32_vector(weight, cols, x.device, "layernorm weight")
    b = _f32_vector(bias, cols, x.device, "layernorm bias")
    y = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    stats = torch.empty((2,) + tuple(x.shape[:-1]), dtype=torch.float32, device=x.device)
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_layernorm_amax_parts(x.data_ptr(), src, w.data_ptr(), b.data_ptr() if b is not None else None, rows, cols,
                                               float(eps), y.data_ptr(), stats[0].data_ptr(), stats[1].data_ptr(), parts.data_ptr(),
                                               _stream()), "odl_fp8_layernorm_amax_parts")
    return y, stats[0], stats[1], parts


def layernorm_bwd(dy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, mean: torch.Tensor, rstd: torch.Tensor):
    """Gradients of :func:`layernorm_amax_parts`'s y for grad_output dy (bf16).
    -> (dx in the dtype of x, d_weight fp32[cols], d_bias fp32[cols])."""
    dy = _bf16_dense(dy, "layernorm dy")
    src = _src_dtype(x)
    x = _dense_16(x)
    if dy.shape != x.shape:
        raise NativeError(f"layernorm backward: dy {tuple(dy.shape)} and x {tuple(x.shape)} differ")
    cols = x.shape[-1]
    rows = x.numel() // max(cols, 1)
    w = _f32_vector(weight, cols, x.device, "layernorm weight")
    mean, rstd = mean.contiguous(), rstd.contiguous()
    _f32_dev(mean.reshape(-1), rows, "layernorm backward mean")
    _f32_dev(rstd.reshape(-1), rows, "layernorm backward rstd")
    dx = torch.empty_like(x)
    dwb = torch.empty(2 * cols, dtype=torch.float32, device=x.device)
    ws = torch.empty(2 * RMSNORM_BWD_SLABS * cols, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_layernorm_bwd(dy.data_ptr(), x.data_ptr(), src, w.data_ptr(), mean.data_ptr(), rstd.data_ptr(), rows, cols,
                                        dx.data_ptr(), dwb.data_ptr(), dwb[cols:].data_ptr(), ws.data_ptr(), _stream()),
           "odl_fp8_layernorm_bwd")
    return dx, dwb[:cols], dwb[cols:]


GELU_TABLE_BYTES = 65536 * 2 + 65536 * 4
_gelu_tables: dict[int, torch.Tensor] = {}


def gelu_table(device: torch.device) -> torch.Tensor:
    """The GELU lookup table of ``device`` (384 KB, filled on first use and kept for the process)."""
    idx = device.index if device.index is not None else torch.cuda.current_device()
    t = _gelu_tables.get(idx)
    if t is None:
        with _lock:
            t = _gelu_tables.get(idx)
            if t is None:
                t = torch.empty(GELU_TABLE_BYTES, dtype=torch.uint8, device=torch.device("cuda", idx))
                with torch.cuda.device(idx):
                    _check(load().odl_fp8_gelu_table(t.data_ptr(), _stream()), "odl_fp8_gelu_table")
                    torch.cuda.current_stream().synchronize()     # other streams may use it right away
                _gelu_tables[idx] = t
    return t


def gelu_amax_parts(x: torch.Tensor):
    """Exact GELU of a bf16 tensor and the partial maxima of the result.  -> (y, parts)."""
    x = _bf16_dense(x, "gelu x")
    cols = x.shape[-1] if x.dim() else 1
    rows = x.numel() // max(cols, 1)
    y = torch.empty_like(x)
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_gelu_amax_parts(x.data_ptr(), rows, cols, gelu_table(x.device).data_ptr(), y.data_ptr(), parts.data_ptr(),
                                          _stream()), "odl_fp8_gelu_amax_parts")
    return y, parts


def gelu_bwd_amax_parts(dy: torch.Tensor, x: torch.Tensor):
    """dx = dy * gelu'(x) in bf16 and its partial maxima.  -> (dx, parts)."""
    dy, x = _bf16_dense(dy, "gelu dy"), _bf16_dense(x, "gelu x")
    if dy.shape != x.shape:
        raise NativeError(f"gelu backward: dy {tuple(dy.shape)} and x {tuple(x.shape)} differ")
    cols = x.shape[-1] if x.dim() else 1
    rows = x.numel() // max(cols, 1)
    dx = torch.empty_like(x)
    parts = torch.empty(AMAX_PARTS, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_gelu_bwd_amax_parts(dy.data_ptr(), x.data_ptr(), rows, cols, gelu_table(x.device).data_ptr(), dx.data_ptr(),
                                              parts.data_ptr(), _stream()), "odl_fp8_gelu_bwd_amax_parts")
    return dx, parts


def quantize_rowcol(x: torch.Tensor, fmt: int, margin: int = 0):
    """Rowwise recipe, both operands of one tensor in two passes over it:
    -> (q [rows, cols] scaled per row, s_row_inv [rows], q_t [cols, rows] scaled per column, s_col_inv [cols],
        amax_row, amax_col)."""
    x = _as_2d(x)
    rows, cols = x.shape
    pr, pc = -(-rows // 4) * 4, -(-cols // 4) * 4            # every vector starts on a 16-byte boundary (the GEMM wants that)
    buf = torch.empty(3 * (pr + pc), dtype=torch.float32, device=x.device)
    a_row, a_col = buf[:rows], buf[pr:pr + cols]
    o = pr + pc
    s_row, s_col = buf[o:o + rows], buf[o + pr:o + pr + cols]
    o = 2 * (pr + pc)
    s_row_inv, s_col_inv = buf[o:o + rows], buf[o + pr:o + pr + cols]
    q = torch.empty((rows, cols), dtype=torch.uint8, device=x.device)
    q_t = torch.empty((cols, rows), dtype=torch.uint8, device=x.device)
    L, stream = load(), _stream()
    _check(L.odl_fp8_amax_rowcol(x.data_ptr(), _src_dtype(x), rows, cols, a_row.data_ptr(), a_col.data_ptr(), stream),
           "odl_fp8_amax_rowcol")
    _check(L.odl_fp8_cast_rowcol(x.data_ptr(), _src_dtype(x), rows, cols, a_row.data_ptr(), a_col.data_ptr(), fmt, margin,
                                 q.data_ptr(), q_t.data_ptr(), s_row.data_ptr(), s_row_inv.data_ptr(), s_col.data_ptr(),
                                 s_col_inv.data_ptr(), stream), "odl_fp8_cast_rowcol")
    return q, s_row_inv, q_t, s_col_inv, a_row, a_col


def scale_from_amax(amax_t: torch.Tensor, fmt: int, margin: int = 0):
    n = amax_t.numel()
    _f32_dev(amax_t, n, "scale_from_amax amax")
    scale = torch.empty_like(amax_t)
    scale_inv = torch.empty_like(amax_t)
    _check(load().odl_fp8_scale_from_amax(amax_t.data_ptr(), n, fmt, margin, scale.data_ptr(), scale_inv.data_ptr(), _stream()),
           "odl_fp8_scale_from_amax")
    return scale, scale_inv


def cast(x: torch.Tensor, scale: torch.Tensor, fmt: int, mode: int = SCALE_TENSOR,
         amax_out: torch.Tensor | None = None, out: torch.Tensor | None = None) -> torch.Tensor:
    x = _as_2d(x)
    rows, cols = x.shape
    _f32_dev(scale, _n_scales(mode, rows, cols), "cast scale")
    if out is None:
        out = torch.empty((rows, cols), dtype=torch.uint8, device=x.device)
    if amax_out is not None:
        _f32_dev(amax_out, 1, "cast amax_out")
    _check(load().odl_fp8_cast(x.data_ptr(), _src_dtype(x), rows, cols, scale.data_ptr(), mode, fmt, out.data_ptr(),
                               amax_out.data_ptr() if amax_out is not None else None, _stream()), "odl_fp8_cast")
    return out


def cast_transpose(x: torch.Tensor, scale: torch.Tensor, fmt: int, mode: int = SCALE_TENSOR,
                   amax_out: torch.Tensor | None = None, want_rowmajor: bool = True):
    """Returns (codes[rows, cols] or None, codes_t[cols, rows])."""
    x = _as_2d(x)
    rows, cols = x.shape
    _f32_dev(scale, _n_scales(mode, rows, cols), "cast_transpose scale")
    out = torch.empty((rows, cols), dtype=torch.uint8, device=x.device) if want_rowmajor else None
    out_t = torch.empty((cols, rows), dtype=torch.uint8, device=x.device)
    if amax_out is not None:
        _f32_dev(amax_out, 1, "cast_transpose amax_out")
    _check(load().odl_fp8_cast_transpose(x.data_ptr(), _src_dtype(x), rows, cols, scale.data_ptr(), mode, fmt,
                                         out.data_ptr() if out is not None else None, out_t.data_ptr(),
                                         amax_out.data_ptr() if amax_out is not None else None, _stream()),
           "odl_fp8_cast_transpose")
    return out, out_t


def cast_delayed(x: torch.Tensor, scale: torch.Tensor, fmt: int, amax_parts: torch.Tensor | None = None,
                 want_rowmajor: bool = True, want_transposed: bool = False, out_t: torch.Tensor | None = None):
    """The cast of the delayed-scaling recipe, one launch: codes with the per-tensor ``scale`` in force
    (row-major, transposed, or both), this step's partial maxima folded into ``amax_parts``
    (AMAX_PARTS floats of a role, accumulated, cleared by the next ``delayed_update``; None: nothing is
    recorded), and 1/scale in a fresh 1-element tensor that later refreshes of ``scale`` do not touch.
    -> (codes or None, codes_t or None, scale_inv[1])."""
    x = _as_2d(x)
    rows, cols = x.shape
    _f32_dev(scale, 1, "cast_delayed scale")
    if amax_parts is not None:
        _f32_dev(amax_parts, AMAX_PARTS, "cast_delayed amax_parts")
    want_transposed = want_transposed or out_t is not None       # out_t: the caller's [cols, rows] buffer, as in cast_dynamic
    if not (want_rowmajor or want_transposed):
        raise NativeError("cast_delayed: neither layout asked for")
    out = torch.empty((rows, cols), dtype=torch.uint8, device=x.device) if want_rowmajor else None
    if out_t is not None:
        _codes_out(out_t, (cols, rows), x.device, "cast_delayed out_t")
    else:
        out_t = torch.empty((cols, rows), dtype=torch.uint8, device=x.device) if want_transposed else None
    scale_inv = torch.empty(1, dtype=torch.float32, device=x.device)
    _check(load().odl_fp8_cast_delayed(x.data_ptr(), _src_dtype(x), rows, cols, scale.data_ptr(), fmt,
                                       out.data_ptr() if out is not None else None,
                                       out_t.data_ptr() if out_t is not None else None,
                                       amax_parts.data_ptr() if amax_parts is not None else None, scale_inv.data_ptr(), _stream()),
           "odl_fp8_cast_delayed")
    return out, out_t, scale_inv


def gemm_nt(a: torch.Tensor, b: torch.Tensor, fmt_a: int, fmt_b: int, sa_inv: torch.Tensor, sb_inv: torch.Tensor,
            bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16,
            out: torch.Tensor | None = None, accumulate: bool = False) -> torch.Tensor:
    """out[M,N] = (a[M,K] . b[N,K]^T) * (sa_inv x sb_inv) (+ bias); a, b uint8 FP8 codes.  A given ``out`` decides the
    output type.  accumulate: out = out + product (needs ``out``; the old value joins the fp32 sum, one rounding)."""
    if accumulate and out is None:
        raise NativeError("gemm_nt(accumulate=True) needs the `out` tensor to add into")
    if out is not None:
        out_dtype = out.dtype
    if a.dtype != torch.uint8 or b.dtype != torch.uint8:
        raise NativeError("gemm_nt operands must be uint8 FP8 codes")
    a, b = _as_2d(a), _as_2d(b)
    M, K = a.shape
    N, K2 = b.shape
    if K != K2:
        raise NativeError(f"gemm_nt: contraction sizes differ ({K} vs {K2})")
    if sa_inv.numel() not in (1, M) or sb_inv.numel() not in (1, N):
        raise NativeError(f"gemm_nt: scale vectors must have 1 or M / N entries, got {sa_inv.numel()}, {sb_inv.numel()}")
    _f32_dev(sa_inv, sa_inv.numel(), "gemm_nt sa_inv")
    _f32_dev(sb_inv, sb_inv.numel(), "gemm_nt sb_inv")
    if bias is not None:
        _f32_dev(bias, N, "gemm_nt bias")
    odt = DT_BF16 if out_dtype == torch.bfloat16 else (DT_F32 if out_dtype == torch.float32 else None)
    if odt is None:
        raise NativeError(f"gemm_nt: output dtype {out_dtype} is not supported (bf16 or fp32)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    elif out.shape != (M, N) or out.dtype != out_dtype or not out.is_contiguous():
        raise NativeError("gemm_nt: `out` has the wrong shape / dtype / layout")
    splits = gemm_split_count(M, N, K)
    if splits > 1:
        return _gemm_splitk(a, b, M, N, K, fmt_a, fmt_b, K_FAST, K_FAST, sa_inv, sb_inv, bias, out, splits, accumulate)
    _check(load().odl_fp8_gemm_nt(a.data_ptr(), b.data_ptr(), M, N, K, fmt_a, fmt_b, sa_inv.data_ptr(), sa_inv.numel(),
                                  sb_inv.data_ptr(), sb_inv.numel(), bias.data_ptr() if bias is not None else None,
                                  DT_F32, out.data_ptr(), odt, int(accumulate), _stream()), "odl_fp8_gemm_nt")
    return out


def gemm_nt_sum(a: "list[torch.Tensor]", b: "list[torch.Tensor]", fmt_a: int, fmt_b: int, sa_inv: "list[torch.Tensor]",
                sb_inv: "list[torch.Tensor]", out_dtype: torch.dtype = torch.bfloat16, out: torch.Tensor | None = None) -> torch.Tensor:
    """out[M,N] = sum_s (a[s][M,K_s] . b[s][N,K_s]^T) * (sa_inv[s] * sb_inv[s]); uint8 FP8 codes, one scale per operand.
    One launch where the shapes suit the streaming kernel (2 .. 4 pairs, M and N multiples of 128, every K_s a multiple
    of 256 and at least 512), otherwise one GEMM per pair, the later ones adding into ``out``."""
    n = len(a)
    if n < 1 or len(b) != n or len(sa_inv) != n or len(sb_inv) != n:
        raise NativeError(f"gemm_nt_sum: {len(a)} / {len(b)} operands, {len(sa_inv)} / {len(sb_inv)} scales")
    if out is not None:
        out_dtype = out.dtype
    odt = DT_BF16 if out_dtype == torch.bfloat16 else (DT_F32 if out_dtype == torch.float32 else None)
    if odt is None:
        raise NativeError(f"gemm_nt_sum: output dtype {out_dtype} is not supported (bf16 or fp32)")
    a, b = [_as_2d(t) for t in a], [_as_2d(t) for t in b]
    M, N = a[0].shape[0], b[0].shape[0]
    for s in range(n):
        if a[s].dtype != torch.uint8 or b[s].dtype != torch.uint8:
            raise NativeError("gemm_nt_sum operands must be uint8 FP8 codes")
        if a[s].shape[0] != M or b[s].shape[0] != N or a[s].shape[1] != b[s].shape[1]:
            raise NativeError(f"gemm_nt_sum: pair {s} is {tuple(a[s].shape)} x {tuple(b[s].shape)}, expected [{M}, K] x [{N}, K]")
        _f32_dev(sa_inv[s], 1, "gemm_nt_sum sa_inv")
        _f32_dev(sb_inv[s], 1, "gemm_nt_sum sb_inv")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a[0].device)
    elif out.shape != (M, N) or not out.is_contiguous():
        raise NativeError("gemm_nt_sum: `out` has the wrong shape / layout")
    ptrs = ctypes.c_void_p * n
    ks = (ctypes.c_int64 * n)(*[t.shape[1] for t in a])
    _check(load().odl_fp8_gemm_nt_sum(n, ptrs(*[t.data_ptr() for t in a]), ptrs(*[t.data_ptr() for t in b]), ks, M, N, fmt_a, fmt_b,
                                      ptrs(*[t.data_ptr() for t in sa_inv]), ptrs(*[t.data_ptr() for t in sb_inv]), out.data_ptr(),
                                      odt, _stream()), "odl_fp8_gemm_nt_sum")
    return out


MX_BLOCK = 32
MX_ROWMAJOR, MX_KSTEP = 0, 1           # ODL_MX_SCALES_*
MX_FLOOR, MX_CEIL = 0, 1               # ODL_MX_SCALE_*: shared exponent floor(log2 amax) - emax / ceil(log2(amax / fp8_max))


def _mx_scales(rows: int, length: int, layout: int | None, device) -> tuple[torch.Tensor, int]:
    """An empty scale tensor for `rows` rows blocked along an axis of `length` elements.  Row-major: [rows, length/32].
    K-step-major: [length/128, rows, 4] (what the streaming GEMM reads; the default whenever length % 128 == 0).  The
    number of dimensions tells the GEMM wrapper which one it got."""
    if layout is None:
        layout = MX_KSTEP if length % 128 == 0 and length > 0 else MX_ROWMAJOR
    if layout == MX_KSTEP:
        if length % 128:
            raise NativeError(f"mx_cast: K-step-major scales need the blocked axis ({length}) to be a multiple of 128")
        return torch.empty((length // 128, rows, 4), dtype=torch.uint8, device=device), layout
    return torch.empty((rows, length // MX_BLOCK), dtype=torch.uint8, device=device), layout


def mx_scales_rowmajor(scales: torch.Tensor) -> torch.Tensor:
    """Scale bytes as [rows, blocks], whichever layout they are stored in."""
    if scales.dim() == 3:
        return scales.permute(1, 0, 2).reshape(scales.shape[1], -1)
    return scales


def mx_cast(x: torch.Tensor, fmt: int, want_rowmajor: bool = True, want_transposed: bool = False, layout: int | None = None,
            scale_rule: int = MX_FLOOR):
    """MXFP8 conversion of ``x`` [rows, cols] in one launch -> (codes [rows, cols], their scales, codes_t [cols, rows],
    their scales); the pair that was not asked for is (None, None).  Scales are E8M0 bytes, one per 32 elements along
    the last axis of the codes they belong to, stored as ``_mx_scales`` describes (layout None: K-step-major where the
    blocked axis allows it).  scale_rule: MX_FLOOR (the OCP formula; a block amax in the top eighth of its binade
    saturates) or MX_CEIL (the exponent rounded up: nothing saturates)."""
    x = _as_2d(x)
    rows, cols = x.shape
    if not (want_rowmajor or want_transposed):
        raise NativeError("mx_cast: neither layout asked for")
    dev = x.device
    out = sc = out_t = sc_t = None
    lay = lay_t = MX_ROWMAJOR
    if want_rowmajor:
        out = torch.empty((rows, cols), dtype=torch.uint8, device=dev)
        sc, lay = _mx_scales(rows, cols, layout, dev)
    if want_transposed:
        out_t = torch.empty((cols, rows), dtype=torch.uint8, device=dev)
        sc_t, lay_t = _mx_scales(cols, rows, layout, dev)
    ptr = lambda t: t.data_ptr() if t is not None else None
    _check(load().odl_fp8_mx_cast(x.data_ptr(), _src_dtype(x), rows, cols, fmt, ptr(out), ptr(sc), lay, ptr(out_t), ptr(sc_t), lay_t,
                                  int(scale_rule), _stream()), "odl_fp8_mx_cast")
    return out, sc, out_t, sc_t


BLOCK = 128


def block_cast(x: torch.Tensor, fmt: int, margin: int = 0, two_d: bool = False, want_rowmajor: bool = True,
               want_transposed: bool = False):
    """The cast of the blockwise recipe in one launch: power-of-two scales per 128 elements of the contraction axis
    (two_d False: per row and 128 columns for the row-major codes, per column and 128 rows for the transposed ones) or
    per 128 x 128 block (two_d True, weights).  -> (codes [rows, cols], scales [cols/128, rows, 4], codes_t [cols, rows],
    scales_t [rows/128, cols, 4]); the scale tensors hold E8M0 bytes in the K-step-major layout, each block's byte four
    times, and go to ``mx_gemm_nt`` as they are.  The pair that was not asked for is (None, None)."""
    x = _as_2d(x)
    rows, cols = x.shape
    if not (want_rowmajor or want_transposed):
        raise NativeError("block_cast: neither layout asked for")
    if rows % BLOCK or cols % BLOCK:
        raise NativeError(f"block_cast: {rows} x {cols}: both sizes must be multiples of 128")
    dev = x.device
    out = sc = out_t = sc_t = None
    if want_rowmajor:
        out = torch.empty((rows, cols), dtype=torch.uint8, device=dev)
        sc = torch.empty((cols // BLOCK, rows, 4), dtype=torch.uint8, device=dev)
    if want_transposed:
        out_t = torch.empty((cols, rows), dtype=torch.uint8, device=dev)
        sc_t = torch.empty((rows // BLOCK, cols, 4), dtype=torch.uint8, device=dev)
    ptr = lambda t: t.data_ptr() if t is not None else None
    _check(load().odl_fp8_block_cast(x.data_ptr(), _src_dtype(x), rows, cols, fmt, margin, 1 if two_d else 0, ptr(out), ptr(sc),
                                     ptr(out_t), ptr(sc_t), _stream()), "odl_fp8_block_cast")
    return out, sc, out_t, sc_t


def mx_gemm_nt(a: torch.Tensor, sa: torch.Tensor, b: torch.Tensor, sb: torch.Tensor, fmt_a: int, fmt_b: int,
               bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16, out: torch.Tensor | None = None,
               accumulate: bool = False) -> torch.Tensor:
    """out[M,N] = sum over 32-blocks of 2^(sa-127) 2^(sb-127) (a_block . b_block) (+ bias); a [M,K], b [N,K] codes,
    sa, sb their E8M0 scale bytes as ``mx_cast`` returns them (both row-major [rows, K/32] or both K-step-major
    [K/128, rows, 4])."""
    for t, what in ((a, "a"), (b, "b"), (sa, "sa"), (sb, "sb")):
        if t.dtype != torch.uint8 or not t.is_cuda or not t.is_contiguous():
            raise NativeError(f"mx_gemm_nt: {what} must be a dense uint8 device tensor")
    if a.dim() != 2 or b.dim() != 2:
        raise NativeError("mx_gemm_nt: operands must be 2-D")
    M, K = a.shape
    N, K2 = b.shape
    if K != K2:
        raise NativeError(f"mx_gemm_nt: contraction sizes differ ({K} vs {K2})")
    if sa.dim() != sb.dim():
        raise NativeError("mx_gemm_nt: the two scale tensors are stored in different layouts")
    layout = MX_KSTEP if sa.dim() == 3 else MX_ROWMAJOR
    want = (lambda rows: (K // 128, rows, 4)) if layout == MX_KSTEP else (lambda rows: (rows, K // MX_BLOCK))
    if K % MX_BLOCK or (layout == MX_KSTEP and K % 128) or tuple(sa.shape) != want(M) or tuple(sb.shape) != want(N):
        raise NativeError(f"mx_gemm_nt: scale shapes {tuple(sa.shape)}, {tuple(sb.shape)} do not fit M, N, K = {M}, {N}, {K}")
    if bias is not None:
        _f32_dev(bias, N, "mx_gemm_nt bias")
    if accumulate and out is None:
        raise NativeError("mx_gemm_nt(accumulate=True) needs the `out` tensor to add into")
    if out is not None:
        out_dtype = out.dtype
        if out.shape != (M, N) or not out.is_contiguous() or not out.is_cuda:
            raise NativeError("mx_gemm_nt: `out` has the wrong shape / layout")
    odt = DT_BF16 if out_dtype == torch.bfloat16 else (DT_F32 if out_dtype == torch.float32 else None)
    if odt is None:
        raise NativeError(f"mx_gemm_nt: output dtype {out_dtype} is not supported (bf16 or fp32)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    # outputs of few tiles with a long contraction: K in runs side by side, like gemm_nt
    splits = gemm_split_count(M, N, K) if layout == MX_KSTEP else 1
    if splits > 1:
        workspace = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
        init_device(a.device)
        _check(load().odl_fp8_mx_gemm_splitk(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), M, N, K, fmt_a, fmt_b,
                                             bias.data_ptr() if bias is not None else None, out.data_ptr(), odt, int(accumulate),
                                             splits, workspace.data_ptr(), workspace.numel() * 4, _stream()), "odl_fp8_mx_gemm_splitk")
        return out
    init_device(a.device)
    _check(load().odl_fp8_mx_gemm_nt(a.data_ptr(), sa.data_ptr(), b.data_ptr(), sb.data_ptr(), layout, M, N, K, fmt_a, fmt_b,
                                     bias.data_ptr() if bias is not None else None, out.data_ptr(), odt, int(accumulate), _stream()),
           "odl_fp8_mx_gemm_nt")
    return out


K_FAST, K_SLOW = 0, 1
split_k = True            # tuning knob: outputs of few tiles with a long contraction are computed as K runs side by side
_tls = threading.local()  # .forced_variant mirrors the library's per-thread switch (see gemm_set_variant)


def gemm_split_count(M: int, N: int, K: int, k_slow: bool = False) -> int:
    """Number of K runs the library proposes for this shape (1: one launch of the ordinary kernel).
    k_slow: an operand is passed with the contraction index slow (only the streaming kernel reads that).
    Always 1 while a kernel variant is forced or ``split_k`` is off."""
    if not split_k or getattr(_tls, "forced_variant", -1) >= 0 or (M + 256) * K >= 2**31 or (N + 256) * K >= 2**31:
        return 1
    return int(load().odl_fp8_gemm_split_count(M, N, K, 1 if k_slow else 0))


def _gemm_splitk(a, b, M, N, K, fmt_a, fmt_b, layout_a, layout_b, sa_inv, sb_inv, bias, out, splits, accumulate=False):
    workspace = torch.empty((splits, M, N), dtype=torch.float32, device=a.device)
    _check(load().odl_fp8_gemm_splitk(a.data_ptr(), b.data_ptr(), M, N, K, fmt_a, fmt_b, layout_a, layout_b, sa_inv.data_ptr(),
                                      sa_inv.numel(), sb_inv.data_ptr(), sb_inv.numel(),
                                      bias.data_ptr() if bias is not None else None, out.data_ptr(), _src_dtype(out), int(accumulate),
                                      splits, workspace.data_ptr(), workspace.numel() * 4, _stream()), "odl_fp8_gemm_splitk")
    return out


def gemm_splitk(a: torch.Tensor, b: torch.Tensor, fmt_a: int, fmt_b: int, sa_inv: torch.Tensor, sb_inv: torch.Tensor,
                splits: int, bias: torch.Tensor | None = None, out_dtype: torch.dtype = torch.bfloat16,
                layout_a: int = K_FAST, layout_b: int = K_FAST, out: torch.Tensor | None = None,
                accumulate: bool = False) -> torch.Tensor:
    """The product of :func:`gemm_nt` / :func:`gemm_layouts` with K cut into ``splits`` runs that are computed
    side by side and added in run order (fp32).  :func:`gemm_nt` and :func:`gemm_layouts` take this route by
    themselves where :func:`gemm_split_count` says so; this entry is for choosing ``splits`` by hand."""
    if a.dtype != torch.uint8 or b.dtype != torch.uint8:
        raise NativeError("gemm_splitk operands must be uint8 FP8 codes")
    a, b = _as_2d(a), _as_2d(b)
    M, K = (a.shape[1], a.shape[0]) if layout_a == K_SLOW else a.shape
    N, K2 = (b.shape[1], b.shape[0]) if layout_b == K_SLOW else b.shape
    if K != K2:
        raise NativeError(f"gemm_splitk: contraction sizes differ ({K} vs {K2})")
    if sa_inv.numel() not in (1, M) or sb_inv.numel() not in (1, N):
        raise NativeError(f"gemm_splitk: scale vectors must have 1 or M / N entries, got {sa_inv.numel()}, {sb_inv.numel()}")
    _f32_dev(sa_inv, sa_inv.numel(), "gemm_splitk sa_inv")
    _f32_dev(sb_inv, sb_inv.numel(), "gemm_splitk sb_inv")
    if bias is not None:
        _f32_dev(bias, N, "gemm_splitk bias")
    if accumulate and out is None:
        raise NativeError("gemm_splitk(accumulate=True) needs the `out` tensor to add into")
    if out is not None:
        out_dtype = out.dtype
        if out.shape != (M, N) or not out.is_contiguous():
            raise NativeError("gemm_splitk: `out` has the wrong shape / layout")
    if out_dtype not in (torch.bfloat16, torch.float32):
        raise NativeError(f"gemm_splitk: output dtype {out_dtype} is not supported (bf16 or fp32)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    return _gemm_splitk(a, b, M, N, K, fmt_a, fmt_b, layout_a, layout_b, sa_inv, sb_inv, bias, out, int(splits), accumulate)


def gemm_layouts_supported(M: int, N: int, K: int, out_dtype: torch.dtype = torch.bfloat16) -> bool:
    """Shapes :func:`gemm_layouts` takes (whole 256 x 256 tiles, operands under 2 GiB)."""
    if out_dtype not in (torch.bfloat16, torch.float32):
        return False
    return (M > 0 and N > 0 and K >= 512 and M % 256 == 0 and N % 256 == 0 and K % 256 == 0
            and (M + 256) * K < 2**31 and (N + 256) * K < 2**31 and N * out_dtype.itemsize * 264 < 2**31)


def wgrad_direct_pays(n_out: int, n_in: int, tokens: int) -> bool:
    """Whether the weight gradient [n_out, n_in] = dY^T . X is better computed from the row-major codes of dY
    (:func:`gemm_layouts`, K-slow operand, no transposed copy of dY) than from a transposed copy with :func:`gemm_nt`.
    The kernel that reads K-slow operands works on whole 256 x 256 tiles: it pays where those fill the chip, and for
    small gradients, where both routes are a handful of short launches and the copy is one more.  In between it either
    leaves compute units idle or splits the contraction and adds a reduction pass, and 128 x 128 tiles over the
    transposed copy are faster.  Measured at 8192 tokens, cast of dY included, direct / transposed in us:
    1024 x 4096 61.7 / 52.2, 2048 x 4096 90.3 / 81.2, 1024 x 3072 53.3 / 48.7, 3072 x 1024 68.2 / 64.6;
    4096 x 4096 129.9 / 136.3, 2048 x 1024 54.2 / 56.2, 2304 x 768 53.8 / 58.7, 1024 x 1024 38.1 / 41.9."""
    tiles = (n_out // 256) * (n_in // 256)
    return tiles >= 192 or n_out * n_in < 2_200_000


def dgrad_sum_in_one_launch(tokens: int, n_in: int, n_outs: "list[int]") -> bool:
    """Whether the data gradient of Linears fed by one tensor, dX [tokens, n_in] = sum_s dY_s [tokens, n_outs[s]] . W_s, runs
    as ONE launch of :func:`gemm_nt_sum` (the streaming kernel carrying its accumulators from one pair to the next): the
    shapes that kernel takes, and an output of more 256 x 256 tiles than half the 256 compute units (smaller ones are better
    served by the per-pair GEMMs that add into dX: those pick 128 x 128 tiles or split the contraction)."""
    if not 2 <= len(n_outs) <= 4 or tokens % 128 or n_in % 128 or any(k % 256 or k < 512 for k in n_outs):
        return False
    tiles = ((tokens + 255) // 256) * ((n_in + 255) // 256)
    return tiles > 128 and all((tokens + 256) * k < 2**31 and (n_in + 256) * k < 2**31 for k in n_outs)


def gemm_layouts(a: torch.Tensor, b: torch.Tensor, fmt_a: int, fmt_b: int, layout_a: int, layout_b: int,
                 sa_inv: torch.Tensor, sb_inv: torch.Tensor, out: torch.Tensor | None = None,
                 out_dtype: torch.dtype = torch.bfloat16, accumulate: bool = False) -> torch.Tensor:
    """out[M,N] (bf16 or fp32) = (A . B^T) * sa_inv * sb_inv where an operand is given either as
    [rows, K] (K_FAST) or as [K, rows] (K_SLOW): no transposed copies for dgrad / wgrad.  A given
    ``out`` decides the output type, else ``out_dtype`` does.  accumulate: out = out + product (needs ``out``); the
    product then passes through an fp32 workspace (``odl_fp8_gemm_splitk``, with one run where K is not worth cutting),
    because the kernel that reads K-slow operands stores a tile where nothing can wait for the old values."""
    if accumulate and out is None:
        raise NativeError("gemm_layouts(accumulate=True) needs the `out` tensor to add into")
    if a.dtype != torch.uint8 or b.dtype != torch.uint8:
        raise NativeError("gemm_layouts operands must be uint8 FP8 codes")
    a, b = _as_2d(a), _as_2d(b)
    M, K = (a.shape[1], a.shape[0]) if layout_a == K_SLOW else a.shape
    N, K2 = (b.shape[1], b.shape[0]) if layout_b == K_SLOW else b.shape
    if K != K2:
        raise NativeError(f"gemm_layouts: contraction sizes differ ({K} vs {K2})")
    _f32_dev(sa_inv, 1, "gemm_layouts sa_inv")
    _f32_dev(sb_inv, 1, "gemm_layouts sb_inv")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    elif out.shape != (M, N) or out.dtype not in (torch.bfloat16, torch.float32) or not out.is_contiguous():
        raise NativeError("gemm_layouts: `out` has the wrong shape / dtype / layout")
    splits = gemm_split_count(M, N, K, layout_a == K_SLOW or layout_b == K_SLOW) if gemm_layouts_supported(M, N, K, out.dtype) else 1
    if splits > 1 or accumulate:
        return _gemm_splitk(a, b, M, N, K, fmt_a, fmt_b, layout_a, layout_b, sa_inv, sb_inv, None, out, splits, accumulate)
    _check(load().odl_fp8_gemm_layouts(a.data_ptr(), b.data_ptr(), M, N, K, fmt_a, fmt_b, layout_a, layout_b, sa_inv.data_ptr(),
                                       sb_inv.data_ptr(), out.data_ptr(), _src_dtype(out), _stream()),
           "odl_fp8_gemm_layouts")
    return out


def delayed_update(history: torch.Tensor, scale: torch.Tensor, scale_inv: torch.Tensor, fmts: torch.Tensor,
                   margin: int = 0, algo: int = AMAX_MAX, amax_parts: torch.Tensor | None = None) -> None:
    """In place: history[H,R] fp32, scale[R], scale_inv[R] fp32, fmts[R] int32 (all on the GPU);
    amax_parts [R, AMAX_PARTS] (optional): partial maxima of this step, folded into history[0] and cleared."""
    if history.dim() != 2:
        raise NativeError("delayed_update: history must be [H, R]")
    H, R = history.shape
    delayed_update_raw(history, H, R, R, scale, scale_inv, fmts, margin, algo, amax_parts)


def delayed_update_raw(history: torch.Tensor, H: int, ld: int, R: int, scale: torch.Tensor, scale_inv: torch.Tensor,
                       fmts: torch.Tensor, margin: int, algo: int, amax_parts: torch.Tensor | None = None) -> None:
    """Same update on the first R roles of an arena whose rows are ld >= R wide."""
    if not (history.is_cuda and history.dtype == torch.float32 and history.is_contiguous() and history.numel() == H * ld):
        raise NativeError("delayed_update_raw: history must be a contiguous fp32 CUDA tensor of H*ld elements")
    for t, name in ((scale, "scale"), (scale_inv, "scale_inv")):
        if not (t.is_cuda and t.dtype == torch.float32 and t.is_contiguous() and t.numel() >= R):
            raise NativeError(f"delayed_update_raw: {name} must be a contiguous fp32 CUDA tensor with >= R entries")
    if not (fmts.is_cuda and fmts.dtype == torch.int32 and fmts.is_contiguous() and fmts.numel() >= R):
        raise NativeError("delayed_update_raw: fmts must be a contiguous int32 CUDA tensor with >= R entries")
    if amax_parts is not None and not (amax_parts.is_cuda and amax_parts.dtype == torch.float32 and amax_parts.is_contiguous()
                                       and amax_parts.numel() >= R * AMAX_PARTS):
        raise NativeError("delayed_update_raw: amax_parts must be a contiguous fp32 CUDA tensor with >= R * AMAX_PARTS entries")
    _check(load().odl_fp8_delayed_update(history.data_ptr(), H, R, ld, scale.data_ptr(), scale_inv.data_ptr(),
                                         fmts.data_ptr(), margin, algo,
                                         amax_parts.data_ptr() if amax_parts is not None else None, _stream()), "odl_fp8_delayed_update")


def gemm_variants() -> list[str]:
    L = load()
    return [L.odl_fp8_gemm_variant_name(i).decode() for i in range(L.odl_fp8_gemm_num_variants())]


def gemm_set_variant(variant: int) -> None:
    """Pin the GEMM kernel variant (-1: choose by shape) for calls made from THIS host thread.  A
    testing / tuning switch: it does not reach other threads, so the GEMMs that autograd's worker
    thread launches in a backward pass keep the automatic choice."""
    _check(load().odl_fp8_gemm_set_variant(variant), "odl_fp8_gemm_set_variant")
    _tls.forced_variant = variant


def gemm_set_clock_probe(records: torch.Tensor | None) -> None:
    """Measurement aid: the streaming GEMM launches that THIS host thread makes from now on record, in turn, into the
    rows of ``records`` (int64 [capacity, 4] on the GPU: shader-clock counter and 100 MHz counter on entry and exit of
    the kernel's first wave).  None switches it off."""
    if records is None:
        _check(load().odl_fp8_gemm_set_clock_probe(None, 0), "odl_fp8_gemm_set_clock_probe")
        return
    if not (records.is_cuda and records.dtype == torch.int64 and records.dim() == 2 and records.shape[1] == 4 and records.is_contiguous()):
        raise NativeError("gemm_set_clock_probe: records must be a contiguous int64 CUDA tensor of shape [capacity, 4]")
    _check(load().odl_fp8_gemm_set_clock_probe(records.data_ptr(), records.shape[0]), "odl_fp8_gemm_set_clock_probe")
