#!/usr/bin/env python3
"""Benchmark of the FP8 Linear path on one MI355X.

Workload (configuration 3 of the benchmark definition, `configs[2]`): the three Linears of a Llama-3-8B SwiGLU MLP,
forward + backward in FP8 with per-tensor dynamic scaling (E4M3 for activations
and weights, E5M2 for gradients), M = 8192 tokens:
    gate, up : X [8192, 4096]   W [14336, 4096]   dY [8192, 14336]
    down     : X [8192, 14336]  W [4096, 14336]   dY [8192, 4096]
One step = fwd + bwd of all three = 9 GEMMs (8.66 TFLOP) plus every amax, cast and
cast+transpose they need (x and w get a transposed FP8 copy for dgrad / wgrad; dY is cast
once and read by wgrad as stored), weights re-quantised each step as after an optimizer
step.  Inputs are synthetic, seeded, and resident in HBM before the clock starts.

Two passes over the same steps: the timed one (`value`, `ms_per_step`) has nothing
on the stream but the work itself; the second records a HIP event on the launch stream
after every native call, and a call's time runs from the previous call's event to its
own (`roofline`, `hbm_kernels`, `time_split_ms_per_step`: kernel + launch gap + one
event each, adding up to the step); the events cost about 2 % of a step, reported as
`ms_per_step_with_kernel_events`.

Prints ONE JSON line: whole-step TFLOP/s, the GEMM kernel's MFMA roofline
fraction, the HBM rates of the memory-bound kernels inside the step and on their own,
the clock and the board power under the GEMM (`clock_probe`, `power_probe`: the board's own sensor against its limit),
and the same arithmetic on the host CPU (the oracle, on a bounded sample) as a
reported baseline.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_FP8_TFLOPS = 5000.0     # MI355X dense FP8 MFMA, published
PEAK_HBM_GBPS = 8000.0       # MI355X HBM3E, published
# Memory-side bytes per GEMM launch come from a tracked data file that names the profiler runs behind it
GEMM_TRAFFIC_FILE = os.path.join(ROOT, "profiles", "gemm_traffic__cfg3_mlp.json")


def gemm_traffic_bytes_per_launch():
    """Mean over the launches of a step of (FETCH_SIZE x its scale + WRITE_SIZE x its scale), from the counter
    values recorded in profiles/gemm_traffic__cfg3_mlp.json; None when the file is not there."""
    try:
        with open(GEMM_TRAFFIC_FILE) as fh:
            t = json.load(fh)
    except OSError:
        return None, None
    n = sum(t["launches_per_step"].values())
    kib = sum(t["launches_per_step"][k] * (t["fetch_size_kib_per_dispatch"][k] * t["fetch_scale"] +
                                           t["write_size_kib_per_dispatch"][k] * t["write_scale"]) for k in t["launches_per_step"])
    return kib * 1024.0 / n, t["source"]


def profiled_kernel_durations():
    """Average kernel durations inside the step from the tracked rocprofv3 summary (kernel time only: no launch gap, no
    event), as recorded in profiles/step_kernel_durations__cfg3_mlp.json; ({}, None) when the file is not there."""
    try:
        with open(os.path.join(ROOT, "profiles", "step_kernel_durations__cfg3_mlp.json")) as fh:
            t = json.load(fh)
    except OSError:
        return {}, None
    return {k: v["avg_us"] for k, v in t["kernels"].items()}, t["source"]


M_TOKENS, D_MODEL, D_FF = 8192, 4096, 14336
LAYERS = (("gate", D_MODEL, D_FF), ("up", D_MODEL, D_FF), ("down", D_FF, D_MODEL))   # name, K(in), N(out)


def step_flops(m: int = M_TOKENS) -> float:
    return sum(6.0 * m * k * n for _, k, n in LAYERS)


class KernelTimer:
    """One HIP event after every native call, on the stream it is launched on (torch's current stream, which is the
    stream the library receives): a call's time runs from the event after the previous call to its own, so the figures
    of a step add up to the step and every launch carries one event, not two."""

    def __init__(self, native, torch):
        self.native, self.torch = native, torch
        self.records: dict[str, list] = {}
        self.enabled = False
        self._orig = {}
        self._last = None

    def start(self):
        self._last = self.torch.cuda.Event(enable_timing=True)
        self._last.record()
        self.enabled = True

    def install(self):
        def wrap(name, work_fn, record_as=None):
            record_as = record_as or name
            orig = getattr(self.native, name)
            self._orig[name] = orig

            def timed(*a, **kw):
                if not self.enabled:
                    return orig(*a, **kw)
                out = orig(*a, **kw)
                e0, e1 = self._last, self.torch.cuda.Event(enable_timing=True)
                e1.record()
                self._last = e1
                key = record_as(*a, **kw) if callable(record_as) else record_as
                self.records.setdefault(key, []).append((e0, e1, work_fn(*a, **kw)))
                return out

            setattr(self.native, name, timed)

        def esz(x):
            return x.element_size()

        wrap("gemm_nt", lambda a, b, *r, **kw: 2.0 * a.shape[0] * b.shape[0] * a.shape[1])            # flops
        # operands stored K-slow are [K, rows]: the product of both shapes is M * K * N * K either way
        wrap("gemm_layouts", lambda a, b, *r, **kw: 2.0 * a.numel() * b.numel() / (a.shape[0] if r[2] else a.shape[1]),
             record_as="gemm_nt")
        wrap("amax", lambda x, *r, **kw: float(x.numel() * esz(x)))                                       # bytes
        wrap("amax_scale", lambda x, *r, **kw: float(x.numel() * esz(x)), record_as="amax")       # amax + scale, one launch
        wrap("amax_parts", lambda x, *r, **kw: float(x.numel() * esz(x)), record_as="amax")
        wrap("cast_dynamic", lambda x, parts, fmt, margin=0, want_rowmajor=True, want_transposed=True, out_t=None:
             float(x.numel() * (esz(x) + int(want_rowmajor) + int(want_transposed or out_t is not None))),
             record_as=lambda x, parts, fmt, margin=0, want_rowmajor=True, want_transposed=True, out_t=None:
             "cast_transpose" if (want_transposed or out_t is not None) else "cast")
        wrap("cast", lambda x, *r, **kw: float(x.numel() * (esz(x) + 1)))
        wrap("cast_transpose",
             lambda x, *r, **kw: float(x.numel() * (esz(x) + (2 if kw.get("want_rowmajor", True) else 1))))

    def summary(self):
        out = {}
        for name, recs in self.records.items():
            ms = [e0.elapsed_time(e1) for e0, e1, _ in recs]
            work = [w for _, _, w in recs]
            out[name] = {"launches": len(recs), "total_ms": sum(ms), "avg_us": 1e3 * sum(ms) / len(ms), "work": sum(work)}
        return out


def weights_changed(module):
    """What an optimizer step does to the module's weight as far as the FP8 path can tell: the Parameter's version
    counter moves, so every cached quantisation of it (per module, per group of siblings, per parameter set) is out of
    date and the next forward quantises the weight again.  No kernel is launched for it."""
    import torch

    torch.autograd.graph.increment_version(module.weight)


def timed_steps(torch, one, steps, warmup):
    """`warmup` untimed calls of `one`, then `steps` timed ones.  ms_per_step is wall time over all of them (host clock,
    synchronised on both sides); min / median / max are per step, from one HIP event between consecutive steps, so a
    single slow step (an allocator that has to grow, a first-use set-up) shows up as max >> median instead of hiding in
    the mean.  host_issue_ms_per_step is the time the host took to queue the launches of the timed steps (close to
    ms_per_step: the host, not the GPU, sets the pace).  `allocator` tells whether torch's caching allocator had to go back
    to the driver during the timed steps."""
    t_w = time.perf_counter()
    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    # short steps: keep warming until the board has been busy for 50 ms.  After an idle spell it runs a handful of
    # launches at a high clock, then drops well below its sustained clock and takes some 10 ms to come back; a step of
    # 1 ms timed right after three warm-up steps sits in that transient (measured: 1.42, 1.24, 1.25 ... 1.13 ms)
    per_step = max((time.perf_counter() - t_w) / max(warmup, 1), 1e-4)
    extra = min(64, max(0, int(0.05 / per_step) - warmup))
    for _ in range(extra):
        one()
    torch.cuda.synchronize()
    before = torch.cuda.memory_stats()
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
    t0 = time.perf_counter()
    marks[0].record()
    for i in range(steps):
        one()
        marks[i + 1].record()
    issued = time.perf_counter() - t0          # the host has queued every launch; the GPU is still working
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    after = torch.cuda.memory_stats()
    in_order = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
    per = sorted(in_order)
    return {"ms_per_step": 1e3 * wall / steps, "host_issue_ms_per_step": 1e3 * issued / steps, "warmup_steps": warmup + extra, "min_ms": per[0], "median_ms": per[len(per) // 2], "max_ms": per[-1],
            "max_over_median": per[-1] / per[len(per) // 2], "slowest_step": in_order.index(per[-1]),
            "per_step_ms": [round(t, 3) for t in in_order],
            "allocator": {"segments_allocated_during_timed_steps": after.get("num_device_alloc", 0) - before.get("num_device_alloc", 0),
                          "alloc_retries_during_timed_steps": after.get("num_alloc_retries", 0) - before.get("num_alloc_retries", 0),
                          "reserved_mib_before": before.get("reserved_bytes.all.current", 0) >> 20,
                          "reserved_mib_after": after.get("reserved_bytes.all.current", 0) >> 20}}


def make_inputs(torch, m=M_TOKENS, device="cuda"):
    g = torch.Generator().manual_seed(0)
    data = {}
    for name, k, n in LAYERS:
        data[name] = {
            "x": torch.randn(m, k, generator=g).bfloat16().to(device),
            "w": (torch.randn(n, k, generator=g) * 0.02).bfloat16().to(device),
            "dy": (torch.randn(m, n, generator=g) * 1e-3).bfloat16().to(device),
        }
    return data


def power_probe(torch, native, step=None, seconds=1.5):
    """The board's own power reading (amdgpu hwmon `power1_input`, microwatts, a value the driver filters over a few
    tenths of a second; `power1_cap` is the limit it regulates to) while one kind of work runs back to back for
    `seconds`: the GEMM on Gaussian and on zero operands, the MXFP8 GEMM, the register-only MFMA loop, the three
    memory-bound kernels and (step given) whole steps of the benchmark.  Per workload: the mean of the readings of the last
    third of the run, the time per launch, and the energy per launch = watts x time (for the GEMM and the loop also
    per flop).  Read-only; {"sensor": None} where the file is not there."""
    import ctypes
    import glob
    import threading

    from bench_probe.build import PROBE_LIB_PATH

    sensors = sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/power1_input"))
    if not sensors:
        return {"sensor": None}
    # the card whose PCI address is that of the device the work runs on (a host may hold several boards)
    sensor, matched = sensors[0], len(sensors) == 1
    try:
        pr = torch.cuda.get_device_properties(torch.cuda.current_device())
        want = f"{pr.pci_domain_id:04x}:{pr.pci_bus_id:02x}:{pr.pci_device_id:02x}."
        for cand in sensors:
            pci = os.path.basename(os.path.realpath(os.path.join(os.path.dirname(cand), "..", "..")))
            if pci.startswith(want):
                sensor, matched = cand, True
                break
    except (AttributeError, OSError):
        pass

    def watts(path=sensor):
        try:
            with open(path) as fh:
                return int(fh.read()) / 1e6
        except (OSError, ValueError):
            return None

    if watts() is None:
        return {"sensor": None}
    out = {"sensor": sensor, "sensor_is_this_device": matched, "cap_w": watts(os.path.join(os.path.dirname(sensor), "power1_cap")), "seconds_per_workload": seconds,
           "workloads": {}}
    torch.cuda.synchronize()
    time.sleep(0.8)
    out["idle_w"] = round(watts(), 1)

    def run(label, fn, flop=None, burst=32):
        # the sensor is read by a second thread (a read takes the driver some 0.1 ms and must not sit between launches)
        reads, done = [], threading.Event()

        def sample():
            while not done.is_set():
                reads.append((time.perf_counter(), watts()))
                time.sleep(0.005)

        torch.cuda.synchronize()
        th = threading.Thread(target=sample, daemon=True)
        t0 = time.perf_counter()
        th.start()
        n = 0
        while time.perf_counter() - t0 < seconds:
            for _ in range(burst):
                fn()
            torch.cuda.synchronize()
            n += burst
        dt = time.perf_counter() - t0
        done.set()
        th.join()
        tail = [w for t, w in reads if t0 + 2.0 * seconds / 3.0 <= t <= t0 + dt and w is not None]
        w = sum(tail) / len(tail) if tail else None
        us = 1e6 * dt / n
        entry = {"watts": round(w, 1) if w is not None else None, "us_per_launch": round(us, 1), "launches": n,
                 "joules_per_launch": round(w * us * 1e-6, 4) if w is not None else None}
        if flop and w is not None:
            entry["pj_per_flop"] = round(w * us * 1e-6 / flop * 1e12, 4)
        out["workloads"][label] = entry
        time.sleep(0.5)          # the reading falls back towards idle before the next workload starts

    M, N, K = M_TOKENS, D_FF, D_MODEL
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn((M, K), generator=g, device="cuda").bfloat16()
    w = (torch.randn((N, K), generator=g, device="cuda") * 0.02).bfloat16()
    xq, _, _, _, sx = native.quantize_dynamic(x, native.E4M3, 0, want_transposed=False)
    wq, _, _, _, sw = native.quantize_dynamic(w, native.E4M3, 0, want_transposed=False)
    c = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    flop = 2.0 * M * N * K
    run("gemm_8192x14336x4096 gaussian_operands", lambda: native.gemm_nt(xq, wq, native.E4M3, native.E4M3, sx, sw, out=c), flop)
    zx, zw = torch.zeros_like(xq), torch.zeros_like(wq)
    run("gemm_8192x14336x4096 zero_operands", lambda: native.gemm_nt(zx, zw, native.E4M3, native.E4M3, sx, sw, out=c), flop)
    del zx, zw
    xm, xs, _, _ = native.mx_cast(x, native.E4M3)
    wm, ws, _, _ = native.mx_cast(w, native.E4M3)
    run("gemm_8192x14336x4096 mxfp8_gaussian_operands", lambda: native.mx_gemm_nt(xm, xs, wm, ws, native.E4M3, native.E4M3), flop)
    del xm, xs, wm, ws, xq, wq, c
    lib = ctypes.CDLL(PROBE_LIB_PATH)
    vp = ctypes.c_void_p
    lib.odl_probe_mfma_loop.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    sink = torch.zeros(1, device="cuda")
    cycles = torch.zeros((cus, 2), dtype=torch.int64, device="cuda")
    iters = 4000
    loop_flop = cus * 4 * iters * 16 * 2.0 * 32 * 32 * 64
    stream = torch.cuda.current_stream().cuda_stream
    for label, rnd in (("mfma_register_loop gaussian_like_operands", 1), ("mfma_register_loop zero_operands", 0)):
        run(label, lambda: lib.odl_probe_mfma_loop(rnd, iters, cus, sink.data_ptr(), cycles.data_ptr(), stream), loop_flop, burst=4)
    big = torch.randn((M_TOKENS, D_FF), generator=g, device="cuda").bfloat16()
    one = torch.ones(1, device="cuda")
    run("amax 8192x14336", lambda: native.amax_parts(big), burst=128)
    run("cast 8192x14336", lambda: native.cast(big, one, native.E5M2), burst=64)
    run("cast_transpose 8192x14336", lambda: native.cast_transpose(big, one, native.E4M3, want_rowmajor=True), burst=64)
    del big
    if step is not None:
        run("whole step (configs[2], tensorwise)", step, step_flops(), burst=4)
    return out


def standalone_hbm(torch, native, iters=24):
    """The memory-bound kernels on their own, on inputs that are not cache-resident: enough
    buffers per shape are walked round-robin to hold three times the 256 MB memory-side cache;
    HIP events around the whole batch, so the GPU's launch gaps are included.  A spin kernel of about a
    millisecond runs in front of every batch so that the host has queued all of it before the GPU starts on it
    (the Python wrappers take 10-20 us per call, more than the small kernels run).  Algorithmic bytes as in the step."""
    out = {}
    spin_cycles = 2_500_000
    # the last three shapes: norm rows of the small presets (per-head q / k norm of Qwen3, GPT-2 and Qwen3 model widths)
    for rows, cols in ((M_TOKENS, 4096), (14336, 4096), (M_TOKENS, 14336), (131072, 128), (16384, 768), (8192, 1024)):
        nbuf = max(4, -(-3 * 256 * 2**20 // (2 * rows * cols)))
        xs = [torch.randn((rows, cols), device="cuda", dtype=torch.bfloat16) for _ in range(nbuf)]
        _, scale, _ = native.amax_scale(xs[0], native.E4M3, 0)
        E = rows * cols
        if cols < 4096:
            w_norm = torch.ones(cols, device="cuda")
            _, rstd_b, _ = native.rmsnorm_amax_parts(xs[0], w_norm, 1e-5)
            _, mean_l, rstd_l, _ = native.layernorm_amax_parts(xs[0], w_norm, w_norm, 1e-5)
            dy_of = {id(x): xs[(i + 1) % nbuf] for i, x in enumerate(xs)}
            kernels = {
                "rmsnorm_amax_bf16_in": (lambda x: native.rmsnorm_amax_parts(x, w_norm, 1e-5), 4 * E),
                "rmsnorm_bwd_bf16": (lambda x: native.rmsnorm_bwd(dy_of[id(x)], x, w_norm, rstd_b), 6 * E),
            }
            if cols >= 768:                # LayerNorm runs over model widths (GPT-2), never over the 128 elements of a head
                kernels["layernorm_amax_bf16_in"] = (lambda x: native.layernorm_amax_parts(x, w_norm, w_norm, 1e-5), 4 * E)
                kernels["layernorm_bwd_bf16"] = (lambda x: native.layernorm_bwd(dy_of[id(x)], x, w_norm, mean_l, rstd_l), 6 * E)
        else:
            kernels = {
                "amax": (lambda x: native.amax_parts(x), 2 * E),
                "amax_rowwise": (lambda x: native.amax(x, native.SCALE_ROW), 2 * E + 4 * rows),
                "amax_and_column_sums": (lambda x: native.amax_parts_colsum(x), 2 * E + 4 * cols),
                "cast": (lambda x: native.cast(x, scale, native.E4M3, native.SCALE_TENSOR), 3 * E),
                "cast_transpose": (lambda x: native.cast_transpose(x, scale, native.E4M3, native.SCALE_TENSOR), 4 * E),
                "amax_then_cast_transpose": (lambda x: native.quantize_dynamic(x, native.E4M3, 0), 6 * E),
                # the block-scaled casts: codes in both layouts plus their scale bytes, no amax pass
                "mx_cast_both_layouts": (lambda x: native.mx_cast(x, native.E4M3, True, True), 4 * E + 2 * (E // 32)),
                "block_cast_1d_both_layouts": (lambda x: native.block_cast(x, native.E4M3, 0, False, True, True), 4 * E + 8 * (E // 128)),
            }
            if cols == D_MODEL and rows == M_TOKENS:   # fp32 sources (master weights, an fp32 residual stream)
                xs32c = [x.float() for x in xs]
                c32 = {id(x): y for x, y in zip(xs, xs32c)}
                kernels["cast_fp32_in"] = (lambda x: native.cast(c32[id(x)], scale, native.E4M3, native.SCALE_TENSOR), 5 * E)
                kernels["cast_transpose_fp32_in"] = (lambda x: native.cast_transpose(c32[id(x)], scale, native.E4M3, native.SCALE_TENSOR), 6 * E)
        if cols == D_FF:                   # the SwiGLU producers run on the [tokens, d_ff] activations
            nxt = {id(x): (xs[(i + 1) % nbuf], xs[(i + 2) % nbuf]) for i, x in enumerate(xs)}
            kernels["swiglu_fwd_amax"] = (lambda x: native.swiglu_amax_parts(x, nxt[id(x)][0]), 6 * E)
            kernels["swiglu_bwd_amax"] = (lambda x: native.swiglu_bwd_amax_parts(x, nxt[id(x)][0], nxt[id(x)][1]), 10 * E)
        if cols == D_MODEL and rows == M_TOKENS:   # RMSNorm in front of q/k/v and gate/up: bf16 and fp32 residual streams
            w_norm = torch.ones(cols, device="cuda")
            kernels["rmsnorm_amax_bf16_in"] = (lambda x: native.rmsnorm_amax_parts(x, w_norm, 1e-5), 4 * E)
            xs32 = [x.float() for x in xs]
            to32 = {id(x): y for x, y in zip(xs, xs32)}
            kernels["rmsnorm_amax_fp32_in"] = (lambda x: native.rmsnorm_amax_parts(to32[id(x)], w_norm, 1e-5), 6 * E)
            kernels["layernorm_amax_bf16_in"] = (lambda x: native.layernorm_amax_parts(x, w_norm, w_norm, 1e-5), 4 * E)
            kernels["gelu_fwd_amax"] = (lambda x: native.gelu_amax_parts(x), 4 * E)
            _, rstd_b, _ = native.rmsnorm_amax_parts(xs[0], w_norm, 1e-5)
            dy_of = {id(x): xs[(i + 1) % nbuf] for i, x in enumerate(xs)}
            kernels["rmsnorm_bwd_bf16"] = (lambda x: native.rmsnorm_bwd(dy_of[id(x)], x, w_norm, rstd_b), 6 * E)
            _, mean_l, rstd_l, _ = native.layernorm_amax_parts(xs[0], w_norm, w_norm, 1e-5)
            kernels["layernorm_bwd_bf16"] = (lambda x: native.layernorm_bwd(dy_of[id(x)], x, w_norm, mean_l, rstd_l), 6 * E)
            kernels["gelu_bwd_amax"] = (lambda x: native.gelu_bwd_amax_parts(dy_of[id(x)], x), 6 * E)
        for name, (fn, nbytes) in kernels.items():
            for x in xs:
                fn(x)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda._sleep(spin_cycles)        # the host queues the whole batch while the GPU spins: GPU time, not host time
            e0.record()
            for i in range(iters):
                fn(xs[i % nbuf])
            e1.record()
            torch.cuda.synchronize()
            us = 1e3 * e0.elapsed_time(e1) / iters
            gbps = nbytes / (us * 1e-6) / 1e9
            out.setdefault(name, {})[f"{rows}x{cols}"] = {"us": round(us, 1), "GB/s": round(gbps), "frac": round(gbps / PEAK_HBM_GBPS, 3)}
        del xs
    return out


def sibling_linears(torch, label, grouped, alone, m, steps=8, warmup=3):
    """Linears fed ONE X (``grouped``: name -> (in, out), names the transform ties into a sibling group) and Linears with
    an input of their own (``alone``), forward + backward of all, weights re-quantised every step.  The transform groups
    the former as it does in a model: X is quantised once, and their data gradients come out as one dX (one GEMM over
    all members' operands, or GEMMs that add into it)."""
    import torch.nn as nn

    from optimus_dl_amd.modules.amp import create_fp8_recipe
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    class Projections(nn.Module):
        def __init__(self):
            super().__init__()
            for name, (k, n) in {**grouped, **alone}.items():
                setattr(self, name, nn.Linear(k, n, bias=False))

        def forward(self, x, others):
            return [getattr(self, name)(x) for name in grouped] + [getattr(self, name)(o) for name, o in zip(alone, others)]

    g = torch.Generator().manual_seed(0)
    net = Projections().to("cuda", torch.bfloat16)
    with torch.no_grad():
        for p in net.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    build_model_transform({"_name": "fp8_linear"}).apply(net)
    recipe = create_fp8_recipe("tensorwise", "hybrid")
    k_in = next(iter(grouped.values()))[0]
    x = torch.randn(m, k_in, generator=g).bfloat16().cuda().requires_grad_(True)
    others = [torch.randn(m, k, generator=g).bfloat16().cuda().requires_grad_(True) for k, _ in alone.values()]
    mods = [getattr(net, name) for name in (*grouped, *alone)]
    dys = [(torch.randn(m, lin.out_features, generator=g) * 1e-3).bfloat16().cuda() for lin in mods]

    def one():
        for lin in mods:
            weights_changed(lin)
            lin.weight.grad = None
        x.grad = None
        for o in others:
            o.grad = None
        with recipe.autocast():
            ys = net(x, others)
        with recipe.backward():
            torch.autograd.backward(ys, dys)

    t = timed_steps(torch, one, steps, warmup)
    flop = sum(6.0 * m * lin.in_features * lin.out_features for lin in mods)
    res = {label: {**t, "TFLOP/s": flop / (t["ms_per_step"] * 1e-3) / 1e12, "flop_per_step": flop}}
    del net, x, others, dys, one
    torch.cuda.empty_cache()
    return res


def attention_projections(torch, steps=8, warmup=3):
    """configs[1] of BASELINE.json as it is written: ONE X [8192, 4096] feeds Wq [4096, 4096], Wk and Wv [1024, 4096]
    (optimus_dl/modules/model/blocks/attention.py:317-319), Wo [4096, 4096] has an input of its own."""
    return sibling_linears(torch, "configs[1] attention projections, tensorwise",
                           {"wq": (4096, 4096), "wk": (4096, 1024), "wv": (4096, 1024)}, {"wo": (4096, 4096)}, 8192, steps, warmup)


def mlp_one_input(torch, steps=8, warmup=3):
    """configs[2] with W_gate and W_up fed the ONE X that BASELINE.json names (optimus_dl/modules/model/blocks/mlp.py:76-78
    feeds w1 and w2 the same tensor); W_down has an input of its own, as in the headline.  Same GEMM work as the
    headline step, which gives every Linear an X of its own: one quantisation of X less, and one dX instead of two."""
    return sibling_linears(torch, "configs[2] with gate and up fed one X (a sibling group)",
                           {"w1": (D_MODEL, D_FF), "w2": (D_MODEL, D_FF)}, {"c_proj": (D_FF, D_MODEL)}, M_TOKENS, steps, warmup)


def other_configs(torch, steps=8, warmup=3, only=""):
    """Whole steps (forward + backward of every Linear, weights re-quantised every step) of the other
    configurations of BASELINE.json and of configuration 3 with fp32 master weights (the reference's
    usual AMP set-up: the weight gradient is then fp32).  Same harness as the headline, fewer steps."""
    from optimus_dl_amd.modules.amp import create_fp8_recipe
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    cases = [
        ("configs[1] attention projections, tensorwise", "tensorwise", {}, [(4096, 4096), (4096, 1024), (4096, 1024), (4096, 4096)], 8192, torch.bfloat16),
        ("configs[2] with fp32 master weights", "tensorwise", {}, [(k, n) for _, k, n in LAYERS], M_TOKENS, torch.float32),
        ("configs[2] under delayed scaling (history 16; the reference's default recipe)", "delayed", {"amax_history_len": 16}, [(k, n) for _, k, n in LAYERS], M_TOKENS, torch.bfloat16),
        ("configs[2] under mxfp8 (32-element blocks, E8M0 scales, scaled MFMA)", "mxfp8", {}, [(k, n) for _, k, n in LAYERS], M_TOKENS, torch.bfloat16),
        ("configs[2] under blockwise (1x128 / 128x128 blocks, power-of-two scales, scaled MFMA)", "blockwise", {}, [(k, n) for _, k, n in LAYERS], M_TOKENS, torch.bfloat16),
        ("configs[3] rowwise, M=16384", "rowwise", {}, [(4096, 14336)], 16384, torch.bfloat16),
        ("configs[4] delayed H=16, Llama-3-70B MLP up/down", "delayed", {"amax_history_len": 16}, [(8192, 28672), (28672, 8192)], 8192, torch.bfloat16),
    ]
    out = {}
    if not only or only in "configs[1] attention projections, tensorwise":
        out.update(attention_projections(torch, steps, warmup))
    if not only or only in "configs[2] with gate and up fed one X (a sibling group)":
        out.update(mlp_one_input(torch, steps, warmup))
    for label, kind, kw, shapes, m, wdtype in cases:
        if only and only not in label:
            continue
        if label.startswith("configs[1]"):
            label += ", as four independent Linears (an X each)"
        recipe = create_fp8_recipe(kind, "hybrid", **kw)
        g = torch.Generator().manual_seed(0)
        mods, xs, dys = [], [], []
        for k, n in shapes:
            lin = FP8Linear(k, n, bias=False, device="cuda", dtype=wdtype)
            with torch.no_grad():
                lin.weight.copy_((torch.randn(n, k, generator=g) * 0.02).to(wdtype))
            mods.append(lin)
            xs.append(torch.randn(m, k, generator=g).bfloat16().cuda().requires_grad_(True))
            dys.append((torch.randn(m, n, generator=g) * 1e-3).bfloat16().cuda())

        def one():
            for lin, x, dy in zip(mods, xs, dys):
                weights_changed(lin)
                lin.weight.grad = None
                x.grad = None
                with recipe.autocast():
                    y = lin(x)
                with recipe.backward():
                    y.backward(dy)

        t = timed_steps(torch, one, steps, warmup)
        flop = sum(6.0 * m * k * n for k, n in shapes)
        out[label] = {**t, "TFLOP/s": flop / (t["ms_per_step"] * 1e-3) / 1e12, "flop_per_step": flop}
        del mods, xs, dys, one
        torch.cuda.empty_cache()
    return out


def mlp_block(torch, native, recipe, steps=10, warmup=3):
    """The same three Linears wired as the MLP they come from (optimus_dl/modules/model/blocks/mlp.py:73-78):
    c_proj(silu(w1 x) * w2 x), forward + backward, weights re-quantised every step; once with the fused
    activation (which also spares the amax passes over h, d_gate, d_up) and once with PyTorch's."""
    from optimus_dl_amd.modules.model.blocks import SwiGLUMLP
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    out = {}
    g = torch.Generator().manual_seed(1)
    x = torch.randn(M_TOKENS, D_MODEL, generator=g).bfloat16().cuda().requires_grad_(True)
    dy = (torch.randn(M_TOKENS, D_MODEL, generator=g) * 1e-3).bfloat16().cuda()
    for label, fuse in (("fused_activation", True), ("pytorch_activation", False)):
        torch.manual_seed(0)
        mlp = SwiGLUMLP(D_MODEL, D_FF).to("cuda", torch.bfloat16)
        build_model_transform({"_name": "fp8_linear", "fuse_swiglu": fuse}).apply(mlp)

        def one():
            for lin in (mlp.w1, mlp.w2, mlp.c_proj):
                weights_changed(lin)
                lin.weight.grad = None
            x.grad = None
            with recipe.autocast():
                y = mlp(x)
            with recipe.backward():
                y.backward(dy)

        t = timed_steps(torch, one, steps, warmup)
        out[label] = {**t, "TFLOP/s": step_flops() / (t["ms_per_step"] * 1e-3) / 1e12}
        del mlp, one
        torch.cuda.empty_cache()
    return out


def llama_block(torch, steps=12, warmup=4):
    """One Llama-3-8B decoder block (RMSNorm, GQA attention with 32 / 8 heads, SwiGLU MLP; fp32 residual stream,
    batch 4 x 2048 tokens), forward + backward, weights re-quantised every step: bf16 autocast, FP8 Linears alone, and FP8
    Linears with the fused RMSNorm / SwiGLU producers.  Attention itself is PyTorch's scaled_dot_product_attention in all three."""
    from optimus_dl_amd.modules import amp as A
    from optimus_dl_amd.modules.model.blocks import LlamaBlock
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    B, T = 4, 2048
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(B, T, D_MODEL, device="cuda", generator=gen).requires_grad_(True)
    dy = torch.randn(B, T, D_MODEL, device="cuda", generator=gen) * 1e-3
    out = {}
    for label, cfg in (("bf16_autocast", None),
                       ("fp8_linears", {"_name": "fp8_linear", "replace_norm": False, "fuse_swiglu": False}),
                       ("fp8_linears_fused_norm_swiglu", {"_name": "fp8_linear"})):
        torch.manual_seed(0)
        blk = LlamaBlock(D_MODEL, 32, 8, D_FF).cuda()
        if cfg:
            build_model_transform(cfg).apply(blk)
        recipe = A.FP8Recipe(recipe_type="tensorwise")

        def one():
            for p_ in blk.parameters():
                p_.grad = None
            x.grad = None
            for m in blk.modules():
                if hasattr(m, "_wcache"):
                    weights_changed(m)
            if cfg:
                with A.fp8_autocast(torch.device("cuda"), recipe):
                    y = blk(x)
                with A.fp8_backward(recipe):
                    y.backward(dy)
            else:
                with torch.autocast("cuda", dtype=torch.bfloat16):
                    y = blk(x)
                y.backward(dy)

        out[label] = timed_steps(torch, one, steps, warmup)
        del blk, one, recipe
        torch.cuda.empty_cache()
    return out


def whole_models(torch, which=("gpt2_124m", "qwen3_0.6b"), steps=5, warmup=3, labels=None, recipe_type="tensorwise"):
    """The reference's own small presets as whole models (GPT-2 124M at 16 x 1024 tokens, Qwen3-0.6B at 4 x 2048;
    fp32 master weights, random init, random tokens): forward + cross-entropy + backward, weights re-quantised every
    step.  bf16 autocast, the FP8 Linears alone, the default transform (fused norms / activations as well), and the same
    with the weights quantised by the `fp8.param` set (two launches per step for all of them); attention and the loss are
    PyTorch's in all four."""
    import torch.nn.functional as F

    from optimus_dl_amd.modules import amp as A
    from optimus_dl_amd.modules.model.families import GPT2, GPT2Config, Qwen3, Qwen3Config
    from optimus_dl_amd.modules.model_transforms import build_model_transform

    def make(name):
        torch.manual_seed(0)
        if name == "gpt2_124m":
            return GPT2(GPT2Config(n_layer=12)), 16, 1024, 50304
        return Qwen3(Qwen3Config(vocab_size=151936, n_layer=28, n_head=16, n_kv_head=8, n_embd=1024, head_dim=128,
                                 intermediate_size=3072)), 4, 2048, 151936

    out = {}
    for name in which:
        out[name] = {}
        for label, cfg in (("bf16_autocast", None),
                           ("fp8_linears", {"_name": "fp8_linear", "replace_norm": False, "fuse_swiglu": False, "fuse_gelu": False}),
                           ("fp8_linears_fused_producers", {"_name": "fp8_linear"}),
                           ("fp8_linears_fused_producers_param_set", {"_name": "fp8_linear"})):
            if labels is not None and label not in labels:
                continue
            model, B, T, V = make(name)
            model = model.cuda()
            if cfg:
                build_model_transform(cfg).apply(model)
            recipe = A.FP8Recipe(recipe_type=recipe_type)
            # `fp8.param`: all weights re-quantised in two launches per step instead of two per weight
            param_set = recipe.attach_params(model) if label.endswith("param_set") else None
            ids = torch.randint(0, V, (B, T), device="cuda")
            tgt = torch.randint(0, V, (B * T,), device="cuda")

            def one():
                for p_ in model.parameters():
                    p_.grad = None
                if param_set is not None:
                    param_set.sync()                 # where the optimizer step's hook would run it
                else:
                    for m in model.modules():
                        if hasattr(m, "_wcache"):
                            weights_changed(m)
                if cfg:
                    with A.fp8_autocast(torch.device("cuda"), recipe):
                        loss = F.cross_entropy(model(ids)["logits"].view(-1, V).float(), tgt)
                    with A.fp8_backward(recipe):
                        loss.backward()
                else:
                    with torch.autocast("cuda", dtype=torch.bfloat16):
                        loss = F.cross_entropy(model(ids)["logits"].view(-1, V).float(), tgt)
                    loss.backward()

            t = timed_steps(torch, one, steps, warmup)
            out[name][label] = {**t, "tokens_per_s": B * T / (t["ms_per_step"] * 1e-3)}
            del model, one, param_set, recipe
            torch.cuda.empty_cache()
    return out


def clock_probe(torch, native, launches=20, settle=40):
    """What clock the board grants while the matrix pipe is busy, and what the pipe delivers at that clock.

    (1) The forward GEMM of the gate projection (8192 x 14336 x 4096) back to back, once on operands quantised from
    Gaussian data and once on all-zero codes: time per launch, TFLOP/s, and the shader clock during the launches (the
    kernel's first wave reads the shader-clock counter and the constant 100 MHz counter on entry and on exit:
    `odl_fp8_gemm_set_clock_probe`).  (2) The same MFMA instruction in a register-only loop (one wave per SIMD on every compute unit, no
    memory traffic), zero and Gaussian-like operands: rate and clock.  `of_peak_at_clock` prices a rate against
    CUs x 8192 flop per clock x the measured clock instead of the nominal 2.4 GHz.
    Every measurement follows `settle` launches of the same work: from idle the board runs a handful of launches
    at a high clock, then drops well below its sustained clock and takes some 30 launches (10 ms) to come back."""
    import ctypes

    from bench_probe.build import PROBE_LIB_PATH

    lib = ctypes.CDLL(PROBE_LIB_PATH)                      # built in-tree by bench_probe/build.py
    vp = ctypes.c_void_p
    lib.odl_probe_mfma_loop.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp]
    lib.odl_probe_mfma_loop_scaled.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp]
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    flop_per_clock = cus * 8192.0                          # dense FP8 MFMA: 4 SIMDs x (2 x 32 x 32 x 64 flop / 64 clocks) per CU

    def stream():
        return torch.cuda.current_stream().cuda_stream

    def priced(tflops, mhz):
        return {"TFLOP/s": round(tflops, 1), "shader_clock_mhz": round(mhz), "of_nominal_peak": round(tflops / PEAK_FP8_TFLOPS, 3),
                "of_peak_at_clock": round(tflops * 1e12 / (flop_per_clock * mhz * 1e6), 3)}

    out = {"compute_units": cus, "flop_per_clock": flop_per_clock, "gemm_8192x14336x4096": {}, "mfma_register_loop": {}}
    M, N, K = M_TOKENS, D_FF, D_MODEL
    g = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn((M, K), generator=g, device="cuda").bfloat16()
    w = (torch.randn((N, K), generator=g, device="cuda") * 0.02).bfloat16()
    xq, _, _, _, sx = native.quantize_dynamic(x, native.E4M3, 0, want_transposed=False)
    wq, _, _, _, sw = native.quantize_dynamic(w, native.E4M3, 0, want_transposed=False)
    c = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
    records = torch.zeros((launches, 4), dtype=torch.int64, device="cuda")     # per launch: clocks and 100 MHz ticks, entry and exit
    for label, a, b in (("gaussian_operands", xq, wq), ("zero_operands", torch.zeros_like(xq), torch.zeros_like(wq))):
        for _ in range(settle):
            native.gemm_nt(a, b, native.E4M3, native.E4M3, sx, sw, out=c)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        native.gemm_set_clock_probe(records)
        e0.record()
        for _ in range(launches):
            native.gemm_nt(a, b, native.E4M3, native.E4M3, sx, sw, out=c)
        e1.record()
        native.gemm_set_clock_probe(None)
        torch.cuda.synchronize()
        r = records.double()
        mhz = float((100.0 * (r[:, 2] - r[:, 0]) / (r[:, 3] - r[:, 1])).mean())     # counters read by one wave inside each launch
        us = 1e3 * e0.elapsed_time(e1) / launches
        entry = priced(2.0 * M * N * K / (us * 1e-6) / 1e12, mhz)
        entry["us_per_launch"] = round(us, 1)
        out["gemm_8192x14336x4096"][label] = entry
    # the same product under MXFP8 (block scales applied by the MFMA, scale dwords fetched beside the operands)
    xm, xs, _, _ = native.mx_cast(x, native.E4M3)
    wm, ws, _, _ = native.mx_cast(w, native.E4M3)
    for _ in range(settle):
        native.mx_gemm_nt(xm, xs, wm, ws, native.E4M3, native.E4M3)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    native.gemm_set_clock_probe(records)
    e0.record()
    for _ in range(launches):
        native.mx_gemm_nt(xm, xs, wm, ws, native.E4M3, native.E4M3)
    e1.record()
    native.gemm_set_clock_probe(None)
    torch.cuda.synchronize()
    r = records.double()
    mhz = float((100.0 * (r[:, 2] - r[:, 0]) / (r[:, 3] - r[:, 1])).mean())
    us = 1e3 * e0.elapsed_time(e1) / launches
    entry = priced(2.0 * M * N * K / (us * 1e-6) / 1e12, mhz)
    entry["us_per_launch"] = round(us, 1)
    out["gemm_8192x14336x4096"]["mxfp8_gaussian_operands"] = entry
    del xm, xs, wm, ws
    sink = torch.zeros(1, device="cuda")
    cycles = torch.zeros((cus, 2), dtype=torch.int64, device="cuda")
    iters = 4000                                           # x 16 MFMAs x 64 clocks: about 2 ms per launch
    for label, rnd, loop in (("gaussian_like_operands", 1, lib.odl_probe_mfma_loop), ("zero_operands", 0, lib.odl_probe_mfma_loop),
                             ("block_scaled_gaussian_like_operands", 1, lib.odl_probe_mfma_loop_scaled)):
        for _ in range(settle // 4):
            loop(rnd, iters, cus, sink.data_ptr(), cycles.data_ptr(), stream())
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(4):
            loop(rnd, iters, cus, sink.data_ptr(), cycles.data_ptr(), stream())
        e1.record()
        torch.cuda.synchronize()
        us = 1e3 * e0.elapsed_time(e1) / 4
        cyc = cycles.double()
        mhz = float((100.0 * cyc[:, 0] / cyc[:, 1]).median())
        entry = priced(cus * 4 * iters * 16 * 2.0 * 32 * 32 * 64 / (us * 1e-6) / 1e12, mhz)
        entry["us_per_launch"] = round(us, 1)
        entry["clocks_per_mfma"] = round(float(cyc[:, 0].median()) / (iters * 16), 2)
        out["mfma_register_loop"][label] = entry
    return out


def cpu_baseline(torch, seconds_hint=20.0):
    """The oracle's emulated-FP8 Linear fwd+bwd on the host cores, on a slice of the rows."""
    from oracle import oracle as O

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    m = 4096
    data = make_inputs(torch, m=m, device="cpu")
    passes, dt = 0, 0.0
    while dt < 10.0 and passes < 8:          # about 10-15 s of CPU work on the GPU box's host share
        t0 = time.perf_counter()
        for name, k, n in LAYERS:
            d = data[name]
            O.linear_fwd_bwd(d["x"], d["w"], d["dy"], O.E4M3, O.E5M2)
        dt += time.perf_counter() - t0
        passes += 1
    return {
        "value": passes * step_flops(m) / dt / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"rows 0..{m - 1} of {M_TOKENS} (all three Linears, fwd+bwd incl. amax/cast), {passes} passes in {dt:.1f} s; "
                  "torch CPU float8 cast + fp32 matmul",
        "seconds": dt,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (for profiler runs)")
    ap.add_argument("--no-standalone", action="store_true",
                    help="skip the stand-alone measurements of the memory-bound kernels (keeps profiler traces to the steps)")
    ap.add_argument("--standalone-only", action="store_true",
                    help="run only the stand-alone measurements of the memory-bound kernels and print them (for profiling)")
    ap.add_argument("--whole-models-only", default="",
                    help="run only the whole-model step of gpt2_124m or qwen3_0.6b with the default transform and print it (for profiling)")
    ap.add_argument("--recipe", default="tensorwise",
                    help="with --whole-models-only: the scaling recipe (tensorwise, delayed, rowwise, mxfp8, blockwise)")
    ap.add_argument("--llama-block-only", action="store_true",
                    help="run only the Llama-3-8B decoder block (bf16 autocast, FP8 Linears, FP8 Linears + fused producers) and print it (for profiling)")
    ap.add_argument("--other-configs-only", default="",
                    help="run only the whole steps of the other configurations whose label contains this text (e.g. mxfp8, rowwise, "
                         "delayed) and print them (for profiling)")
    ap.add_argument("--no-dgrad-sum-fusion", action="store_true",
                    help="leave the data-gradient sums of Linears fed by one tensor (q/k/v, gate/up) to autograd instead of the "
                         "GEMMs' accumulate flag (FP8Recipe.fuse_dgrad_sum = False), for A/B traces")
    ap.add_argument("--dgrad-sum-by-accumulate", action="store_true",
                    help="sum those data gradients with the GEMMs' accumulate flag only, not by one GEMM over all members' "
                         "operands (FP8Recipe.fuse_dgrad_gemm = False), for A/B traces")
    ap.add_argument("--clock-probe-only", action="store_true",
                    help="run only the clock probe (GEMM back to back on Gaussian / zero operands, register-only MFMA loop) and print it")
    ap.add_argument("--power-probe-only", action="store_true",
                    help="run only the board-power probe (GEMM, MFMA loop, memory-bound kernels, whole steps back to back) and print it")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 256 MiB device copy (reference kernel for scaling FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU; --gpus {args.gpus} is not supported "
              "(no collectives are part of the FP8 Linear path).", file=sys.stderr)
        return 2

    import torch

    from optimus_dl_amd import native
    from optimus_dl_amd.modules.amp import create_fp8_recipe
    from optimus_dl_amd.modules.fp8_linear import FP8Linear

    native.load()   # raises if the HIP library is missing: there is no fallback
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    if args.standalone_only:
        print(json.dumps({"hbm_kernels_standalone": standalone_hbm(torch, native)}))
        return 0
    if args.clock_probe_only:
        print(json.dumps({"clock_probe": clock_probe(torch, native)}))
        return 0
    if args.no_dgrad_sum_fusion or args.dgrad_sum_by_accumulate:
        from optimus_dl_amd.modules.amp import fp8 as _fp8

        _recipe_init = _fp8.FP8Recipe.__init__

        def _init_without_fusion(self, *a, **k):
            _recipe_init(self, *a, **k)
            self.fuse_dgrad_sum = not args.no_dgrad_sum_fusion
            self.fuse_dgrad_gemm = not args.dgrad_sum_by_accumulate

        _fp8.FP8Recipe.__init__ = _init_without_fusion
    if args.llama_block_only:
        print(json.dumps({"llama3_8b_block_fwd_bwd": llama_block(torch, steps=args.steps)}))
        return 0
    if args.other_configs_only:
        print(json.dumps({"other_configs_fwd_bwd": other_configs(torch, steps=args.steps, only=args.other_configs_only)}))
        return 0
    if args.whole_models_only:
        print(json.dumps({"whole_models_fwd_bwd": whole_models(torch, which=(args.whole_models_only,), steps=args.steps,
                                                                   labels=("fp8_linears_fused_producers",), recipe_type=args.recipe),
                          "recipe": args.recipe}))
        return 0
    dev = "cuda"
    data = make_inputs(torch, device=dev)
    recipe = create_fp8_recipe("tensorwise", "hybrid")
    layers = {}
    for name, k, n in LAYERS:
        lin = torch.nn.Linear(k, n, bias=False, device=dev, dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.copy_(data[name]["w"])
        layers[name] = FP8Linear.from_linear(lin)
        data[name]["x"].requires_grad_(True)

    timer = KernelTimer(native, torch)
    timer.install()

    def one_step():
        for name, _, _ in LAYERS:
            lin, d = layers[name], data[name]
            weights_changed(lin)              # weights change every optimizer step: re-quantise them every step
            lin.weight.grad = None
            d["x"].grad = None
            with recipe.autocast():
                y = lin(d["x"])
            with recipe.backward():
                y.backward(d["dy"])

    if args.copy_calibration:
        src = torch.empty(256 * 1024 * 1024, dtype=torch.uint8, device=dev).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        del src, dst
    for _ in range(args.warmup):
        one_step()
    torch.cuda.synchronize()
    if args.power_probe_only:
        print(json.dumps({"power_probe": power_probe(torch, native, step=one_step)}))
        return 0
    # the timed region: exactly `steps` steps, nothing else on the stream
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    # the same steps again with a HIP event after every native call (per-kernel figures)
    timer.start()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_step()
    torch.cuda.synchronize()
    wall_instrumented = time.perf_counter() - t0
    timer.enabled = False

    ks = timer.summary()
    ms_per_step = 1e3 * wall / args.steps
    tflops = step_flops() / (wall / args.steps) / 1e12
    gemm = ks["gemm_nt"]
    gemm_tflops = gemm["work"] / (gemm["total_ms"] * 1e-3) / 1e12
    hbm = {}
    for name in ("amax", "cast", "cast_transpose"):
        if name in ks:
            gbps = ks[name]["work"] / (ks[name]["total_ms"] * 1e-3) / 1e9
            hbm[name] = {"achieved": gbps, "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": gbps / PEAK_HBM_GBPS,
                         "avg_us": ks[name]["avg_us"], "launches": ks[name]["launches"]}
    # for orientation, what the same kernels took inside the step in the tracked rocprofv3 run (kernel time only: no launch
    # gap, no event).  These are CONSTANTS read from a committed file, made on another box at another time; nothing in
    # `tracked_profile_reference` is measured by this run, and no figure of this run is derived from it.
    prof_us, prof_src = profiled_kernel_durations()
    tracked_reference = None
    if prof_us:
        tracked_reference = {"not_measured_by_this_run": True, "source": prof_src, "kernel_avg_us": {}}
        for name in hbm:
            if name in prof_us:
                per_launch = ks[name]["work"] / ks[name]["launches"]
                tracked_reference["kernel_avg_us"][name] = {"avg_us": prof_us[name],
                                                            "frac_of_hbm_peak_at_this_run_s_bytes": per_launch / (prof_us[name] * 1e-6) / 1e9 / PEAK_HBM_GBPS}
    quant_bytes = sum(ks[n]["work"] for n in ("amax", "cast", "cast_transpose") if n in ks)
    quant_ms = sum(ks[n]["total_ms"] for n in ("amax", "cast", "cast_transpose") if n in ks)

    line = {
        "metric": "fp8 Linear fwd+bwd TFLOP/s (Llama-3-8B MLP, M=8192) + cast/amax HBM GB/s",
        "value": tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8 (e4m3 x/w, e5m2 grads; fp32 accumulate; bf16 out)",
        "data": "synthetic",
        "config": {
            "workload": "configs[2] of BASELINE.json: Llama-3-8B SwiGLU MLP Linears (gate, up [14336x4096]; down [4096x14336]), "
                        "M=8192, FP8 fwd+bwd, per-tensor dynamic scaling, fused cast+transpose of x and w, dY read by wgrad as stored",
            "flop_per_step": step_flops(),
            "gemms_per_step": 9,
            "gemm_variant": "auto",
        },
        "frac_of_fp8_peak": tflops / PEAK_FP8_TFLOPS,
        "gemm_only_tflops": gemm_tflops,
        "cast_amax_gbps": quant_bytes / (quant_ms * 1e-3) / 1e9 if quant_ms else None,
        "cast_amax_frac_of_hbm_peak": (quant_bytes / (quant_ms * 1e-3) / 1e9) / PEAK_HBM_GBPS if quant_ms else None,
        "tracked_profile_reference": tracked_reference,
        "time_split_ms_per_step": {n: ks[n]["total_ms"] / args.steps for n in ks},
        "ms_per_step_with_kernel_events": 1e3 * wall_instrumented / args.steps,
        "roofline": {
            "kernel": "gemm_nt_stream_kernel (FP8 MFMA GEMM; fwd, dgrad, wgrad launches)",
            "bound": "mfma",
            "achieved": gemm_tflops,
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": gemm_tflops / PEAK_FP8_TFLOPS,
            "traffic": gemm_traffic_bytes_per_launch()[0],
            "traffic_unit": "bytes per launch (FETCH_SIZE + WRITE_SIZE counters, measured separately)",
            "traffic_source": gemm_traffic_bytes_per_launch()[1],
            "algorithmic_bytes": (sum(m_ * k_ + n_ * k_ + 2 * m_ * n_ for m_, n_, k_ in
                                      [(M_TOKENS, n, k) for _, k, n in LAYERS] + [(M_TOKENS, k, n) for _, k, n in LAYERS] +
                                      [(n, k, M_TOKENS) for _, k, n in LAYERS]) / 9.0),
            "avg_launch_us": gemm["avg_us"],
            "launches": gemm["launches"],
        },
        "hbm_kernels": hbm,
    }
    if not args.no_standalone:
        line["clock_probe"] = clock_probe(torch, native)
        # the same GEMM back to back with the clock measured: what the roofline fraction is at the clock the board grants
        line["roofline"]["granted_clock"] = line["clock_probe"]["gemm_8192x14336x4096"]["gaussian_operands"]
        line["hbm_kernels_standalone"] = standalone_hbm(torch, native)
        # what the board draws under each kind of work, against the limit it regulates to
        line["power_probe"] = power_probe(torch, native, step=one_step)
    if not args.no_standalone:
        del layers, data
        line["mlp_block_fwd_bwd"] = mlp_block(torch, native, recipe)
        line["llama3_8b_block_fwd_bwd"] = llama_block(torch)
        line["other_configs_fwd_bwd"] = other_configs(torch)
        line["whole_models_fwd_bwd"] = whole_models(torch)
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch)
    # processes this run started that are still alive (none are expected: nothing here forks or spawns)
    try:
        import psutil

        line["child_processes_at_exit"] = [" ".join(c.cmdline()[:4]) or c.name() for c in psutil.Process().children(recursive=True)]
    except Exception as exc:  # psutil missing or /proc unreadable: say so, the figures above do not depend on it
        line["child_processes_at_exit"] = f"unknown ({type(exc).__name__})"
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
