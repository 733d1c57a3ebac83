#!/usr/bin/env python3
"""Benchmark of the gfx950 backend on BASELINE.json's headline workload.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only sdpa|chains|gemm|f32|survey]

A step is one pass of the hot path over one batch of synthetic input already
resident in HBM: causal bf16 scaled-dot-product attention, B=4 H=32 S=4096
D=128 (BASELINE.json configs[3], the configuration the metric is quoted on).
Prints ONE JSON line.  `value` is TFLOP/s over the algorithmic FLOP count
4*B*H*S^2*D/2.  The same line carries the roofline of the SDPA kernel, the
fused-chain kernels' achieved HBM bandwidth (configs[1] and configs[2]), the
MFMA GEMM behind nn::Linear, the timings of the C++ host layer and a
CPU baseline (the oracle's restatement of Axiom's CPU algorithm, timed on this
host on a bounded sample).

The defaults (50 warm-up, 200 timed launches per kernel) are sized for the device's clock
governor: coming from idle the first ~20 ms of MFMA work run at reduced clocks (the same SDPA
launch measures ~650 us in a 5+20 run and ~550 us from the 50th launch on), so a short run
reports the ramp, not the kernel.  Every kernel is therefore warmed up for at least 100 ms.

Everything runs on ONE GPU; --gpus above 1 is refused.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E
# HBM bytes per launch, measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and scaled by a copy kernel of known size:
# read from the committed summary of those runs (a table whose rows start with the workload's key in backticks and end
# with the bytes per launch); a workload the summary does not hold reports null
TRAFFIC_PROFILE = ROOT / "profiles" / "bench_kernels_hbm_traffic.md"


def traffic_from_profile() -> dict:
    out = {}
    if not TRAFFIC_PROFILE.exists():
        return out
    for ln in TRAFFIC_PROFILE.read_text().splitlines():
        cells = [c.strip() for c in ln.strip().strip("|").split("|")]
        if len(cells) >= 3 and cells[0].startswith("`") and cells[0].endswith("`"):
            try:
                out[cells[0].strip("`")] = float(cells[-1].replace(" ", ""))
            except ValueError:
                pass
    return out


MIN_WARMUP_MS = 100.0  # clocks and power settle within about this much work of one kind ...
MAX_SETTLE_MS = 1500.0  # ... but a leg that follows a very different one can take longer: see time_launches


def time_launches(torch, stream, launch, steps: int, warmup: int):
    """(average launch duration in ms over exactly `steps` launches, shortest single launch in ms, number of
    warm-up launches that ran before the timed region).  The average is the time between two HIP events on `stream`
    that bracket the `steps` launches; the shortest launch comes from a second, untimed round with an event after
    every launch.  Warm-up: `warmup` launches, continued until MIN_WARMUP_MS of work has run (short kernels would
    otherwise be timed while the device is still changing clocks), then batches of launches until two consecutive
    batches agree within 1 % (at most MAX_SETTLE_MS): the figure is the steady state of this kernel, not the tail of
    the previous leg's power state."""
    ran = 0
    with torch.cuda.stream(stream):
        t0 = time.time()
        for _ in range(warmup):
            launch()
        ran += warmup
        stream.synchronize()
        spent_ms = (time.time() - t0) * 1e3
        if warmup > 0 and spent_ms < MIN_WARMUP_MS:
            more = int((MIN_WARMUP_MS - spent_ms) / (spent_ms / warmup)) + 1
            for _ in range(more):
                launch()
            ran += more
            stream.synchronize()
        if warmup > 0:
            batch = max(10, warmup)
            prev, agree, settle_t0 = None, 0, time.time()
            while (time.time() - settle_t0) * 1e3 < MAX_SETTLE_MS:
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(stream)
                for _ in range(batch):
                    launch()
                e1.record(stream)
                stream.synchronize()
                ran += batch
                t = e0.elapsed_time(e1)
                agree = agree + 1 if prev is not None and abs(t - prev) <= 0.01 * prev else 0
                prev = t
                if agree >= 2:
                    break
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(stream)
        for _ in range(steps):
            launch()
        e1.record(stream)
        stream.synchronize()
        total = e0.elapsed_time(e1)
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
        evs[0].record(stream)
        for i in range(steps):
            launch()
            evs[i + 1].record(stream)
        stream.synchronize()
    per = [evs[i].elapsed_time(evs[i + 1]) for i in range(steps)]
    return total / steps, min(per), ran


def bench_sdpa(torch, capi, stream, steps, warmup):
    B, H, S, D = 4, 32, 4096, 128
    g = torch.Generator(device="cuda").manual_seed(42)
    q, k, v = (torch.randn((B, H, S, D), generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16) for _ in range(3))
    o = torch.empty_like(q)
    p = capi.SdpaParams()
    p.dtype, p.batch, p.heads, p.seq_q, p.seq_kv, p.head_dim = capi.DTYPE_BF16, B, H, S, S, D
    p.scale, p.is_causal = -1.0, 1
    for arr in (p.q_strides, p.k_strides, p.v_strides, p.o_strides):
        arr[:] = (H * S * D, S * D, D)
    lib = capi.lib()
    sp = C.c_void_p(stream.cuda_stream)
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, C.byref(p), sp)

    def launch():
        capi.check(lib.axhip_sdpa_fwd(*args))

    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
    flops = 4.0 * B * H * S * S * D / 2.0
    return {
        "kernel": lib.axhip_sdpa_kernel_name(C.byref(p)).decode(),
        "avg_ms": avg_ms, "min_ms": min_ms, "warmup_launches": warm_n,
        "flops": flops, "tflops": flops / (avg_ms * 1e-3) / 1e12,
        "finite": bool(torch.isfinite(o.float()).all().item()),
    }


def _rows_program(capi, x, out, dt, out_dt):
    p = capi.RowsProgram()
    p.rows, p.cols = x.shape[0], x.shape[1]
    p.input, p.input_dtype = x.data_ptr(), dt
    p.output, p.output_dtype = out.data_ptr(), out_dt
    p.norm_weight = p.norm_bias = -1
    return p


COLD_MIN_BYTES = 1 << 30  # bytes of other buffers touched between two uses of one buffer set in the rotating ("cold") timing


class ColdTimer:
    """Duration of single launches whose inputs come from HBM: between two timed launches a reduction reads 1 GiB of
    other data through the caches (read only: a flush that writes leaves hundreds of MiB of modified lines behind,
    whose write-back then competes with the launch that is being timed).  Every launch is bracketed by two HIP events
    of its own; what that bracketing adds to a launch is measured once per use (the same bracketing without the
    flush, against the back-to-back average) and taken off."""

    def __init__(self, torch, stream):
        self.torch, self.stream = torch, stream
        self.src = torch.zeros((1 << 30) // 4, device="cuda", dtype=torch.float32)
        self.acc = torch.zeros((), device="cuda", dtype=torch.float32)

    def _bracketed(self, launch, steps, flush):
        torch, stream = self.torch, self.stream
        pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        with torch.cuda.stream(stream):
            for e0, e1 in pairs:
                if flush:
                    torch.amax(self.src, dim=0, out=self.acc)
                e0.record(stream)
                launch()
                e1.record(stream)
            stream.synchronize()
        t = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)
        return t[len(t) // 2]

    def cold_ms(self, launch, steps, hot_avg_ms):
        """median cold launch in ms, and the event overhead that was taken off"""
        steps = max(steps, 20)
        overhead = max(0.0, self._bracketed(launch, steps, False) - hot_avg_ms)
        return max(self._bracketed(launch, steps, True) - overhead, 1e-6), overhead


def time_rotating(torch, stream, launchers, steps, warmup):
    """Average launch duration in ms over exactly `steps` launches that rotate through `launchers` (the same program
    over independent buffer sets, sized by the caller so that at least COLD_MIN_BYTES of other data pass through the
    caches between two uses of one set: the inputs then come from HBM, not from the 256 MiB memory-side cache)."""
    state = {"i": 0}

    def launch():
        launchers[state["i"] % len(launchers)]()
        state["i"] += 1

    avg_ms, min_ms, ran = time_launches(torch, stream, launch, steps, warmup)
    return avg_ms, min_ms, ran


def _chain_record(lib, capi, p, avg_ms, min_ms, warm_n, cold_ms, cold_min_ms, n_sets, set_bytes, nbytes):
    import ctypes as C

    return {
        "kernel": lib.axhip_fused_rows_kernel_name(C.byref(p)).decode(), "bytes": nbytes,
        # inputs from HBM: launches rotate over `buffer_sets` independent input/output sets
        "avg_ms": cold_ms, "min_ms": cold_min_ms, "gbs": nbytes / (cold_ms * 1e-3) / 1e9,
        "frac_of_hbm_peak": nbytes / (cold_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "frac_of_hbm_peak_cold": nbytes / (cold_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "buffer_sets": n_sets, "bytes_touched_between_reuse": (n_sets - 1) * set_bytes,
        # back-to-back launches on ONE buffer set: part of the input is re-found in the memory-side cache
        "avg_ms_same_buffers": avg_ms, "min_ms_same_buffers": min_ms, "warmup_launches": warm_n,
        "frac_of_hbm_peak_same_buffers": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
    }


def _sets_for(set_bytes: int) -> int:
    return max(3, -(-COLD_MIN_BYTES // set_bytes) + 1)


def bench_chains(torch, capi, stream, steps, warmup):
    """The fused-chain kernels of BASELINE.json configs[1] and [2].  Two timings each: `frac_of_hbm_peak` (=
    `frac_of_hbm_peak_cold`) rotates every launch over enough independent buffer sets that at least 1 GiB of other
    data is touched between two uses of a buffer -- the inputs come from HBM; `frac_of_hbm_peak_same_buffers` is the
    back-to-back figure on one set, part of whose input survives in the 256 MiB memory-side cache."""
    lib = capi.lib()
    sp = C.c_void_p(stream.cuda_stream)
    res = {}
    g = torch.Generator(device="cuda").manual_seed(42)

    # configs[1]: softmax((relu(a)+1)*b, -1).sum(1), fp32 [8192, 8192]
    R = Cc = 8192
    set_bytes = 2 * R * Cc * 4
    n_sets = _sets_for(set_bytes)
    one = torch.ones(1, device="cuda")
    sets, progs = [], []
    for _ in range(n_sets):
        a = torch.randn((R, Cc), generator=g, device="cuda")
        b = torch.randn((R, Cc), generator=g, device="cuda")
        out = torch.empty(R, device="cuda")
        p = _rows_program(capi, a, out, capi.DTYPE_F32, capi.DTYPE_F32)
        p.n_operands = 2
        p.operands[0].ptr, p.operands[0].dtype, p.operands[0].kind = one.data_ptr(), capi.DTYPE_F32, capi.BK["scalar"]
        p.operands[1].ptr, p.operands[1].dtype, p.operands[1].kind = b.data_ptr(), capi.DTYPE_F32, capi.BK["full"]
        p.n_pre = 3
        p.pre[0].op, p.pre[0].operand = capi.OP["relu"], -1
        p.pre[1].op, p.pre[1].operand = capi.OP["add"], 0
        p.pre[2].op, p.pre[2].operand = capi.OP["mul"], 1
        p.row_op = capi.ROWOP["softmax"]
        p.reduce = capi.RED["sum"]
        sets.append((a, b, out))
        progs.append(p)
    launchers = [(lambda q=q: capi.check(lib.axhip_fused_rows(C.byref(q), sp))) for q in progs]
    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, launchers[0], steps, warmup)
    cold_ms, cold_min, _ = time_rotating(torch, stream, launchers, steps, warmup)
    nbytes = 2 * R * Cc * 4 + R * 4
    rec = _chain_record(lib, capi, progs[0], avg_ms, min_ms, warm_n, cold_ms, cold_min, n_sets, set_bytes, nbytes)
    rec["rows_sum_to_one"] = bool(all(torch.allclose(s[2], torch.ones_like(s[2]), atol=1e-4) for s in sets))
    res["chain_relu_add_mul_softmax_sum_f32_8192x8192"] = rec
    # plain copy of the same matrix through the elementwise kernel (empty chain): the kernel of
    # known traffic that the rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by
    a = sets[0][0]
    cp = torch.empty_like(a)
    pc = _rows_program(capi, a, cp, capi.DTYPE_F32, capi.DTYPE_F32)
    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, lambda: capi.check(lib.axhip_fused_rows(C.byref(pc), sp)), steps, warmup)
    nbytes = 2 * R * Cc * 4
    res["copy_f32_8192x8192"] = {
        "kernel": lib.axhip_fused_rows_kernel_name(C.byref(pc)).decode(), "avg_ms": avg_ms, "min_ms": min_ms, "warmup_launches": warm_n,
        "bytes": nbytes, "gbs": nbytes / (avg_ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "bit_exact": bool(torch.equal(cp, a)),
    }
    del a, cp, sets, progs, launchers

    # configs[2]: gelu(layernorm(x)*gamma+beta) and the RMSNorm variant, bf16 [16384, 4096]
    R, Cc = 16384, 4096
    set_bytes = 2 * R * Cc * 2
    n_sets = _sets_for(set_bytes)
    xs = [torch.randn((R, Cc), generator=g, device="cuda").to(torch.bfloat16) for _ in range(n_sets)]
    ys = [torch.empty_like(x) for x in xs]
    gamma = (torch.rand(Cc, generator=g, device="cuda") + 0.5).to(torch.bfloat16)
    beta = (torch.rand(Cc, generator=g, device="cuda") * 0.2 - 0.1).to(torch.bfloat16)
    for name, rowop, has_bias in (("layernorm", "layernorm", True), ("rmsnorm", "rmsnorm", False)):
        progs = []
        for x, y in zip(xs, ys):
            p = _rows_program(capi, x, y, capi.DTYPE_BF16, capi.DTYPE_BF16)
            p.n_operands = 2
            p.operands[0].ptr, p.operands[0].dtype, p.operands[0].kind = gamma.data_ptr(), capi.DTYPE_BF16, capi.BK["rowvec"]
            p.operands[1].ptr, p.operands[1].dtype, p.operands[1].kind = beta.data_ptr(), capi.DTYPE_BF16, capi.BK["rowvec"]
            p.row_op, p.eps = capi.ROWOP[rowop], 1e-5
            p.norm_weight, p.norm_bias = 0, (1 if has_bias else -1)
            p.n_post = 1
            p.post[0].op, p.post[0].operand = capi.OP["gelu"], -1
            p.reduce = capi.RED["none"]
            progs.append(p)
        launchers = [(lambda q=q: capi.check(lib.axhip_fused_rows(C.byref(q), sp))) for q in progs]
        torch.cuda.synchronize()
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launchers[0], steps, warmup)
        cold_ms, cold_min, _ = time_rotating(torch, stream, launchers, steps, warmup)
        nbytes = 2 * R * Cc * 2 + Cc * 2 * (2 if has_bias else 1)
        rec = _chain_record(lib, capi, progs[0], avg_ms, min_ms, warm_n, cold_ms, cold_min, n_sets, set_bytes, nbytes)
        rec["finite"] = bool(all(torch.isfinite(y.float()).all().item() for y in ys))
        res[f"chain_gelu_{name}_bf16_16384x4096"] = rec
    # What the memory system gives a one-read-one-write stream of this size when nothing is found in the caches: the
    # runtime's own device-to-device copy (hipMemcpyAsync behind axhip_memcpy_d2d_async) and the library's elementwise
    # copy kernel (an empty chain), on the same rotation of 128 MiB buffers as the norm chains above
    copy_launchers = [(lambda x=x, y=y: capi.check(lib.axhip_memcpy_d2d_async(y.data_ptr(), x.data_ptr(), R * Cc * 2, sp))) for x, y in zip(xs, ys)]
    cold_ms, cold_min, _ = time_rotating(torch, stream, copy_launchers, steps, warmup)
    same_ms, _, _ = time_launches(torch, stream, copy_launchers[0], steps, warmup)
    nbytes = 2 * R * Cc * 2
    res["hbm_copy_reference_128MiB"] = {
        "what": "hipMemcpyAsync device-to-device, 128 MiB in + 128 MiB out per launch, same buffer rotation as the norm chains",
        "avg_ms": cold_ms, "min_ms": cold_min, "bytes": nbytes, "buffer_sets": n_sets,
        "frac_of_hbm_peak_cold": nbytes / (cold_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "frac_of_hbm_peak_same_buffers": nbytes / (same_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
    }
    progs = [_rows_program(capi, x, y, capi.DTYPE_BF16, capi.DTYPE_BF16) for x, y in zip(xs, ys)]
    ew_launchers = [(lambda q=q: capi.check(lib.axhip_fused_rows(C.byref(q), sp))) for q in progs]
    cold_ms, cold_min, _ = time_rotating(torch, stream, ew_launchers, steps, warmup)
    same_ms, _, _ = time_launches(torch, stream, ew_launchers[0], steps, warmup)
    res["elementwise_copy_bf16_16384x4096"] = {
        "kernel": lib.axhip_fused_rows_kernel_name(C.byref(progs[0])).decode(), "avg_ms": cold_ms, "min_ms": cold_min, "bytes": nbytes, "buffer_sets": n_sets,
        "frac_of_hbm_peak_cold": nbytes / (cold_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "frac_of_hbm_peak_same_buffers": nbytes / (same_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
        "bit_exact": bool(torch.equal(ys[0], xs[0])),
    }
    for name in ("chain_gelu_layernorm_bf16_16384x4096", "chain_gelu_rmsnorm_bf16_16384x4096"):
        res[name]["frac_of_cold_copy_reference"] = res[name]["frac_of_hbm_peak_cold"] / res["hbm_copy_reference_128MiB"]["frac_of_hbm_peak_cold"]
    del xs, ys, progs
    # a row length that the 16-byte vector does not divide (Whisper's 1500 frames): the kernels' ragged variant
    Rr, Cr = 30000, 1500
    set_bytes = 2 * Rr * Cr * 2
    n_sets = _sets_for(set_bytes)
    xs = [torch.randn((Rr, Cr), generator=g, device="cuda").to(torch.bfloat16) for _ in range(n_sets)]
    ys = [torch.empty_like(x) for x in xs]
    progs = []
    for x, y in zip(xs, ys):
        p = _rows_program(capi, x, y, capi.DTYPE_BF16, capi.DTYPE_BF16)
        p.row_op, p.reduce = capi.ROWOP["softmax"], capi.RED["none"]
        progs.append(p)
    launchers = [(lambda q=q: capi.check(lib.axhip_fused_rows(C.byref(q), sp))) for q in progs]
    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, launchers[0], steps, warmup)
    cold_ms, cold_min, _ = time_rotating(torch, stream, launchers, steps, warmup)
    nbytes = 2 * Rr * Cr * 2
    rec = _chain_record(lib, capi, progs[0], avg_ms, min_ms, warm_n, cold_ms, cold_min, n_sets, set_bytes, nbytes)
    rec["rows_sum_to_one"] = bool(all(((y.float().sum(1) - 1.0).abs() < 2e-2).all().item() for y in ys))
    res["softmax_bf16_30000x1500_odd_row_length"] = rec
    return res



class _Prog:
    """A row program over torch device tensors (bench-side builder for the survey)."""

    def __init__(self, capi, x, out_dtype=None):
        import torch

        self.capi, self.x, self.keep = capi, x, []
        self.dt = {torch.float32: capi.DTYPE_F32, torch.float16: capi.DTYPE_F16, torch.bfloat16: capi.DTYPE_BF16}[x.dtype]
        self.p = capi.RowsProgram()
        self.p.rows, self.p.cols = x.shape
        self.p.input, self.p.input_dtype = x.data_ptr(), self.dt
        self.p.norm_weight = self.p.norm_bias = -1
        self.post_stage = False
        self.read_bytes = x.numel() * x.element_size()
        self.out_dtype = out_dtype

    def _operand(self, t, kind):
        i = self.p.n_operands
        self.keep.append(t)
        self.p.operands[i].ptr, self.p.operands[i].kind = t.data_ptr(), self.capi.BK[kind]
        self.p.operands[i].dtype = self.dt if t.dtype == self.x.dtype else self.capi.DTYPE_F32
        self.p.n_operands = i + 1
        self.read_bytes += t.numel() * t.element_size()
        return i

    def op(self, name, operand=None, kind="full", imm=None):
        chain, n = (self.p.post, self.p.n_post) if self.post_stage else (self.p.pre, self.p.n_pre)
        chain[n].op = self.capi.OP[name]
        chain[n].operand = -1 if operand is None else self._operand(operand, kind)
        if imm is not None:
            chain[n].imm, chain[n].imm_kind = imm, self.capi.BK["imm"]
        if self.post_stage:
            self.p.n_post = n + 1
        else:
            self.p.n_pre = n + 1
        return self

    def row(self, name, w=None, b=None):
        self.p.row_op, self.p.eps = self.capi.ROWOP[name], 1e-5
        if w is not None:
            self.p.norm_weight = self._operand(w, "rowvec")
        if b is not None:
            self.p.norm_bias = self._operand(b, "rowvec")
        self.post_stage = True
        return self

    def finish(self, torch, reduce="none"):
        self.p.reduce = self.capi.RED[reduce]
        odt = self.out_dtype or self.x.dtype
        shape = self.x.shape if reduce == "none" else (self.x.shape[0],)
        self.out = torch.empty(shape, device="cuda", dtype=odt)
        self.p.output = self.out.data_ptr()
        self.p.output_dtype = {torch.float32: self.capi.DTYPE_F32, torch.float16: self.capi.DTYPE_F16, torch.bfloat16: self.capi.DTYPE_BF16}[odt]
        self.bytes = self.read_bytes + self.out.numel() * self.out.element_size()
        return self


def bench_survey(torch, capi, stream, steps, warmup):
    """Achieved HBM bandwidth of a spread of row programs: the built-in kernel shapes, shapes the library compiles
    at run time (rows_jit_*), and rows of odd length.  Bytes are the algorithmic ones: every operand read once, the
    result written once."""
    lib = capi.lib()
    sp = C.c_void_p(stream.cuda_stream)
    g = torch.Generator(device="cuda").manual_seed(7)
    res = {}

    def rnd(shape, dtype, scale=1.0, shift=0.0):
        return (torch.randn(shape, generator=g, device="cuda") * scale + shift).to(dtype)

    cold = ColdTimer(torch, stream)

    def with_cold(rec, launch, avg_ms, nbytes):
        # the same launch with its inputs flushed out of the caches first (frac_of_hbm_peak is the back-to-back figure)
        cold_ms, overhead_ms = cold.cold_ms(launch, steps, avg_ms)
        rec["cold_us"] = cold_ms * 1e3
        rec["event_overhead_us"] = overhead_ms * 1e3
        rec["frac_of_hbm_peak_cold"] = nbytes / (cold_ms * 1e-3) / 1e9 / PEAK_HBM_GBS
        return rec

    def run(name, prog):
        lib.axhip_fused_rows_prepare(C.byref(prog.p))
        torch.cuda.synchronize()
        launch = lambda: capi.check(lib.axhip_fused_rows(C.byref(prog.p), sp))
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
        res[name] = with_cold({"kernel": lib.axhip_fused_rows_kernel_name(C.byref(prog.p)).decode(), "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3,
                               "bytes": prog.bytes, "frac_of_hbm_peak": prog.bytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                               "finite": bool(torch.isfinite(prog.out.float()).all().item())}, launch, avg_ms, prog.bytes)

    bf, f32 = torch.bfloat16, torch.float32
    R, Cc = 16384, 4096
    x, y = rnd((R, Cc), bf), rnd((R, Cc), bf)
    w, b = rnd((Cc,), bf, 0.3, 1.0), rnd((Cc,), bf, 0.1)
    cvec, half = rnd((R,), bf), torch.full((1,), 0.5, device="cuda", dtype=bf)
    P = lambda t=x, od=None: _Prog(capi, t, od)
    tag = "bf16_16384x4096"
    run(f"softmax_{tag}", P().row("softmax").finish(torch))
    run(f"softmax(x*s)_{tag}", P().op("mul", imm=0.125).row("softmax").finish(torch))
    run(f"softmax(x+y)_{tag}", P().op("add", y).row("softmax").finish(torch))
    run(f"softmax(x*s+y)_{tag}", P().op("mul", half, "scalar").op("add", y).row("softmax").finish(torch))
    run(f"logsoftmax_{tag}", P().row("logsoftmax").finish(torch))
    run(f"layernorm_{tag}", P().row("layernorm", w, b).finish(torch))
    run(f"layernorm(x+y)_{tag}", P().op("add", y).row("layernorm", w, b).finish(torch))
    run(f"gelu(layernorm)_{tag}", P().row("layernorm", w, b).op("gelu").finish(torch))
    run(f"silu(layernorm)_{tag}", P().row("layernorm", w, b).op("silu").finish(torch))
    run(f"rmsnorm_{tag}", P().row("rmsnorm", w).finish(torch))
    run(f"gelu(rmsnorm)_{tag}", P().row("rmsnorm", w).op("gelu").finish(torch))
    run(f"rmsnorm(x+y)_{tag}", P().op("add", y).row("rmsnorm", w).finish(torch))
    run(f"sum(x)_{tag}", P().finish(torch, "sum"))
    run(f"mean(x^2)_{tag}", P(od=f32).op("square").finish(torch, "mean"))
    run(f"sum(x*y)_{tag}", P().op("mul", y).finish(torch, "sum"))
    run(f"max(|x|)_{tag}", P().op("abs").finish(torch, "max"))
    # shapes without a built-in kernel: compiled when first seen
    run(f"sigmoid(layernorm)_{tag}", P().row("layernorm", w, b).op("sigmoid").finish(torch))
    run(f"softmax(exp(x))_{tag}", P().op("exp").row("softmax").finish(torch))
    run(f"softmax(tanh(x*s)+y)_{tag}", P().op("mul", imm=0.5).op("tanh").op("add", y).row("softmax").finish(torch))
    run(f"layernorm(relu(x)*y+r)_{tag}", P().op("relu").op("mul", y).op("add", w, "rowvec").row("layernorm", w, b).finish(torch))
    run(f"softmax(x*c)*y_{tag}", P().op("mul", cvec, "colvec").row("softmax").op("mul", y).finish(torch))
    run(f"rmsnorm(x)*sigmoid(y)_fp32out_{tag}", P(od=f32).row("rmsnorm", w).op("mul", y).finish(torch))
    del x, y
    a, c = rnd((8192, 8192), f32), rnd((8192, 8192), f32)
    w32, b32 = rnd((8192,), f32, 0.3, 1.0), rnd((8192,), f32, 0.1)
    one = torch.ones(1, device="cuda")
    tag = "f32_8192x8192"
    run(f"softmax((relu(a)+1)*b).sum_{tag}", P(a).op("relu").op("add", one, "scalar").op("mul", c).row("softmax").finish(torch, "sum"))
    run(f"softmax_{tag}", P(a).row("softmax").finish(torch))
    run(f"layernorm_{tag}", P(a).row("layernorm", w32, b32).finish(torch))
    run(f"gelu(layernorm(a+b))_{tag}", P(a).op("add", c).row("layernorm", w32, b32).op("gelu").finish(torch))
    run(f"sum(a)_{tag}", P(a).finish(torch, "sum"))
    del a, c
    # the wider operator table: a comparison to a Bool array, where() on it, a leaky ReLU chain, any() per row
    xb, yb = rnd((16384, 4096), bf), rnd((16384, 4096), bf)
    mask = torch.empty((16384, 4096), device="cuda", dtype=torch.uint8)
    pg = _Prog(capi, xb)
    pg.op("gt", yb)
    pg.p.output, pg.p.output_dtype, pg.p.reduce = mask.data_ptr(), capi.DTYPE_U8, capi.RED["none"]
    pg.out, pg.bytes = mask, 2 * xb.numel() * 2 + mask.numel()
    run("x>y_to_bool_bf16_16384x4096", pg)
    run("leaky_relu(x)*y_bf16_16384x4096", _Prog(capi, xb).op("leaky_relu", imm=0.01).op("mul", yb).finish(torch))
    # (elementwise chains of 8 MiB or more: compiled, the array seen as rows of 512 chunks)
    run("gelu(x)_bf16_16384x4096", _Prog(capi, xb).op("gelu").finish(torch))
    run("relu(x)_as_vector_bf16_1x67108864", _Prog(capi, xb.view(1, -1)).op("relu").finish(torch))
    anyout = torch.empty((16384,), device="cuda", dtype=torch.uint8)
    pa = _Prog(capi, xb)
    pa.op("gt", imm=3.5)
    pa.p.output, pa.p.output_dtype, pa.p.reduce = anyout.data_ptr(), capi.DTYPE_U8, capi.RED["max"]
    pa.out, pa.bytes = anyout, xb.numel() * 2 + anyout.numel()
    run("any(x>3.5)_bf16_16384x4096", pa)
    wout = torch.empty_like(xb)
    shp, st = (C.c_int64 * 2)(16384, 4096), (C.c_int64 * 2)(4096, 1)
    launch = lambda: capi.check(lib.axhip_where(mask.data_ptr(), capi.DTYPE_U8, xb.data_ptr(), capi.DTYPE_BF16, yb.data_ptr(), capi.DTYPE_BF16, wout.data_ptr(),
                                               capi.DTYPE_BF16, 2, shp, st, st, st, sp))
    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
    nbytes = 3 * xb.numel() * 2 + mask.numel()
    res["where(mask,x,y)_bf16_16384x4096"] = with_cold(
        {"kernel": "where_vec", "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes, "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
         "finite": bool(torch.equal(wout, torch.where(mask.bool(), xb, yb)))}, launch, avg_ms, nbytes)
    del yb, mask, wout
    # the convolution front end's mover: reflect padding of a (N, C, L) signal along L (Whisper pads its mel frames this way)
    pin = xb.view(16, 1024, 4096)
    pout = torch.empty((16, 1024, 4096 + 512), dtype=bf, device="cuda")
    pshape, pstr = (C.c_int64 * 3)(16, 1024, 4096), (C.c_int64 * 3)(1024 * 4096, 4096, 1)
    pb, pa_ = (C.c_int64 * 3)(0, 0, 256), (C.c_int64 * 3)(0, 0, 256)
    launch = lambda: capi.check(lib.axhip_pad_mode(pin.data_ptr(), pout.data_ptr(), capi.DTYPE_BF16, 3, pshape, pstr, pb, pa_, capi.PAD["reflect"], 0.0, sp))
    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
    nbytes = (pin.numel() + pout.numel()) * 2
    res["pad_reflect_bf16_16x1024x4096_by_256"] = with_cold(
        {"kernel": "pad", "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes, "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
         "finite": bool(torch.equal(pout, torch.nn.functional.pad(pin.float(), (256, 256), mode="reflect").to(bf)))}, launch, avg_ms, nbytes)
    del xb, pin, pout
    # transposed copies (axhip_strided_copy: 16 x 16 vector tiles through LDS)
    for tname, shape, perm, dt in (("transpose_bf16_8192x8192", (8192, 8192), (1, 0), bf), ("transpose_f32_8192x8192", (8192, 8192), (1, 0), f32),
                                   ("nchw_to_nhwc_bf16_64x64x128x128", (64, 64, 128, 128), (0, 2, 3, 1), bf),
                                   ("transpose_bf16_32x1500x1280_to_32x1280x1500", (32, 1500, 1280), (0, 2, 1), bf)):
        tin = rnd(shape, dt)
        tv = tin.permute(*perm)
        tout = torch.empty(tv.shape, dtype=dt, device="cuda")
        tshape, tstr = (C.c_int64 * tv.dim())(*tv.shape), (C.c_int64 * tv.dim())(*tv.stride())
        code = capi.DTYPE_BF16 if dt == bf else capi.DTYPE_F32
        launch = lambda: capi.check(lib.axhip_strided_copy(tin.data_ptr(), code, tout.data_ptr(), code, tv.dim(), tshape, tstr, sp))
        torch.cuda.synchronize()
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
        nbytes = 2 * tin.numel() * tin.element_size()
        res[tname] = with_cold({"kernel": "strided_copy (transpose tiles)", "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes,
                                "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "finite": bool(torch.equal(tout, tv))}, launch, avg_ms, nbytes)
        del tin, tv, tout
    # rows of odd length
    for rows, cols, dt, name in ((30000, 1500, bf, "bf16"), (16384, 4100, bf, "bf16"), (16384, 4097, bf, "bf16"), (16384, 1501, f32, "f32")):
        t = rnd((rows, cols), dt)
        run(f"softmax_{name}_{rows}x{cols}", P(t).row("softmax").finish(torch))
    t, u = rnd((30000, 1001), bf), rnd((30000, 1001), bf)
    wr, br = rnd((1001,), bf, 0.3, 1.0), rnd((1001,), bf, 0.1)
    run("layernorm_bf16_30000x1001", P(t).row("layernorm", wr, br).finish(torch))
    run("softmax(|x|*y)_bf16_30000x1001", P(t).op("abs").op("mul", u).row("softmax").finish(torch))
    t, u = rnd((16384, 4099), bf), rnd((16384, 4099), bf)
    wr, br = rnd((4099,), bf, 0.3, 1.0), rnd((4099,), bf, 0.1)
    run("layernorm(x+y)_bf16_16384x4099", P(t).op("add", u).row("layernorm", wr, br).finish(torch))
    run("mean(x^2)_bf16_16384x4099", P(t, f32).op("square").finish(torch, "mean"))
    del t, u
    # short rows (attention scores over short sequences, per-head norms, class logits): 4 to 32 lanes per row, several
    # rows to a wavefront; odd lengths on the 16-byte grid
    for rows, cols, dt, name in ((1 << 20, 64, bf, "bf16"), (1 << 19, 128, bf, "bf16"), (1 << 20, 64, f32, "f32"), (1 << 22, 16, bf, "bf16")):
        t = rnd((rows, cols), dt, 2.0)
        wr = rnd((cols,), dt, 0.3, 1.0)
        run(f"softmax_{name}_{rows}x{cols}", P(t).row("softmax").finish(torch))
        run(f"rmsnorm_{name}_{rows}x{cols}", P(t).row("rmsnorm", wr).finish(torch))
        del t
    # (from 32768 rows on: 64 / L consecutive rows per wavefront staged in LDS, L lanes per row)
    for rows, cols, dt, name in ((3000000, 10, f32, "f32"), (400000, 77, bf, "bf16"), (170000, 197, bf, "bf16"), (200000, 250, bf, "bf16"),
                                 (100000, 513, bf, "bf16")):
        t = rnd((rows, cols), dt, 2.0)
        run(f"softmax_{name}_{rows}x{cols}", P(t).row("softmax").finish(torch))
        if cols in (77, 197):
            wr, br = rnd((cols,), dt, 0.3, 1.0), rnd((cols,), dt, 0.1)
            run(f"rmsnorm_{name}_{rows}x{cols}", P(t).row("rmsnorm", wr).finish(torch))
            run(f"layernorm_{name}_{rows}x{cols}", P(t).row("layernorm", wr, br).finish(torch))
        del t
    # vocabulary-sized rows (language-model logits): 1024-thread blocks; beyond 8 chunks per thread the row stays in
    # registers as raw words, beyond 16 (fp32 logits over 128 256 entries) the block walks the row once per pass
    for rows, cols, dt, name in ((4096, 50304, bf, "bf16"), (2048, 128256, bf, "bf16"), (2048, 50304, f32, "f32"), (4096, 50257, bf, "bf16"),
                                 (1024, 128256, f32, "f32")):
        t = rnd((rows, cols), dt, 3.0)
        run(f"softmax_{name}_{rows}x{cols}", P(t).row("softmax").finish(torch))
        run(f"logsoftmax(x*s)_{name}_{rows}x{cols}", P(t).op("mul", imm=0.5).row("logsoftmax").finish(torch))
        run(f"max(x)_{name}_{rows}x{cols}", P(t).finish(torch, "max"))
        del t
    # argmax along the last axis (greedy decoding over logits) and along other axes of a contiguous array
    for (outer, axis, inner), dt, name in (((16384, 4096, 1), bf, "bf16"), ((4096, 50304, 1), bf, "bf16"), ((8192, 8192, 1), f32, "f32"),
                                           ((1 << 20, 64, 1), bf, "bf16"), ((64, 4096, 1024), bf, "bf16"), ((1, 4096, 16384), f32, "f32")):
        t = rnd((outer, axis, inner), dt, 3.0)
        out = torch.empty((outer * inner,), device="cuda", dtype=torch.int64)
        code = capi.DTYPE_BF16 if dt == bf else capi.DTYPE_F32
        torch.cuda.synchronize()
        launch = lambda: capi.check(lib.axhip_argreduce(t.data_ptr(), code, outer, axis, inner, 0, out.data_ptr(), sp))
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
        nbytes = t.numel() * t.element_size() + out.numel() * 8
        res[f"argmax_axis1_{name}_{outer}x{axis}x{inner}"] = with_cold(
            {"kernel": "argreduce_rows" if inner == 1 else "argreduce_strided", "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes,
             "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "finite": bool(torch.equal(out.view(outer, inner), t.float().argmax(1)))},
            launch, avg_ms, nbytes)
        del t, out
    # reductions and softmax along an inner axis of a contiguous array (no transposing copy)
    for (outer, axis, inner), dt, name in (((1, 4096, 16384), f32, "f32"), ((64, 4096, 1024), bf, "bf16"), ((8192, 8, 1024), f32, "f32")):
        t = rnd((outer, axis, inner), dt, 3.0)
        code = capi.DTYPE_BF16 if dt == bf else capi.DTYPE_F32
        out = torch.empty((outer, inner), device="cuda", dtype=dt)
        torch.cuda.synchronize()
        launch = lambda: capi.check(lib.axhip_reduce_axis(t.data_ptr(), code, outer, axis, inner, capi.RED["sum"], out.data_ptr(), code, sp))
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
        nbytes = (t.numel() + out.numel()) * t.element_size()
        res[f"sum_axis1_{name}_{outer}x{axis}x{inner}"] = with_cold(
            {"kernel": "reduce_axis", "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes,
             "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "finite": bool(torch.isfinite(out.float()).all().item())}, launch, avg_ms, nbytes)
        full = torch.empty_like(t)
        torch.cuda.synchronize()
        launch = lambda: capi.check(lib.axhip_softmax_axis(t.data_ptr(), code, outer, axis, inner, 0, full.data_ptr(), sp))
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
        nbytes = 2 * t.numel() * t.element_size()
        res[f"softmax_axis1_{name}_{outer}x{axis}x{inner}"] = with_cold(
            {"kernel": "softmax_axis", "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes,
             "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "finite": bool(torch.isfinite(full.float()).all().item())}, launch, avg_ms, nbytes)
        del t, out, full
    # the movers around attention scores and convolutions: a [queries, keys] mask and a key-padding mask filled into
    # [batch, heads, queries, keys] scores, where() under the same mask, a convolution input padded by one on each side
    i64 = lambda *v: (C.c_int64 * len(v))(*v)
    S = (4, 32, 1024, 1024)
    full_st = i64(32 << 20, 1 << 20, 1024, 1)
    scores, other, out = rnd(S, bf, 2.0), rnd(S, bf, 2.0), torch.empty(S, device="cuda", dtype=bf)
    mask = (torch.rand((1024, 1024), device="cuda") > 0.5).to(torch.uint8)
    keys = (torch.rand((4, 1024), device="cuda") > 0.5).to(torch.uint8)
    BF, U8 = capi.DTYPE_BF16, capi.DTYPE_U8

    def mover(name, kernel, launch, nbytes, check):
        torch.cuda.synchronize()
        avg_ms, min_ms, warm_n = time_launches(torch, stream, launch, steps, warmup)
        res[name] = with_cold({"kernel": kernel, "avg_us": avg_ms * 1e3, "min_us": min_ms * 1e3, "bytes": nbytes,
                               "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, "finite": bool(check())}, launch, avg_ms, nbytes)

    nb = 2 * scores.numel() * 2
    mover("masked_fill_bf16_4x32x1024x1024_mask_1024x1024", "masked_fill_vec",
          lambda: capi.check(lib.axhip_masked_fill(scores.data_ptr(), BF, mask.data_ptr(), out.data_ptr(), 4, i64(*S), full_st, i64(0, 0, 1024, 1), -1e9, sp)),
          nb, lambda: torch.equal(out, scores.masked_fill(mask.bool(), -1e9)))
    mover("masked_fill_bf16_4x32x1024x1024_key_padding_4x1x1x1024", "masked_fill_vec",
          lambda: capi.check(lib.axhip_masked_fill(scores.data_ptr(), BF, keys.data_ptr(), out.data_ptr(), 4, i64(*S), full_st, i64(1024, 0, 0, 1), -1e9, sp)),
          nb, lambda: torch.equal(out, scores.masked_fill(keys.bool()[:, None, None, :], -1e9)))
    mover("where_bf16_4x32x1024x1024_cond_1024x1024", "where_rows",
          lambda: capi.check(lib.axhip_where(mask.data_ptr(), U8, scores.data_ptr(), BF, other.data_ptr(), BF, out.data_ptr(), BF, 4, i64(*S), i64(0, 0, 1024, 1), full_st, full_st, sp)),
          3 * scores.numel() * 2, lambda: torch.equal(out, torch.where(mask.bool(), scores, other)))
    del scores, other, out
    x = rnd((32, 1280, 3000), bf, 1.0)
    padded = torch.empty((32, 1280, 3002), device="cuda", dtype=bf)
    mover("pad_bf16_32x1280x3000_by_1_1_last", "pad_vec",
          lambda: capi.check(lib.axhip_pad(x.data_ptr(), padded.data_ptr(), BF, 3, i64(32, 1280, 3000), i64(1280 * 3000, 3000, 1), i64(0, 0, 1), i64(0, 0, 1), 0.0, sp)),
          (x.numel() + padded.numel()) * 2, lambda: torch.equal(padded, torch.nn.functional.pad(x, (1, 1))))
    del x, padded
    return res


def bench_gemm(torch, capi, stream, steps, warmup):
    """x W^T through axhip_gemm (the nn::Linear product): a large square, the tall product of a
    long batch, the Whisper-block projection of BASELINE.json configs[4], and two decoding steps."""
    lib = capi.lib()
    sp = C.c_void_p(stream.cuda_stream)
    res = {}
    g = torch.Generator(device="cuda").manual_seed(42)
    # (the last three: decoding steps, one and four tokens against a weight matrix -- bound by reading the weights; the 512 MiB
    # matrix is larger than the 256 MiB memory-side cache, so its rate is an HBM rate)
    for M, N, K in ((4096, 4096, 4096), (8192, 4096, 4096), (1500, 1280, 1280), (1, 4096, 4096), (4, 4096, 4096), (1, 16384, 16384)):
        a = torch.randn((M, K), generator=g, device="cuda").to(torch.bfloat16)
        w = (torch.randn((N, K), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
        c = torch.empty((M, N), device="cuda", dtype=torch.bfloat16)
        p = capi.GemmParams()
        p.dtype, p.trans_a, p.trans_b = capi.DTYPE_BF16, 0, 1
        p.m, p.n, p.k = M, N, K
        p.lda, p.ldb, p.ldc, p.batch = K, K, N, 1
        args = (a.data_ptr(), w.data_ptr(), c.data_ptr(), C.byref(p), sp)
        torch.cuda.synchronize()
        avg_ms, min_ms, warm_n = time_launches(torch, stream, lambda: capi.check(lib.axhip_gemm(*args)), steps, warmup)
        flops = 2.0 * M * N * K
        # the vendor library on the same operands (torch.matmul -> hipBLASLt), for context only
        with torch.cuda.stream(stream):
            wt = w.t()
            lib_ms, _, _ = time_launches(torch, stream, lambda: torch.matmul(a, wt), steps, warmup)
        res[f"gemm_nt_bf16_{M}x{N}x{K}"] = {"avg_ms": avg_ms, "min_ms": min_ms, "warmup_launches": warm_n, "flops": flops, "tflops": flops / (avg_ms * 1e-3) / 1e12,
                                             "frac_of_mfma_peak": flops / (avg_ms * 1e-3) / 1e12 / PEAK_BF16_TFLOPS,
                                             "finite": bool(torch.isfinite(c.float()).all().item()),
                                             "hipblaslt_avg_ms": lib_ms}
        if M <= 8:  # what bounds a decoding step is the one read of W
            nbytes = 2.0 * (N * K + M * K + M * N)
            res[f"gemm_nt_bf16_{M}x{N}x{K}"].update({"bytes": nbytes, "gbs": nbytes / (avg_ms * 1e-3) / 1e9})
        del a, w, c
    # a decoding step of attention: one query per (batch, head) against 16384 keys -- the keys are split between
    # work-groups and the partial states merged by a second kernel; K and V (1 GiB) are larger than the memory-side cache
    B, H, S, D = 4, 32, 16384, 128
    q = torch.randn((B, H, 1, D), generator=g, device="cuda").to(torch.bfloat16)
    k, v = (torch.randn((B, H, S, D), generator=g, device="cuda").to(torch.bfloat16) for _ in range(2))
    o = torch.empty_like(q)
    p = capi.SdpaParams()
    p.dtype, p.batch, p.heads, p.seq_q, p.seq_kv, p.head_dim = capi.DTYPE_BF16, B, H, 1, S, D
    p.scale, p.is_causal = -1.0, 0
    p.q_strides[:] = (H * D, D, D)
    p.o_strides[:] = (H * D, D, D)
    for arr in (p.k_strides, p.v_strides):
        arr[:] = (H * S * D, S * D, D)
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, C.byref(p), sp)
    torch.cuda.synchronize()
    avg_ms, min_ms, warm_n = time_launches(torch, stream, lambda: capi.check(lib.axhip_sdpa_fwd(*args)), steps, warmup)
    nbytes = 2.0 * (2 * B * H * S * D + 2 * B * H * D)
    ref = torch.nn.functional.scaled_dot_product_attention(q.float(), k.float(), v.float())
    res[f"sdpa_decode_bf16_b{B}h{H}s{S}d{D}"] = {"kernel": lib.axhip_sdpa_kernel_name(C.byref(p)).decode(), "avg_ms": avg_ms, "min_ms": min_ms, "warmup_launches": warm_n,
                                                  "bytes": nbytes, "gbs": nbytes / (avg_ms * 1e-3) / 1e9, "frac_of_hbm_peak": nbytes / (avg_ms * 1e-3) / 1e9 / PEAK_HBM_GBS,
                                                  "max_abs_err_vs_fp32": float((o.float() - ref).abs().max().item())}
    del q, k, v, o, ref
    return res


PEAK_F32_MFMA_TFLOPS = 157.3  # MI355X dense fp32 matrix peak


def bench_f32(torch, capi, stream, steps, warmup):
    """The fp32 matrix-instruction kernels (the dtype the reference's GPU path and its Whisper example run in):
    attention on BASELINE.json configs[0] and on a chip-filling shape, x W^T on the Whisper projection and a
    large square.  fp32 products and sums; priced against the 157.3 TFLOP/s fp32 matrix peak."""
    lib = capi.lib()
    sp = C.c_void_p(stream.cuda_stream)
    res = {}
    g = torch.Generator(device="cuda").manual_seed(42)
    steps_f32, warmup_f32 = max(10, steps // 4), max(5, warmup // 4)  # these launches are 10-1000x longer than the 16-bit ones
    for B, H, S, D in ((1, 8, 512, 64), (4, 32, 2048, 64)):
        q, k, v = (torch.randn((B, H, S, D), generator=g, device="cuda") for _ in range(3))
        o = torch.empty_like(q)
        p = capi.SdpaParams()
        p.dtype, p.batch, p.heads, p.seq_q, p.seq_kv, p.head_dim = capi.DTYPE_F32, B, H, S, S, D
        p.scale, p.is_causal = -1.0, 0
        for arr in (p.q_strides, p.k_strides, p.v_strides, p.o_strides):
            arr[0], arr[1], arr[2] = H * S * D, S * D, D
        args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), None, C.byref(p), sp)
        torch.cuda.synchronize()
        avg_ms, min_ms, warm_n = time_launches(torch, stream, lambda: capi.check(lib.axhip_sdpa_fwd(*args)), steps_f32, warmup_f32)
        flops = 4.0 * B * H * S * S * D
        res[f"sdpa_f32_b{B}h{H}s{S}d{D}"] = {"kernel": lib.axhip_sdpa_kernel_name(C.byref(p)).decode(), "avg_ms": avg_ms, "min_ms": min_ms, "warmup_launches": warm_n, "flops": flops,
                                             "tflops": flops / (avg_ms * 1e-3) / 1e12, "frac_of_f32_mfma_peak": flops / (avg_ms * 1e-3) / 1e12 / PEAK_F32_MFMA_TFLOPS,
                                             "finite": bool(torch.isfinite(o).all().item())}
        del q, k, v, o
    for M, N, K in ((1500, 1280, 1280), (4096, 4096, 4096)):
        a = torch.randn((M, K), generator=g, device="cuda")
        w = torch.randn((N, K), generator=g, device="cuda") * 0.02
        c = torch.empty((M, N), device="cuda")
        p = capi.GemmParams()
        p.dtype, p.trans_a, p.trans_b = capi.DTYPE_F32, 0, 1
        p.m, p.n, p.k = M, N, K
        p.lda, p.ldb, p.ldc, p.batch = K, K, N, 1
        args = (a.data_ptr(), w.data_ptr(), c.data_ptr(), C.byref(p), sp)
        torch.cuda.synchronize()
        avg_ms, min_ms, warm_n = time_launches(torch, stream, lambda: capi.check(lib.axhip_gemm(*args)), steps_f32, warmup_f32)
        flops = 2.0 * M * N * K
        res[f"gemm_nt_f32_{M}x{N}x{K}"] = {"avg_ms": avg_ms, "min_ms": min_ms, "warmup_launches": warm_n, "flops": flops, "tflops": flops / (avg_ms * 1e-3) / 1e12,
                                            "frac_of_f32_mfma_peak": flops / (avg_ms * 1e-3) / 1e12 / PEAK_F32_MFMA_TFLOPS,
                                            "finite": bool(torch.isfinite(c).all().item())}
        del a, w, c
    return res


def _oracle_build_flags() -> str:
    """The compiler line the oracle library was built with (oracle/Makefile), for the baseline's description."""
    cc, flags = "gcc", "?"
    for ln in (ROOT / "oracle" / "Makefile").read_text().splitlines():
        if ln.startswith("CFLAGS ?="):
            flags = ln.split("=", 1)[1].strip()
        if ln.startswith("CC ?="):
            cc = ln.split("=", 1)[1].strip()
    return f"{cc} {flags}"


def cpu_baseline(seconds_budget: float = 20.0):
    """Axiom's CPU flash attention (oracle restatement, native BLAS tier) on a bounded
    sample of the same workload: `n` (batch, head) slices of the bf16 S=4096 D=128 causal
    problem, all host threads.  Reported in the metric's unit over the algorithmic
    (causal) FLOP count, although the CPU algorithm also evaluates the masked blocks."""
    import numpy as np

    from oracle import axo

    S, D = 4096, 128
    threads = axo.num_threads()
    g = axo.PCG64(42)
    # calibrate with one slice per thread on a short sequence, then size the sample
    n = max(threads, 1)
    q, k, v = (axo.to_bits(g.normal((1, n, S, D)), axo.BF16) for _ in range(3))
    t0 = time.time()
    axo.sdpa(q[:, :, :512], k[:, :, :512], v[:, :, :512], axo.BF16, -1.0, True)
    t_small = time.time() - t0
    est_full = t_small * (S / 512) ** 2
    reps = 1
    if est_full > seconds_budget:  # keep the sample bounded: fewer slices
        n = max(1, int(n * seconds_budget / est_full))
    t0 = time.time()
    axo.sdpa(q[:, :n], k[:, :n], v[:, :n], axo.BF16, -1.0, True)
    dt = time.time() - t0
    flops = n * reps * 4.0 * S * S * D / 2.0
    return {
        "value": flops / dt / 1e12, "unit": "TFLOP/s", "cores": threads, "kind": "port",
        "sample": f"{n} of 128 (batch, head) slices of the bf16 B4 H32 S4096 D128 causal problem, {dt:.2f} s wall, "
                  f"tiled CPU flash attention (64x64 blocks, native sgemm tier, masked blocks not skipped), "
                  f"{threads} OpenMP threads; FLOPs counted as 4*S^2*D/2 per slice; built with `{_oracle_build_flags()}` "
                  f"(x86-64-v3 = AVX2+FMA, not -march=native: the library is compiled on another host than the one it is timed on)",
    }


def cpu_baselines_other_configs():
    """The oracle's restatement of Axiom's CPU path on the other configurations (BASELINE.json configs[0], [1], [2]
    and [4]) in full size, each in the unit of its GPU figure: one untimed pass, then the median of three."""
    import numpy as np

    from oracle import axo

    threads = axo.num_threads()
    g = axo.PCG64(42)
    how = f"{threads} OpenMP threads, 1 warm-up + median of 3 passes, built with `{_oracle_build_flags()}`"

    def median3(fn):
        fn()
        ts = []
        for _ in range(3):
            t0 = time.time()
            fn()
            ts.append(time.time() - t0)
        return sorted(ts)[1]

    res = {}
    # configs[0]: fp32 attention B1 H8 S512 D64
    q, k, v = (g.normal((1, 8, 512, 64)).astype(np.float32) for _ in range(3))
    t = median3(lambda: axo.sdpa(q, k, v, axo.F32, -1.0, False))
    res["c1_sdpa_f32_b1h8s512d64"] = {"value": 4.0 * 8 * 512 * 512 * 64 / t / 1e9, "unit": "GFLOP/s", "seconds": t, "cores": threads, "kind": "port",
                                      "sample": "the whole configuration; tiled CPU flash attention, native sgemm tier; " + how}
    # configs[1]: softmax((relu(a)+1)*b).sum(1), fp32 [8192, 8192], op by op as the CPU path runs it
    R = Cc = 8192
    a, b = g.normal((R, Cc)).astype(np.float32), g.normal((R, Cc)).astype(np.float32)
    t = median3(lambda: axo.chain_relu_add_mul_softmax_sum(a, b))
    res["c2_chain_f32_8192x8192"] = {"value": (2 * R * Cc * 4 + R * 4) / t / 1e9, "unit": "GB/s", "seconds": t, "cores": threads, "kind": "port",
                                     "sample": "the whole configuration; one pass per operation (relu, +1, *b, 3-pass softmax, row sum), "
                                               "rate over the fused kernel's algorithmic bytes; " + how}
    del a, b
    # configs[2]: gelu(layernorm(x)*gamma+beta) and the RMSNorm variant, bf16 [16384, 4096]
    R, Cc = 16384, 4096
    x = axo.to_bits(g.normal((R, Cc)), axo.BF16)
    gamma, beta = axo.to_bits(g.uniform((Cc,), 0.5, 1.5), axo.BF16), axo.to_bits(g.uniform((Cc,), -0.1, 0.1), axo.BF16)
    t = median3(lambda: axo.unary("gelu", axo.to_bits(axo.layer_norm(x, gamma, beta, axo.BF16, 1e-5), axo.BF16), axo.BF16))
    res["c3_gelu_layernorm_bf16_16384x4096"] = {"value": (2 * R * Cc * 2 + 2 * Cc * 2) / t / 1e9, "unit": "GB/s", "seconds": t, "cores": threads, "kind": "port",
                                                "sample": "the whole configuration; decomposed layer norm, conversion to bf16, gelu pass; rate over the fused "
                                                          "kernel's algorithmic bytes; " + how}
    t = median3(lambda: axo.unary("gelu", axo.to_bits(axo.rms_norm(x, gamma, axo.BF16, 1e-5), axo.BF16), axo.BF16))
    res["c3_gelu_rmsnorm_bf16_16384x4096"] = {"value": (2 * R * Cc * 2 + Cc * 2) / t / 1e9, "unit": "GB/s", "seconds": t, "cores": threads, "kind": "port",
                                              "sample": "as the layer-norm variant, with the decomposed RMS norm"}
    del x
    # configs[4]: x + out_proj(attention(q_proj x, k_proj x, v_proj x)), then layer norm; x [1500, 1280] bf16, 20 heads of 64
    S, Dm, Hh = 1500, 1280, 20
    xb = axo.to_bits(g.normal((S, Dm)), axo.BF16)
    w = [axo.to_bits(g.normal((Dm, Dm)) * 0.02, axo.BF16) for _ in range(4)]
    ones, zeros = axo.to_bits(np.ones(Dm), axo.BF16), axo.to_bits(np.zeros(Dm), axo.BF16)

    def block():
        heads = [np.ascontiguousarray(axo.matmul(xb, w[i], axo.BF16, False, True).reshape(1, S, Hh, Dm // Hh).transpose(0, 2, 1, 3)) for i in range(3)]
        o = axo.sdpa(heads[0], heads[1], heads[2], axo.BF16, -1.0, False)
        o = np.ascontiguousarray(o.transpose(0, 2, 1, 3)).reshape(S, Dm)
        y = axo.binary("add", xb, axo.matmul(o, w[3], axo.BF16, False, True), axo.BF16)
        return axo.layer_norm(y, ones, zeros, axo.BF16, 1e-5)

    t0 = time.time()  # its 16-bit x W^T is a plain triple loop on the CPU path: ~15 s a pass, so one pass only
    block()
    t = time.time() - t0
    res["c5_whisper_block_bf16_s1500_d1280_h20"] = {"value": (8.0 * S * Dm * Dm + 4.0 * S * S * Dm) / t / 1e9, "unit": "GFLOP/s", "seconds": t, "cores": threads,
                                                    "kind": "port", "sample": "the whole configuration; four x W^T on the native sgemm tier, tiled attention, "
                                                                              "residual add, decomposed layer norm; "
                                                                              f"ONE pass, no warm-up, {threads} OpenMP threads, built with `{_oracle_build_flags()}`"}
    return res


def host_layer_bench():
    """The same configurations along the whole drop-in path (C++ host layer: lazy graph, plan cache,
    caching allocator, launches, one device synchronisation per materialisation): wall-clock
    microseconds per materialisation from axiom_amd/lib/host_bench."""
    import subprocess

    exe = ROOT / "axiom_amd" / "lib" / "host_bench"
    if not exe.exists():
        return {"error": "axiom_amd/lib/host_bench is not built (python -m axiom_amd.build_host)"}
    p = subprocess.run([str(exe), "100", "20"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    if p.returncode != 0:
        return {"error": f"host_bench exited with {p.returncode}: {p.stderr[-300:]}"}
    return json.loads(p.stdout)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--min-warmup-ms", type=float, default=None, help="warm every kernel for at least this long (default 100)")
    ap.add_argument("--only", choices=["sdpa", "chains", "gemm", "f32", "survey"], default=None)
    args = ap.parse_args()
    if args.min_warmup_ms is not None:
        global MIN_WARMUP_MS
        MIN_WARMUP_MS = args.min_warmup_ms
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU (both hot paths shard without communication; "
              "no multi-GPU figure is produced). Re-run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    from axiom_amd import capi

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the gfx950 backend has no CPU fallback", file=sys.stderr)
        return 3
    capi.check(capi.lib().axhip_init(0))
    stream = torch.cuda.Stream()

    t_wall0 = time.time()
    sd = bench_sdpa(torch, capi, stream, args.steps, args.warmup) if args.only in (None, "sdpa") else None
    ch = bench_chains(torch, capi, stream, args.steps, args.warmup) if args.only in (None, "chains") else None
    gm = bench_gemm(torch, capi, stream, args.steps, args.warmup) if args.only in (None, "gemm") else None
    f32 = bench_f32(torch, capi, stream, args.steps, args.warmup) if args.only in (None, "f32") else None
    survey = bench_survey(torch, capi, stream, args.steps, args.warmup) if args.only == "survey" else None
    cpu = None if (args.no_cpu or sd is None) else cpu_baseline()
    cpu_other = None if (args.no_cpu or args.only is not None) else cpu_baselines_other_configs()
    traffic = traffic_from_profile()

    line = {
        "metric": "SDPA TFLOP/s (bf16 B4 H32 S4096 D128) + fused-chain HBM GB/s, % of peak",
        "value": sd["tflops"] if sd else None,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "warmup_launches_run": sd["warmup_launches"] if sd else None,
        "ms_per_step": sd["avg_ms"] if sd else None,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": "causal SDPA forward, bf16, B=4 H=32 S=4096 D=128, scale 1/sqrt(128), fp32 accumulate, bf16 out "
                               "(BASELINE.json configs[3]); inputs resident in HBM"},
    }
    if sd:
        line["roofline"] = {
            "bound": "mfma", "kernel": "sdpa_" + sd["kernel"], "achieved": sd["tflops"], "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s", "frac": sd["tflops"] / PEAK_BF16_TFLOPS, "traffic": traffic.get("sdpa_bf16_causal_b4h32s4096d128"),
            "traffic_source": str(TRAFFIC_PROFILE.relative_to(ROOT)),
            "algorithmic_flops_per_launch": sd["flops"], "avg_launch_ms": sd["avg_ms"], "min_launch_ms": sd["min_ms"],
        }
        line["output_finite"] = sd["finite"]
    if ch:
        for name, rec in ch.items():
            rec["traffic"] = traffic.get(name)
        line["fused_chains"] = ch
    if gm:
        line["gemm"] = gm
    if f32:
        line["f32_matrix_kernels"] = f32
    if survey:
        line["row_program_survey"] = survey
    if args.only is None:
        hl = host_layer_bench()
        # fractions of peak along the whole drop-in path: one materialisation with its own wait, and 16 queued per wait
        for rec in hl.values():
            if not isinstance(rec, dict):
                continue
            for key, peak, tag in (("GB_per_s", PEAK_HBM_GBS, "frac_of_hbm_peak"), ("GFLOP_per_s", PEAK_BF16_TFLOPS * 1e3, "frac_of_bf16_mfma_peak")):
                if key in rec:
                    rec[tag] = rec[key] / peak
                    if "queued_" + key in rec:
                        rec["queued_" + tag] = rec["queued_" + key] / peak
        line["host_layer"] = hl
    if cpu:
        line["cpu_baseline"] = cpu
    if cpu_other:
        # the GPU figure of the same configuration beside each CPU figure, in the same unit
        hl = line.get("host_layer", {})
        gpu = {"c1_sdpa_f32_b1h8s512d64": (f32 or {}).get("sdpa_f32_b1h8s512d64", {}).get("tflops", 0.0) * 1e3 or None,
               "c2_chain_f32_8192x8192": (ch or {}).get("chain_relu_add_mul_softmax_sum_f32_8192x8192", {}).get("gbs"),
               "c3_gelu_layernorm_bf16_16384x4096": (ch or {}).get("chain_gelu_layernorm_bf16_16384x4096", {}).get("gbs"),
               "c3_gelu_rmsnorm_bf16_16384x4096": (ch or {}).get("chain_gelu_rmsnorm_bf16_16384x4096", {}).get("gbs"),
               "c5_whisper_block_bf16_s1500_d1280_h20": hl.get("c5_whisper_block_bf16_s1500_d1280_h20", {}).get("GFLOP_per_s")}
        for name, rec in cpu_other.items():
            rec["gpu_value"] = gpu.get(name)
        line["cpu_baselines_other_configs"] = cpu_other
    line["bench_wall_s"] = time.time() - t_wall0
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
