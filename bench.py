#!/usr/bin/env python3
"""Benchmark of the MI355X chill-attention hot path.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3] [--mode fwd+bwd|fwd]

One "step" is one pass of the hot path over one batch of synthetic input that is already
resident in HBM: forward (chill_fwd) and, in fwd+bwd mode, the backward launches (chill_bwd_dq_delta, which
computes delta on its way, then chill_bwd_dkdv: what the operator's backward launches), all through the C ABI
on pre-allocated buffers.  Prints ONE JSON line.

  value      effective TFLOP/s over unmasked score entries (4*B*H*D*nnz forward, 2.5x for backward)
  roofline   for the kernel that takes the largest share of the step: algorithmic FLOPs per launch
             divided by its mean launch duration, measured here with HIP events on the launch stream
  cpu_baseline  the reference's CPU path (dense boolean mask -> torch SDPA on the host cores), timed
             on a bounded sample of the same workload

Only one GPU is used; --gpus N with N > 1 exits with a message.
"""

from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "chill-attention_amd"))

PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}  # MI355X dense MFMA
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch), scaled by what
# the same counters read for a plain 1 GiB copy in the same run (FETCH_SIZE x 2.000, WRITE_SIZE x 1.000).
# The figures come from the summary named in TRAFFIC_SOURCE, which records the digest of the kernel
# sources it was measured on (kernel_sources_digest below); with other sources the line reports null.
TRAFFIC_SOURCE = "profiles/c3_causal_bf16_fwd_bwd_kernels.md"
MEASURED_TRAFFIC = {
    ("C3", "chill_fwd"): (594702 * 2.0 + 344064) * 1024,
    ("C3", "chill_bwd_dq_delta"): (924862 * 2.0 + 290374) * 1024,
    ("C3", "chill_bwd_dkdv"): (830308 * 2.0 + 577536) * 1024,
}


def kernel_sources_digest():
    """sha1 over the kernel sources (csrc/*.h, *.hip, *.cpp, *.py, Makefile): names the build a profile
    summary belongs to."""
    import hashlib

    csrc = os.path.join(ROOT, "chill-attention_amd", "csrc")
    h = hashlib.sha1()
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".h", ".hip", ".cpp", ".py")) or name == "Makefile":
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:12]


def traffic_is_current():
    try:
        with open(os.path.join(ROOT, TRAFFIC_SOURCE)) as f:
            return f"kernel sources digest: {kernel_sources_digest()}" in f.read()
    except OSError:
        return False


class ClockSampler:
    """Shader clock (MHz) while the GPU works, as `rocm-smi --showclocks` reports it, sampled from a thread."""

    def __init__(self, period_s=0.4):
        import threading

        self.samples, self.period, self._stop = [], period_s, threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    def _run(self):
        import re
        import subprocess

        while not self._stop.is_set():
            try:
                out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=10).stdout
                m = re.search(r"sclk clock level[^\n]*\((\d+)Mhz\)", out)
                if m:
                    self.samples.append(int(m.group(1)))
            except Exception:
                return
            self._stop.wait(self.period)

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join(timeout=15)

    def mean(self):
        return sum(self.samples) / len(self.samples) if self.samples else None

# name -> (mask ctor name, args, dtype, B, H, T, D, seed, sigma)
WORKLOADS = {
    "C1": ("CausalChillMask", (), "f32", 1, 2, 256, 64, 0, 1.0),
    "C2": ("SlidingWindowChillMask", (128, 128), "bf16", 4, 16, 4096, 64, 1, 1.0),
    "C3": ("CausalChillMask", (), "bf16", 8, 16, 8192, 128, 2, 1.0),
    "C4": ("ChunkwiseChillMask", (128, 2), "f16", 2, 32, 16384, 128, 3, 0.5),
    "C5a": ("PrefixLMChillMask", (1024,), "bf16", 4, 32, 8192, 64, 4, 1.0),
    "C5b": ("PrefixLMChillMask", (1024,), "f32", 1, 8, 2048, 64, 4, 1.0),
    # not a BASELINE configuration: the widest head dim, for inspecting its kernels
    "D256": ("CausalChillMask", (), "bf16", 4, 8, 8192, 256, 5, 1.0),
}


def make_inputs(torch, B, H, T, D, dtype, seed, sigma, device):
    g = torch.Generator("cpu").manual_seed(seed)
    ts = [torch.randn(B, H, T, D, generator=g, dtype=torch.float32) * sigma for _ in range(4)]
    return [t.to(dtype).to(device) for t in ts]  # q, k, v, dO


def raising_q_tiles(torch, ca, mask, q, k, T, D, dname, heads=4):
    """Fraction of the forward's q-tiles in which at least one row has its softmax reference raised inside the
    loop, from a host-side model on `heads` (batch, head) slices: a row takes the max of the first 32-key block its
    wave visits as reference; the reference is raised when the exponents climb more than 40 (bf16) / 15 (fp16) log2
    units above it."""
    from chill_attention import _lib
    from chill_attention.tiles import tile_config

    dtype = q.dtype
    B, H = q.shape[:2]
    rows = tile_config(mask, D, dtype, _lib.PASS_FWD, seq_len=T, batch_heads=B * H)["rows"]
    dense = mask.make_mask(T).to(q.device)  # [T, T] bool
    c = D ** -0.5 * 1.4426950408889634
    first_key = dense.float().argmax(dim=1)  # first visible key of a row
    first_block = first_key.view(T // 32, 32).amin(dim=1) // 32  # first block of the wave that owns the row
    first_block = first_block.repeat_interleave(32)
    cols = torch.arange(T, device=q.device)
    in_first = (cols[None, :] // 32) == first_block[:, None]
    climb = 40.0 if dname == "bf16" else 15.0
    raising = total = 0
    for i in range(heads):
        b, h = (i * 7) % B, (i * 5) % H
        hk = h // (H // k.shape[1])
        s2 = ((q[b, h].float() * c).to(dtype).float() @ k[b, hk].float().T).masked_fill(~dense, float("-inf"))
        m0 = s2.masked_fill(~in_first, float("-inf")).amax(dim=1)
        m0 = torch.where(torch.isfinite(m0), m0, torch.zeros_like(m0))
        up = (s2.amax(dim=1) - m0) > climb
        raising += int(up.view(T // rows, rows).any(dim=1).sum())
        total += T // rows
    return {"fraction": raising / total, "q_tiles_sampled": total, "rows_per_q_tile": rows}


class Runner:
    """Pre-allocated buffers + raw C-ABI launches for one workload."""

    def __init__(self, torch, ca, mask, q, k, v, do, sm_scale):
        from chill_attention import _lib

        self.torch, self._lib, self.mask = torch, _lib, mask
        self.q, self.k, self.v, self.do = q, k, v, do
        B, H, T, D = q.shape
        self.shape = (B, H, k.shape[1], T, D)
        self.dtype = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[q.dtype]
        self.o = torch.empty_like(q)
        self.lse = torch.empty(B, H, T, dtype=torch.float32, device=q.device)
        self.delta = torch.empty(B, H, T, dtype=torch.float32, device=q.device)
        self.dq, self.dk, self.dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        self.desc = mask.descriptor()
        self.sm_scale = float(sm_scale)
        t4 = _lib.tensor4
        self.t = {n: t4(getattr(self, n)) for n in ("q", "k", "v", "do", "o", "dq", "dk", "dv")}
        self.s_lse, self.s_delta = _lib.strides3(self.lse), _lib.strides3(self.delta)
        self.stream = torch.cuda.current_stream().cuda_stream

    def _r(self, n):
        return ctypes.byref(self.t[n])

    def fwd(self):
        B, H, Hkv, T, D = self.shape
        L = self._lib
        L.check("chill_fwd", L.lib.chill_fwd(
            self._r("q"), self._r("k"), self._r("v"), self._r("o"), ctypes.c_void_p(self.lse.data_ptr()), self.s_lse,
            None, 0, B, H, Hkv, T, D, self.dtype, self.sm_scale, ctypes.byref(self.desc), ctypes.c_void_p(self.stream)))

    def delta_(self):
        B, H, Hkv, T, D = self.shape
        L = self._lib
        L.check("chill_bwd_delta", L.lib.chill_bwd_delta(
            self._r("o"), self._r("do"), ctypes.c_void_p(self.delta.data_ptr()), self.s_delta,
            B, H, T, D, self.dtype, ctypes.c_void_p(self.stream)))

    def dkdv(self):
        B, H, Hkv, T, D = self.shape
        L = self._lib
        L.check("chill_bwd_dkdv", L.lib.chill_bwd_dkdv(
            self._r("q"), self._r("k"), self._r("v"), self._r("do"), self._r("dk"), self._r("dv"),
            ctypes.c_void_p(self.lse.data_ptr()), self.s_lse, ctypes.c_void_p(self.delta.data_ptr()), self.s_delta,
            None, 0, B, H, Hkv, T, D, self.dtype, self.sm_scale, ctypes.byref(self.desc), ctypes.c_void_p(self.stream)))

    def dq_(self):
        B, H, Hkv, T, D = self.shape
        L = self._lib
        L.check("chill_bwd_dq", L.lib.chill_bwd_dq(
            self._r("q"), self._r("k"), self._r("v"), self._r("do"), self._r("dq"),
            ctypes.c_void_p(self.lse.data_ptr()), self.s_lse, ctypes.c_void_p(self.delta.data_ptr()), self.s_delta,
            None, 0, B, H, Hkv, T, D, self.dtype, self.sm_scale, ctypes.byref(self.desc), ctypes.c_void_p(self.stream)))

    def dq_delta_(self):
        B, H, Hkv, T, D = self.shape
        L = self._lib
        L.check("chill_bwd_dq_delta", L.lib.chill_bwd_dq_delta(
            self._r("q"), self._r("k"), self._r("v"), self._r("o"), self._r("do"), self._r("dq"),
            ctypes.c_void_p(self.lse.data_ptr()), self.s_lse, ctypes.c_void_p(self.delta.data_ptr()), self.s_delta,
            None, 0, B, H, Hkv, T, D, self.dtype, self.sm_scale, ctypes.byref(self.desc), ctypes.c_void_p(self.stream)))

    def kernels(self, mode, separate_delta=False):
        """The launches of one step.  separate_delta: the backward as the three launches of the reference's
        structure (delta, dK/dV, dQ) instead of the two the operator uses."""
        ks = [("chill_fwd", self.fwd)]
        if mode == "fwd+bwd" and separate_delta:
            ks += [("chill_bwd_delta", self.delta_), ("chill_bwd_dkdv", self.dkdv), ("chill_bwd_dq", self.dq_)]
        elif mode == "fwd+bwd":
            ks += [("chill_bwd_dq_delta", self.dq_delta_), ("chill_bwd_dkdv", self.dkdv)]
        return ks


def cpu_baseline(torch, mask_name, margs, dtype_name, T, D, mode, seed, sigma, budget_s=15.0):
    """Reference CPU path on a bounded sample: dense mask -> torch SDPA (fp32 on upcast inputs, as
    the reference's tests run it), one (batch, head) slice of the workload at full T per call,
    repeated for about budget_s seconds (at least 3 calls, at most 64)."""
    sys.path.insert(0, ROOT)
    from oracle import chill_oracle as orc

    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except AttributeError:
        pass
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    q, k, v, do = make_inputs(torch, 1, 1, T, D, torch.float32, seed, sigma, "cpu")
    times = []
    t_begin = time.perf_counter()
    while True:
        qq, kk, vv = (x.clone().requires_grad_(mode == "fwd+bwd") for x in (q, k, v))
        t0 = time.perf_counter()
        out, _ = orc.reference_naive(mask_name, margs, qq, kk, vv, None)
        if mode == "fwd+bwd":
            out.backward(do)
        times.append(time.perf_counter() - t0)
        elapsed = time.perf_counter() - t_begin
        if (elapsed > budget_s and len(times) >= 3) or len(times) >= 64 or elapsed > 4 * budget_s:
            break
    used = times[1:] if len(times) > 1 else times  # the first run warms the allocator up
    timed = len(used)
    sec = sum(used) / timed
    fl = orc.flops(mask_name, margs, 1, 1, T, D, mode)
    return {
        "value": fl / sec / 1e12,
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"1 (batch, head) slice of the workload at full T={T}, D={D}, fp32 dense-mask torch SDPA "
                  f"{mode}, mean of {timed} run(s), {sec:.2f} s each",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3", choices=sorted(WORKLOADS))
    ap.add_argument("--mode", default="fwd+bwd", choices=["fwd", "fwd+bwd"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--separate-delta", action="store_true",
                    help="time the backward as three launches (delta, dK/dV, dQ) instead of the operator's two")
    ap.add_argument("--sustained-seconds", type=float, default=3.0,
                    help="length of the continuous loop behind the `sustained` figure (0: leave it out)")
    ap.add_argument("--sigma", type=float, default=None,
                    help="standard deviation of q, k, v, dO instead of the workload's (inspection: the forward of "
                         "16-bit inputs at head dims 64 and 128 raises a row's softmax reference only when the "
                         "exponents climb far above it; the line then carries `fwd_q_tiles_raising_reference`)")
    ap.add_argument("--dtype", default=None, choices=["f32", "f16", "bf16"], help="element type instead of the workload's")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also launch one plain 1 GiB device copy (1 GiB read + 1 GiB written) before the warm-up: "
                         "the known-size dispatch that scales the FETCH_SIZE / WRITE_SIZE counters of a "
                         "rocprofv3 --pmc run")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build measures ONE MI355X; every box has one GPU and the hot path "
                 "shards over (batch, head) without communication, so --gpus must be 1")

    import torch

    import chill_attention as ca

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    mask_name, margs, dname, B, H, T, D, seed, sigma = WORKLOADS[args.workload]
    mode = "fwd" if args.workload == "C1" else args.mode
    if args.sigma is not None:
        sigma = args.sigma
    if args.dtype is not None:
        dname = args.dtype
    dtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dname]
    mask = getattr(ca, mask_name)(*margs)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    q, k, v, do = make_inputs(torch, B, H, T, D, dtype, seed, sigma, dev)
    run = Runner(torch, ca, mask, q, k, v, do, D ** -0.5)
    kernels = run.kernels(mode, args.separate_delta)

    if args.copy_probe:
        src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        for _, fn in kernels:
            fn()
    torch.cuda.synchronize()

    # per-kernel HIP events on the launch stream (torch's current stream) + whole-step wall clock
    ev = [[(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in kernels]
          for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for s in range(args.steps):
        for i, (_, fn) in enumerate(kernels):
            ev[s][i][0].record()
            fn()
            ev[s][i][1].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    per_launch = [[ev[s][i][0].elapsed_time(ev[s][i][1]) for s in range(args.steps)] for i in range(len(kernels))]
    k_ms = [sum(x) / len(x) for x in per_launch]
    k_min = [min(x) for x in per_launch]
    k_med = [sorted(x)[len(x) // 2] for x in per_launch]

    nnz = mask.nnz(T)
    fwd_flops = 4.0 * B * H * D * nnz
    step_flops = fwd_flops * (3.5 if mode == "fwd+bwd" else 1.0)
    value = step_flops / (ms_per_step * 1e-3) / 1e12
    peak = PEAK_TFLOPS[dname]

    # The timed region above is short (the board has not settled at its power limit yet).  `sustained`: the
    # same launches in one continuous loop of a few seconds, with the shader clock sampled meanwhile.
    sustained = None
    if args.sustained_seconds > 0:
        n_loop = max(int(args.sustained_seconds / (ms_per_step * 1e-3)), args.steps)
        with ClockSampler() as clock:
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(n_loop):
                for _, fn in kernels:
                    fn()
            torch.cuda.synchronize()
            loop_s = time.perf_counter() - t0
        sustained = {"value": step_flops * n_loop / loop_s / 1e12, "unit": "TFLOP/s", "steps": n_loop,
                     "seconds": loop_s, "ms_per_step": loop_s * 1e3 / n_loop, "sm_clock_mhz": clock.mean(),
                     "frac_of_peak": step_flops * n_loop / loop_s / 1e12 / peak}

    # the same step through the public operator (chill_attention + autograd): allocation and dispatch included
    op_ms = None
    if args.sustained_seconds > 0:
        qa, ka, va = (x.detach().clone().requires_grad_(mode == "fwd+bwd") for x in (q, k, v))

        def op_step():
            o = ca.chill_attention(qa, ka, va, mask=mask)
            if mode == "fwd+bwd":
                o.backward(do)
                qa.grad = ka.grad = va.grad = None

        for _ in range(3):
            op_step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            op_step()
        torch.cuda.synchronize()
        op_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # algorithmic FLOPs per launch: forward 4*D per unmasked entry (2 GEMMs); of the backward's
    # 10*D (5 GEMMs: S, dP, dV, dK, dQ) the dK/dV kernel is charged S, dP, dV, dK = 8*D and the dQ
    # kernel dQ = 2*D (its own S and dP are recomputation, not algorithmic work)
    per_entry = {"chill_fwd": 4.0, "chill_bwd_dkdv": 8.0, "chill_bwd_dq": 2.0, "chill_bwd_dq_delta": 2.0, "chill_bwd_delta": 0.0}
    es = 4 if dname == "f32" else 2
    dom = max(range(len(kernels)), key=lambda i: k_ms[i])
    dom_name = kernels[dom][0]
    alg_bytes = {
        "chill_fwd": 4.0 * B * H * T * D * es + 4.0 * B * H * T,
        "chill_bwd_delta": 2.0 * B * H * T * D * es + 4.0 * B * H * T,
        "chill_bwd_dkdv": 6.0 * B * H * T * D * es + 8.0 * B * H * T,
        "chill_bwd_dq": 5.0 * B * H * T * D * es + 8.0 * B * H * T,
        "chill_bwd_dq_delta": 6.0 * B * H * T * D * es + 8.0 * B * H * T,
    }
    alg_flops = per_entry[dom_name] * B * H * D * nnz
    # the roof that bounds the kernel: max(FLOPs / peak, algorithmic bytes / HBM bandwidth)
    t_mfma = alg_flops / (peak * 1e12)
    t_hbm = alg_bytes[dom_name] / (PEAK_HBM_GBS * 1e9)
    if t_hbm >= t_mfma:
        roof = {"kernel": dom_name, "bound": "hbm", "achieved": alg_bytes[dom_name] / (k_ms[dom] * 1e-3) / 1e9,
                "peak": PEAK_HBM_GBS, "unit": "GB/s"}
    else:
        roof = {"kernel": dom_name, "bound": "mfma", "achieved": alg_flops / (k_ms[dom] * 1e-3) / 1e12, "peak": peak,
                "unit": "TFLOP/s"}
    roof["bound_ms"] = {"mfma": t_mfma * 1e3, "hbm": t_hbm * 1e3}
    roof["frac"] = roof["achieved"] / roof["peak"]
    current = traffic_is_current()
    roof["traffic"] = MEASURED_TRAFFIC.get((args.workload, dom_name)) if current else None
    roof["traffic_unit"] = "bytes per launch (rocprofv3 FETCH_SIZE + WRITE_SIZE, copy-scaled)"
    roof["traffic_source"] = TRAFFIC_SOURCE if current else f"none: {TRAFFIC_SOURCE} was measured on other kernel sources"
    roof["algorithmic_bytes"] = alg_bytes[dom_name]
    roof["avg_launch_ms"] = k_ms[dom]

    out = {
        "metric": f"effective TFLOP/s {mode}, {mask} {dname} B{B} H{H} T{T} D{D}",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dname,
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: {mask} {mode} {dname} B={B} H={H} T={T} D={D} seed={seed} "
                               f"sigma={sigma}, inputs resident in HBM"},
        "frac_of_peak": value / peak,
        "kernel_ms": {kernels[i][0]: k_ms[i] for i in range(len(kernels))},
        "kernel_ms_median": {kernels[i][0]: k_med[i] for i in range(len(kernels))},
        "kernel_ms_min": {kernels[i][0]: k_min[i] for i in range(len(kernels))},
        "fwd_tflops": fwd_flops / (k_ms[0] * 1e-3) / 1e12,
        "fwd_frac_of_peak": fwd_flops / (k_ms[0] * 1e-3) / 1e12 / peak,
        "roofline": roof,
        "kernel_frac_of_own_roof": {
            kernels[i][0]: max(per_entry[kernels[i][0]] * B * H * D * nnz / (peak * 1e12),
                               alg_bytes[kernels[i][0]] / (PEAK_HBM_GBS * 1e9)) / (k_ms[i] * 1e-3)
            for i in range(len(kernels))},
        # the matrix work each kernel EXECUTES (dQ recomputes S and dP: 6*D per entry for its algorithmic 2*D)
        # over its time, as a fraction of the peak
        "kernel_executed_frac_of_peak": {
            kernels[i][0]: {"chill_fwd": 4.0, "chill_bwd_dkdv": 8.0, "chill_bwd_dq": 6.0, "chill_bwd_dq_delta": 6.0}[kernels[i][0]] * B * H * D * nnz
            / (k_ms[i] * 1e-3) / (peak * 1e12)
            for i in range(len(kernels)) if kernels[i][0] != "chill_bwd_delta"},
        "sustained": sustained,
        "sm_clock_mhz": sustained["sm_clock_mhz"] if sustained else None,
        "operator_ms_per_step": op_ms,
        "kernel_sources_digest": kernel_sources_digest(),
    }
    if args.sigma is not None and dname != "f32" and D in (64, 128):
        out["fwd_q_tiles_raising_reference"] = raising_q_tiles(torch, ca, mask, q, k, T, D, dname)
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, mask_name, margs, dname, T, D, mode, seed, sigma)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
