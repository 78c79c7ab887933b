#!/usr/bin/env python3
"""Sweep of chill_attention over masks, sequence lengths and head shapes on one MI355X, next to
what PyTorch itself offers on the same GPU.  The counterpart of the reference's
benchmark/benchmark.py (same masks, shapes, dtype, input scale and correctness checks,
benchmark.py:26-75, 112-131, 216-239); timing is done with HIP events, optionally over a captured
HIP graph, instead of triton.testing.

    python chill-attention_amd/benchmark/benchmark.py [--providers chill,sdpa,flex] [--modes fwd,bwd]
        [--masks causal,full,...] [--points 4] [--max-time 6000] [--graph] [--out DIR]

providers
  chill  this package, through the public op (autograd included in "bwd" mode)
  sdpa   torch.nn.functional.scaled_dot_product_attention: is_causal for the causal mask, no mask
         for the full one, the dense boolean mask otherwise (the reference's "torch" line)
  flex   torch.compile(flex_attention) with the mask's make_flex_mask(); skipped with a note when
         the compiler stack of the box cannot build it

"bwd" times forward + backward of one call, as the reference does (benchmark.py:176-183).  TFLOP/s
count unmasked score entries only: 4 * B * H * D * nnz forward, 3.5 x that for forward + backward.
Writes results.csv and results.md under --out (default: benchmark/results).
"""

from __future__ import annotations

import argparse
import csv
import os
import sys
import time

import numpy as np
import torch
import torch.nn.functional as F

HERE = os.path.dirname(os.path.realpath(__file__))
sys.path.insert(0, os.path.join(HERE, ".."))

import chill_attention as ca  # noqa: E402

MASKS = {
    "sliding_window": lambda: ca.SlidingWindowChillMask(16, 16),
    "causal": lambda: ca.CausalChillMask(),
    "chunkwise": lambda: ca.ChunkwiseChillMask(16, 8),
    "prefix_lm": lambda: ca.PrefixLMChillMask(128),
    "full": lambda: ca.FullChillMask(),
}
SHAPES = {"small": dict(batch=8, heads=12, dim=64), "medium": dict(batch=8, heads=4, dim=128)}


def make_inputs(batch, heads, T, dim, dtype, device, seed):
    g = torch.Generator(device=device).manual_seed(seed)
    mk = lambda std: torch.empty(batch, heads, T, dim, dtype=torch.float32, device=device).normal_(0.0, std, generator=g)
    q, k, v = (mk(0.01).to(dtype).requires_grad_() for _ in range(3))
    do = mk(0.1)
    return q, k, v, do


def build_provider(provider, mask, q, k, v, T):
    """Returns a function () -> O, or raises if the provider cannot serve this case."""
    if provider == "chill":
        return lambda: ca.chill_attention(q, k, v, mask=mask)
    if provider == "sdpa":
        if isinstance(mask, ca.CausalChillMask):
            return lambda: F.scaled_dot_product_attention(q, k, v, is_causal=True)
        if isinstance(mask, ca.FullChillMask):
            return lambda: F.scaled_dot_product_attention(q, k, v)
        dense = mask.make_mask(T).to(q.device)
        return lambda: F.scaled_dot_product_attention(q, k, v, attn_mask=dense)
    if provider == "flex":
        from torch.nn.attention.flex_attention import flex_attention

        block_mask = mask.make_flex_mask(T)
        compiled = torch.compile(flex_attention)
        return lambda: compiled(q, k, v, block_mask=block_mask)
    raise ValueError(provider)


def time_ms(fn, use_graph, min_ms=200.0, max_iters=400):
    """Mean milliseconds per call, HIP events around a batch of calls sized to run >= min_ms."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    runner = fn
    if use_graph:
        # the library allocates nothing and every launch goes to the current stream, so a call can be
        # captured once and replayed; torch's allocations live in the graph's private pool
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        with torch.cuda.graph(graph):
            fn()
        runner = graph.replay
        runner()
        torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    runner()
    b.record()
    torch.cuda.synchronize()
    one = max(a.elapsed_time(b), 1e-3)
    iters = int(min(max_iters, max(5, min_ms / one)))
    a.record()
    for _ in range(iters):
        runner()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / iters


def run_case(provider, mode, mask, shape, T, dtype, use_graph, check):
    device = torch.device("cuda")
    q, k, v, do = make_inputs(shape["batch"], shape["heads"], T, shape["dim"], dtype, device, seed=T)
    fn = build_provider(provider, mask, q, k, v, T)
    note = ""
    if check:
        # the reference's checks (benchmark.py:216-239): O within 3e-3, gradients within 1e-2 of the
        # dense-mask SDPA result on the same inputs.  The oracle runs on fp32 copies of the inputs: in
        # fp16 PyTorch's dense-mask kernel is itself up to 3.5e-3 away from the fp32 result on these
        # inputs, which makes the 3e-3 check fail now and then whatever is being checked.
        ref, res_mask = ca._chill_reference_naive(mask, q.float(), k.float(), v.float(), None)
        out = fn()
        torch.testing.assert_close((out * res_mask.broadcast_to(out.shape)).float(), ref, atol=3e-3, rtol=0)
        if mode == "bwd" and provider != "flex":
            grads_ref = torch.autograd.grad(ref, (q, k, v), do.to(ref.dtype) * res_mask)
            grads = torch.autograd.grad(out, (q, k, v), do.to(out.dtype) * res_mask)
            for g, gr in zip(grads, grads_ref):
                torch.testing.assert_close(g.float(), gr.float(), atol=1e-2, rtol=0)
        del ref, out
        note = "checked"
    if mode == "fwd":
        def target():
            with torch.no_grad():
                return fn()
    else:
        dout = do.to(dtype)

        def target():
            q.grad = k.grad = v.grad = None
            fn().backward(dout)
    ms = time_ms(target, use_graph)
    nnz = mask.nnz(T)
    flops = 4.0 * shape["batch"] * shape["heads"] * shape["dim"] * nnz * (3.5 if mode == "bwd" else 1.0)
    return ms, flops / (ms * 1e-3) / 1e12, note


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--providers", default="chill,sdpa")
    ap.add_argument("--modes", default="fwd,bwd")
    ap.add_argument("--masks", default=",".join(MASKS))
    ap.add_argument("--shapes", default=",".join(SHAPES))
    ap.add_argument("--points", type=int, default=4)
    ap.add_argument("--max-time", type=int, default=6000)
    ap.add_argument("--dtype", default="f16", choices=["f16", "bf16"])
    ap.add_argument("--graph", action="store_true", help="time replays of a captured HIP graph")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--out", default=os.path.join(HERE, "results"))
    args = ap.parse_args()
    if not torch.cuda.is_available():
        sys.exit("benchmark.py: no GPU visible")
    dtype = {"f16": torch.float16, "bf16": torch.bfloat16}[args.dtype]
    times = sorted({int(t) for t in np.linspace(128, args.max_time, args.points)})
    os.makedirs(args.out, exist_ok=True)
    rows = []
    dead = set()  # providers that failed to build once are not tried again
    t_start = time.time()
    for mask_name in args.masks.split(","):
        mask = MASKS[mask_name]()
        for shape_name in args.shapes.split(","):
            shape = SHAPES[shape_name]
            for mode in args.modes.split(","):
                for T in times:
                    for provider in args.providers.split(","):
                        if provider in dead:
                            continue
                        tag = f"{mask} {shape_name} {mode} T={T} {provider}"
                        try:
                            ms, tflops, note = run_case(provider, mode, mask, shape, T, dtype,
                                                        args.graph and provider == "chill", not args.no_check)
                        except torch.OutOfMemoryError:
                            print(f"{tag}: out of memory, skipped", flush=True)
                            torch.cuda.empty_cache()
                            continue
                        except AssertionError as e:
                            print(f"{tag}: MISMATCH {str(e).splitlines()[0]}", flush=True)
                            rows.append([str(mask), shape_name, mode, T, provider, "", "", "mismatch"])
                            continue
                        except Exception as e:  # a provider the box cannot build (flex without a compiler)
                            if provider == "chill":
                                raise
                            print(f"{tag}: unavailable ({type(e).__name__}: {str(e)[:120]})", flush=True)
                            dead.add(provider)
                            continue
                        print(f"{tag}: {ms:.3f} ms {tflops:.1f} TFLOP/s {note} [{time.time() - t_start:.0f} s]", flush=True)
                        rows.append([str(mask), shape_name, mode, T, provider, f"{ms:.4f}", f"{tflops:.2f}", note])
    with open(os.path.join(args.out, "results.csv"), "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(["mask", "shape", "mode", "T", "provider", "ms", "tflops", "note"])
        w.writerows(rows)
    providers = [p for p in args.providers.split(",") if p not in dead]
    by_case = {}
    for mask_s, shape_name, mode, T, provider, ms, tflops, note in rows:
        by_case.setdefault((mask_s, shape_name, mode, T), {})[provider] = (ms, tflops)
    with open(os.path.join(args.out, "results.md"), "w") as f:
        f.write(f"dtype {args.dtype}, {torch.cuda.get_device_name(0)}, torch {torch.__version__}"
                f"{', chill timed as HIP-graph replays' if args.graph else ''}\n\n")
        f.write("| mask | shape | mode | T | " + " | ".join(f"{p} ms | {p} TFLOP/s" for p in providers) + " |\n")
        f.write("|---|---|---|---|" + "---|---|" * len(providers) + "\n")
        for (mask_s, shape_name, mode, T), res in by_case.items():
            cells = " | ".join(" | ".join(res.get(p, ("", ""))) for p in providers)
            f.write(f"| {mask_s} | {shape_name} | {mode} | {T} | {cells} |\n")
    print(f"wrote {args.out}/results.csv and results.md")


if __name__ == "__main__":
    main()
