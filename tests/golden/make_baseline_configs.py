"""Writes tests/golden/baseline_configs.json: the five benchmark configurations with the unmasked
entry counts and forward GFLOP figures from an independent hand derivation
(closed forms per mask and the reference's FLOP convention, benchmark/benchmark.py:271-276).
The numbers are typed in, NOT computed by this repository's code, so they are an
independent check of the oracle's nnz() / flops().

    python tests/golden/make_baseline_configs.py
"""

import json
import os

CONFIGS = [
    dict(name="C1", mask="CausalChillMask", args=[], dtype="f32", B=1, H=2, T=256, D=64, seed=0, sigma=1.0,
         nnz_per_head=32896, fwd_gflop=0.017),
    dict(name="C2", mask="SlidingWindowChillMask", args=[128, 128], dtype="bf16", B=4, H=16, T=4096, D=64, seed=1,
         sigma=1.0, nnz_per_head=1036160, fwd_gflop=16.98),
    dict(name="C3", mask="CausalChillMask", args=[], dtype="bf16", B=8, H=16, T=8192, D=128, seed=2, sigma=1.0,
         nnz_per_head=33558528, fwd_gflop=2199.3),
    dict(name="C4", mask="ChunkwiseChillMask", args=[128, 2], dtype="f16", B=2, H=32, T=16384, D=128, seed=3,
         sigma=0.5, nnz_per_head=6242304, fwd_gflop=204.6),
    dict(name="C5a", mask="PrefixLMChillMask", args=[1024], dtype="bf16", B=4, H=32, T=8192, D=64, seed=4, sigma=1.0,
         nnz_per_head=34082304, fwd_gflop=1116.8),
    dict(name="C5b", mask="PrefixLMChillMask", args=[1024], dtype="f32", B=1, H=8, T=2048, D=64, seed=4, sigma=1.0,
         nnz_per_head=2621952, fwd_gflop=5.37),
]

if __name__ == "__main__":
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "baseline_configs.json")
    with open(out, "w") as f:
        json.dump({"source": "hand-derived closed forms for the benchmark configurations of alexdremov/chill-attention v2.1.0", "configs": CONFIGS}, f, indent=1)
    print("wrote", out)
