"""Seeded random sweep over the op's argument surface: mask class and arguments, dtype, head dim,
GQA group, sequence length (not a multiple of anything), lens, strided views.  Every case is
checked against the oracle (dense mask -> torch SDPA + autograd on fp32-upcast inputs) at the
tolerances of the reference's own tests (test_chill_attention.py:167-172, 316-321) and, for head
dims >= 64, at the benchmark's atol = rtol (1e-2 for the 16-bit types, 1e-4 for fp32) as well."""

import numpy as np
import pytest
import torch

import chill_attention as ca
from oracle import chill_oracle as orc
from test_attention_gpu import check_close

pytestmark = pytest.mark.gpu
DEV = "cuda"
OUT_TOL = {torch.float32: (2e-6, 1e-4), torch.float16: (1e-2, 1e-3), torch.bfloat16: (5e-2, 1e-2)}
GRAD_TOL = {torch.float32: (5e-5, 1e-3), torch.float16: (5e-3, 1e-3), torch.bfloat16: (1e-1, 1e-2)}


def draw_case(rng):
    T = int(rng.choice([1, 2, 31, 33, 64, 65, 127, 129, 255, 257, 300, 511, 513, 640, 777]))
    kind = rng.choice(["Full", "Causal", "SlidingWindow", "Chunkwise", "PrefixLM"])
    if kind == "SlidingWindow":
        args = (int(rng.integers(0, 2 * T + 2)), int(rng.integers(0, 2 * T + 2)))
    elif kind == "Chunkwise":
        args = (int(rng.integers(1, T + 40)), int(rng.integers(0, 5)))
    elif kind == "PrefixLM":
        args = (int(rng.integers(0, T + 40)),)
    else:
        args = ()
    dtype = [torch.float32, torch.float16, torch.bfloat16][int(rng.integers(0, 3))]
    D = int(rng.choice([16, 32, 64, 128, 256]))
    Hkv = int(rng.choice([1, 2, 3]))
    H = Hkv * int(rng.choice([1, 2, 4]))
    B = int(rng.choice([1, 2, 3]))
    lens_kind = rng.choice(["none", "random", "short"])
    layout = rng.choice(["contiguous", "bthd", "padded"])
    return kind + "ChillMask", args, dtype, B, H, Hkv, T, D, lens_kind, layout


def make(shape, dtype, layout, gen):
    B, H, T, D = shape
    if layout == "bthd":  # [B, T, H, D] memory seen as [B, H, T, D]
        return torch.randn(B, T, H, D, device=DEV, dtype=dtype, generator=gen).transpose(1, 2)
    if layout == "padded":  # rows inside a wider buffer
        return torch.randn(B, H, T, D + 8, device=DEV, dtype=dtype, generator=gen)[..., :D]
    return torch.randn(B, H, T, D, device=DEV, dtype=dtype, generator=gen)


@pytest.mark.parametrize("seed", range(48))
def test_random_case(seed):
    rng = np.random.default_rng(1000 + seed)
    name, args, dtype, B, H, Hkv, T, D, lens_kind, layout = draw_case(rng)
    gen = torch.Generator(DEV).manual_seed(seed)
    mask = getattr(ca, name)(*args)
    q = make((B, H, T, D), dtype, layout, gen).requires_grad_(True)
    k = make((B, Hkv, T, D), dtype, layout, gen).requires_grad_(True)
    v = make((B, Hkv, T, D), dtype, layout, gen).requires_grad_(True)
    do = make((B, H, T, D), dtype, "contiguous", gen)
    lens = None
    if lens_kind == "random":
        lens = torch.from_numpy(rng.integers(0, T + 1, size=B).astype(np.int32)).to(DEV)
    elif lens_kind == "short":
        lens = torch.from_numpy(rng.integers(0, min(T, 3) + 1, size=B).astype(np.int32)).to(DEV)
    print(f"seed {seed}: {mask} {dtype} B{B} H{H}/{Hkv} T{T} D{D} lens={None if lens is None else lens.tolist()} {layout}", flush=True)
    out, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens, return_lse=True)
    out.backward(do)
    qr, kr, vr = (x.detach().float().clone().requires_grad_(True) for x in (q, k, v))
    ref, res_mask = orc.reference_naive(name, args, qr, kr, vr, lens)
    (ref * res_mask).backward(do.float() * res_mask)
    assert out.shape == q.shape and lse.shape == q.shape[:3]
    check_close(out.detach() * res_mask, (ref * res_mask).detach(), dtype, OUT_TOL[dtype], D, "O")
    for nm, got, want in (("dq", q.grad, qr.grad), ("dk", k.grad, kr.grad), ("dv", v.grad, vr.grad)):
        assert got.shape == want.shape
        check_close(got, want, dtype, GRAD_TOL[dtype], D, nm)
    # rows at or beyond lens are exactly zero in the output and in dQ
    if lens is not None:
        dead = ~(torch.arange(T, device=DEV)[None, :] < lens[:, None])
        assert (out.detach().transpose(1, 2)[dead] == 0).all() and (q.grad.transpose(1, 2)[dead] == 0).all()
