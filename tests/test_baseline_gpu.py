"""The five BASELINE configurations at their full sizes.

Inputs follow the benchmark protocol: q, k, v, dO drawn in that order from
torch.Generator('cpu').manual_seed(seed) as fp32 N(0, sigma), cast to the config dtype.  Checked
  * against the oracle (dense mask -> torch SDPA + autograd on fp32-upcast inputs) on eight (batch, head)
    slices per configuration (every one for the small ones), spread over the work-item order of the
    launch (first, last and middle items of the runs the eight XCDs get), with the tolerance of the
    benchmark definition: atol = rtol = 1e-2 for bf16 / fp16, 1e-4 for fp32 (O, dQ, dK, dV); the largest
    errors are printed;
  * through size-independent properties on the full outputs: V = 1 gives O = 1 (rows of P sum to 1),
    O stays inside [min V, max V], sum(dQ*Q) == sum(dK*K), and a (batch, head) slice run alone stays
    within the same tolerance (bit for bit where the slice's launch uses the same tile shape).
"""

import json
import os

import pytest
import torch

import chill_attention as ca
from oracle import chill_oracle as orc

pytestmark = pytest.mark.gpu
DEV = "cuda"
with open(os.path.join(os.path.dirname(__file__), "golden", "baseline_configs.json")) as f:
    CONFIGS = {c["name"]: c for c in json.load(f)["configs"]}
DT = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
TOL = {torch.float32: 1e-4, torch.float16: 1e-2, torch.bfloat16: 1e-2}


def oracle_slices(B, H):
    """(batch, head) pairs for the oracle.  Work items are (batch * H + head) * tiles + tile, dealt to
    the 8 XCDs in contiguous runs: the first and the last item, items on both sides of XCD run
    boundaries, and some from the middle of runs."""
    n = B * H
    if n <= 8:
        return [(i // H, i % H) for i in range(n)]
    per = -(-n // 8)
    picks = {0, n - 1, per - 1, per, 3 * per + per // 2, 4 * per - 1, 4 * per, 6 * per + 1}
    return [(i // H, i % H) for i in sorted(min(max(i, 0), n - 1) for i in picks)]


def report(name, what, got, want):
    diff = (got.float() - want.float()).abs()
    rel = (diff / want.float().abs().clamp_min(1e-3)).max().item()
    print(f"  {name} {what}: max abs err {diff.max().item():.3e}, max rel err (|want| >= 1e-3) {rel:.3e}", flush=True)


def inputs(c):
    g = torch.Generator("cpu").manual_seed(c["seed"])
    shape = (c["B"], c["H"], c["T"], c["D"])
    return [(torch.randn(shape, generator=g, dtype=torch.float32) * c["sigma"]).to(DT[c["dtype"]]).to(DEV) for _ in range(4)]


@pytest.mark.parametrize("name", ["C1", "C2", "C3", "C4", "C5a", "C5b"])
def test_baseline_config(name):
    c = CONFIGS[name]
    dtype = DT[c["dtype"]]
    tol = TOL[dtype]
    mask = getattr(ca, c["mask"])(*c["args"])
    q, k, v, do = inputs(c)
    fwd_only = name == "C1"
    for x in (q, k, v):
        x.requires_grad_(not fwd_only)
    print(f"baseline {name}: {mask} {dtype} B{c['B']} H{c['H']} T{c['T']} D{c['D']}", flush=True)
    out, lse = ca.chill_attention(q, k, v, mask=mask, return_lse=True)
    if not fwd_only:
        out.backward(do)
    torch.cuda.synchronize()
    assert torch.isfinite(out).all() and torch.isfinite(lse).all()

    # oracle on a few (batch, head) slices
    from chill_attention import _lib
    from chill_attention.tiles import tile_config

    slices = oracle_slices(c["B"], c["H"])
    assert len(slices) >= min(8, c["B"] * c["H"])
    for b, h in slices:
        qs, ks, vs = (x.detach()[b : b + 1, h : h + 1].float().clone().requires_grad_(not fwd_only) for x in (q, k, v))
        ref, _ = orc.reference_naive(c["mask"], tuple(c["args"]), qs, ks, vs, None)
        report(name, f"slice {(b, h)} O", out.detach()[b : b + 1, h : h + 1], ref.detach().to(dtype))
        torch.testing.assert_close(out.detach()[b : b + 1, h : h + 1], ref.detach().to(dtype), atol=tol, rtol=tol)
        if not fwd_only:
            ref.backward(do[b : b + 1, h : h + 1].float())
            for nm, got, want in (("dq", q.grad, qs.grad), ("dk", k.grad, ks.grad), ("dv", v.grad, vs.grad)):
                report(name, f"slice {(b, h)} {nm}", got[b : b + 1, h : h + 1], want.to(dtype))
                torch.testing.assert_close(got[b : b + 1, h : h + 1], want.to(dtype), atol=tol, rtol=tol, msg=lambda s: f"{name} {nm} slice {(b, h)}: {s}")
        del ref, qs, ks, vs
    # a slice run on its own is the same computation: within the tolerance always, and bit-identical when
    # its launch takes the same row of the tile table (small launches take the short-sequence row)
    for b, h in (slices[0], slices[-1]):
        with torch.no_grad():
            alone = ca.chill_attention(q.detach()[b : b + 1, h : h + 1], k.detach()[b : b + 1, h : h + 1], v.detach()[b : b + 1, h : h + 1], mask=mask)
        full = out.detach()[b : b + 1, h : h + 1]
        torch.testing.assert_close(alone, full, atol=tol, rtol=tol)
        same_shape = (tile_config(mask, c["D"], dtype, _lib.PASS_FWD, seq_len=c["T"], batch_heads=1)
                      == tile_config(mask, c["D"], dtype, _lib.PASS_FWD, seq_len=c["T"], batch_heads=c["B"] * c["H"]))
        if same_shape:
            assert torch.equal(alone, full)

    # properties on the full tensors
    with torch.no_grad():
        vmin = v.detach().float().amin(dim=2, keepdim=True)
        vmax = v.detach().float().amax(dim=2, keepdim=True)
        o32 = out.detach().float()
        slack = 2e-2 if dtype != torch.float32 else 1e-5
        assert (o32 <= vmax + slack * (1 + vmax.abs())).all() and (o32 >= vmin - slack * (1 + vmin.abs())).all()
        ones = ca.chill_attention(q.detach(), k.detach(), torch.ones_like(v), mask=mask)
        torch.testing.assert_close(ones.float(), torch.ones_like(o32), atol=1e-2 if dtype != torch.float32 else 1e-5, rtol=0)
        if not fwd_only:
            assert all(torch.isfinite(x.grad).all() for x in (q, k, v))
            a = (q.grad.double() * q.detach().double()).sum()
            b_ = (k.grad.double() * k.detach().double()).sum()
            scale = (q.grad.double() * q.detach().double()).abs().sum()
            assert abs(a - b_) <= 2e-3 * scale, (a.item(), b_.item(), scale.item())


def test_c1_against_cpu_oracle_f64():
    """C1 is small enough for the textbook float64 oracle on the CPU, LSE2 included."""
    c = CONFIGS["C1"]
    q, k, v, _ = inputs(c)
    out, lse = ca.chill_attention(q, k, v, mask=ca.CausalChillMask(), return_lse=True)
    ref = orc.attention_f64(c["mask"], (), q.cpu().numpy(), k.cpu().numpy(), v.cpu().numpy())
    torch.testing.assert_close(out.cpu().double(), torch.from_numpy(ref["o"]), atol=1e-4, rtol=1e-4)
    torch.testing.assert_close(lse.cpu().double(), torch.from_numpy(ref["lse2"]), atol=1e-4, rtol=1e-5)
