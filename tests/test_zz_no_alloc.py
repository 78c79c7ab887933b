"""The backward entry point that takes no delta workspace (chill_bwd_noalloc) against the two entry
points it stands for (chill_bwd_dq_delta + chill_bwd_dkdv with a caller-owned delta), through
the C ABI: two calls in a row, the second with a smaller input, so that what the first call left in the
library's array cannot pass for the second call's rows.  Integer-exact comparison: the same kernels run on
the same values."""

import ctypes

import pytest
import torch

import chill_attention as ca
from chill_attention import _lib

pytestmark = pytest.mark.gpu
DEV = "cuda"


def backward_both_ways(mask, B, H, Hkv, T, D, dtype, lens, seed):
    g = torch.Generator(DEV).manual_seed(seed)
    q = torch.randn(B, H, T, D, device=DEV, dtype=dtype, generator=g)
    k = torch.randn(B, Hkv, T, D, device=DEV, dtype=dtype, generator=g)
    v = torch.randn(B, Hkv, T, D, device=DEV, dtype=dtype, generator=g)
    do = torch.randn(B, H, T, D, device=DEV, dtype=dtype, generator=g)
    o, lse = ca.chill_attention(q, k, v, mask=mask, lens=lens, return_lse=True)
    code = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}[dtype]
    desc = mask.descriptor()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    lens_p = (None, 0) if lens is None else (ctypes.c_void_p(lens.data_ptr()), lens.stride(0))
    t = {n: _lib.tensor4(x) for n, x in (("q", q), ("k", k), ("v", v), ("o", o), ("do", do))}
    r = lambda n: ctypes.byref(t[n])
    lse_p, s_lse = ctypes.c_void_p(lse.data_ptr()), _lib.strides3(lse)
    sm_scale = D ** -0.5

    def outputs():
        out = {"dq": torch.full_like(q, float("nan")), "dk": torch.full_like(k, float("nan")), "dv": torch.full_like(v, float("nan"))}
        return out, {n: _lib.tensor4(x) for n, x in out.items()}

    # the existing entry points, with a delta buffer of the caller
    want, tw = outputs()
    delta = torch.empty(B, H, T, dtype=torch.float32, device=DEV)
    delta_p, s_delta = ctypes.c_void_p(delta.data_ptr()), _lib.strides3(delta)
    L = _lib.lib
    _lib.check("chill_bwd_dq_delta", L.chill_bwd_dq_delta(r("q"), r("k"), r("v"), r("o"), r("do"), ctypes.byref(tw["dq"]), lse_p, s_lse,
                                                          delta_p, s_delta, *lens_p, B, H, Hkv, T, D, code, sm_scale, ctypes.byref(desc), stream))
    _lib.check("chill_bwd_dkdv", L.chill_bwd_dkdv(r("q"), r("k"), r("v"), r("do"), ctypes.byref(tw["dk"]), ctypes.byref(tw["dv"]),
                                                  lse_p, s_lse, delta_p, s_delta, *lens_p, B, H, Hkv, T, D, code, sm_scale,
                                                  ctypes.byref(desc), stream))
    # the entry point without a workspace
    got, tg = outputs()
    _lib.check("chill_bwd_noalloc", L.chill_bwd_noalloc(
        r("q"), r("k"), r("v"), r("o"), r("do"), ctypes.byref(tg["dq"]), ctypes.byref(tg["dk"]), ctypes.byref(tg["dv"]),
        lse_p, s_lse, *lens_p, B, H, Hkv, T, D, code, sm_scale, ctypes.byref(desc), stream))
    torch.cuda.synchronize()
    return got, want


def test_backward_without_workspace_equals_backward_with_one():
    cases = [
        # the first call fills many rows of the library's array ...
        (ca.CausalChillMask(), 2, 8, 2, 1500, 128, torch.bfloat16, None),
        # ... the second is smaller (fewer rows, other head count, lens): stale rows would show
        (ca.SlidingWindowChillMask(37, 5), 3, 2, 2, 333, 64, torch.float32, [333, 100, 0]),
        (ca.PrefixLMChillMask(50), 1, 4, 1, 200, 64, torch.float16, None),
    ]
    for i, (mask, B, H, Hkv, T, D, dtype, lens) in enumerate(cases):
        lens_t = None if lens is None else torch.tensor(lens, dtype=torch.int32, device=DEV)
        print(f"no-alloc backward, call {i}: {mask} {dtype} B{B} H{H}/{Hkv} T{T} D{D} lens={lens}", flush=True)
        got, want = backward_both_ways(mask, B, H, Hkv, T, D, dtype, lens_t, seed=i)
        for name in ("dq", "dk", "dv"):
            assert torch.isfinite(want[name]).all(), name
            assert torch.equal(got[name], want[name]), f"call {i}: {name} differs"


def test_captured_in_a_hip_graph_after_a_first_call():
    """chill_bwd_noalloc recorded into a HIP graph (its first call on the device has happened before, outside the
    capture, as the header asks: that call looks the array's address up): every replay, with new contents in the
    static inputs and eager work and synchronisations in between, equals the operator's own backward run eagerly."""
    mask = ca.ChunkwiseChillMask(40, 1)
    B, H, Hkv, T, D, dtype = 2, 4, 2, 300, 128, torch.bfloat16
    backward_both_ways(mask, 1, 2, 2, 64, 64, dtype, None, seed=5)  # the first call on this device, if none was made yet
    q, k, v, do = (torch.randn(B, h, T, D, device=DEV, dtype=dtype) for h in (H, Hkv, Hkv, H))
    o = torch.empty_like(q)
    lse = torch.empty(B, H, T, device=DEV)
    dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
    desc = mask.descriptor()
    t = {n: _lib.tensor4(x) for n, x in (("q", q), ("k", k), ("v", v), ("o", o), ("do", do), ("dq", dq), ("dk", dk), ("dv", dv))}
    r = lambda n: ctypes.byref(t[n])
    L = _lib.lib
    sm_scale = D ** -0.5

    def forward(stream):
        _lib.check("chill_fwd", L.chill_fwd(r("q"), r("k"), r("v"), r("o"), ctypes.c_void_p(lse.data_ptr()), _lib.strides3(lse), None, 0,
                                            B, H, Hkv, T, D, _lib.BF16, sm_scale, ctypes.byref(desc), stream))

    def backward(stream):
        _lib.check("chill_bwd_noalloc", L.chill_bwd_noalloc(
            r("q"), r("k"), r("v"), r("o"), r("do"), r("dq"), r("dk"), r("dv"), ctypes.c_void_p(lse.data_ptr()), _lib.strides3(lse),
            None, 0, B, H, Hkv, T, D, _lib.BF16, sm_scale, ctypes.byref(desc), stream))

    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        forward(stream)
        backward(stream)
    for replay in range(4):
        for x in (q, k, v, do):
            x.copy_(torch.randn_like(x) * (1.0 + 0.5 * replay))
        graph.replay()
        torch.cuda.synchronize()
        got = [x.clone() for x in (dq, dk, dv)]
        # eagerly, with a delta buffer of the caller, through the public operator's own backward
        qe, ke, ve = (x.clone().requires_grad_() for x in (q, k, v))
        out = ca.chill_attention(qe, ke, ve, mask=mask)
        want = torch.autograd.grad(out, (qe, ke, ve), do)
        torch.cuda.synchronize()
        assert torch.equal(out, o), f"replay {replay}: forward"
        for name, g, w in zip(("dq", "dk", "dv"), got, want):
            assert torch.equal(g, w), f"replay {replay}: {name}"


def test_sizes_beyond_the_array_are_refused():
    mask = ca.CausalChillMask()
    desc = mask.descriptor()
    x = torch.zeros(1, 1, 16, 64, device=DEV, dtype=torch.bfloat16)
    lse = torch.zeros(1, 1, 16, device=DEV)
    t = _lib.tensor4(x)
    B = _lib.BWD_NOALLOC_MAX_ROWS // 16 + 1  # B * H * T one row block over the limit; nothing is launched
    status = _lib.lib.chill_bwd_noalloc(*([ctypes.byref(t)] * 8), ctypes.c_void_p(lse.data_ptr()), _lib.strides3(lse), None, 0,
                                        B, 1, 1, 16, 64, _lib.BF16, 0.125, ctypes.byref(desc), None)
    assert status == -9  # CHILL_ERR_TOO_LARGE
    with pytest.raises(_lib.ChillLibraryError, match="too large|TOO_LARGE|32-bit|fit"):
        _lib.check("chill_bwd_noalloc", status)
