"""User-written masks ("Creating Your Own Mask", reference README.md:124-179): a mask whose device
statement is a C++ functor compiled into a library of its own.

The example mask (attention sinks + causal window) has holes inside its key limits and a
non-monotone upper query limit, so it exercises what the built-in masks do not: tile ranges as the
hull over a tile's rows, and a position-by-position count of unmasked pairs.
"""

import ctypes

import numpy as np
import pytest
import torch

import chill_attention as ca
from chill_attention import _lib, user_mask
from chill_attention.examples import SinkWindowChillMask
from oracle import chill_oracle as orc


def sink_window(q, k, args):
    """The test's own statement of the predicate."""
    sinks, window = args
    return (k <= q) & ((k < sinks) | (q - k <= window))


INSTANCES = [(4, 16), (0, 7), (33, 0), (100, 50)]


def test_library_is_built_around_the_functor():
    lib = SinkWindowChillMask._library()
    assert lib is not _lib.lib
    assert lib.chill_has_user_mask() == 1 and _lib.lib.chill_has_user_mask() == 0
    # the stock library refuses the user id, the user library refuses the built-in ids
    d = _lib.mask_desc(_lib.MASK_USER, [4, 16])
    out = np.empty((8, 8), dtype=np.uint8)
    ptr = out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))
    assert _lib.lib.chill_mask_eval(ctypes.byref(d), 8, ptr) < 0
    assert lib.chill_mask_eval(ctypes.byref(d), 8, ptr) == 0
    d2 = _lib.mask_desc(_lib.MASK_CAUSAL, [])
    assert lib.chill_mask_eval(ctypes.byref(d2), 8, ptr) < 0
    # wrong number of arguments
    d3 = _lib.mask_desc(_lib.MASK_USER, [4])
    assert lib.chill_mask_eval(ctypes.byref(d3), 8, ptr) < 0


@pytest.mark.parametrize("args", INSTANCES)
def test_verify_and_enumeration(args):
    m = SinkWindowChillMask(*args)
    for n in (1, 10, 16, 200, 333):
        m.verify(n)
        want = orc.mask_pred(sink_window, args, np.arange(n), np.arange(n))
        assert (m.make_mask(n).cpu().numpy() == want).all()
        assert m.nnz(n) == int(want.sum())


@pytest.mark.parametrize("args", INSTANCES)
@pytest.mark.parametrize("tiles", [(32, 64), (64, 64), (256, 64), (128, 32)])
def test_tile_ranges_cover_every_unmasked_tile(args, tiles):
    """Non-monotone limits: the tile range of a row tile is the hull of its rows' ranges, so every
    tile that holds an unmasked pair is visited — for query rows (forward, dQ) and key rows (dK/dV)."""
    tile_in, tile_out = tiles
    m = SinkWindowChillMask(*args)
    for n in (130, 700):
        dense = orc.mask_pred(sink_window, args, np.arange(n), np.arange(n))
        for pass_id, matrix in ((_lib.PASS_FWD, dense), (_lib.PASS_DKDV, dense.T)):
            ranges = m._calc_tile_ranges(n, tile_in, tile_out, pass_id).numpy()
            for i, (start, end, fs, fe) in enumerate(ranges):
                rows = matrix[i * tile_in : (i + 1) * tile_in]
                used = np.nonzero(rows.any(axis=0))[0]
                if used.size:
                    assert start <= used[0] // tile_out and end >= used[-1] // tile_out + 1
                    assert start == used[0] // tile_out and end == used[-1] // tile_out + 1  # exact hull
                assert fs >= fe or rows[:, fs * tile_out : fe * tile_out].all()


def test_tile_config_of_a_user_mask():
    from chill_attention.tiles import tile_config

    c = tile_config(SinkWindowChillMask(4, 16), 128, torch.bfloat16, _lib.PASS_FWD)
    assert c["rows"] == 32 * c["waves"] and c["lds_bytes"] <= 160 * 1024


def test_a_mask_without_functor_is_refused():
    class Bare(ca.ChillMask):
        @staticmethod
        def mask(q, k, seq_len, args):
            return q[:, None] >= k[None, :]

        @staticmethod
        def q_range_for_k(k, seq_len, args):
            return k, np.zeros_like(k) + seq_len - 1

        @staticmethod
        def k_range_for_q(q, seq_len, args):
            return np.zeros_like(q), q

    with pytest.raises(NotImplementedError):
        Bare().descriptor()


def test_functor_text_is_wrapped_and_keyed_by_content():
    class A(ca.ChillMask):
        hip_functor = "static constexpr int kNumArgs = 0; /* ... */"
        mask = q_range_for_k = k_range_for_q = staticmethod(lambda *a: None)

    src = user_mask.functor_source(A)
    assert "struct Mask<CHILL_MASK_USER> : MaskDefaults" in src and A.hip_functor in src
    p1 = user_mask.library_path(A)
    A.hip_functor += " "
    assert user_mask.library_path(A) != p1


# ---------------------------------------------------------------------------------------- GPU
DEV = "cuda"


# the reference's tolerances (atol, rtol): test_chill_attention.py:167-172 (outputs), :316-321 (gradients)
OUT_TOL = {torch.float32: (2e-6, 1e-4), torch.float16: (1e-2, 1e-3), torch.bfloat16: (5e-2, 1e-2)}
GRAD_TOL = {torch.float32: (5e-5, 1e-3), torch.float16: (5e-3, 1e-3), torch.bfloat16: (1e-1, 1e-2)}


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=str)
@pytest.mark.parametrize("args,T", [((4, 16), 500), ((33, 100), 1025), ((0, 7), 300)])
def test_attention_with_a_user_mask_matches_the_oracle(args, T, dtype):
    """O, dQ, dK, dV through the custom op of a user mask against dense-mask SDPA with the test's
    own statement of the predicate, at the tolerances of the reference's own tests and (head dim 64)
    at the benchmark's atol = rtol as well."""
    from test_attention_gpu import check_close

    torch.manual_seed(0)
    B, H, Hkv, D = 2, 4, 2, 64
    mask = SinkWindowChillMask(*args)
    q = torch.randn(B, H, T, D, device=DEV, dtype=dtype, requires_grad=True)
    k = torch.randn(B, Hkv, T, D, device=DEV, dtype=dtype, requires_grad=True)
    v = torch.randn(B, Hkv, T, D, device=DEV, dtype=dtype, requires_grad=True)
    lens = torch.tensor([T, T // 3], device=DEV, dtype=torch.int32)
    do = torch.randn(B, H, T, D, device=DEV, dtype=dtype)
    print(f"user mask {mask} {dtype} T={T}", flush=True)
    out = ca.chill_attention(q, k, v, mask=mask, lens=lens)
    out.backward(do)
    qr, kr, vr = (x.detach().float().clone().requires_grad_(True) for x in (q, k, v))
    ref, res_mask = orc.reference_naive(sink_window, args, qr, kr, vr, lens)
    (ref * res_mask).backward(do.float() * res_mask)
    check_close((out * res_mask).detach(), (ref * res_mask).detach(), dtype, OUT_TOL[dtype], D, "O")
    for nm, got, want in (("dq", q.grad, qr.grad), ("dk", k.grad, kr.grad), ("dv", v.grad, vr.grad)):
        check_close(got, want, dtype, GRAD_TOL[dtype], D, nm)


@pytest.mark.gpu
def test_device_functor_of_a_user_mask_equals_host():
    """The functor the kernels run, dumped from the device, against the host enumeration."""
    m = SinkWindowChillMask(5, 9)
    lib = m._library()
    n = 200
    desc = m.descriptor()
    out = torch.empty(n, n, dtype=torch.uint8, device=DEV)
    _lib.check("chill_mask_eval_device", lib.chill_mask_eval_device(ctypes.byref(desc), n, ctypes.c_void_p(out.data_ptr()), None))
    torch.cuda.synchronize()
    assert (out.cpu().numpy().astype(bool) == orc.mask_pred(sink_window, (5, 9), np.arange(n), np.arange(n))).all()
    for pass_id, tile_in, tile_out in ((_lib.PASS_FWD, 32, 64), (_lib.PASS_DKDV, 32, 64), (_lib.PASS_DQ, 256, 64)):
        host = m._calc_tile_ranges(n, tile_in, tile_out, pass_id).numpy()
        dev = torch.empty(host.shape, dtype=torch.int32, device=DEV)
        _lib.check("chill_tile_ranges_device", lib.chill_tile_ranges_device(
            ctypes.byref(desc), pass_id, n, n, tile_in, tile_out, ctypes.c_void_p(dev.data_ptr()), None))
        torch.cuda.synchronize()
        assert (dev.cpu().numpy() == host).all()
