"""The C-ABI shared library on the CPU: it loads, exports every symbol the header declares, and its
argument validation answers with error codes before anything is launched (no GPU needed)."""

import ctypes
import os
import re

import pytest

from chill_attention import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "chill_attention.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(chill_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_symbols()
    assert len(names) >= 15
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), f"{n} declared in include/chill_attention.h but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == names
    assert _lib.lib.chill_abi_version() == _lib.ABI_VERSION


def test_status_strings():
    for code in range(0, -10, -1):
        s = _lib.lib.chill_status_string(code).decode()
        assert s and s != "unknown status"
    assert _lib.lib.chill_status_string(-99).decode() == "unknown status"


def _t4(ptr=0x1000, strides=(1 << 20, 1 << 16, 128, 1)):
    t = _lib.ChillTensor4()
    t.ptr = ptr
    for i, s in enumerate(strides):
        t.stride[i] = s
    return t


def _call_fwd(q=None, k=None, v=None, o=None, B=1, H=2, Hkv=2, T=64, D=128, dtype=_lib.BF16, mask=None, null_q=False):
    q, k, v, o = (x if x is not None else _t4() for x in (q, k, v, o))
    mask = mask if mask is not None else _lib.mask_desc(_lib.MASK_CAUSAL, [])
    s3 = (ctypes.c_int64 * 3)(H * T, T, 1)
    return _lib.lib.chill_fwd(
        None if null_q else ctypes.byref(q), ctypes.byref(k), ctypes.byref(v), ctypes.byref(o), None, s3, None, 0,
        B, H, Hkv, T, D, dtype, 0.1, ctypes.byref(mask), None)


def test_forward_validation_returns_codes_without_launching():
    E = {"null": -1, "dtype": -2, "dim": -3, "mask": -4, "shape": -5, "stride": -6, "large": -9}
    assert _call_fwd(null_q=True) == E["null"]
    assert _call_fwd(q=_t4(ptr=None)) == E["null"]
    assert _call_fwd(dtype=7) == E["dtype"]
    assert _call_fwd(D=48) == E["dim"]
    assert _call_fwd(D=0) == E["dim"]
    assert _call_fwd(mask=_lib.mask_desc(9, [])) == E["mask"]
    assert _call_fwd(mask=_lib.mask_desc(_lib.MASK_SLIDING_WINDOW, [3])) == E["mask"]  # wrong arg count
    assert _call_fwd(mask=_lib.mask_desc(_lib.MASK_CHUNKWISE, [0, 1])) == E["mask"]  # zero chunk size
    assert _call_fwd(mask=_lib.mask_desc(_lib.MASK_PREFIX_LM, [-1])) == E["mask"]
    assert _call_fwd(B=0) == E["shape"]
    assert _call_fwd(H=6, Hkv=4) == E["shape"]
    assert _call_fwd(T=(1 << 29) + 1) == E["large"]
    assert _call_fwd(q=_t4(strides=(1 << 20, 1 << 16, 128, 2))) == E["stride"]  # inner stride
    assert _call_fwd(q=_t4(strides=(1 << 20, 1 << 16, 100, 1))) == E["stride"]  # rows not 16-byte aligned
    assert _call_fwd(q=_t4(ptr=0x1004)) == E["stride"]  # misaligned base
    assert _call_fwd(q=_t4(strides=(-1, 1 << 16, 128, 1))) == E["stride"]
    with pytest.raises(_lib.ChillLibraryError) as ei:
        _lib.check("chill_fwd", _call_fwd(D=48))
    assert ei.value.status == E["dim"] and "head dim" in str(ei.value)


def test_backward_and_debug_validation():
    t = _t4()
    s3 = (ctypes.c_int64 * 3)(128, 64, 1)
    m = _lib.mask_desc(_lib.MASK_CAUSAL, [])
    assert _lib.lib.chill_bwd_delta(ctypes.byref(t), ctypes.byref(t), None, s3, 1, 2, 64, 128, _lib.BF16, None) == -1
    assert _lib.lib.chill_bwd_delta(ctypes.byref(t), ctypes.byref(t), 0x1000, s3, 1, 2, 64, 100, _lib.BF16, None) == -3
    bad_s3 = (ctypes.c_int64 * 3)(128, 64, 2)
    assert _lib.lib.chill_bwd_delta(ctypes.byref(t), ctypes.byref(t), 0x1000, bad_s3, 1, 2, 64, 128, _lib.BF16, None) == -6
    r = _lib.lib.chill_bwd_dq(ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t),
                              None, s3, 0x1000, s3, None, 0, 1, 2, 2, 64, 128, _lib.BF16, 0.1, ctypes.byref(m), None)
    assert r == -1  # lse missing
    r = _lib.lib.chill_bwd_dkdv(ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), ctypes.byref(t), None,
                                0x1000, s3, 0x1000, s3, None, 0, 1, 2, 2, 64, 128, _lib.BF16, 0.1, ctypes.byref(m), None)
    assert r == -1  # dv missing
    assert _lib.lib.chill_mask_eval_device(ctypes.byref(m), 16, None, None) == -1
    assert _lib.lib.chill_tile_ranges_device(ctypes.byref(m), 5, 64, 64, 32, 32, 0x1000, None) == -8
    out = (ctypes.c_int32 * 8)()
    assert _lib.lib.chill_tile_ranges(ctypes.byref(m), 0, 64, 65, 32, 32, out) == -5  # seq_len > T
    assert _lib.lib.chill_tile_ranges(ctypes.byref(m), 0, 64, 64, 0, 32, out) == -8
    assert _lib.lib.chill_mask_limits(ctypes.byref(m), 2, 4, 4, out) == -8


def test_tile_table():
    import torch

    import chill_attention as ca
    from chill_attention.tiles import _get_default_config_bwd, _get_default_config_fwd, tile_config

    for mask in (ca.CausalChillMask(), ca.SlidingWindowChillMask(1, 1)):
        for dt in (torch.float32, torch.float16, torch.bfloat16):
            for D in (16, 32, 64, 128, 256):
                for p in (_lib.PASS_FWD, _lib.PASS_DQ, _lib.PASS_DKDV):
                    c = tile_config(mask, D, dt, p)
                    # one wave per 32 resident rows, or (dK/dV) two or four waves per 32 rows, or one wave per 64
                    assert c["rows"] in (64 * c["waves"], 32 * c["waves"], 16 * c["waves"], 8 * c["waves"]) and c["streamed"] % 32 == 0
                    assert 0 < c["lds_bytes"] <= 160 * 1024
    # fp32 rows of 512 bytes and more: the waves of a 32-key block split its state
    assert tile_config(ca.CausalChillMask(), 128, torch.float32, _lib.PASS_DKDV)["waves"] == 8
    assert tile_config(ca.CausalChillMask(), 128, torch.float32, _lib.PASS_DKDV)["rows"] == 128
    assert tile_config(ca.CausalChillMask(), 256, torch.float32, _lib.PASS_DKDV)["rows"] == 32
    # rows the tile sweep put into the table (mask- and head-dim-specific)
    causal, window = ca.CausalChillMask(), ca.SlidingWindowChillMask(128, 128)
    assert tile_config(causal, 128, torch.bfloat16, _lib.PASS_FWD)["streamed"] == 64
    assert tile_config(causal, 64, torch.float16, _lib.PASS_FWD)["streamed"] == 64
    assert tile_config(causal, 32, torch.float16, _lib.PASS_FWD)["streamed"] == 64
    assert tile_config(window, 64, torch.bfloat16, _lib.PASS_FWD)["streamed"] == 64
    # banded masks, and every mask at head dims <= 64: 4 waves with a two-stage ring, two or more workgroups per CU
    for p, mask, D, waves in ((_lib.PASS_FWD, window, 64, 4), (_lib.PASS_FWD, window, 128, 4), (_lib.PASS_FWD, causal, 64, 4), (_lib.PASS_FWD, causal, 128, 8),
                              (_lib.PASS_DQ, window, 128, 4), (_lib.PASS_DQ, causal, 64, 4)):
        c = tile_config(mask, D, torch.bfloat16, p)
        assert c["waves"] == waves, (p, D, c)
        if waves == 4:
            assert c["streamed"] == 64 and 2 * c["lds_bytes"] <= 160 * 1024
    # the fast forward (16-bit, head dim 64 / 128) keeps a tile resident ahead: three stages at D = 64, four at D = 128
    assert tile_config(causal, 64, torch.bfloat16, _lib.PASS_FWD)["lds_bytes"] == 3 * 64 * (144 + 192)
    assert tile_config(causal, 128, torch.bfloat16, _lib.PASS_FWD)["lds_bytes"] == 4 * 64 * (272 + 320)
    # short sequences and small grids at head dim 128: the 4-wave shape in forward (T <= 1024) and dQ (T <= 4096)
    for p, T, bh, waves in ((_lib.PASS_FWD, 1024, 128, 4), (_lib.PASS_FWD, 1025, 128, 8), (_lib.PASS_DQ, 4096, 128, 4),
                            (_lib.PASS_DQ, 4097, 30, 8), (_lib.PASS_DQ, 8191, 15, 8), (_lib.PASS_FWD, 8192, 8, 8), (_lib.PASS_FWD, 8192, 16, 8),
                            (_lib.PASS_DQ, 8192, 8, 4), (_lib.PASS_DKDV, 2048, 8, 4), (_lib.PASS_DKDV, 2048, 16, 8)):
        assert tile_config(causal, 128, torch.bfloat16, p, seq_len=T, batch_heads=bh)["waves"] == waves, (p, T, bh)
    # (under a full mask the forward takes its 8-wave shape from 769 keys on)
    assert tile_config(ca.FullChillMask(), 128, torch.bfloat16, _lib.PASS_FWD, seq_len=768, batch_heads=128)["waves"] == 4
    assert tile_config(ca.FullChillMask(), 128, torch.bfloat16, _lib.PASS_FWD, seq_len=769, batch_heads=128)["waves"] == 8
    assert tile_config(causal, 128, torch.float32, _lib.PASS_DQ, seq_len=128) == tile_config(causal, 128, torch.float32, _lib.PASS_DQ)
    assert _lib.lib.chill_tile_config_for_shape(1, 128, _lib.BF16, 0, 1, 0, (ctypes.c_int32 * 4)()) == -8
    # launches far too small for the chip: 32 rows per workgroup; fp32 much further up than 16-bit inputs, and furthest
    # under masks whose rows grow with their index (tiles = B * H * T / 32)
    prefix, full = ca.PrefixLMChillMask(100), ca.FullChillMask()
    for mask, dt, D, p, bh, T, small in (
            (full, torch.bfloat16, 64, _lib.PASS_FWD, 8, 1024, True), (full, torch.bfloat16, 64, _lib.PASS_FWD, 9, 1024, False),
            (causal, torch.bfloat16, 64, _lib.PASS_FWD, 16, 1024, True), (prefix, torch.float16, 32, _lib.PASS_FWD, 17, 1024, False),
            (causal, torch.bfloat16, 128, _lib.PASS_FWD, 16, 1024, True), (causal, torch.bfloat16, 128, _lib.PASS_FWD, 17, 1024, False),
            (causal, torch.float32, 64, _lib.PASS_FWD, 32, 2048, True), (causal, torch.float32, 64, _lib.PASS_FWD, 33, 2048, False),
            (prefix, torch.float32, 128, _lib.PASS_FWD, 24, 2048, True), (prefix, torch.float32, 128, _lib.PASS_FWD, 25, 2048, False),
            (full, torch.float32, 64, _lib.PASS_FWD, 24, 2048, True), (window, torch.float32, 64, _lib.PASS_FWD, 25, 2048, False),
            (causal, torch.float32, 64, _lib.PASS_FWD, 1, 16384, True), (causal, torch.float32, 64, _lib.PASS_FWD, 1, 16385, False),
            (causal, torch.bfloat16, 64, _lib.PASS_FWD, 1, 16384, True), (causal, torch.bfloat16, 64, _lib.PASS_FWD, 1, 16385, False),
            (full, torch.float32, 128, _lib.PASS_DQ, 2, 8192, True), (full, torch.float32, 64, _lib.PASS_DKDV, 2, 8192, True),
            (causal, torch.float32, 64, _lib.PASS_DQ, 128, 4096, True), (causal, torch.float32, 32, _lib.PASS_DQ, 129, 4096, False),
            (causal, torch.float32, 128, _lib.PASS_DQ, 64, 4096, True), (causal, torch.float32, 128, _lib.PASS_DQ, 65, 4096, False),
            (full, torch.float32, 64, _lib.PASS_DQ, 24, 2048, True), (full, torch.float32, 64, _lib.PASS_DQ, 25, 2048, False),
            (causal, torch.float16, 64, _lib.PASS_DQ, 16, 1024, True), (full, torch.float16, 128, _lib.PASS_DQ, 16, 1024, True),
            (causal, torch.float16, 128, _lib.PASS_DQ, 17, 1024, False), (window, torch.float16, 128, _lib.PASS_DQ, 2, 8192, True),
            (causal, torch.float32, 64, _lib.PASS_DKDV, 64, 2048, True), (causal, torch.float32, 64, _lib.PASS_DKDV, 65, 2048, False),
            (prefix, torch.float32, 32, _lib.PASS_DKDV, 8, 4096, True), (prefix, torch.float32, 32, _lib.PASS_DKDV, 9, 4096, False),
            (full, torch.float32, 64, _lib.PASS_DKDV, 8, 2048, True), (full, torch.float32, 64, _lib.PASS_DKDV, 9, 2048, False),
            (causal, torch.float32, 128, _lib.PASS_DKDV, 1, 512, False), (causal, torch.bfloat16, 64, _lib.PASS_DKDV, 8, 1024, True),
            (causal, torch.bfloat16, 64, _lib.PASS_DKDV, 9, 1024, False), (causal, torch.bfloat16, 64, _lib.PASS_DKDV, 4, 4096, True),
            (full, torch.bfloat16, 64, _lib.PASS_DKDV, 4, 4096, False), (causal, torch.bfloat16, 64, _lib.PASS_DKDV, 5, 4096, False)):
        c = tile_config(mask, D, dt, p, seq_len=T, batch_heads=bh)
        assert (c["rows"] == 32 and c["streamed"] == 32) == small, (mask, dt, D, p, bh, T, c)
    # (more tiles than CUs: forward and dQ workgroups hold two tiles where two LDS areas fit)
    one = tile_config(causal, 64, torch.float32, _lib.PASS_FWD, seq_len=1024, batch_heads=8)["lds_bytes"]
    assert tile_config(causal, 64, torch.float32, _lib.PASS_FWD, seq_len=1024, batch_heads=9)["lds_bytes"] == 2 * one
    assert tile_config(causal, 128, torch.float32, _lib.PASS_FWD, seq_len=1024, batch_heads=9)["lds_bytes"] == 4 * (2 * 32 * 512 + 512)
    # dK/dV at 16-bit head dims <= 64: 64 key rows per workgroup of 4 waves, several workgroups per CU (at head dim 64
    # for short sequences, small grids and banded masks; long sequences: K in registers, below)
    for D, T, rows, waves in ((64, 3499, 64, 4), (32, None, 64, 4), (32, 8192, 64, 4)):
        c = tile_config(causal, D, torch.bfloat16, _lib.PASS_DKDV, seq_len=T, batch_heads=1 << 12)
        assert (c["rows"], c["waves"]) == (rows, waves), (D, c)
    assert tile_config(window, 64, torch.bfloat16, _lib.PASS_DKDV)["rows"] == 64
    # dQ at 16-bit head dim 128 from 4097 keys on (full masks: 2048), full grids, masks that are not banded: Q and dO in
    # registers
    regs2 = {"rows": 256, "streamed": 32, "waves": 4, "lds_bytes": 4 * 2 * 32 * 256}
    assert tile_config(causal, 128, torch.bfloat16, _lib.PASS_DQ) == regs2
    assert tile_config(causal, 128, torch.float16, _lib.PASS_DQ, seq_len=8192, batch_heads=16) == regs2
    assert tile_config(causal, 128, torch.float16, _lib.PASS_DQ, seq_len=4097, batch_heads=31) == regs2
    assert tile_config(ca.PrefixLMChillMask(7), 128, torch.bfloat16, _lib.PASS_DQ, seq_len=6000, batch_heads=32) == regs2
    assert tile_config(ca.FullChillMask(), 128, torch.bfloat16, _lib.PASS_DQ, seq_len=2048, batch_heads=64) == regs2
    for mask, T, bh in ((causal, 4096, 128), (causal, 8192, 15), (causal, 4097, 30), (window, 16384, 128), (ca.FullChillMask(), 2047, 128),
                        (ca.FullChillMask(), 2048, 63), (ca.ChunkwiseChillMask(1024, 1), 8192, 128)):
        assert tile_config(mask, 128, torch.bfloat16, _lib.PASS_DQ, seq_len=T, batch_heads=bh)["streamed"] == 64, (mask, T, bh)
    assert tile_config(causal, 64, torch.bfloat16, _lib.PASS_DQ, seq_len=8192, batch_heads=128)["streamed"] == 64
    # dK/dV at 16-bit head dim 128: K in registers, two 32-key blocks per wave (256 key rows, 4 waves, 32-row tiles in
    # four stages) for long sequences on a grid of two workgroups per CU, except under banded masks; else the paired kernel
    regs = {"rows": 256, "streamed": 32, "waves": 4, "lds_bytes": 256 * 256 + 4 * (2 * 32 * 256 + 2 * 32 * 4)}
    assert tile_config(causal, 128, torch.bfloat16, _lib.PASS_DKDV) == regs
    assert tile_config(causal, 128, torch.float16, _lib.PASS_DKDV, seq_len=8192, batch_heads=128) == regs
    assert tile_config(causal, 128, torch.float16, _lib.PASS_DKDV, seq_len=4096, batch_heads=32) == regs
    # (from 3072 keys on under causal-like masks, 3500 at head dim 64; under a full mask from 1024)
    assert tile_config(causal, 128, torch.float16, _lib.PASS_DKDV, seq_len=3072, batch_heads=64) == regs
    assert tile_config(ca.PrefixLMChillMask(9), 128, torch.float16, _lib.PASS_DKDV, seq_len=3500, batch_heads=64) == regs
    assert tile_config(ca.FullChillMask(), 128, torch.bfloat16, _lib.PASS_DKDV, seq_len=1024, batch_heads=128) == regs
    assert tile_config(ca.FullChillMask(), 128, torch.bfloat16, _lib.PASS_DKDV, seq_len=4096, batch_heads=16) == regs
    for mask, T, bh in ((causal, 3071, 128), (causal, 4096, 31), (window, 8192, 128), (window, None, 1 << 20), (ca.FullChillMask(), 1023, 256),
                        (ca.FullChillMask(), 1024, 63), (ca.FullChillMask(), 4096, 15), (ca.ChunkwiseChillMask(128, 2), 4095, 128)):
        c = tile_config(mask, 128, torch.bfloat16, _lib.PASS_DKDV, seq_len=T, batch_heads=bh)
        assert (c["rows"], c["waves"], c["streamed"]) == (128, 8, 64), (mask, T, bh, c)
    # chunkwise masks whose chunks are a multiple of a wave's 64 key rows (no partly masked block inside the band) take
    # it too; other chunk sizes do not, nor does the report that is not told the mask's arguments
    for chunk, T, bh, row in ((128, 16384, 64, regs), (64, 4096, 32, regs), (1024, 8192, 64, regs), (192, 4096, 32, regs)):
        assert tile_config(ca.ChunkwiseChillMask(chunk, 2), 128, torch.float16, _lib.PASS_DKDV, seq_len=T, batch_heads=bh) == row
    for mask, T, bh in ((ca.ChunkwiseChillMask(96, 3), 8192, 64), (ca.ChunkwiseChillMask(32, 3), 8192, 64), (ca.ChunkwiseChillMask(128, 2), 4095, 64),
                        (ca.ChunkwiseChillMask(128, 2), 4096, 31), (ca.ChunkwiseChillMask(128, 2), None, 1 << 20)):
        c = tile_config(mask, 128, torch.float16, _lib.PASS_DKDV, seq_len=T, batch_heads=bh)
        assert (c["rows"], c["waves"], c["streamed"]) == (128, 8, 64), (mask, T, bh, c)
    # a banded mask whose rows see many keys is a long loop again: the forward at head dim 128 takes its 8-wave shape from
    # 1024 keys on, dK/dV under a sliding window its register-resident kernel from 4096 keys on (dQ keeps the 4-wave shape)
    for mask, waves in ((ca.SlidingWindowChillMask(1023, 0), 8), (ca.SlidingWindowChillMask(1000, 22), 4), (ca.SlidingWindowChillMask(128, 128), 4),
                        (ca.ChunkwiseChillMask(512, 1), 8), (ca.ChunkwiseChillMask(128, 2), 4), (ca.ChunkwiseChillMask(341, 2), 4)):
        assert tile_config(mask, 128, torch.bfloat16, _lib.PASS_FWD, seq_len=8192, batch_heads=128)["waves"] == waves, mask
        assert tile_config(mask, 128, torch.bfloat16, _lib.PASS_FWD, seq_len=1024, batch_heads=128)["waves"] == 4, mask
        assert tile_config(mask, 64, torch.bfloat16, _lib.PASS_FWD, seq_len=8192, batch_heads=128)["waves"] == 4, mask
        assert tile_config(mask, 128, torch.bfloat16, _lib.PASS_DQ, seq_len=8192, batch_heads=128)["waves"] == 4, mask
    assert tile_config(ca.SlidingWindowChillMask(4095, 0), 128, torch.bfloat16, _lib.PASS_DKDV, seq_len=8192, batch_heads=128) == regs
    assert tile_config(ca.SlidingWindowChillMask(2000, 2095), 128, torch.float16, _lib.PASS_DKDV, seq_len=8192, batch_heads=128) == regs
    for mask, T, bh in ((ca.SlidingWindowChillMask(4094, 0), 8192, 128), (ca.SlidingWindowChillMask(4095, 0), 4095, 128),
                        (ca.SlidingWindowChillMask(4095, 0), 8192, 15)):
        c = tile_config(mask, 128, torch.bfloat16, _lib.PASS_DKDV, seq_len=T, batch_heads=bh)
        assert (c["rows"], c["waves"], c["streamed"]) == (128, 8, 64), (mask, T, bh, c)
    out4 = (ctypes.c_int32 * 4)()
    assert _lib.lib.chill_tile_config_for_shape(3, 128, _lib.F16, _lib.PASS_DKDV, 64, 16384, out4) == 0 and out4[0] == 128
    assert _lib.lib.chill_tile_config_for_shape(2, 128, _lib.F16, _lib.PASS_FWD, 64, 16384, out4) == 0 and out4[2] == 4
    desc = ca.ChunkwiseChillMask(128, 2).descriptor()
    assert _lib.lib.chill_tile_config_for_launch(ctypes.byref(desc), 128, _lib.F16, _lib.PASS_DKDV, 64, 16384, out4) == 0
    assert list(out4) == [regs["rows"], regs["streamed"], regs["waves"], regs["lds_bytes"]]
    assert _lib.lib.chill_tile_config_for_launch(None, 128, _lib.F16, _lib.PASS_DKDV, 64, 16384, out4) == -1
    assert _lib.lib.chill_tile_config_for_launch(ctypes.byref(desc), 128, _lib.F16, _lib.PASS_DKDV, 64, 16384, None) == -1
    desc.nargs = 1
    assert _lib.lib.chill_tile_config_for_launch(ctypes.byref(desc), 128, _lib.F16, _lib.PASS_DKDV, 64, 16384, out4) == -4
    # the same kernel at head dim 64 (rows of 128 bytes), on grids of at least four workgroups per CU; of the chunkwise
    # masks only chunks of 320 rows and more
    regs64 = {"rows": 256, "streamed": 32, "waves": 4, "lds_bytes": 256 * 128 + 4 * (2 * 32 * 128 + 2 * 32 * 4)}
    assert tile_config(causal, 64, torch.bfloat16, _lib.PASS_DKDV) == regs64
    assert tile_config(ca.PrefixLMChillMask(1024), 64, torch.float16, _lib.PASS_DKDV, seq_len=8192, batch_heads=128) == regs64
    assert tile_config(ca.ChunkwiseChillMask(512, 1), 64, torch.float16, _lib.PASS_DKDV, seq_len=8192, batch_heads=128) == regs64
    assert tile_config(causal, 64, torch.float16, _lib.PASS_DKDV, seq_len=4096, batch_heads=64) == regs64
    assert tile_config(causal, 64, torch.float16, _lib.PASS_DKDV, seq_len=3500, batch_heads=74) == regs64
    assert tile_config(ca.FullChillMask(), 64, torch.bfloat16, _lib.PASS_DKDV, seq_len=1024, batch_heads=64) == regs64
    assert tile_config(causal, 64, torch.bfloat16, _lib.PASS_DKDV, seq_len=8192, batch_heads=16) == regs64
    assert tile_config(ca.PrefixLMChillMask(5), 64, torch.bfloat16, _lib.PASS_DKDV, seq_len=16384, batch_heads=8) == regs64
    assert tile_config(ca.SlidingWindowChillMask(4096, 100), 64, torch.bfloat16, _lib.PASS_DKDV, seq_len=8192, batch_heads=128) == regs64
    for mask, T, bh in ((causal, 4096, 63), (causal, 8192, 15), (causal, 8191, 31), (ca.ChunkwiseChillMask(512, 1), 8192, 31), (ca.ChunkwiseChillMask(128, 2), 16384, 64),
                        (ca.ChunkwiseChillMask(256, 1), 8192, 128), (window, 8192, 128)):
        c = tile_config(mask, 64, torch.bfloat16, _lib.PASS_DKDV, seq_len=T, batch_heads=bh)
        assert (c["rows"], c["waves"], c["streamed"]) == (64, 4, 64), (mask, T, bh, c)
    assert 2 * tile_config(window, 64, torch.bfloat16, _lib.PASS_DKDV)["lds_bytes"] <= 160 * 1024
    tq, tk, waves = _get_default_config_fwd(128, torch.bfloat16)
    assert tq == 32 * waves and tk % 32 == 0
    (dq_q, dq_k, _), (dk_q, dk_k, _) = _get_default_config_bwd(128, torch.bfloat16)
    assert dq_q % 32 == 0 and dk_k % 32 == 0
    out = (ctypes.c_int32 * 4)()
    assert _lib.lib.chill_tile_config(0, 100, _lib.BF16, 0, out) == -3
    assert _lib.lib.chill_tile_config(0, 64, 5, 0, out) == -2
    assert _lib.lib.chill_tile_config(9, 64, _lib.BF16, 0, out) == -4
    assert _lib.lib.chill_tile_config(0, 64, _lib.BF16, 3, out) == -8


def test_work_items_are_a_permutation_and_resident_grids_balance():
    """chill_work_item (the kernels' workgroup -> work item order, compiled for the host): over a grid the items are a
    permutation of 0 .. total-1 for every grid size and every number of resident workgroups; a grid that the chip holds
    at once gives the two (three) workgroups that share a CU items whose causal weights add up alike."""
    f = _lib.lib.chill_work_item
    for resident in (1, 2, 3):
        for total in list(range(1, 530)) + [600, 767, 768, 769, 1000, 1024, 4096]:
            grid = -(-total // 8) * 8
            items = [f(w, total, resident) for w in range(grid)]
            assert sorted(i for i in items if i >= 0) == list(range(total)), (resident, total)
            if resident == 1 or total <= 256 or total > 256 * resident:
                # one workgroup per CU, or a grid dealt out as CUs become free: XCD x takes items x * per .. in order
                per = -(-total // 8)
                assert all(items[w] in (-1, (w % 8) * per + w // 8) for w in range(grid)), (resident, total)
    assert f(-1, 8, 1) == -8 and f(0, 0, 1) == -8 and f(0, 8, 0) == -8
    # 512 workgroups, two per CU, tiles of n_tiles per head ordered longest first (weight = n_tiles - 1 - item % n_tiles):
    # workgroups l and l + 32 of an XCD share a CU
    for n_tiles in (16, 32, 64):
        weight = lambda item: n_tiles - 1 - item % n_tiles
        for xcd in range(8):
            sums = {weight(f(8 * l + xcd, 512, 2)) + weight(f(8 * (l + 32) + xcd, 512, 2)) for l in range(32)}
            assert sums == {n_tiles - 1}, (n_tiles, xcd, sums)
            plain = {weight(f(8 * l + xcd, 512, 1)) + weight(f(8 * (l + 32) + xcd, 512, 1)) for l in range(32)}
            assert len(plain) > 1


def test_cpu_tensors_are_refused():
    import torch

    import chill_attention as ca

    q = torch.randn(1, 1, 16, 16)
    with pytest.raises((RuntimeError, NotImplementedError)):
        ca.chill_attention(q, q, q, mask=ca.CausalChillMask())


def test_inputs_on_other_devices_are_refused_before_any_launch():
    """A k, v, lens, o, lse or dO that does not live on q's device would reach the kernels as a bad
    pointer: the adapters refuse it (checked here without a GPU, on the validation function)."""
    import torch

    from chill_attention import chill

    q = torch.empty(2, 2, 16, 16, device="meta")
    cpu = torch.zeros(2, 2, 16, 16)
    with pytest.raises(ValueError, match="k is on cpu"):
        chill._check_inputs(q, cpu, q, None, 1.0)
    with pytest.raises(ValueError, match="lens is on cpu"):
        chill._check_inputs(q, q, q, torch.ones(2, dtype=torch.int32), 1.0)
    with pytest.raises(ValueError, match="do is on cpu"):
        chill._check_inputs(q, q, q, None, 1.0, others=(("o", q), ("do", cpu)))
    with pytest.raises(ValueError, match="finite"):
        chill._check_inputs(q, q, q, None, float("nan"))
    with pytest.raises(ValueError, match="head dim"):
        bad = torch.empty(2, 2, 16, 24, device="meta")
        chill._check_inputs(bad, bad, bad, None, 1.0)
    with pytest.raises(RuntimeError, match="GPU only"):
        chill._check_inputs(cpu, cpu, cpu, None, 1.0)


def test_build_refuses_unsound_register_use():
    """__graft_entry__.build() and user_mask.build() end with tune.check_hand_managed_registers: a build in
    which the compiler touches the accumulation registers that the head-dim-256 kernels manage themselves
    is refused (here: a build with a macro that makes it do so on purpose)."""
    import inspect
    import shutil

    import __graft_entry__ as entry
    from chill_attention import tune, user_mask

    assert "check_hand_managed_registers" in inspect.getsource(entry.build)
    assert "check_hand_managed_registers" in inspect.getsource(user_mask.build)
    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not on PATH")
    tune.check_hand_managed_registers()  # the shipped build is sound
    with pytest.raises(RuntimeError, match="unsound"):
        tune.check_hand_managed_registers({"CHILL_TEST_UNSOUND_REGISTERS": 1})


def test_tile_sweep_candidates():
    """The sweep tool's candidate list: the shipped shape comes first and overrides nothing."""
    from chill_attention import tune

    names = [n for n, _ in tune.CANDIDATES]
    assert len(set(names)) == len(names) and tune.CANDIDATES[0][1] == {}
    allowed = {"CHILL_TUNE_FWD_WAVES", "CHILL_TUNE_FWD_STREAMED", "CHILL_TUNE_FWD_STAGES", "CHILL_TUNE_DQ_WAVES",
               "CHILL_TUNE_DQ_STREAMED", "CHILL_TUNE_DQ_STAGES", "CHILL_TUNE_DKDV_WAVES", "__flags__"}
    header = open(os.path.join(ROOT, "chill-attention_amd", "csrc", "chill_tiles.h")).read()
    for _, macros in tune.CANDIDATES:
        assert set(macros) <= allowed and all(m in header for m in macros if m != "__flags__")
    assert tune.candidate_library("w8_s64").endswith(os.path.join("lib", "tune", "w8_s64", "libchill_attention_hip.so"))


@pytest.mark.parametrize("elem", ["bf16", "f16"])
def test_hand_managed_accumulation_registers(elem):
    """The 16-bit head-dim-256 kernels keep their accumulator blocks in accumulation registers that they
    name themselves (dK/dV: a0..a255, forward and dQ: a128..a255); the compiler does not know they are
    live.  Sound only while the compiler stays below them and spills nothing in those kernels: checked on
    the generated assembly."""
    import shutil

    from chill_attention import tune

    if shutil.which("hipcc") is None:
        pytest.skip("hipcc not on PATH")
    rows = tune.hand_managed_registers(elem, 256)
    assert len(rows) == 15  # three kernels per built-in mask
    for kernel, lowest in (("fwd_regs_kernel", 128), ("dq_regs_kernel", 128), ("dkdv_regs_kernel", 0)):
        assert sum(kernel in name for name, *_ in rows) == 5, kernel
        for name, compiler_max, hand_min, spilled in rows:
            if kernel in name:
                assert compiler_max < hand_min, (name, compiler_max, hand_min)
                assert hand_min == lowest and spilled == 0, (name, hand_min, spilled)
    # dK/dV with register-resident K at head dim 128 (a0..a255 named by the kernel and its generated loop): the
    # compiler touches no accumulation register there, so what it spills is in scratch memory
    rows = tune.hand_managed_registers(elem, 128)
    assert len(rows) == 10 and sum("dkdv_regs_kernel" in name for name, *_ in rows) == 5 and sum("dq_regs2_kernel" in name for name, *_ in rows) == 5
    for name, compiler_max, hand_min, spilled in rows:
        assert compiler_max == -1 and hand_min == 0, (name, compiler_max, hand_min)


def test_eager_operator_library_loads():
    """The operator registered from C++ (csrc/chill_torch.cpp) is built next to the kernel library, loads
    into this PyTorch and has the schema the Python side calls it with."""
    import torch

    assert os.path.exists(_lib.TORCH_LIB_PATH), "libchill_attention_torch.so has not been built"
    op = _lib.torch_operator()
    assert op is not None
    schema = str(torch.ops.chill_attention_amd.attention.default._schema)
    assert schema == ("chill_attention_amd::attention(Tensor q, Tensor k, Tensor v, Tensor? lens, int entry_points, "
                      "int mask_id, int[] mask_args, float sm_scale, bool return_lse) -> (Tensor, Tensor)")
    table = _lib.entry_points(_lib.lib)
    assert all(getattr(table, n) for n, *_ in _lib.EntryPoints._fields_)
    # the operator takes a handle of a registered table, and tables that are not one are refused
    import ctypes

    reg = ctypes.CDLL(_lib.TORCH_LIB_PATH).chill_torch_register_entry_points
    reg.argtypes, reg.restype = [ctypes.c_void_p], ctypes.c_int64
    handle = _lib.register_entry_points(_lib.lib)
    assert handle >= 0 and _lib.register_entry_points(_lib.lib) == handle + 1
    bad = _lib.entry_points(_lib.lib)
    bad.magic ^= 1
    assert reg(ctypes.addressof(bad)) == -1 and reg(None) == -1
    old = _lib.entry_points(_lib.lib)
    old.abi_version += 1
    assert reg(ctypes.addressof(old)) == -2
    q = torch.zeros(1, 1, 8, 16)
    with pytest.raises(RuntimeError, match="not a handle"):
        op(q, q, q, None, handle + 1000, 1, [], 0.25, False)
    with pytest.raises((RuntimeError, NotImplementedError)):
        op(q, q, q, None, handle, 1, [], 0.25, False)  # CPU tensors: no kernel for them, no crash
