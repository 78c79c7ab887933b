"""ctypes loader of the C oracle (``chill_oracle.c``).  TEST INFRASTRUCTURE ONLY.

Builds ``_build/libchill_oracle.so`` with gcc on first use if it is missing (the library is tiny
and CPU-only).
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "_build", "libchill_oracle.so")

MASK_IDS = {
    "FullChillMask": 0,
    "CausalChillMask": 1,
    "SlidingWindowChillMask": 2,
    "ChunkwiseChillMask": 3,
    "PrefixLMChillMask": 4,
}


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(os.path.join(_DIR, "chill_oracle.c")):
        subprocess.check_call(["make", "-C", _DIR, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _SO


def _load():
    lib = ctypes.CDLL(build())
    i64, i32 = ctypes.c_int64, ctypes.c_int
    p64 = ctypes.POINTER(ctypes.c_int64)
    lib.oracle_pred.restype = i32
    lib.oracle_pred.argtypes = [i32, i64, i64, i64, i64]
    lib.oracle_dense_mask.restype = None
    lib.oracle_dense_mask.argtypes = [i32, i64, i64, i64, ctypes.POINTER(ctypes.c_uint8)]
    lib.oracle_nnz_bruteforce.restype = i64
    lib.oracle_nnz_bruteforce.argtypes = [i32, i64, i64, i64]
    lib.oracle_tile_ranges.restype = None
    lib.oracle_tile_ranges.argtypes = [i32, i64, i64, i32, i64, i64, i64, i64, i32, p64]
    lib.oracle_check_tile_ranges.restype = i64
    lib.oracle_check_tile_ranges.argtypes = [i32, i64, i64, i32, i64, i64, i64, i64, p64]
    lib.oracle_true_limits.restype = None
    lib.oracle_true_limits.argtypes = [i32, i64, i64, i32, i64, p64]
    lib.oracle_rule_limits.restype = None
    lib.oracle_rule_limits.argtypes = [i32, i64, i64, i32, i64, i64, p64]
    lib.oracle_is_full_block.restype = i32
    lib.oracle_is_full_block.argtypes = [i32, i64, i64, i64, i64, i64, i64]
    lib.oracle_has_full_blocks.restype = i32
    lib.oracle_has_full_blocks.argtypes = [i32, i64, i64, i64, i64, i64]
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def _ida(name, args):
    a = list(args) + [0, 0]
    return MASK_IDS[name], int(a[0]), int(a[1])


def _p64(arr):
    return arr.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))


def dense_mask(name, args, n):
    out = np.empty((n, n), dtype=np.uint8)
    lib().oracle_dense_mask(*_ida(name, args), n, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)))
    return out.astype(bool)


def nnz_bruteforce(name, args, n):
    return int(lib().oracle_nnz_bruteforce(*_ida(name, args), n))


def tile_ranges(name, args, qrows, T, seq_len, tile_in, tile_out, widened_q_full=False):
    n_tiles = -(-T // tile_in)
    out = np.zeros((n_tiles, 4), dtype=np.int64)
    lib().oracle_tile_ranges(*_ida(name, args), int(qrows), T, seq_len, tile_in, tile_out, int(widened_q_full), _p64(out))
    return out


def check_tile_ranges(name, args, qrows, T, seq_len, tile_in, tile_out, ranges):
    r = np.ascontiguousarray(ranges, dtype=np.int64)
    return int(lib().oracle_check_tile_ranges(*_ida(name, args), int(qrows), T, seq_len, tile_in, tile_out, _p64(r)))


def true_limits(name, args, which, n):
    out = np.zeros((n, 2), dtype=np.int64)
    lib().oracle_true_limits(*_ida(name, args), which, n, _p64(out))
    return out


def rule_limits(name, args, which, n, seq_len):
    out = np.zeros((n, 2), dtype=np.int64)
    lib().oracle_rule_limits(*_ida(name, args), which, n, seq_len, _p64(out))
    return out
