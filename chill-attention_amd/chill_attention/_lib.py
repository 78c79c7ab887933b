"""ctypes binding of the gfx950 shared library (C ABI declared in ``include/chill_attention.h``).

The library is the only compute path: if it has not been built, importing this module raises, and
nothing in the package falls back to another implementation.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_uint8, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# CHILL_ATTENTION_LIB names another build of the same library (for A/B measurements)
LIB_PATH = os.environ.get("CHILL_ATTENTION_LIB") or os.path.join(os.path.dirname(_PKG_DIR), "lib", "libchill_attention_hip.so")

ABI_VERSION = 1

# ChillDType / ChillMaskId / ChillPass of the header
F32, F16, BF16 = 0, 1, 2
MASK_FULL, MASK_CAUSAL, MASK_SLIDING_WINDOW, MASK_CHUNKWISE, MASK_PREFIX_LM = range(5)
MASK_USER = 5  # the one mask of a library built around a user-written functor
PASS_FWD, PASS_DQ, PASS_DKDV = 0, 1, 2


class ChillMaskDesc(ctypes.Structure):
    _fields_ = [("id", c_int32), ("nargs", c_int32), ("args", c_int64 * 4)]


class ChillTensor4(ctypes.Structure):
    _fields_ = [("ptr", c_void_p), ("stride", c_int64 * 4)]


class ChillLibraryError(RuntimeError):
    """A C-ABI call returned a negative status."""

    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed with status {status}: {text}")
        self.status = status


def load_library(path: str) -> ctypes.CDLL:
    """Load one build of the library (the stock one, or one built around a user mask) and declare
    the C ABI on it."""
    if not os.path.exists(path):
        raise ImportError(
            f"chill_attention: the HIP library {path} has not been built "
            "(run `make -C chill-attention_amd/csrc -j8` or `python -c 'import __graft_entry__ as g; g.build()'`). "
            "There is no fallback implementation."
        )
    lib = ctypes.CDLL(path)
    P = POINTER
    T4 = P(ChillTensor4)
    MD = P(ChillMaskDesc)
    I64_3 = P(c_int64)
    sig = {
        "chill_fwd": (c_int32, [T4, T4, T4, T4, c_void_p, I64_3, c_void_p, c_int64,
                                c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_float, MD, c_void_p]),
        "chill_bwd_delta": (c_int32, [T4, T4, c_void_p, I64_3, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p]),
        "chill_bwd_dq": (c_int32, [T4, T4, T4, T4, T4, c_void_p, I64_3, c_void_p, I64_3, c_void_p, c_int64,
                                   c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_float, MD, c_void_p]),
        "chill_bwd_dq_delta": (c_int32, [T4, T4, T4, T4, T4, T4, c_void_p, I64_3, c_void_p, I64_3, c_void_p, c_int64,
                                         c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_float, MD, c_void_p]),
        "chill_bwd_dkdv": (c_int32, [T4, T4, T4, T4, T4, T4, c_void_p, I64_3, c_void_p, I64_3, c_void_p, c_int64,
                                     c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_float, MD, c_void_p]),
        "chill_bwd_noalloc": (c_int32, [T4, T4, T4, T4, T4, T4, T4, T4, c_void_p, I64_3, c_void_p, c_int64,
                                        c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_float, MD, c_void_p]),
        "chill_mask_eval_device": (c_int32, [MD, c_int32, c_void_p, c_void_p]),
        "chill_tile_ranges_device": (c_int32, [MD, c_int32, c_int32, c_int32, c_int32, c_int32, c_void_p, c_void_p]),
        "chill_mask_eval": (c_int32, [MD, c_int32, P(c_uint8)]),
        "chill_mask_limits": (c_int32, [MD, c_int32, c_int32, c_int32, P(c_int32)]),
        "chill_tile_ranges": (c_int32, [MD, c_int32, c_int32, c_int32, c_int32, c_int32, P(c_int32)]),
        "chill_mask_is_full_block": (c_int32, [MD, c_int32, c_int32, c_int32, c_int32, c_int32]),
        "chill_mask_has_full_blocks": (c_int32, [MD, c_int32, c_int32, c_int32]),
        "chill_tile_config": (c_int32, [c_int32, c_int32, c_int32, c_int32, P(c_int32)]),
        "chill_tile_config_for_shape": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int64, c_int32, P(c_int32)]),
        "chill_tile_config_for_launch": (c_int32, [P(ChillMaskDesc), c_int32, c_int32, c_int32, c_int64, c_int32, P(c_int32)]),
        "chill_work_item": (c_int32, [c_int32, c_int32, c_int32]),
        "chill_mask_nnz": (c_int64, [MD, c_int32]),
        "chill_status_string": (c_char_p, [c_int32]),
        "chill_abi_version": (c_int32, []),
        "chill_has_user_mask": (c_int32, []),
    }
    for name, (restype, argtypes) in sig.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.chill_abi_version()
    if got != ABI_VERSION:
        raise ImportError(f"chill_attention: library ABI version {got}, binding expects {ABI_VERSION}")
    return lib


lib = load_library(LIB_PATH)
EXPORTED_SYMBOLS = (
    "chill_fwd", "chill_bwd_delta", "chill_bwd_dq", "chill_bwd_dq_delta", "chill_bwd_dkdv", "chill_bwd_noalloc", "chill_mask_eval_device",
    "chill_tile_ranges_device", "chill_mask_eval", "chill_mask_limits", "chill_tile_ranges",
    "chill_mask_is_full_block", "chill_mask_has_full_blocks", "chill_tile_config", "chill_tile_config_for_shape",
    "chill_tile_config_for_launch", "chill_work_item",
    "chill_mask_nnz",
    "chill_status_string", "chill_abi_version", "chill_has_user_mask",
)


BWD_NOALLOC_MAX_ROWS = 4 * 1024 * 1024  # CHILL_BWD_NOALLOC_MAX_ROWS of the header

# The eager-mode operator registered from C++ (csrc/chill_torch.cpp): the same adapters and autograd
# formula as the torch.library layer of chill.py without its per-call Python cost.  It links against no
# kernel library; a call names the entry points it is to use through a table built here.
TORCH_LIB_PATH = os.path.join(os.path.dirname(LIB_PATH), "libchill_attention_torch.so")


ENTRY_POINTS_MAGIC = 0x4350454C4C494843  # "CHILLEPC", as csrc/chill_torch.cpp checks it


class EntryPoints(ctypes.Structure):
    """Addresses of one kernel library's entry points behind a magic word, the ABI version and the size
    of the table, in the order csrc/chill_torch.cpp declares."""

    _fields_ = [("magic", ctypes.c_uint64), ("abi_version", ctypes.c_uint32), ("bytes", ctypes.c_uint32)] + [
        (n, c_void_p) for n in ("fwd", "dq_delta", "dkdv", "status_string")]


def entry_points(cdll: ctypes.CDLL) -> EntryPoints:
    names = ("chill_fwd", "chill_bwd_dq_delta", "chill_bwd_dkdv", "chill_status_string")
    return EntryPoints(ENTRY_POINTS_MAGIC, cdll.chill_abi_version(), ctypes.sizeof(EntryPoints),
                       *(ctypes.cast(getattr(cdll, n), c_void_p).value for n in names))


def register_entry_points(cdll: ctypes.CDLL) -> int:
    """Hands the entry points of one kernel library to the C++ operator; returns the handle its calls name
    the library by."""
    assert torch_operator() is not None
    reg = ctypes.CDLL(TORCH_LIB_PATH).chill_torch_register_entry_points
    reg.argtypes, reg.restype = [c_void_p], ctypes.c_int64
    table = entry_points(cdll)
    handle = reg(ctypes.addressof(table))
    if handle < 0:
        raise RuntimeError(f"{TORCH_LIB_PATH} refuses the entry points of {cdll._name} "
                           f"({'another ABI version' if handle == -2 else 'not a table'})")
    return handle


_torch_operator = False  # not looked for yet


def torch_operator():
    """``torch.ops.chill_attention_amd.attention``, or None when its library has not been built or
    CHILL_ATTENTION_EAGER_OP=0 asks for the Python operator layer."""
    global _torch_operator
    if _torch_operator is False:
        _torch_operator = None
        if os.environ.get("CHILL_ATTENTION_EAGER_OP", "1") != "0" and os.path.exists(TORCH_LIB_PATH):
            import torch

            try:
                torch.ops.load_library(TORCH_LIB_PATH)
                _torch_operator = torch.ops.chill_attention_amd.attention
            except (OSError, RuntimeError) as e:
                # built against another PyTorch: the torch.library operators do the same work
                import warnings

                warnings.warn(f"chill_attention: {TORCH_LIB_PATH} does not load ({e}); eager calls take the "
                              "torch.library operators (rebuild with `make -C chill-attention_amd/csrc`)")
    return _torch_operator


def check(fn: str, status: int) -> int:
    """Raise for a negative status, pass non-negative values through."""
    if status < 0:
        raise ChillLibraryError(fn, status, lib.chill_status_string(status).decode())
    return status


def mask_desc(mask_id: int, args) -> ChillMaskDesc:
    d = ChillMaskDesc()
    d.id = mask_id
    d.nargs = len(args)
    if len(args) > 4:
        raise ValueError("a mask descriptor carries at most 4 arguments")
    for i, a in enumerate(args):
        d.args[i] = int(a)
    return d


def tensor4(t) -> ChillTensor4:
    """View of a 4-d torch tensor: raw pointer + element strides."""
    v = ChillTensor4()
    v.ptr = t.data_ptr()
    for i in range(4):
        v.stride[i] = t.stride(i)
    return v


def strides3(t):
    return (c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))
