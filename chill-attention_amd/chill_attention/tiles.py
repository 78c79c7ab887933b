"""Static MI355X tile table (the counterpart of the reference's ``autotune.py`` default tables).

The table itself is compiled into the HIP library (``csrc/chill_tiles.h``) so the kernels and this
report cannot disagree; these helpers only read it.
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}


def tile_config(mask, head_dim: int, dtype: torch.dtype, pass_id: int, seq_len: int | None = None,
                batch_heads: int = 1 << 20) -> dict:
    """Tile shape the library uses for ``(mask class, head_dim, dtype, pass)``; with ``seq_len`` (and
    ``batch_heads`` = B * H) for a launch of that shape: the forward and dQ rows of 16-bit inputs at
    head dim 128 use a smaller workgroup for short sequences and for grids that would not fill the chip.
    Without ``seq_len``: the row of long sequences on a full chip.

    Returns ``{"rows", "streamed", "waves", "lds_bytes"}``: resident rows per workgroup (query
    rows for forward / dQ, key rows for dK/dV), rows of one streamed tile, wavefronts per
    workgroup and LDS bytes per workgroup.
    """
    out = (ctypes.c_int32 * 4)()
    mask_id = mask.mask_id if mask.mask_id is not None else _lib.MASK_USER
    lib = mask._library()
    if seq_len is None:
        _lib.check("chill_tile_config", lib.chill_tile_config(mask_id, head_dim, _DTYPES[dtype], pass_id, out))
    else:
        # (with the mask's arguments: the dK/dV row of a chunkwise mask depends on the chunk size)
        desc = mask.descriptor()
        _lib.check(
            "chill_tile_config_for_launch",
            lib.chill_tile_config_for_launch(ctypes.byref(desc), head_dim, _DTYPES[dtype], pass_id, batch_heads, seq_len, out),
        )
    return {"rows": out[0], "streamed": out[1], "waves": out[2], "lds_bytes": out[3]}


def _get_default_config_fwd(head_dim, dtype, mask=None):
    """(TILE_Q, TILE_K, waves) of the forward kernel — cf. reference autotune.py:98-107."""
    from .mask import CausalChillMask

    c = tile_config(mask or CausalChillMask(), head_dim, dtype, _lib.PASS_FWD)
    return c["rows"], c["streamed"], c["waves"]


def _get_default_config_bwd(head_dim, dtype, mask=None):
    """((TILE_DQ_Q, TILE_DQ_K, waves), (TILE_DK_Q, TILE_DK_K, waves)) — cf. reference autotune.py:110-119."""
    from .mask import CausalChillMask

    m = mask or CausalChillMask()
    dq = tile_config(m, head_dim, dtype, _lib.PASS_DQ)
    dk = tile_config(m, head_dim, dtype, _lib.PASS_DKDV)
    return (dq["rows"], dq["streamed"], dq["waves"]), (dk["streamed"], dk["rows"], dk["waves"])
