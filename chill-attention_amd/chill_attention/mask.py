"""The ``ChillMask`` family: parametric attention masks that lower to a mask-id + args descriptor.

Same public surface as the reference's ``chill_attention/mask.py`` (class names, constructor
arguments, ``name`` / ``constargs`` / ``__str__``, the rule methods and their inclusive /
half-open conventions, ``make_mask`` and ``verify``), but the rules here are plain integer / numpy
functions on the host, and the copy the GPU runs is the ``__host__ __device__`` functor of the same
mask id in ``csrc/chill_mask.h``.  ``make_mask`` and ``verify`` go through the compiled functors, so
verifying a mask verifies the code the kernels execute.

Rule conventions (reference mask.py:79-151):
  * ``k_range_for_q`` / ``q_range_for_k`` return INCLUSIVE ``(lo, hi)`` limits;
  * ``k_full_range_for_q`` / ``q_full_range_for_k`` return HALF-OPEN ``[lo, hi)`` ranges.
"""

from __future__ import annotations

import ctypes
import typing
from abc import ABC, abstractmethod

import numpy as np
import torch

from . import _lib


def _best_device() -> str:
    return "cuda" if torch.cuda.is_available() else "cpu"


class ChillMask(ABC):
    """Base class of attention masks (reference mask.py:15-250).

    Attributes:
        name: class name; custom ops are registered once per name.
        constargs: tuple of int / float / bool parameters, passed to the kernels at run time.
        mask_id: id of the compiled functor in the HIP library, ``None`` for masks that have none.
    """

    name: str
    constargs: typing.Tuple[typing.Union[int, float, bool], ...]
    mask_id: typing.Optional[int] = None

    def __init__(self, constargs=None):
        self.constargs = constargs or tuple()
        self.name = type(self).__name__
        assert isinstance(self.constargs, tuple), "mask arguments are given as one tuple"
        for i in self.constargs:
            assert isinstance(i, (int, float, bool)), "a mask argument must be an int, a float or a bool (operator schema)"

    def __str__(self):
        return f"{self.name}({', '.join(map(str, self.constargs))})"

    __repr__ = __str__

    # ------------------------------------------------------------------ rules (host statement)
    @staticmethod
    @abstractmethod
    def mask(q, k, seq_len, args):
        """Boolean ``[len(q), len(k)]`` array: True where query position q may attend key position k.
        The ``< seq_len`` limit is applied by the callers, not here."""

    @staticmethod
    @abstractmethod
    def q_range_for_k(k, seq_len, args):
        """Inclusive ``(lo, hi)`` query limits for key position(s) ``k``."""

    @staticmethod
    @abstractmethod
    def k_range_for_q(q, seq_len, args):
        """Inclusive ``(lo, hi)`` key limits for query position(s) ``q``."""

    @staticmethod
    def k_full_range_for_q(qb, TILE_Q, seq_len, args):
        """Half-open key range visible to EVERY query of the tile ``[qb, qb + TILE_Q)``."""
        return 0, 0

    @staticmethod
    def q_full_range_for_k(kb, TILE_K, seq_len, args):
        """Half-open query range that sees EVERY key of the tile ``[kb, kb + TILE_K)``."""
        return 0, 0

    @staticmethod
    def has_k_full_range():
        return False

    @staticmethod
    def has_q_full_range():
        return False

    @staticmethod
    def q_lims_continious():
        """Limits of a key tile are (q_range_for_k(first)[0], q_range_for_k(last)[1])."""
        return True

    @staticmethod
    def k_lims_continious():
        """Limits of a query tile are (k_range_for_q(first)[0], k_range_for_q(last)[1])."""
        return True

    @staticmethod
    def is_guaranteed_safe():
        """True if every query row sees at least one key."""
        return False

    @staticmethod
    def has_full_blocks(q_tile_size, k_tile_size, seq_len, args):
        return False

    @staticmethod
    def is_full_block(q, k, q_tile_size, k_tile_size, seq_len, args):
        return False

    # ------------------------------------------------------------------ lowering
    def descriptor(self) -> "_lib.ChillMaskDesc":
        """The mask-id + args descriptor handed to the C ABI."""
        return _descriptor(type(self), self.constargs)

    @classmethod
    def _library(cls):
        """The loaded library that holds this class's functor: the stock one for the built-in masks,
        a library of its own (built on first use, see ``user_mask``) for a user-written mask."""
        from . import user_mask

        return user_mask.library_for(cls) if user_mask.is_user_mask(cls) else _lib.lib

    # ------------------------------------------------------------------ enumeration
    def make_mask(self, max_pos: int) -> torch.Tensor:
        """Dense boolean mask ``[max_pos, max_pos]`` (rows = queries), reference mask.py:379-412.

        Enumerated by the compiled functor (host build of the header the kernels use)."""
        out = np.empty((max_pos, max_pos), dtype=np.uint8)
        desc = self.descriptor()
        _lib.check(
            "chill_mask_eval",
            self._library().chill_mask_eval(ctypes.byref(desc), max_pos, out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))),
        )
        return torch.from_numpy(out).to(torch.bool).to(_best_device())

    def _calc_limits(self, max_pos: int, which: int) -> torch.Tensor:
        """Per-position inclusive limits, evaluated like the reference's ``_calc_limits``
        (mask.py:414-454): rule called with ``seq_len`` rounded up to 32, values ``>= max_pos``
        clamped to ``max_pos - 1``.  ``which``: 0 = k_range_for_q, 1 = q_range_for_k."""
        total_pos = -(-max_pos // 32) * 32
        out = np.empty((max_pos, 2), dtype=np.int32)
        desc = self.descriptor()
        _lib.check(
            "chill_mask_limits",
            self._library().chill_mask_limits(
                ctypes.byref(desc), which, max_pos, total_pos, out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))
            ),
        )
        out = np.where(out >= max_pos, max_pos - 1, out)
        return torch.from_numpy(out)

    def _calc_tile_ranges(self, max_pos: int, tile_in: int, tile_out: int, pass_id: int = _lib.PASS_FWD,
                          seq_len: typing.Optional[int] = None) -> torch.Tensor:
        """``[n_tiles, 4]`` int32: (start_tile, end_tile, full_start_tile, full_end_tile) per row
        tile, exactly as the kernels compute them."""
        seq_len = max_pos if seq_len is None else seq_len
        n_tiles = -(-max_pos // tile_in)
        out = np.empty((n_tiles, 4), dtype=np.int32)
        desc = self.descriptor()
        _lib.check(
            "chill_tile_ranges",
            self._library().chill_tile_ranges(
                ctypes.byref(desc), pass_id, max_pos, seq_len, tile_in, tile_out,
                out.ctypes.data_as(ctypes.POINTER(ctypes.c_int32)),
            ),
        )
        return torch.from_numpy(out)

    def _calc_full_block_indices(self, max_pos, q_tile_size, k_tile_size):
        res = []
        for q in range(0, max_pos, q_tile_size):
            for k in range(0, max_pos, k_tile_size):
                if self.is_full_block(q, k, q_tile_size, k_tile_size, max_pos, self.constargs):
                    res.append((q, k))
        return res

    def nnz(self, max_pos: int) -> int:
        """Number of unmasked (q, k) pairs below ``max_pos`` (effective-FLOP numerator)."""
        desc = self.descriptor()
        return int(_lib.check("chill_mask_nnz", self._library().chill_mask_nnz(ctypes.byref(desc), max_pos)))

    def verify(self, max_pos: int):
        """Check every rule of the mask against brute-force enumeration of the dense mask.

        Same properties as the reference's ``verify`` (mask.py:700-803), plus two the reference
        does not check: ``q_full_range_for_k`` is sound, and the Python rules of this class agree
        with the compiled functors.

        Raises:
            AssertionError: on any inconsistency.
        """
        mask = self.make_mask(max_pos).cpu().numpy()
        assert mask.dtype == np.bool_, "Mask must be boolean"
        args = self.constargs
        pos = np.arange(max_pos)

        # python statement == compiled functor
        py_mask = np.asarray(self.mask(pos, pos, max_pos, args), dtype=bool)
        assert py_mask.shape == mask.shape and (py_mask == mask).all(), "python mask rule != compiled functor"

        k_lims_for_q = self._calc_limits(max_pos, 0).numpy()
        q_lims_for_k = self._calc_limits(max_pos, 1).numpy()
        total_pos = -(-max_pos // 32) * 32
        for rule, compiled in ((self.k_range_for_q, k_lims_for_q), (self.q_range_for_k, q_lims_for_k)):
            lo, hi = rule(pos, total_pos, args)
            py = np.stack([np.broadcast_to(lo, pos.shape), np.broadcast_to(hi, pos.shape)], axis=1)
            py = np.where(py >= max_pos, max_pos - 1, py)
            assert (py == compiled).all(), f"python {rule.__name__} != compiled functor"

        # analytical limits == true min / max of every non-empty row / column
        for name, dense, lims in (("k lims for q", mask, k_lims_for_q), ("q lims for k", mask.T, q_lims_for_k)):
            rows = np.nonzero(dense.any(axis=1))[0]
            real_lo = dense.argmax(axis=1)
            real_hi = dense.shape[1] - 1 - dense[:, ::-1].argmax(axis=1)
            bad = rows[(real_lo[rows] != lims[rows, 0]) | (real_hi[rows] != lims[rows, 1])]
            assert bad.size == 0, (
                f"Mismatch real vs analytical {name} at position {bad[:1]}: "
                f"real = {(real_lo[bad[:1]], real_hi[bad[:1]])}, analytical = {lims[bad[:1]]}"
            )

        # blocks flagged full are homogeneous
        tile_sizes = [16, 32, 64, 128, 256]
        for tq in tile_sizes:
            for tk in tile_sizes:
                if not self.has_full_blocks(tq, tk, seq_len=max_pos, args=args):
                    continue
                for q, k in self._calc_full_block_indices(max_pos, tq, tk):
                    tile = mask[q : q + tq, k : k + tk]
                    assert tile.all() or (~tile).all(), (
                        "Encountered unmasked block, while the mask says otherwise. "
                        f"{q = }, {k = }, {tq = }, {tk = }"
                    )

        # full ranges are all-True
        for has, rule, dense, what in (
            (self.has_k_full_range(), self.k_full_range_for_q, mask, "k_full_range_for_q"),
            (self.has_q_full_range(), self.q_full_range_for_k, mask.T, "q_full_range_for_k"),
        ):
            if not has:
                continue
            for tile in [16, 32, 64]:
                for b in range(0, max_pos, tile):
                    lo, hi = (int(x) for x in rule(b, tile, max_pos, args))
                    e = min(b + tile, max_pos)
                    hi = min(hi, max_pos)
                    if hi > lo:
                        assert dense[b:e, lo:hi].all(), (
                            f"{what} returned [{lo}, {hi}) for tile [{b}, {e}), but some tokens are masked"
                        )

    def make_flex_mask(self, max_pos):
        """FlexAttention ``BlockMask`` of the same pattern, or None (reference mask.py:473-483)."""
        return None

    def _calc_full_ranges(self, max_pos: int, TILE_Q: int) -> torch.Tensor:
        """``[n_tiles, 2]`` int32: the half-open predicate-free key range of every query tile
        (reference mask.py:507-534)."""
        n_tiles = -(-max_pos // TILE_Q)
        out = np.zeros((n_tiles, 2), dtype=np.int32)
        for i in range(n_tiles):
            lo, hi = self.k_full_range_for_q(i * TILE_Q, TILE_Q, max_pos, self.constargs)
            out[i] = (int(lo), int(hi))
        return torch.from_numpy(out)

    def plot(
        self,
        max_pos,
        draw_full_blocks: typing.Union[bool, int, typing.Tuple[int, int]] = False,
        plot_block_types: bool = False,
        TILE_Q: int = 32,
        TILE_K: int = 32,
    ):
        """Draw the mask (reference mask.py:536-698): left panel rows = queries, right panel its
        transpose, each with the analytical limits of the streamed axis drawn over it.

        Args:
            max_pos: number of positions to draw.
            draw_full_blocks: outline the blocks ``is_full_block`` reports — ``True`` for tile sizes
                16..256, an int for one square tile size, a pair for one ``(q, k)`` tile size.
            plot_block_types: shade, per query tile of ``TILE_Q`` rows, the key range that the
                kernels run without predicate (``k_full_range_for_q``).
            TILE_Q, TILE_K: tile sizes for ``plot_block_types``.

        Returns:
            matplotlib.figure.Figure
        """
        import itertools

        import matplotlib

        if not matplotlib.get_backend():
            matplotlib.use("Agg")
        import matplotlib.patches as patches
        import matplotlib.pyplot as plt

        dense = self.make_mask(max_pos).cpu().numpy()
        k_lims = self._calc_limits(max_pos, 0).numpy()  # per query: [lo, hi] over keys
        q_lims = self._calc_limits(max_pos, 1).numpy()  # per key: [lo, hi] over queries
        pos = np.arange(max_pos)

        fig, axes = plt.subplots(1, 2, figsize=(10, 5))
        panels = (
            (axes[0], dense, q_lims, "k index", "q index", "q_lims_for_k"),
            (axes[1], dense.T, k_lims, "q index", "k index", "k_lims_for_q"),
        )
        for ax, image, lims, xlabel, ylabel, what in panels:
            ax.imshow(image, origin="lower", vmin=0, vmax=1)
            ax.plot(pos, np.clip(lims[:, 0] - 0.5, -0.5, max_pos - 1), color="red", label=f"min {what}")
            ax.plot(pos, np.clip(lims[:, 1] + 0.5, -0.5, max_pos - 1), color="blue", label=f"max {what}")
            ax.set_xlabel(xlabel)
            ax.set_ylabel(ylabel)

        if draw_full_blocks:
            if isinstance(draw_full_blocks, bool):
                sizes_q = sizes_k = [16, 32, 64, 128, 256]
            elif isinstance(draw_full_blocks, int):
                sizes_q = sizes_k = [draw_full_blocks]
            else:
                sizes_q, sizes_k = [draw_full_blocks[0]], [draw_full_blocks[1]]
            styles = itertools.cycle(
                itertools.product(["black", "green", "violet", "purple", "darkorange", "white", "lightblue"], ["-", "--", ":"])
            )
            for tq in sizes_q:
                for tk in sizes_k:
                    if not self.has_full_blocks(tq, tk, seq_len=max_pos, args=self.constargs):
                        continue
                    color, style = next(styles)
                    for q, k in self._calc_full_block_indices(max_pos, tq, tk):
                        if q + tq > max_pos or k + tk > max_pos or not dense[q : q + tq, k : k + tk].any():
                            continue
                        for ax, (x, y, w, h) in zip(axes, ((k, q, tk, tq), (q, k, tq, tk))):
                            ax.add_patch(
                                patches.Rectangle((x - 0.5, y - 0.5), w, h, ls=style, ec=color, zorder=2, alpha=0.3, fill=False)
                            )

        if plot_block_types and self.has_k_full_range():
            full_ranges = self._calc_full_ranges(max_pos, TILE_Q).numpy()
            first = True
            for i, (ks, ke) in enumerate(full_ranges):
                if ke <= ks:
                    continue
                qb = i * TILE_Q
                style = dict(color="yellow", alpha=0.6, zorder=4, ec="red", ls="-", lw=1.5)
                axes[0].add_patch(
                    patches.Rectangle((ks - 0.5, qb - 0.5), ke - ks, TILE_Q, label="predicate-free range" if first else None, **style)
                )
                axes[1].add_patch(patches.Rectangle((qb - 0.5, ks - 0.5), TILE_Q, ke - ks, **style))
                first = False

        axes[0].legend()
        axes[1].legend()
        return fig


_DESC_IDS: dict = {}


def _descriptor(cls, constargs) -> "_lib.ChillMaskDesc":
    from . import user_mask

    mask_id = cls.mask_id
    if mask_id is None:
        if not user_mask.is_user_mask(cls):
            raise NotImplementedError(
                f"{cls.__name__} has no compiled functor: the built-in masks (Full, Causal, SlidingWindow, "
                "Chunkwise, PrefixLM) lower to a mask id, a mask of your own needs a `hip_functor` "
                "(see chill_attention.user_mask)"
            )
        mask_id = _lib.MASK_USER
    for a in constargs:
        if isinstance(a, float) and not float(a).is_integer():
            raise ValueError(f"{cls.__name__}: mask arguments must be integers, got {a!r}")
    return _lib.mask_desc(mask_id, [int(a) for a in constargs])


def _flex(mask_mod, max_pos):
    from torch.nn.attention.flex_attention import create_block_mask

    return create_block_mask(mask_mod, B=None, H=None, Q_LEN=max_pos, KV_LEN=max_pos, device=_best_device())


def _col(x):
    return np.asarray(x)[:, None]


def _row(x):
    return np.asarray(x)[None, :]


class FullChillMask(ChillMask):
    """Every query attends to every key (reference mask.py:806-889)."""

    mask_id = _lib.MASK_FULL

    def __init__(self):
        super().__init__()

    @staticmethod
    def mask(q, k, seq_len, args):
        return np.ones((len(np.atleast_1d(q)), len(np.atleast_1d(k))), dtype=bool)

    @staticmethod
    def q_range_for_k(k, seq_len, args):
        return np.zeros_like(k), np.zeros_like(k) + (seq_len - 1)

    @staticmethod
    def k_range_for_q(q, seq_len, args):
        return np.zeros_like(q), np.zeros_like(q) + (seq_len - 1)

    @staticmethod
    def k_full_range_for_q(qb, TILE_Q, seq_len, args):
        return 0, seq_len

    @staticmethod
    def q_full_range_for_k(kb, TILE_K, seq_len, args):
        return 0, seq_len

    @staticmethod
    def has_k_full_range():
        return True

    @staticmethod
    def has_q_full_range():
        return True

    @staticmethod
    def is_guaranteed_safe():
        return True

    @staticmethod
    def has_full_blocks(q_tile_size, k_tile_size, seq_len, args):
        return True

    @staticmethod
    def is_full_block(q, k, q_tile_size, k_tile_size, seq_len, args):
        return True

    def make_flex_mask(self, max_pos):
        return _flex(lambda b, h, q_idx, kv_idx: q_idx >= 0, max_pos)


class CausalChillMask(ChillMask):
    """Query q attends to keys k <= q (reference mask.py:892-976)."""

    mask_id = _lib.MASK_CAUSAL

    def __init__(self):
        super().__init__()

    @staticmethod
    def mask(q, k, seq_len, args):
        return _col(q) >= _row(k)

    @staticmethod
    def q_range_for_k(k, seq_len, args):
        return k, np.zeros_like(k) + (seq_len - 1)

    @staticmethod
    def k_range_for_q(q, seq_len, args):
        return np.zeros_like(q), q

    @staticmethod
    def k_full_range_for_q(qb, TILE_Q, seq_len, args):
        return 0, qb + 1

    @staticmethod
    def q_full_range_for_k(kb, TILE_K, seq_len, args):
        return max(0, kb + TILE_K - 1), seq_len

    @staticmethod
    def has_k_full_range():
        return True

    @staticmethod
    def has_q_full_range():
        return True

    @staticmethod
    def is_guaranteed_safe():
        return True

    @staticmethod
    def has_full_blocks(q_tile_size, k_tile_size, seq_len, args):
        return (k_tile_size - 1) <= seq_len - q_tile_size

    @staticmethod
    def is_full_block(q, k, q_tile_size, k_tile_size, seq_len, args):
        return (k + k_tile_size - 1) <= q

    def make_flex_mask(self, max_pos):
        return _flex(lambda b, h, q_idx, kv_idx: q_idx >= kv_idx, max_pos)


class SlidingWindowChillMask(ChillMask):
    """Query q attends to keys in ``[q - left_context, q + right_context]`` (reference mask.py:979-1108).

    Args:
        left_context: number of preceding positions visible.
        right_context: number of following positions visible.
    """

    mask_id = _lib.MASK_SLIDING_WINDOW

    def __init__(self, left_context, right_context):
        super().__init__((left_context, right_context))

    @staticmethod
    def mask(q, k, seq_len, args):
        left, right = args
        return (_row(k) <= _col(q) + right) & (_row(k) >= _col(q) - left)

    @staticmethod
    def q_range_for_k(k, seq_len, args):
        left, right = args
        return np.maximum(0, k - right), np.minimum(k + left, seq_len - 1)

    @staticmethod
    def k_range_for_q(q, seq_len, args):
        left, right = args
        return np.maximum(0, q - left), np.minimum(q + right, seq_len - 1)

    @staticmethod
    def k_full_range_for_q(qb, TILE_Q, seq_len, args):
        left, right = args
        start = max(0, qb + TILE_Q - 1 - left)
        end = min(seq_len, qb + right + 1)
        return start, max(start, end)

    @staticmethod
    def q_full_range_for_k(kb, TILE_K, seq_len, args):
        # not defined by the reference (it inherits (0, 0)); the window transposed
        left, right = args
        start = max(0, kb + TILE_K - 1 - right)
        end = min(seq_len, kb + left + 1)
        return start, max(start, end)

    @staticmethod
    def has_k_full_range():
        return True

    @staticmethod
    def has_q_full_range():
        return True

    @staticmethod
    def is_guaranteed_safe():
        return False

    @staticmethod
    def has_full_blocks(q_tile_size, k_tile_size, seq_len, args):
        left, right = args
        return (
            (q_tile_size <= left and k_tile_size <= right)
            or (q_tile_size * 2 <= left)
            or (k_tile_size * 2 <= right)
        )

    @staticmethod
    def is_full_block(q, k, q_tile_size, k_tile_size, seq_len, args):
        left, right = args

        def inside(diff):
            return (0 <= diff <= left) or (-right <= diff <= 0)

        return inside((q + q_tile_size - 1) - k) and inside(q - (k + k_tile_size - 1))

    def make_flex_mask(self, max_pos):
        left, right = self.constargs

        def sliding_window(b, h, q_idx, kv_idx):
            diff = q_idx - kv_idx
            return ((diff <= left) & (diff >= 0)) | ((diff >= -right) & (diff <= 0))

        return _flex(sliding_window, max_pos)


class ChunkwiseChillMask(ChillMask):
    """The sequence is cut into chunks of ``context_size``; a query attends to its own chunk and the
    ``back_contexts`` chunks before it (reference mask.py:1111-1266).

    Args:
        context_size: chunk length.
        back_contexts: number of preceding chunks visible.
    """

    mask_id = _lib.MASK_CHUNKWISE

    def __init__(self, context_size, back_contexts):
        super().__init__((context_size, back_contexts))

    @staticmethod
    def mask(q, k, seq_len, args):
        context, back = args
        diff = _col(q) // context - _row(k) // context
        return (diff >= 0) & (diff <= back)

    @staticmethod
    def q_range_for_k(k, seq_len, args):
        context, back = args
        kc = k // context
        return kc * context, np.minimum((kc + back + 1) * context - 1, seq_len - 1)

    @staticmethod
    def k_range_for_q(q, seq_len, args):
        context, back = args
        qc = q // context
        return np.maximum(0, (qc - back) * context), np.minimum((qc + 1) * context - 1, seq_len - 1)

    @staticmethod
    def k_full_range_for_q(qb, TILE_Q, seq_len, args):
        context, back = args
        start = max(0, ((qb + TILE_Q - 1) // context - back) * context)
        end = min(seq_len, (qb // context + 1) * context)
        return start, max(start, end)

    @staticmethod
    def q_full_range_for_k(kb, TILE_K, seq_len, args):
        # not defined by the reference (it inherits (0, 0))
        context, back = args
        start = ((kb + TILE_K - 1) // context) * context
        end = min(seq_len, (kb // context + back + 1) * context)
        return start, max(start, end)

    @staticmethod
    def has_k_full_range():
        return True

    @staticmethod
    def has_q_full_range():
        return True

    @staticmethod
    def is_guaranteed_safe():
        return False

    @staticmethod
    def has_full_blocks(q_tile_size, k_tile_size, seq_len, args):
        context, back = args
        # worst case: the last query tile that still sees chunk 0
        return ChunkwiseChillMask.is_full_block(
            context * (back + 1) - q_tile_size, 0, q_tile_size, k_tile_size, seq_len, args
        )

    @staticmethod
    def is_full_block(q, k, q_tile_size, k_tile_size, seq_len, args):
        context, back = args
        d0 = q // context - (k + k_tile_size - 1) // context
        d1 = (q + q_tile_size - 1) // context - k // context
        return bool((0 <= d0 <= back) and (0 <= d1 <= back))

    def make_flex_mask(self, max_pos):
        context, back = self.constargs

        def chunkwise(b, h, q_idx, kv_idx):
            diff = q_idx // context - kv_idx // context
            return (diff >= 0) & (diff <= back)

        return _flex(chunkwise, max_pos)


class PrefixLMChillMask(ChillMask):
    """Bidirectional attention inside the first ``prefix_size`` positions, causal after
    (reference mask.py:1269-1394).

    Args:
        prefix_size: length of the bidirectional prefix.
    """

    mask_id = _lib.MASK_PREFIX_LM

    def __init__(self, prefix_size):
        super().__init__((prefix_size,))

    @staticmethod
    def mask(q, k, seq_len, args):
        prefix = args[0]
        return (_row(k) < prefix) | (_col(q) >= _row(k))

    @staticmethod
    def q_range_for_k(k, seq_len, args):
        prefix = args[0]
        return np.where(k < prefix, 0, k), np.zeros_like(k) + (seq_len - 1)

    @staticmethod
    def k_range_for_q(q, seq_len, args):
        prefix = args[0]
        return np.zeros_like(q), np.minimum(np.maximum(q, prefix - 1), seq_len - 1)

    @staticmethod
    def k_full_range_for_q(qb, TILE_Q, seq_len, args):
        prefix = args[0]
        return 0, min(max(prefix, qb + 1), seq_len)

    @staticmethod
    def q_full_range_for_k(kb, TILE_K, seq_len, args):
        # not defined by the reference (it inherits (0, 0))
        prefix = args[0]
        if kb + TILE_K <= prefix:
            return 0, seq_len
        return min(kb + TILE_K - 1, seq_len), seq_len

    @staticmethod
    def has_k_full_range():
        return True

    @staticmethod
    def has_q_full_range():
        return True

    @staticmethod
    def is_guaranteed_safe():
        return True

    @staticmethod
    def has_full_blocks(q_tile_size, k_tile_size, seq_len, args):
        return True

    @staticmethod
    def is_full_block(q, k, q_tile_size, k_tile_size, seq_len, args):
        prefix = args[0]
        causal_full = (k + k_tile_size - 1) <= q
        in_prefix = (q + q_tile_size <= prefix) and (k + k_tile_size <= prefix)
        return bool(causal_full or in_prefix)

    def make_flex_mask(self, max_pos):
        prefix = self.constargs[0]
        return _flex(lambda b, h, q, k: (k < prefix) | (q >= k), max_pos)


if __name__ == "__main__":
    # python -m chill_attention.mask: draw a mask and check its rules (reference mask.py:1397-1407)
    import matplotlib

    matplotlib.use("Agg")
    demo = SlidingWindowChillMask(10, 4)
    demo.plot(200, True).savefig("mask.png")
    demo.verify(1024)
    print(f"{demo}: rules verified up to 1024 positions, drawing in mask.png")
