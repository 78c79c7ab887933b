"""A worked example of a user-written mask (see ``user_mask``): attention sinks plus a causal window.

A query sees the first ``sinks`` keys and the ``window`` keys before it (itself included) — the
pattern of streaming LLM inference.  The device statement is the functor in
``csrc/chill_user_mask.h``; the numpy statements below are what ``verify()`` checks it against.
"""

from __future__ import annotations

import os

import numpy as np

from .mask import ChillMask, _col, _row
from .user_mask import CSRC_DIR


class SinkWindowChillMask(ChillMask):
    """``k <= q`` and (``k < sinks`` or ``q - k <= window``)."""

    hip_header = os.path.join(CSRC_DIR, "chill_user_mask.h")

    def __init__(self, sinks: int, window: int):
        super().__init__((sinks, window))

    @staticmethod
    def mask(q, k, seq_len, args):
        sinks, window = args
        q, k = _col(q), _row(k)
        return (k <= q) & ((k < sinks) | (q - k <= window))

    @staticmethod
    def k_range_for_q(q, seq_len, args):
        sinks, window = args
        lo = np.zeros_like(q) if sinks > 0 else np.maximum(0, q - window)
        return lo, q

    @staticmethod
    def q_range_for_k(k, seq_len, args):
        # the upper limit drops when k leaves the sinks: the limits are not monotone, and the
        # functor says so (kMonotoneLimits = false)
        sinks, window = args
        return k, np.where(k < sinks, seq_len - 1, np.minimum(k + window, seq_len - 1))

    @staticmethod
    def is_guaranteed_safe():
        return True

    @staticmethod
    def q_lims_continious():
        return False
