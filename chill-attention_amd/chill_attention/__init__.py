"""chill_attention for MI355X: sparse flash attention with parametric masks on hand-written
gfx950 kernels.  Same exports as the reference package (chill_attention/__init__.py:1-13)."""

from .chill import (
    _chill_reference_naive,
    chill_attention,
    register_chill_mask,
)
from .mask import (
    CausalChillMask,
    ChillMask,
    ChunkwiseChillMask,
    FullChillMask,
    PrefixLMChillMask,
    SlidingWindowChillMask,
)

__all__ = [
    "chill_attention",
    "register_chill_mask",
    "_chill_reference_naive",
    "ChillMask",
    "FullChillMask",
    "CausalChillMask",
    "SlidingWindowChillMask",
    "ChunkwiseChillMask",
    "PrefixLMChillMask",
]
