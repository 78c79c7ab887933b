"""CPU oracle for the chill-attention hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, on the CPU, the algorithm of the reference (alexdremov/chill-attention
v2.1.0) for the path the HIP library implements.  Only ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py`` may import it; the product never does.

It deliberately shares no code with the product: the mask rules below are written from the
reference's second, plain-PyTorch statement of every mask (the FlexAttention ``mask_mod``s) and
from its range rules, independently of ``csrc/chill_mask.h`` and ``chill_attention/mask.py``.

What each function follows (paths relative to the reference repository), and how it is pinned:

  mask_pred            mask.py:870-871, 957-958, 1069-1073, 1224-1227, 1368-1371 (mask_mod) and
                       :825, 911, 1010-1012, 1145-1148, 1301-1304 (Triton rule).
                       Pinned by tests/test_oracle.py: the two statements agree for n <= 1030 and
                       special cases reduce to each other (SW(0,0) = identity, PrefixLM(p >= n) = Full,
                       Chunkwise(c >= n) = Full, Chunkwise(1, b) = SW(b, 0), Causal = tril).
  k_range_for_q,       mask.py:828-835, 914-921, 1015-1038, 1151-1185, 1307-1336.
  q_range_for_k        Pinned by brute force: equal to the per-row / per-column min and max of the
                       dense mask (the property mask.verify checks, mask.py:737-761).
  k_full_range_for_q,  mask.py:838-853, 924-940, 1041-1051, 1188-1206, 1339-1350 (+ base class
  q_full_range_for_k   (0, 0), mask.py:110-151).  Pinned by brute force: the range is all-True, and
                       for k_full_range_for_q maximal when non-empty.
  is_full_block,       mask.py:876-889, 963-976, 1080-1108, 1234-1266, 1378-1394.  Pinned by brute
  has_full_blocks      force: flagged blocks are homogeneous (mask.py:763-779).
  min_max_tiles        utils.py:221-272 (continuous path).  Pinned by brute force against the hull
                       of non-empty tiles of the dense mask.
  split_tiles          chill_fwd.py:161-185 (same logic chill_bwd_dq.py:279-293,
                       chill_bwd_dkdv.py:329-344).  Pinned by brute force: tiles inside the full
                       sub-range are all-True.
  reference_naive      chill.py:498-544 (dense mask -> torch SDPA, lens / GQA handling).  Pinned
                       against attention_f64 (textbook softmax in float64) and against torch's own
                       is_causal / unmasked SDPA special cases.
  attention_f64        textbook forward and analytic backward in float64; pinned by central finite
                       differences on tiny inputs and by autograd through reference_naive.
  lse2                 chill_fwd.py:328 (base-2 LSE including the scale); closed form via logsumexp.
  delta                utils.py:190.
  nnz, flops           benchmark/benchmark.py:271-276; closed forms pinned against dense_mask().sum().
"""

from __future__ import annotations

import math

import numpy as np

MASK_NAMES = (
    "FullChillMask",
    "CausalChillMask",
    "SlidingWindowChillMask",
    "ChunkwiseChillMask",
    "PrefixLMChillMask",
)


# --------------------------------------------------------------------------------------------
# mask predicate — two independent statements
# --------------------------------------------------------------------------------------------
def mask_pred(name, args, q, k):
    """Boolean [len(q), len(k)] from the reference's Triton rule (mask.py:825, 911, 1010-1012,
    1145-1148, 1301-1304).  For a user-written mask ``name`` is the test's own statement of the
    predicate, a callable ``(q[:, None], k[None, :], args) -> bool array``."""
    q = np.asarray(q, dtype=np.int64)[:, None]
    k = np.asarray(k, dtype=np.int64)[None, :]
    if callable(name):
        return np.broadcast_to(np.asarray(name(q, k, args), dtype=bool), (q.shape[0], k.shape[1])).copy()
    if name == "FullChillMask":
        return np.ones((q.shape[0], k.shape[1]), dtype=bool)
    if name == "CausalChillMask":
        return q >= k
    if name == "SlidingWindowChillMask":
        left, right = args
        return (k <= q + right) & (k >= q - left)
    if name == "ChunkwiseChillMask":
        c, back = args
        d = q // c - k // c
        return (d >= 0) & (d <= back)
    if name == "PrefixLMChillMask":
        (prefix,) = args
        return (k < prefix) | (q >= k)
    raise KeyError(name)


def mask_pred_flex(name: str, args, q, k):
    """The reference's second statement: its FlexAttention mask_mod bodies (mask.py:870-871,
    957-958, 1069-1073, 1224-1227, 1368-1371)."""
    q = np.asarray(q, dtype=np.int64)[:, None]
    k = np.asarray(k, dtype=np.int64)[None, :]
    if name == "FullChillMask":
        return np.broadcast_to(q >= 0, (q.shape[0], k.shape[1])).copy()
    if name == "CausalChillMask":
        return q >= k
    if name == "SlidingWindowChillMask":
        left, right = args
        diff = q - k
        return ((diff <= left) & (diff >= 0)) | ((diff >= -right) & (diff <= 0))
    if name == "ChunkwiseChillMask":
        c, back = args
        d = q // c - k // c
        return (d >= 0) & (d <= back)
    if name == "PrefixLMChillMask":
        (prefix,) = args
        return (k < prefix) | (q >= k)
    raise KeyError(name)


def dense_mask(name: str, args, n: int) -> np.ndarray:
    """make_mask(n): pred & q < n & k < n (mask.py:313-315, 379-412)."""
    pos = np.arange(n)
    return mask_pred(name, args, pos, pos)


# --------------------------------------------------------------------------------------------
# range rules (inclusive) and full ranges (half-open)
# --------------------------------------------------------------------------------------------
def k_range_for_q(name, args, q: int, seq_len: int):
    if name == "FullChillMask":
        return 0, seq_len - 1
    if name == "CausalChillMask":
        return 0, q
    if name == "SlidingWindowChillMask":
        left, right = args
        return max(0, q - left), min(q + right, seq_len - 1)
    if name == "ChunkwiseChillMask":
        c, back = args
        qc = q // c
        return max(0, (qc - back) * c), min((qc + 1) * c - 1, seq_len - 1)
    if name == "PrefixLMChillMask":
        (prefix,) = args
        return 0, min(max(q, prefix - 1), seq_len - 1)
    raise KeyError(name)


def q_range_for_k(name, args, k: int, seq_len: int):
    if name == "FullChillMask":
        return 0, seq_len - 1
    if name == "CausalChillMask":
        return k, seq_len - 1
    if name == "SlidingWindowChillMask":
        left, right = args
        return max(0, k - right), min(k + left, seq_len - 1)
    if name == "ChunkwiseChillMask":
        c, back = args
        kc = k // c
        return kc * c, min((kc + back + 1) * c - 1, seq_len - 1)
    if name == "PrefixLMChillMask":
        (prefix,) = args
        return (0 if k < prefix else k), seq_len - 1
    raise KeyError(name)


def k_full_range_for_q(name, args, qb: int, tile_q: int, seq_len: int):
    if name == "FullChillMask":
        return 0, seq_len
    if name == "CausalChillMask":
        return 0, qb + 1
    if name == "SlidingWindowChillMask":
        left, right = args
        start = max(0, qb + tile_q - 1 - left)
        end = min(seq_len, qb + right + 1)
        return start, max(start, end)
    if name == "ChunkwiseChillMask":
        c, back = args
        k_end = (qb // c + 1) * c
        k_start = ((qb + tile_q - 1) // c - back) * c
        start = max(0, k_start)
        return start, max(start, min(seq_len, k_end))
    if name == "PrefixLMChillMask":
        (prefix,) = args
        return 0, min(max(prefix, qb + 1), seq_len)
    raise KeyError(name)


def q_full_range_for_k(name, args, kb: int, tile_k: int, seq_len: int):
    """The reference defines this only for Full and Causal (mask.py:847-853, 933-940); the other
    masks inherit the empty range (mask.py:131-151)."""
    if name == "FullChillMask":
        return 0, seq_len
    if name == "CausalChillMask":
        return max(0, kb + tile_k - 1), seq_len
    return 0, 0


def q_full_range_exact(name, args, kb: int, tile_k: int, seq_len: int):
    """Largest interval of queries that see every key of [kb, kb + tile_k) (keys clipped to
    seq_len), by brute force.  Used to judge ranges the reference leaves undefined.  Returns
    (lo, hi) half-open, or (0, 0) if no query qualifies, or None if the qualifying set is not an
    interval."""
    ke = min(kb + tile_k, seq_len)
    if ke <= kb:
        return 0, 0
    sub = mask_pred(name, args, np.arange(seq_len), np.arange(kb, ke)).all(axis=1)
    idx = np.nonzero(sub)[0]
    if idx.size == 0:
        return 0, 0
    if idx[-1] - idx[0] + 1 != idx.size:
        return None
    return int(idx[0]), int(idx[-1]) + 1


def is_full_block(name, args, q: int, k: int, tq: int, tk: int, seq_len: int) -> bool:
    if name == "FullChillMask":
        return True
    if name == "CausalChillMask":
        return (k + tk - 1) <= q
    if name == "SlidingWindowChillMask":
        left, right = args

        def inside(diff):
            return ((diff <= left) and (diff >= 0)) or ((diff >= -right) and (diff <= 0))

        return inside((q + tq - 1) - k) and inside(q - (k + tk - 1))
    if name == "ChunkwiseChillMask":
        c, back = args
        d0 = q // c - (k + tk - 1) // c  # Python floor division, q may be negative (mask.py:1239-1246)
        d1 = (q + tq - 1) // c - k // c
        return (0 <= d0 <= back) and (0 <= d1 <= back)
    if name == "PrefixLMChillMask":
        (prefix,) = args
        return ((k + tk - 1) <= q) or ((q + tq <= prefix) and (k + tk <= prefix))
    raise KeyError(name)


def has_full_blocks(name, args, tq: int, tk: int, seq_len: int) -> bool:
    if name in ("FullChillMask", "PrefixLMChillMask"):
        return True
    if name == "CausalChillMask":
        return (tk - 1) <= seq_len - tq
    if name == "SlidingWindowChillMask":
        left, right = args
        return (tq <= left and tk <= right) or (tq * 2 <= left) or (tk * 2 <= right)
    if name == "ChunkwiseChillMask":
        c, back = args
        return is_full_block(name, args, c * (back + 1) - tq, 0, tq, tk, seq_len)
    raise KeyError(name)


# --------------------------------------------------------------------------------------------
# tile decisions
# --------------------------------------------------------------------------------------------
def min_max_tiles(lims, i: int, seq_len: int, tile_in: int, tile_out: int):
    """_get_min_max_tiles, continuous path (utils.py:249-256, 270-272).  ``lims(pos, seq_len)``
    is one of the inclusive range rules."""
    i_max = min(i + tile_in, seq_len) - 1
    start, _ = lims(i, seq_len)
    _, end = lims(i_max, seq_len)
    return start // tile_out, -(-(end + 1) // tile_out)


def split_tiles(start_tile, end_tile, full_range, i, seq_len, tile_in, tile_out, split, hfb):
    """Loop split (chill_fwd.py:161-185).  ``full_range`` = (lo, hi) half-open token range or a
    callable returning it.  Returns (full_start_tile, full_end_tile)."""
    fs, fe = end_tile, start_tile
    if split and hfb and (i + tile_in <= seq_len):
        lo, hi = full_range() if callable(full_range) else full_range
        fs = -(-lo // tile_out)
        fe = hi // tile_out
    fs = max(start_tile, fs)
    fe = min(end_tile, fe)
    if fs >= fe:
        fs = fe = end_tile
    return fs, fe


def tile_ranges(name, args, pass_q_rows: bool, T: int, seq_len: int, tile_in: int, tile_out: int,
                q_full=None):
    """[n_tiles, 4] int array (start, end, full_start, full_end) for every row tile, the way the
    reference's kernels decide them.  ``pass_q_rows``: True for forward / dQ (rows = queries),
    False for dK/dV (rows = keys).  ``q_full`` optionally overrides q_full_range_for_k."""
    n_tiles = -(-T // tile_in)
    out = np.zeros((n_tiles, 4), dtype=np.int64)
    if pass_q_rows:
        lims = lambda p, s: k_range_for_q(name, args, p, s)  # noqa: E731
        hfb = has_full_blocks(name, args, tile_in, tile_out, T)
        full = lambda i: k_full_range_for_q(name, args, i, tile_in, seq_len)  # noqa: E731
    else:
        lims = lambda p, s: q_range_for_k(name, args, p, s)  # noqa: E731
        hfb = has_full_blocks(name, args, tile_out, tile_in, T)
        rule = q_full or q_full_range_for_k
        full = lambda i: rule(name, args, i, tile_in, seq_len)  # noqa: E731
    for t in range(n_tiles):
        i = t * tile_in
        if i >= seq_len:
            continue
        s, e = min_max_tiles(lims, i, seq_len, tile_in, tile_out)
        fs, fe = split_tiles(s, e, lambda: full(i), i, seq_len, tile_in, tile_out, True, hfb)
        out[t] = (s, e, fs, fe)
    return out


# --------------------------------------------------------------------------------------------
# counts
# --------------------------------------------------------------------------------------------
def nnz(name, args, T: int) -> int:
    """Unmasked (q, k) pairs, closed forms."""
    if name == "FullChillMask":
        return T * T
    if name == "CausalChillMask":
        return T * (T + 1) // 2
    if name == "PrefixLMChillMask":
        p = min(args[0], T)
        return T * (T + 1) // 2 + p * (p - 1) // 2
    if name == "SlidingWindowChillMask":
        left, right = args
        q = np.arange(T, dtype=np.int64)
        return int((np.minimum(q + right, T - 1) - np.maximum(0, q - left) + 1).sum())
    if name == "ChunkwiseChillMask":
        c, back = args
        q = np.arange(T, dtype=np.int64)
        return int((np.minimum((q // c + 1) * c - 1, T - 1) - np.maximum(0, (q // c - back) * c) + 1).sum())
    raise KeyError(name)


def flops(name, args, B: int, H: int, T: int, D: int, mode: str) -> float:
    """Effective FLOPs counting unmasked entries only: forward 4*B*H*D*nnz, backward 2.5x that
    (benchmark/benchmark.py:271-276)."""
    fwd = 4.0 * B * H * D * nnz(name, args, T)
    return {"fwd": fwd, "bwd": 2.5 * fwd, "fwd+bwd": 3.5 * fwd}[mode]


# --------------------------------------------------------------------------------------------
# attention
# --------------------------------------------------------------------------------------------
def _full_mask(name, args, B, T, lens):
    """[B, 1, T, T] boolean mask including the lens limit on keys AND queries (chill.py:530-537)."""
    m = dense_mask(name, args, T)[None, None]
    if lens is None:
        return np.broadcast_to(m, (B, 1, T, T))
    lens = np.asarray(lens)
    inside = np.arange(T)[None, :] < lens[:, None]  # [B, T]
    pair = inside[:, :, None] & inside[:, None, :]
    return m & pair[:, None]


def reference_naive(name, args, q, k, v, lens=None):
    """Dense-mask torch SDPA (chill.py:498-544): GQA expand, mask, lens padding, default scale
    D**-0.5.  torch tensors in, (out * res_mask, res_mask) out."""
    import torch
    import torch.nn.functional as F

    if q.shape[1] != k.shape[1]:
        g = q.shape[1] // k.shape[1]
        k = k.repeat_interleave(g, dim=1)
        v = v.repeat_interleave(g, dim=1)
    B, _, T, _ = q.shape
    lens_np = None if lens is None else lens.detach().cpu().numpy()
    attn_mask = torch.from_numpy(np.array(_full_mask(name, args, B, T, lens_np))).to(q.device)
    if lens is None:
        res_mask = torch.as_tensor(1, device=q.device)
    else:
        res_mask = (torch.arange(T, device=q.device)[None, :] < lens[:, None])[:, None, :, None]
    out = F.scaled_dot_product_attention(q, k, v, attn_mask=attn_mask)
    return out * res_mask, res_mask


def attention_f64(name, args, q, k, v, do=None, lens=None, sm_scale=None):
    """Textbook masked attention in float64 (numpy), with the analytic backward.

    Returns dict(o, lse2, delta, dq, dk, dv) — gradients only when ``do`` is given.  Rows with no
    visible key give o = 0, lse2 = -inf and contribute nothing to the gradients; rows >= lens are
    zero.  GQA: k, v may have fewer heads; dk, dv are summed over each group.
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    B, H, T, D = q.shape
    Hkv = k.shape[1]
    g = H // Hkv
    ke = np.repeat(k, g, axis=1)
    ve = np.repeat(v, g, axis=1)
    scale = D ** -0.5 if sm_scale is None else sm_scale
    m = _full_mask(name, args, B, T, lens)
    s = np.einsum("bhqd,bhkd->bhqk", q, ke) * scale
    s = np.where(m, s, -np.inf)
    smax = s.max(axis=-1, keepdims=True)
    smax_safe = np.where(np.isfinite(smax), smax, 0.0)
    e = np.exp(s - smax_safe)
    l = e.sum(axis=-1, keepdims=True)
    p = e / np.where(l == 0, 1.0, l)
    o = np.einsum("bhqk,bhkd->bhqd", p, ve)
    with np.errstate(divide="ignore"):
        lse2 = (smax_safe[..., 0] + np.log(l[..., 0])) * math.log2(math.e)
    lse2 = np.where(l[..., 0] == 0, -np.inf, lse2)
    res = {"o": o, "lse2": lse2}
    if do is not None:
        do = np.asarray(do, dtype=np.float64)
        delta = (o * do).sum(-1)
        dp = np.einsum("bhqd,bhkd->bhqk", do, ve)
        ds = p * (dp - delta[..., None])
        dq = np.einsum("bhqk,bhkd->bhqd", ds, ke) * scale
        dk_e = np.einsum("bhqk,bhqd->bhkd", ds, q) * scale
        dv_e = np.einsum("bhqk,bhqd->bhkd", p, do)
        res.update(
            delta=delta,
            dq=dq,
            dk=dk_e.reshape(B, Hkv, g, T, D).sum(2),
            dv=dv_e.reshape(B, Hkv, g, T, D).sum(2),
        )
    return res


def lse2(name, args, q, k, lens=None, sm_scale=None):
    """Base-2 log-sum-exp of the scaled, masked scores (chill_fwd.py:328): natural LSE * log2(e)."""
    return attention_f64(name, args, q, k, k, lens=lens, sm_scale=sm_scale)["lse2"]


def lse2_dense(name, args, q, k, lens=None, sm_scale=None):
    """The same LSE2 as `lse2`, on torch tensors of any device, in float64 (for inputs too large for the
    numpy textbook): [B, H, T]; -inf for rows without a visible key, rows >= lens included."""
    import torch

    if q.shape[1] != k.shape[1]:
        k = k.repeat_interleave(q.shape[1] // k.shape[1], dim=1)
    B, _, T, D = q.shape
    scale = D ** -0.5 if sm_scale is None else sm_scale
    lens_np = None if lens is None else lens.detach().cpu().numpy()
    m = torch.from_numpy(np.array(_full_mask(name, args, B, T, lens_np))).to(q.device)
    s = torch.einsum("bhqd,bhkd->bhqk", q.double(), k.double()) * scale
    s = torch.where(m, s, torch.full_like(s, -math.inf))
    return torch.logsumexp(s, dim=-1) * math.log2(math.e)


def delta(o, do):
    """delta[b,h,t] = sum_d o*do in fp32-or-better (utils.py:190)."""
    return (np.asarray(o, dtype=np.float64) * np.asarray(do, dtype=np.float64)).sum(-1)
