// Mask algebra: predicate + range functors, one specialisation per mask id.
//
// The same header is compiled for the host (enumeration entry points, validation) and for the
// device (the attention kernels), so what the CPU tests check is the code the GPU runs.
//
// Conventions follow the reference's ChillMask contract (chill_attention/mask.py:15-250):
//   - *_range_for_* return INCLUSIVE [lo, hi] limits (mask.py:79-107);
//   - *_full_range_for_* return HALF-OPEN [lo, hi) ranges (mask.py:110-151);
//   - positions are non-negative 32-bit ints; mask arguments are validated to fit on the host.
#pragma once

#include <stdint.h>

#include "../../include/chill_attention.h"

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define CHILL_HD __host__ __device__ __forceinline__
#else
#define CHILL_HD inline
#endif

namespace chill {

struct MaskArgs {
    int a0;
    int a1;
    int a2;
    int a3;
};

struct Range {
    int lo;
    int hi;
};

CHILL_HD int imin(int a, int b) { return a < b ? a : b; }
CHILL_HD int imax(int a, int b) { return a > b ? a : b; }
CHILL_HD int cdiv(int a, int b) { return (a + b - 1) / b; }
// floor division for a possibly negative numerator, positive denominator (Python's //)
CHILL_HD int floordiv(int a, int b) {
    int q = a / b;
    return (a % b != 0 && a < 0) ? q - 1 : q;
}

template <int ID>
struct Mask;

// What a mask functor inherits unless it says otherwise — the defaults of the reference's ChillMask
// base class (mask.py:110-250): no predicate-free ranges, no full blocks, rows may be empty, and
// limits that never decrease from one row to the next (the reference's *_lims_continious = True).
// kRowIsRange = true states that the visible positions of a row ARE its range: pred(q, k) holds for
// exactly the k in k_range_for_q(q) and exactly the q in q_range_for_k(k) (true of the five
// built-in masks; the kernels then mask a partial block with two comparisons per entry instead of
// evaluating the predicate).
// A functor whose limits are NOT monotone sets kMonotoneLimits = false; tile ranges then come
// from the minimum / maximum over the rows of a tile (utils.py:259-268).
struct MaskDefaults {
    static constexpr int kNumArgs = 0;
    static constexpr bool kSafe = false;
    static constexpr bool kHasKFullRange = false;
    static constexpr bool kHasQFullRange = false;
    static constexpr bool kMonotoneLimits = true;
    static constexpr bool kRowIsRange = false;
    CHILL_HD static Range k_full_range_for_q(int, int, int, MaskArgs) { return {0, 0}; }
    CHILL_HD static Range q_full_range_for_k(int, int, int, MaskArgs) { return {0, 0}; }
    CHILL_HD static bool has_full_blocks(int, int, int, MaskArgs) { return false; }
    CHILL_HD static bool is_full_block(int, int, int, int, int, MaskArgs) { return false; }
};

// ---------------------------------------------------------------- Full (mask.py:806-889)
template <>
struct Mask<CHILL_MASK_FULL> : MaskDefaults {
    static constexpr int kNumArgs = 0;
    static constexpr bool kSafe = true;        // every row sees at least one key (mask.py:864)
    static constexpr bool kHasKFullRange = true;
    static constexpr bool kHasQFullRange = true;
    static constexpr bool kRowIsRange = true;
    CHILL_HD static bool pred(int, int, int, MaskArgs) { return true; }
    CHILL_HD static Range k_range_for_q(int, int seq_len, MaskArgs) { return {0, seq_len - 1}; }
    CHILL_HD static Range q_range_for_k(int, int seq_len, MaskArgs) { return {0, seq_len - 1}; }
    CHILL_HD static Range k_full_range_for_q(int, int, int seq_len, MaskArgs) { return {0, seq_len}; }
    CHILL_HD static Range q_full_range_for_k(int, int, int seq_len, MaskArgs) { return {0, seq_len}; }
    CHILL_HD static bool has_full_blocks(int, int, int, MaskArgs) { return true; }
    CHILL_HD static bool is_full_block(int, int, int, int, int, MaskArgs) { return true; }
};

// ---------------------------------------------------------------- Causal (mask.py:892-976)
template <>
struct Mask<CHILL_MASK_CAUSAL> : MaskDefaults {
    static constexpr int kNumArgs = 0;
    static constexpr bool kSafe = true;
    static constexpr bool kHasKFullRange = true;
    static constexpr bool kHasQFullRange = true;
    static constexpr bool kRowIsRange = true;
    CHILL_HD static bool pred(int q, int k, int, MaskArgs) { return q >= k; }
    CHILL_HD static Range k_range_for_q(int q, int, MaskArgs) { return {0, q}; }
    CHILL_HD static Range q_range_for_k(int k, int seq_len, MaskArgs) { return {k, seq_len - 1}; }
    CHILL_HD static Range k_full_range_for_q(int qb, int, int, MaskArgs) { return {0, qb + 1}; }
    CHILL_HD static Range q_full_range_for_k(int kb, int tk, int seq_len, MaskArgs) {
        return {imax(0, kb + tk - 1), seq_len};
    }
    CHILL_HD static bool has_full_blocks(int tq, int tk, int seq_len, MaskArgs) {
        return (tk - 1) <= seq_len - tq;
    }
    CHILL_HD static bool is_full_block(int q, int k, int, int tk, int, MaskArgs) {
        return (k + tk - 1) <= q;
    }
};

// ---------------------------------------------------------------- SlidingWindow (mask.py:979-1108)
// args: a0 = left_context, a1 = right_context
template <>
struct Mask<CHILL_MASK_SLIDING_WINDOW> : MaskDefaults {
    static constexpr int kNumArgs = 2;
    static constexpr bool kSafe = false;
    static constexpr bool kHasKFullRange = true;
    static constexpr bool kHasQFullRange = true;
    static constexpr bool kRowIsRange = true;
    CHILL_HD static bool pred(int q, int k, int, MaskArgs a) {
        return (k <= q + a.a1) & (k >= q - a.a0);
    }
    CHILL_HD static Range k_range_for_q(int q, int seq_len, MaskArgs a) {
        return {imax(0, q - a.a0), imin(q + a.a1, seq_len - 1)};
    }
    CHILL_HD static Range q_range_for_k(int k, int seq_len, MaskArgs a) {
        return {imax(0, k - a.a1), imin(k + a.a0, seq_len - 1)};
    }
    CHILL_HD static Range k_full_range_for_q(int qb, int tq, int seq_len, MaskArgs a) {
        int start = imax(0, qb + tq - 1 - a.a0);
        int end = imin(seq_len, qb + a.a1 + 1);
        return {start, imax(start, end)};
    }
    // The reference leaves this at the base-class (0, 0) (mask.py:131-151), which makes its
    // dK/dV kernel run every tile with the predicate.  The transposed window is used here: all
    // k in [kb, kb+tk) are visible to q iff q - left <= kb and kb + tk - 1 <= q + right.
    CHILL_HD static Range q_full_range_for_k(int kb, int tk, int seq_len, MaskArgs a) {
        int start = imax(0, kb + tk - 1 - a.a1);
        int end = imin(seq_len, kb + a.a0 + 1);
        return {start, imax(start, end)};
    }
    CHILL_HD static bool has_full_blocks(int tq, int tk, int, MaskArgs a) {
        return ((tq <= a.a0) && (tk <= a.a1)) || (tq * 2 <= a.a0) || (tk * 2 <= a.a1);
    }
    CHILL_HD static bool in_window(int diff, MaskArgs a) {
        return ((diff <= a.a0) & (diff >= 0)) | ((diff >= -a.a1) & (diff <= 0));
    }
    CHILL_HD static bool is_full_block(int q, int k, int tq, int tk, int, MaskArgs a) {
        int diff_left = (q + tq - 1) - k;
        int diff_right = q - (k + tk - 1);
        return in_window(diff_left, a) && in_window(diff_right, a);
    }
};

// ---------------------------------------------------------------- Chunkwise (mask.py:1111-1266)
// args: a0 = context_size (> 0), a1 = back_contexts (>= 0)
template <>
struct Mask<CHILL_MASK_CHUNKWISE> : MaskDefaults {
    static constexpr int kNumArgs = 2;
    static constexpr bool kSafe = false;
    static constexpr bool kHasKFullRange = true;
    static constexpr bool kHasQFullRange = true;
    static constexpr bool kRowIsRange = true;
    CHILL_HD static bool pred(int q, int k, int, MaskArgs a) {
        int d = q / a.a0 - k / a.a0;
        return (d >= 0) & (d <= a.a1);
    }
    CHILL_HD static Range k_range_for_q(int q, int seq_len, MaskArgs a) {
        int qc = q / a.a0;
        return {imax(0, (qc - a.a1) * a.a0), imin((qc + 1) * a.a0 - 1, seq_len - 1)};
    }
    CHILL_HD static Range q_range_for_k(int k, int seq_len, MaskArgs a) {
        int kc = k / a.a0;
        return {kc * a.a0, imin((kc + a.a1 + 1) * a.a0 - 1, seq_len - 1)};
    }
    CHILL_HD static Range k_full_range_for_q(int qb, int tq, int seq_len, MaskArgs a) {
        int qc_min = qb / a.a0;
        int qc_max = (qb + tq - 1) / a.a0;
        int start = imax(0, (qc_max - a.a1) * a.a0);
        int end = imin(seq_len, (qc_min + 1) * a.a0);
        return {start, imax(start, end)};
    }
    // Not provided by the reference (base-class (0, 0), mask.py:131-151).  q sees the whole
    // k-tile iff chunk(q) >= chunk(last k) and chunk(q) <= chunk(first k) + back.
    CHILL_HD static Range q_full_range_for_k(int kb, int tk, int seq_len, MaskArgs a) {
        int kc_min = kb / a.a0;
        int kc_max = (kb + tk - 1) / a.a0;
        int start = kc_max * a.a0;
        int end = imin(seq_len, (kc_min + a.a1 + 1) * a.a0);
        return {start, imax(start, end)};
    }
    CHILL_HD static bool is_full_block(int q, int k, int tq, int tk, int, MaskArgs a) {
        int d0 = floordiv(q, a.a0) - floordiv(k + tk - 1, a.a0);
        int d1 = floordiv(q + tq - 1, a.a0) - floordiv(k, a.a0);
        return (d0 >= 0) & (d0 <= a.a1) & (d1 >= 0) & (d1 <= a.a1);
    }
    CHILL_HD static bool has_full_blocks(int tq, int tk, int seq_len, MaskArgs a) {
        // worst case: the last q-tile that still sees chunk 0 (mask.py:1234-1246)
        return is_full_block(a.a0 * (a.a1 + 1) - tq, 0, tq, tk, seq_len, a);
    }
};

// ---------------------------------------------------------------- PrefixLM (mask.py:1269-1394)
// args: a0 = prefix_size
template <>
struct Mask<CHILL_MASK_PREFIX_LM> : MaskDefaults {
    static constexpr int kNumArgs = 1;
    static constexpr bool kSafe = true;
    static constexpr bool kHasKFullRange = true;
    static constexpr bool kHasQFullRange = true;
    static constexpr bool kRowIsRange = true;
    CHILL_HD static bool pred(int q, int k, int, MaskArgs a) { return (k < a.a0) | (q >= k); }
    CHILL_HD static Range k_range_for_q(int q, int seq_len, MaskArgs a) {
        return {0, imin(imax(q, a.a0 - 1), seq_len - 1)};
    }
    CHILL_HD static Range q_range_for_k(int k, int seq_len, MaskArgs a) {
        return {k < a.a0 ? 0 : k, seq_len - 1};
    }
    CHILL_HD static Range k_full_range_for_q(int qb, int, int seq_len, MaskArgs a) {
        return {0, imin(imax(a.a0, qb + 1), seq_len)};
    }
    // Not provided by the reference (base-class (0, 0), mask.py:131-151).  A k-tile inside the
    // prefix is visible to every q; otherwise the causal rule of its last key applies.
    CHILL_HD static Range q_full_range_for_k(int kb, int tk, int seq_len, MaskArgs a) {
        if (kb + tk <= a.a0) return {0, seq_len};
        int start = imin(kb + tk - 1, seq_len);
        return {start, seq_len};
    }
    CHILL_HD static bool has_full_blocks(int, int, int, MaskArgs) { return true; }
    CHILL_HD static bool is_full_block(int q, int k, int tq, int tk, int, MaskArgs a) {
        bool causal_full = (k + tk - 1) <= q;
        bool in_prefix = (q + tq <= a.a0) & (k + tk <= a.a0);
        return causal_full | in_prefix;
    }
};

// Visible positions of one row as an inclusive range clipped to the sequence (QROWS: the keys of
// query `row`, else the queries of key `row`); empty (lo > hi) for a row past the end.
template <int ID, bool QROWS>
CHILL_HD Range visible_range(int row, int seq_len, MaskArgs a) {
    if (row >= seq_len) return {1, 0};
    const Range r = QROWS ? Mask<ID>::k_range_for_q(row, seq_len, a) : Mask<ID>::q_range_for_k(row, seq_len, a);
    return {imax(r.lo, 0), imin(r.hi, seq_len - 1)};
}

// ---------------------------------------------------------------- tile decisions
// Tiles of the streamed axis one row tile has to visit, and the sub-range of them that needs no
// predicate.  Loop order in the kernels: [start, full_start) predicated, [full_start, full_end)
// predicate-free, [full_end, end) predicated.
struct TileRange {
    int start;
    int end;
    int full_start;
    int full_end;
};

// `i` = first position of the row tile, tile_in = its size, tile_out = size of streamed tiles.
// QROWS = true: rows are queries (forward, dQ), limits come from k_range_for_q / k_full_range_for_q;
// QROWS = false: rows are keys (dK/dV), limits come from q_range_for_k / q_full_range_for_k.
// Restates _get_min_max_tiles' continuous path (utils.py:249-256, 270-272) and the loop split
// (chill_fwd.py:161-185; chill_bwd_dq.py:279-293; chill_bwd_dkdv.py:329-344).  The caller
// guarantees i < seq_len.
template <int ID, bool QROWS>
CHILL_HD TileRange tile_range(int i, int tile_in, int tile_out, int seq_len, bool has_full_blocks,
                              MaskArgs a) {
    using M = Mask<ID>;
    int i_max = imin(i + tile_in, seq_len) - 1;
    Range first = QROWS ? M::k_range_for_q(i, seq_len, a) : M::q_range_for_k(i, seq_len, a);
    Range last = QROWS ? M::k_range_for_q(i_max, seq_len, a) : M::q_range_for_k(i_max, seq_len, a);
    if (!M::kMonotoneLimits) {
        // hull of the rows' ranges; rows without any visible position (hi < lo) do not count
        int lo = 0x7fffffff, hi = -1;
        for (int row = i; row <= i_max; row++) {
            Range rr = QROWS ? M::k_range_for_q(row, seq_len, a) : M::q_range_for_k(row, seq_len, a);
            if (rr.hi >= rr.lo) {
                lo = imin(lo, rr.lo);
                hi = imax(hi, rr.hi);
            }
        }
        if (hi < 0) lo = 0;
        first.lo = lo;
        last.hi = hi;
    }
    TileRange r;
    r.start = first.lo / tile_out;
    r.end = cdiv(last.hi + 1, tile_out);
    int fs = r.end, fe = r.start;
    constexpr bool kSplit = QROWS ? M::kHasKFullRange : M::kHasQFullRange;
    if (kSplit && has_full_blocks && (i + tile_in <= seq_len)) {
        Range f = QROWS ? M::k_full_range_for_q(i, tile_in, seq_len, a)
                        : M::q_full_range_for_k(i, tile_in, seq_len, a);
        fs = cdiv(f.lo, tile_out);
        fe = f.hi / tile_out;
    }
    fs = imax(r.start, fs);
    fe = imin(r.end, fe);
    if (fs >= fe) {
        fs = r.end;
        fe = r.end;
    }
    r.full_start = fs;
    r.full_end = fe;
    return r;
}

// The same for a kernel that computes the rows of a ragged last row tile like any others and throws them
// away: the rows of [i, i + tile_in) at and beyond seq_len exist in memory or read as zero, they are never
// stored, and no row's result depends on another row's.  The predicate-free range of the COMPLETE tile
// (every mask states it from the tile's first row and size) holds for the rows that exist, so the tile
// need not end inside the sequence as the reference's loop split asks (chill_bwd_dq.py:279-293,
// chill_bwd_dkdv.py:329-344); the streamed tiles of the range do lie inside it.  Without this the one
// ragged workgroup of a head runs every tile under the predicate and finishes long after the others
// (causal B4 H16 D128 dQ: T = 8192 1.39 ms, T = 8200 1.63 ms).
template <int ID, bool QROWS>
CHILL_HD TileRange tile_range_rows_discarded(int i, int tile_in, int tile_out, int seq_len, bool has_full_blocks,
                                             MaskArgs a) {
    using M = Mask<ID>;
    TileRange r = tile_range<ID, QROWS>(i, tile_in, tile_out, seq_len, has_full_blocks, a);
    constexpr bool kSplit = QROWS ? M::kHasKFullRange : M::kHasQFullRange;
    if (kSplit && has_full_blocks && i + tile_in > seq_len) {
        const Range f = QROWS ? M::k_full_range_for_q(i, tile_in, seq_len, a) : M::q_full_range_for_k(i, tile_in, seq_len, a);
        const int fs = imax(r.start, cdiv(f.lo, tile_out));
        const int fe = imin(imin(r.end, f.hi / tile_out), seq_len / tile_out);
        if (fs < fe) {
            r.full_start = fs;
            r.full_end = fe;
        }
    }
    return r;
}

// has_full_blocks for a pass: the row tile is (tq) for QROWS passes and (tk) for the dK/dV pass,
// but the mask rule always takes (q_tile, k_tile) in that order (chill.py:159-164, 375-386).
template <int ID>
CHILL_HD bool pass_has_full_blocks(bool qrows, int tile_in, int tile_out, int T, MaskArgs a) {
    return qrows ? Mask<ID>::has_full_blocks(tile_in, tile_out, T, a)
                 : Mask<ID>::has_full_blocks(tile_out, tile_in, T, a);
}

}  // namespace chill

// A library built with -DCHILL_USER_MASK_HEADER='"file"' compiles ONE extra functor, written by the
// user, and serves only that one (so that the build stays a fifth of the stock one).  The file
// specialises chill::Mask<CHILL_MASK_USER>; chill_user_mask.h documents what it must contain.
#ifdef CHILL_USER_MASK_HEADER
#include CHILL_USER_MASK_HEADER
#endif

namespace chill {

// Runtime dispatch over the mask id for host-side entry points and launchers.
#ifdef CHILL_USER_MASK_HEADER
#define CHILL_DISPATCH_MASK(id, ...)                                                  \
    switch (id) {                                                                     \
        case CHILL_MASK_USER: { constexpr int MASK_ID = CHILL_MASK_USER; __VA_ARGS__; } break; \
        default: break;                                                               \
    }
inline bool mask_id_served(int id) { return id == CHILL_MASK_USER; }
inline int mask_num_args(int) { return Mask<CHILL_MASK_USER>::kNumArgs; }
#else
#define CHILL_DISPATCH_MASK(id, ...)                                                  \
    switch (id) {                                                                     \
        case CHILL_MASK_FULL: { constexpr int MASK_ID = CHILL_MASK_FULL; __VA_ARGS__; } break; \
        case CHILL_MASK_CAUSAL: { constexpr int MASK_ID = CHILL_MASK_CAUSAL; __VA_ARGS__; } break; \
        case CHILL_MASK_SLIDING_WINDOW: { constexpr int MASK_ID = CHILL_MASK_SLIDING_WINDOW; __VA_ARGS__; } break; \
        case CHILL_MASK_CHUNKWISE: { constexpr int MASK_ID = CHILL_MASK_CHUNKWISE; __VA_ARGS__; } break; \
        case CHILL_MASK_PREFIX_LM: { constexpr int MASK_ID = CHILL_MASK_PREFIX_LM; __VA_ARGS__; } break; \
        default: break;                                                               \
    }
inline bool mask_id_served(int id) { return id >= 0 && id < CHILL_MASK_COUNT; }
inline int mask_num_args(int id) {
    static const int nargs[CHILL_MASK_COUNT] = {0, 0, 2, 2, 1};
    return nargs[id];
}
#endif

// Validates a descriptor and lowers it to kernel arguments.  Returns a ChillStatus.
inline int lower_mask(const ChillMaskDesc* d, MaskArgs* out) {
    if (d == nullptr) return CHILL_ERR_NULL_POINTER;
    if (!mask_id_served(d->id)) return CHILL_ERR_BAD_MASK;
    if (d->nargs != mask_num_args(d->id) || d->nargs > 4) return CHILL_ERR_BAD_MASK;
    // arguments are position-like: keep sums with positions inside int32
    const int64_t kMaxArg = (int64_t)1 << 29;
    for (int i = 0; i < d->nargs; i++) {
        if (d->args[i] < 0 || d->args[i] > kMaxArg) return CHILL_ERR_BAD_MASK;
    }
    out->a0 = d->nargs > 0 ? (int)d->args[0] : 0;
    out->a1 = d->nargs > 1 ? (int)d->args[1] : 0;
    out->a2 = d->nargs > 2 ? (int)d->args[2] : 0;
    out->a3 = d->nargs > 3 ? (int)d->args[3] : 0;
    if (d->id == CHILL_MASK_CHUNKWISE) {
        if (out->a0 <= 0) return CHILL_ERR_BAD_MASK;
        // (chunk + back + 1) * context must stay inside int32 for T < 2^29
        if ((int64_t)out->a1 * out->a0 > kMaxArg) out->a1 = (int)(kMaxArg / out->a0);
    }
    return CHILL_OK;
}

}  // namespace chill
