/*
 * CPU oracle, integer part, in plain C.  TEST INFRASTRUCTURE ONLY: nothing the product ships or
 * measures links or loads this file; tests load it to brute-force the mask rules and tile
 * decisions at sizes where Python loops are too slow.
 *
 * Restates, independently of the HIP library's functor header, the reference's
 *   - mask predicates          chill_attention/mask.py:825, 911, 1010-1012, 1145-1148, 1301-1304
 *   - inclusive range rules    mask.py:828-835, 914-921, 1015-1038, 1151-1185, 1307-1336
 *   - k_full_range_for_q       mask.py:838-844, 924-930, 1041-1051, 1188-1206, 1339-1350
 *   - q_full_range_for_k       mask.py:847-853, 933-940 (Full, Causal); others (0,0), mask.py:131-151
 *   - has_full_blocks          mask.py:876-877, 963-964, 1080-1086, 1234-1246, 1378-1379
 *   - _get_min_max_tiles       chill_attention/utils.py:249-256, 270-272 (continuous path)
 *   - the loop split           chill_attention/chill_fwd.py:161-185
 * and provides exhaustive checkers over the dense mask (the method of ChillMask.verify,
 * mask.py:700-803).
 *
 * Mask ids: 0 Full, 1 Causal, 2 SlidingWindow(left,right), 3 Chunkwise(context,back), 4 PrefixLM(prefix).
 */
#include <stdint.h>
#include <stdlib.h>

static int64_t imin64(int64_t a, int64_t b) { return a < b ? a : b; }
static int64_t imax64(int64_t a, int64_t b) { return a > b ? a : b; }
static int64_t fdiv(int64_t a, int64_t b) { /* Python // */
    int64_t q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) q--;
    return q;
}
static int64_t cdiv64(int64_t a, int64_t b) { return -fdiv(-a, b); }

int oracle_pred(int id, int64_t a0, int64_t a1, int64_t q, int64_t k) {
    switch (id) {
        case 0: return 1;
        case 1: return q >= k;
        case 2: return (k <= q + a1) && (k >= q - a0);
        case 3: { int64_t d = fdiv(q, a0) - fdiv(k, a0); return d >= 0 && d <= a1; }
        case 4: return (k < a0) || (q >= k);
        default: return 0;
    }
}

static void k_range_for_q(int id, int64_t a0, int64_t a1, int64_t q, int64_t n, int64_t* lo, int64_t* hi) {
    switch (id) {
        case 0: *lo = 0; *hi = n - 1; break;
        case 1: *lo = 0; *hi = q; break;
        case 2: *lo = imax64(0, q - a0); *hi = imin64(q + a1, n - 1); break;
        case 3: { int64_t c = fdiv(q, a0); *lo = imax64(0, (c - a1) * a0); *hi = imin64((c + 1) * a0 - 1, n - 1); } break;
        default: *lo = 0; *hi = imin64(imax64(q, a0 - 1), n - 1); break;
    }
}

static void q_range_for_k(int id, int64_t a0, int64_t a1, int64_t k, int64_t n, int64_t* lo, int64_t* hi) {
    switch (id) {
        case 0: *lo = 0; *hi = n - 1; break;
        case 1: *lo = k; *hi = n - 1; break;
        case 2: *lo = imax64(0, k - a1); *hi = imin64(k + a0, n - 1); break;
        case 3: { int64_t c = fdiv(k, a0); *lo = c * a0; *hi = imin64((c + a1 + 1) * a0 - 1, n - 1); } break;
        default: *lo = (k < a0) ? 0 : k; *hi = n - 1; break;
    }
}

static void k_full_range_for_q(int id, int64_t a0, int64_t a1, int64_t qb, int64_t tq, int64_t n, int64_t* lo, int64_t* hi) {
    switch (id) {
        case 0: *lo = 0; *hi = n; break;
        case 1: *lo = 0; *hi = qb + 1; break;
        case 2: { int64_t s = imax64(0, qb + tq - 1 - a0), e = imin64(n, qb + a1 + 1); *lo = s; *hi = imax64(s, e); } break;
        case 3: {
            int64_t ke = (fdiv(qb, a0) + 1) * a0, ks = (fdiv(qb + tq - 1, a0) - a1) * a0;
            int64_t s = imax64(0, ks), e = imin64(n, ke);
            *lo = s; *hi = imax64(s, e);
        } break;
        default: *lo = 0; *hi = imin64(imax64(a0, qb + 1), n); break;
    }
}

/* mode 0: the reference's rule (empty for ids 2..4); mode 1: the widened rules the HIP library adds */
static void q_full_range_for_k(int id, int64_t a0, int64_t a1, int64_t kb, int64_t tk, int64_t n, int mode, int64_t* lo, int64_t* hi) {
    if (id == 0) { *lo = 0; *hi = n; return; }
    if (id == 1) { *lo = imax64(0, kb + tk - 1); *hi = n; return; }
    if (mode == 0) { *lo = 0; *hi = 0; return; }
    if (id == 2) { /* q - left <= kb and kb + tk - 1 <= q + right */
        int64_t s = imax64(0, kb + tk - 1 - a1), e = imin64(n, kb + a0 + 1);
        *lo = s; *hi = imax64(s, e);
    } else if (id == 3) { /* chunk(q) in [chunk(last k), chunk(first k) + back] */
        int64_t s = fdiv(kb + tk - 1, a0) * a0, e = imin64(n, (fdiv(kb, a0) + a1 + 1) * a0);
        *lo = s; *hi = imax64(s, e);
    } else { /* inside the prefix every q sees the tile; otherwise causal on its last key */
        if (kb + tk <= a0) { *lo = 0; *hi = n; }
        else { *lo = imin64(kb + tk - 1, n); *hi = n; }
    }
}

static int sw_inside(int64_t d, int64_t l, int64_t r) { return (d <= l && d >= 0) || (d >= -r && d <= 0); }

int oracle_is_full_block(int id, int64_t a0, int64_t a1, int64_t q, int64_t k, int64_t tq, int64_t tk) {
    switch (id) {
        case 0: return 1;
        case 1: return (k + tk - 1) <= q;
        case 2: return sw_inside((q + tq - 1) - k, a0, a1) && sw_inside(q - (k + tk - 1), a0, a1);
        case 3: {
            int64_t d0 = fdiv(q, a0) - fdiv(k + tk - 1, a0), d1 = fdiv(q + tq - 1, a0) - fdiv(k, a0);
            return d0 >= 0 && d0 <= a1 && d1 >= 0 && d1 <= a1;
        }
        default: return ((k + tk - 1) <= q) || ((q + tq <= a0) && (k + tk <= a0));
    }
}

int oracle_has_full_blocks(int id, int64_t a0, int64_t a1, int64_t tq, int64_t tk, int64_t n) {
    switch (id) {
        case 0: case 4: return 1;
        case 1: return (tk - 1) <= n - tq;
        case 2: return (tq <= a0 && tk <= a1) || (tq * 2 <= a0) || (tk * 2 <= a1);
        default: return oracle_is_full_block(3, a0, a1, a0 * (a1 + 1) - tq, 0, tq, tk);
    }
}

void oracle_dense_mask(int id, int64_t a0, int64_t a1, int64_t n, uint8_t* out) {
    for (int64_t q = 0; q < n; q++)
        for (int64_t k = 0; k < n; k++) out[q * n + k] = (uint8_t)oracle_pred(id, a0, a1, q, k);
}

int64_t oracle_nnz_bruteforce(int id, int64_t a0, int64_t a1, int64_t n) {
    int64_t c = 0;
    for (int64_t q = 0; q < n; q++)
        for (int64_t k = 0; k < n; k++) c += oracle_pred(id, a0, a1, q, k);
    return c;
}

/* Tile decisions for every row tile: out[t*4 + {0..3}] = start, end, full_start, full_end.
 * qrows != 0: rows are queries (forward, dQ); else rows are keys (dK/dV).  qfull_mode as above. */
void oracle_tile_ranges(int id, int64_t a0, int64_t a1, int qrows, int64_t T, int64_t seq_len,
                        int64_t tile_in, int64_t tile_out, int qfull_mode, int64_t* out) {
    int64_t tiles = cdiv64(T, tile_in);
    int hfb = qrows ? oracle_has_full_blocks(id, a0, a1, tile_in, tile_out, T)
                    : oracle_has_full_blocks(id, a0, a1, tile_out, tile_in, T);
    for (int64_t t = 0; t < tiles; t++) {
        int64_t i = t * tile_in;
        int64_t* o = out + 4 * t;
        o[0] = o[1] = o[2] = o[3] = 0;
        if (i >= seq_len) continue;
        int64_t i_max = imin64(i + tile_in, seq_len) - 1, lo, hi, dummy;
        if (qrows) { k_range_for_q(id, a0, a1, i, seq_len, &lo, &dummy); k_range_for_q(id, a0, a1, i_max, seq_len, &dummy, &hi); }
        else { q_range_for_k(id, a0, a1, i, seq_len, &lo, &dummy); q_range_for_k(id, a0, a1, i_max, seq_len, &dummy, &hi); }
        int64_t s = fdiv(lo, tile_out), e = cdiv64(hi + 1, tile_out);
        int64_t fs = e, fe = s;
        if (hfb && (i + tile_in <= seq_len)) {
            int64_t flo, fhi;
            if (qrows) k_full_range_for_q(id, a0, a1, i, tile_in, seq_len, &flo, &fhi);
            else q_full_range_for_k(id, a0, a1, i, tile_in, seq_len, qfull_mode, &flo, &fhi);
            fs = cdiv64(flo, tile_out);
            fe = fdiv(fhi, tile_out);
        }
        fs = imax64(s, fs);
        fe = imin64(e, fe);
        if (fs >= fe) { fs = e; fe = e; }
        o[0] = s; o[1] = e; o[2] = fs; o[3] = fe;
    }
}

/* Exhaustive check of tile decisions `r` (layout as above, any producer) against the predicate,
 * restricted to positions < seq_len.  For every row tile that starts below seq_len:
 *   1. no visible pair lies in a streamed tile outside [start, end);
 *   2. the first and the last tile of a non-empty range each hold a visible pair (tight hull),
 *      and an empty range has start >= end only if the row tile sees nothing;
 *   3. every pair of a tile inside [full_start, full_end) is visible and the tile lies below seq_len.
 * Returns 0 if all hold, else 1000000 * rule + failing row tile + 1. */
int64_t oracle_check_tile_ranges(int id, int64_t a0, int64_t a1, int qrows, int64_t T, int64_t seq_len,
                                 int64_t tile_in, int64_t tile_out, const int64_t* r) {
    int64_t tiles = cdiv64(T, tile_in), otiles = cdiv64(T, tile_out);
    uint8_t* any = (uint8_t*)malloc((size_t)otiles);
    uint8_t* all = (uint8_t*)malloc((size_t)otiles);
    int64_t bad = 0;
    for (int64_t t = 0; t < tiles && !bad; t++) {
        int64_t i0 = t * tile_in, i1 = imin64(i0 + tile_in, seq_len);
        if (i0 >= seq_len) continue;
        for (int64_t ot = 0; ot < otiles; ot++) {
            int64_t j0 = ot * tile_out, j1 = imin64(j0 + tile_out, seq_len);
            int a = 0, f = (j0 + tile_out <= seq_len) && (i0 + tile_in <= seq_len);
            for (int64_t i = i0; i < i1; i++)
                for (int64_t j = j0; j < j1; j++) {
                    int p = qrows ? oracle_pred(id, a0, a1, i, j) : oracle_pred(id, a0, a1, j, i);
                    a |= p;
                    f &= p;
                }
            any[ot] = (uint8_t)a;
            all[ot] = (uint8_t)f;
        }
        const int64_t* o = r + 4 * t;
        for (int64_t ot = 0; ot < otiles; ot++)
            if (any[ot] && (ot < o[0] || ot >= o[1])) bad = 1000000 + t + 1;
        if (!bad && o[0] < o[1] && (!any[o[0]] || !any[o[1] - 1])) bad = 2000000 + t + 1;
        for (int64_t ot = o[2]; ot < o[3] && !bad; ot++)
            if (ot < 0 || ot >= otiles || !all[ot]) bad = 3000000 + t + 1;
    }
    free(any);
    free(all);
    return bad;
}

/* True inclusive limits of every row (which = 0: keys per query) or column (which = 1: queries per
 * key) of the n x n dense mask: out[i*2] = min, out[i*2+1] = max, or (-1, -1) for an empty line. */
void oracle_true_limits(int id, int64_t a0, int64_t a1, int which, int64_t n, int64_t* out) {
    for (int64_t i = 0; i < n; i++) {
        int64_t lo = -1, hi = -1;
        for (int64_t j = 0; j < n; j++) {
            int p = which == 0 ? oracle_pred(id, a0, a1, i, j) : oracle_pred(id, a0, a1, j, i);
            if (p) { if (lo < 0) lo = j; hi = j; }
        }
        out[2 * i] = lo;
        out[2 * i + 1] = hi;
    }
}

/* The range rules themselves, for comparison with oracle_true_limits. */
void oracle_rule_limits(int id, int64_t a0, int64_t a1, int which, int64_t n, int64_t seq_len, int64_t* out) {
    for (int64_t i = 0; i < n; i++) {
        if (which == 0) k_range_for_q(id, a0, a1, i, seq_len, &out[2 * i], &out[2 * i + 1]);
        else q_range_for_k(id, a0, a1, i, seq_len, &out[2 * i], &out[2 * i + 1]);
    }
}
