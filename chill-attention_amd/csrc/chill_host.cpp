// Host-only entry points of the C ABI: dense mask / limits / tile-range enumeration, the static
// tile table and the closed-form unmasked-entry count.  They run the same functor header the
// kernels are compiled from, so CPU tests exercise the device logic without a GPU.
#include <stddef.h>

#include "chill_mask.h"
#include "chill_tiles.h"

using namespace chill;

extern "C" {

int chill_mask_eval(const ChillMaskDesc* mask, int32_t n, uint8_t* out) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (out == nullptr) return CHILL_ERR_NULL_POINTER;
    if (n < 0) return CHILL_ERR_BAD_SHAPE;
    CHILL_DISPATCH_MASK(mask->id, {
        for (int q = 0; q < n; q++)
            for (int k = 0; k < n; k++)
                out[(size_t)q * n + k] = Mask<MASK_ID>::pred(q, k, n, a) ? 1 : 0;
    });
    return CHILL_OK;
}

int chill_mask_limits(const ChillMaskDesc* mask, int32_t which, int32_t n, int32_t seq_len,
                      int32_t* out) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (out == nullptr) return CHILL_ERR_NULL_POINTER;
    if (n < 0 || seq_len < 0) return CHILL_ERR_BAD_SHAPE;
    if (which != 0 && which != 1) return CHILL_ERR_BAD_ARGUMENT;
    CHILL_DISPATCH_MASK(mask->id, {
        for (int i = 0; i < n; i++) {
            Range r = which == 0 ? Mask<MASK_ID>::k_range_for_q(i, seq_len, a)
                                 : Mask<MASK_ID>::q_range_for_k(i, seq_len, a);
            out[2 * i] = r.lo;
            out[2 * i + 1] = r.hi;
        }
    });
    return CHILL_OK;
}

int chill_tile_ranges(const ChillMaskDesc* mask, int32_t pass, int32_t T, int32_t seq_len,
                      int32_t tile_in, int32_t tile_out, int32_t* out) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (out == nullptr) return CHILL_ERR_NULL_POINTER;
    if (T <= 0 || seq_len < 0 || seq_len > T) return CHILL_ERR_BAD_SHAPE;
    if (tile_in <= 0 || tile_out <= 0) return CHILL_ERR_BAD_ARGUMENT;
    if (pass != CHILL_PASS_FWD && pass != CHILL_PASS_DQ && pass != CHILL_PASS_DKDV)
        return CHILL_ERR_BAD_ARGUMENT;
    const bool qrows = pass != CHILL_PASS_DKDV;
    const int tiles = cdiv(T, tile_in);
    CHILL_DISPATCH_MASK(mask->id, {
        const bool hfb = pass_has_full_blocks<MASK_ID>(qrows, tile_in, tile_out, T, a);
        for (int t = 0; t < tiles; t++) {
            int i = t * tile_in;
            TileRange r = {0, 0, 0, 0};
            if (i < seq_len) {
                r = qrows ? tile_range<MASK_ID, true>(i, tile_in, tile_out, seq_len, hfb, a)
                          : tile_range<MASK_ID, false>(i, tile_in, tile_out, seq_len, hfb, a);
            }
            out[4 * t + 0] = r.start;
            out[4 * t + 1] = r.end;
            out[4 * t + 2] = r.full_start;
            out[4 * t + 3] = r.full_end;
        }
    });
    return CHILL_OK;
}

int chill_mask_is_full_block(const ChillMaskDesc* mask, int32_t q, int32_t k, int32_t tile_q,
                             int32_t tile_k, int32_t seq_len) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (tile_q <= 0 || tile_k <= 0) return CHILL_ERR_BAD_ARGUMENT;
    int res = 0;
    CHILL_DISPATCH_MASK(mask->id, { res = Mask<MASK_ID>::is_full_block(q, k, tile_q, tile_k, seq_len, a) ? 1 : 0; });
    return res;
}

int chill_mask_has_full_blocks(const ChillMaskDesc* mask, int32_t tile_q, int32_t tile_k,
                               int32_t seq_len) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (tile_q <= 0 || tile_k <= 0) return CHILL_ERR_BAD_ARGUMENT;
    int res = 0;
    CHILL_DISPATCH_MASK(mask->id, { res = Mask<MASK_ID>::has_full_blocks(tile_q, tile_k, seq_len, a) ? 1 : 0; });
    return res;
}

int64_t chill_mask_nnz(const ChillMaskDesc* mask, int32_t T) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (T < 0) return CHILL_ERR_BAD_SHAPE;
    // every built-in mask row is one interval [lo, hi] of keys, so the count is a sum of lengths;
    // a user mask may have holes inside its limits and is counted position by position
    int64_t total = 0;
    CHILL_DISPATCH_MASK(mask->id, {
        for (int q = 0; q < T; q++) {
            Range r = Mask<MASK_ID>::k_range_for_q(q, T, a);
            if (r.hi < r.lo) continue;
            if (MASK_ID == CHILL_MASK_USER) {
                for (int k = r.lo; k <= r.hi; k++) total += Mask<MASK_ID>::pred(q, k, T, a) ? 1 : 0;
            } else {
                total += (int64_t)(r.hi - r.lo + 1);
            }
        }
    });
    return total;
}

int chill_tile_config(int32_t mask_id, int32_t D, int32_t dtype, int32_t pass, int32_t out[4]) {
    return chill_tile_config_for_shape(mask_id, D, dtype, pass, 1, kLongSequence, out);
}

static int report_tile_config(int mask_id, long long mask_arg0, long long band_keys, int32_t D, int32_t dtype, int32_t pass,
                              int64_t batch_heads, int32_t T, int32_t out[4]) {
    if (out == nullptr) return CHILL_ERR_NULL_POINTER;
    if (!mask_id_served(mask_id)) return CHILL_ERR_BAD_MASK;
    if (T < 1 || batch_heads < 1) return CHILL_ERR_BAD_ARGUMENT;
    TileConfig c;
    int st = tile_config(mask_id, mask_arg0, band_keys, D, dtype, pass, batch_heads, T, &c);
    if (st != CHILL_OK) return st;
    out[0] = c.rows;
    out[1] = c.streamed;
    out[2] = c.waves;
    out[3] = c.lds_bytes;
    return CHILL_OK;
}

int chill_tile_config_for_shape(int32_t mask_id, int32_t D, int32_t dtype, int32_t pass, int64_t batch_heads,
                                int32_t T, int32_t out[4]) {
    // (a mask id alone: the row of a mask whose arguments do not change the route; of a banded mask, a narrow one)
    return report_tile_config(mask_id, 1, mask_is_banded(mask_id) ? kNarrowBand : kWholeSequence, D, dtype, pass, batch_heads, T, out);
}

int chill_tile_config_for_launch(const ChillMaskDesc* mask, int32_t D, int32_t dtype, int32_t pass,
                                 int64_t batch_heads, int32_t T, int32_t out[4]) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    return report_tile_config(mask->id, a.a0, mask_band_keys(mask->id, a.a0, a.a1), D, dtype, pass, batch_heads, T, out);
}

int chill_work_item(int32_t workgroup, int32_t total, int32_t resident) {
    if (workgroup < 0 || total < 1 || resident < 1) return CHILL_ERR_BAD_ARGUMENT;
    return xcd_contiguous_item(workgroup, total, resident);
}

const char* chill_status_string(int32_t status) {
    switch (status) {
        case CHILL_OK: return "ok";
        case CHILL_ERR_NULL_POINTER: return "null pointer";
        case CHILL_ERR_BAD_DTYPE: return "unsupported dtype (expected fp32, fp16 or bf16)";
        case CHILL_ERR_BAD_HEAD_DIM: return "unsupported head dim (expected 16, 32, 64, 128 or 256)";
        case CHILL_ERR_BAD_MASK: return "bad mask descriptor (unknown id, wrong argument count or argument out of range)";
        case CHILL_ERR_BAD_SHAPE: return "bad shape (non-positive extent or H not divisible by H_kv)";
        case CHILL_ERR_BAD_STRIDE: return "bad stride (inner stride must be 1, strides non-negative, rows 16-byte aligned)";
        case CHILL_ERR_HIP: return "HIP launch failure";
        case CHILL_ERR_BAD_ARGUMENT: return "bad argument";
        case CHILL_ERR_TOO_LARGE: return "problem too large (32-bit position arithmetic, or the fixed array of chill_bwd_noalloc)";
        default: return "unknown status";
    }
}

int32_t chill_abi_version(void) { return CHILL_ABI_VERSION; }

int32_t chill_has_user_mask(void) {
#ifdef CHILL_USER_MASK_HEADER
    return 1;
#else
    return 0;
#endif
}

}  // extern "C"
