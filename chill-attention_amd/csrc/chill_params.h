// Plain-data kernel arguments, filled by the C-ABI entry points after validation.
#pragma once

#include <stdint.h>

#include "chill_mask.h"

namespace chill {

struct Strides3 {  // element strides of a [B, H, T, D] tensor with unit inner stride
    int64_t b, h, t;
};

struct FwdParams {
    const void* q;
    const void* k;
    const void* v;
    void* o;
    float* lse;  // nullable
    const int32_t* lens;  // nullable
    Strides3 sq, sk, sv, so;
    int64_t lse_b, lse_h;  // fp32 [B, H, T], unit inner stride
    int64_t lens_stride;
    int32_t B, H, H_kv, T;
    int32_t group;         // H / H_kv
    float scale_log2;      // sm_scale * log2(e)
    MaskArgs margs;
};

struct DeltaParams {
    const void* o;
    const void* d_o;
    float* delta;
    Strides3 so, sdo;
    int64_t delta_b, delta_h;
    int32_t B, H, T;
};

struct BwdParams {
    const void* q;
    const void* k;
    const void* v;
    const void* d_o;
    void* dq;
    void* dk;
    void* dv;
    const float* lse;
    const float* delta;
    const int32_t* lens;  // nullable
    // dQ that computes delta itself (chill_bwd_dq_delta): the forward's output, and where the rows of
    // delta = rowsum(O * dO) go for the dK/dV launch that follows; both null otherwise
    const void* o;
    float* delta_out;
    Strides3 sq, sk, sv, sdo, sdq, sdk, sdv, so;
    int64_t lse_b, lse_h;
    int64_t delta_b, delta_h;
    int64_t lens_stride;
    int32_t B, H, H_kv, T;
    int32_t group;
    float sm_scale;
    float scale_log2;
    MaskArgs margs;
};

// One row of the static tile table (the replacement for the reference's autotune tables,
// autotune.py:11-119): rows per workgroup = 32 * waves, streamed tile size.
struct TileConfig {
    int rows;      // resident rows per workgroup (q rows for fwd / dQ, k rows for dK/dV)
    int streamed;  // rows of one streamed tile
    int waves;
    int lds_bytes;
};

}  // namespace chill
