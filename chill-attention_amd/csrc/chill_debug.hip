// Device-side dumps of the mask functors and tile decisions.  They exist so tests can show that
// the code the attention kernels run agrees bit-for-bit with the host enumeration; they play the
// role ChillMask._mask_infer / _limits_infer / _full_ranges_infer (chill_attention/mask.py:282-377,
// 485-534) play for the reference's Triton functions.
#include <hip/hip_runtime.h>

#include "chill_mask.h"

namespace chill {

template <int MASK>
__global__ void mask_eval_kernel(int n, MaskArgs a, uint8_t* out) {
    int k = blockIdx.x * blockDim.x + threadIdx.x;
    int q = blockIdx.y;
    if (k < n && q < n) out[(size_t)q * n + k] = Mask<MASK>::pred(q, k, n, a) ? 1 : 0;
}

template <int MASK>
__global__ void tile_ranges_kernel(int pass, int T, int seq_len, int tile_in, int tile_out, MaskArgs a,
                                   int32_t* out) {
    int t = blockIdx.x * blockDim.x + threadIdx.x;
    int tiles = cdiv(T, tile_in);
    if (t >= tiles) return;
    const bool qrows = pass != CHILL_PASS_DKDV;
    const bool hfb = pass_has_full_blocks<MASK>(qrows, tile_in, tile_out, T, a);
    int i = t * tile_in;
    TileRange r = {0, 0, 0, 0};
    if (i < seq_len) {
        r = qrows ? tile_range<MASK, true>(i, tile_in, tile_out, seq_len, hfb, a)
                  : tile_range<MASK, false>(i, tile_in, tile_out, seq_len, hfb, a);
    }
    out[4 * t + 0] = r.start;
    out[4 * t + 1] = r.end;
    out[4 * t + 2] = r.full_start;
    out[4 * t + 3] = r.full_end;
}

}  // namespace chill

using namespace chill;

extern "C" {

int chill_mask_eval_device(const ChillMaskDesc* mask, int32_t n, uint8_t* out, void* stream) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (out == nullptr) return CHILL_ERR_NULL_POINTER;
    if (n <= 0 || n > 65535) return CHILL_ERR_BAD_SHAPE;
    dim3 grid(cdiv(n, 256), n), block(256);
    CHILL_DISPATCH_MASK(mask->id, {
        hipLaunchKernelGGL(mask_eval_kernel<MASK_ID>, grid, block, 0, static_cast<hipStream_t>(stream), n, a, out);
    });
    return hipGetLastError() == hipSuccess ? CHILL_OK : CHILL_ERR_HIP;
}

int chill_tile_ranges_device(const ChillMaskDesc* mask, int32_t pass, int32_t T, int32_t seq_len,
                             int32_t tile_in, int32_t tile_out, int32_t* out, void* stream) {
    MaskArgs a;
    int st = lower_mask(mask, &a);
    if (st != CHILL_OK) return st;
    if (out == nullptr) return CHILL_ERR_NULL_POINTER;
    if (T <= 0 || seq_len < 0 || seq_len > T) return CHILL_ERR_BAD_SHAPE;
    if (tile_in <= 0 || tile_out <= 0) return CHILL_ERR_BAD_ARGUMENT;
    if (pass != CHILL_PASS_FWD && pass != CHILL_PASS_DQ && pass != CHILL_PASS_DKDV)
        return CHILL_ERR_BAD_ARGUMENT;
    int tiles = cdiv(T, tile_in);
    dim3 grid(cdiv(tiles, 64)), block(64);
    CHILL_DISPATCH_MASK(mask->id, {
        hipLaunchKernelGGL(tile_ranges_kernel<MASK_ID>, grid, block, 0, static_cast<hipStream_t>(stream), pass, T,
                           seq_len, tile_in, tile_out, a, out);
    });
    return hipGetLastError() == hipSuccess ? CHILL_OK : CHILL_ERR_HIP;
}

}  // extern "C"
