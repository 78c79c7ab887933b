/*
 * chill_attention.h — C ABI of the MI355X (gfx950) sparse flash-attention library.
 *
 * This is the boundary the Python host code binds with ctypes.  Every entry point takes plain
 * pointers, sizes and strides; no torch types cross it.  The library never allocates or frees
 * device memory: the caller owns every buffer (outputs, the fp32 delta scratch of the backward,
 * LSE).  All device entry points are asynchronous on the given stream and hold no mutable global
 * state, so they are re-entrant.
 *
 * Each entry point cites the piece of the reference (alexdremov/chill-attention v2.1.0) whose
 * kernel launch it replaces.
 *
 * Conventions
 *   - tensors are [B, H, T, D] (q, o, do, dq) or [B, H_kv, T, D] (k, v, dk, dv); strides are in
 *     ELEMENTS; the innermost stride must be 1 and every row start must be 16-byte aligned;
 *   - lse / delta are fp32 [B, H, T] with element strides, innermost stride 1;
 *   - lens is int32 [B] (element stride given) or NULL; a sequence length is min(lens[b], T);
 *   - LSE is base-2 and includes the softmax scale: LSE2 = log2 sum_k 2^(scale*log2(e)*q.k);
 *     a row with no unmasked key has LSE2 = -inf and O = 0;
 *   - return value: CHILL_OK (0) or a negative ChillStatus; nothing is launched on error.
 */
#ifndef CHILL_ATTENTION_H
#define CHILL_ATTENTION_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define CHILL_ABI_VERSION 1

typedef enum ChillStatus {
    CHILL_OK = 0,
    CHILL_ERR_NULL_POINTER = -1,
    CHILL_ERR_BAD_DTYPE = -2,
    CHILL_ERR_BAD_HEAD_DIM = -3,   /* D must be one of 16, 32, 64, 128, 256 */
    CHILL_ERR_BAD_MASK = -4,       /* unknown mask id, wrong nargs, or argument out of range */
    CHILL_ERR_BAD_SHAPE = -5,      /* B, H, H_kv, T non-positive or H % H_kv != 0 */
    CHILL_ERR_BAD_STRIDE = -6,     /* inner stride != 1, negative stride, or misaligned rows */
    CHILL_ERR_HIP = -7,            /* hipGetLastError() reported a launch failure */
    CHILL_ERR_BAD_ARGUMENT = -8,   /* anything else (bad pass id, bad tile size, ...) */
    CHILL_ERR_TOO_LARGE = -9       /* an index would not fit the kernels' 32-bit position math */
} ChillStatus;

typedef enum ChillDType {
    CHILL_F32 = 0,
    CHILL_F16 = 1,
    CHILL_BF16 = 2
} ChillDType;

/* Mask ids: one per ChillMask class of the reference (chill_attention/mask.py:806-1394), plus
 * CHILL_MASK_USER for a library built around one user-written functor — the counterpart of the
 * reference's "Creating Your Own Mask" (README.md:124-179; ChillMask contract mask.py:54-250).
 * Such a library (make USER_MASK=functor.h, see csrc/chill_user_mask.h) serves ONLY
 * CHILL_MASK_USER; the stock library serves only the five built-in ids. */
typedef enum ChillMaskId {
    CHILL_MASK_FULL = 0,           /* FullChillMask            mask.py:806-889,   no args          */
    CHILL_MASK_CAUSAL = 1,         /* CausalChillMask          mask.py:892-976,   no args          */
    CHILL_MASK_SLIDING_WINDOW = 2, /* SlidingWindowChillMask   mask.py:979-1108,  (left, right)    */
    CHILL_MASK_CHUNKWISE = 3,      /* ChunkwiseChillMask       mask.py:1111-1266, (context, back)  */
    CHILL_MASK_PREFIX_LM = 4,      /* PrefixLMChillMask        mask.py:1269-1394, (prefix,)        */
    CHILL_MASK_COUNT = 5,          /* number of built-in masks */
    CHILL_MASK_USER = 5            /* user-written functor, up to 4 integer args      */
} ChillMaskId;

/* The "mask-ID-plus-args" descriptor a ChillMask instance lowers to.  The reference bakes
 * mask.constargs into the Triton kernel as constexpr (chill.py:151); here they are runtime
 * values, so one compiled kernel serves every instance of a mask class. */
typedef struct ChillMaskDesc {
    int32_t id;      /* ChillMaskId */
    int32_t nargs;   /* number of meaningful entries of args */
    int64_t args[4];
} ChillMaskDesc;

/* A 4-d strided tensor view (element strides). */
typedef struct ChillTensor4 {
    void* ptr;
    int64_t stride[4];
} ChillTensor4;

/* Kernel passes, for chill_tile_config / chill_tile_ranges. */
typedef enum ChillPass {
    CHILL_PASS_FWD = 0,   /* q-tile rows, streams k-tiles   (chill_fwd.py)      */
    CHILL_PASS_DQ = 1,    /* q-tile rows, streams k-tiles   (chill_bwd_dq.py)   */
    CHILL_PASS_DKDV = 2   /* k-tile rows, streams q-tiles   (chill_bwd_dkdv.py) */
} ChillPass;

/* ------------------------------------------------------------------------------------------
 * Device entry points
 * ---------------------------------------------------------------------------------------- */

/* Forward: O = softmax(mask(Q K^T * sm_scale)) V, optional LSE2.
 * Replaces the launch of _chill_attn_fwd (chill_fwd.py:21-359) at chill.py:207, grid chill.py:122-123.
 * Every row of `o` (and of `lse`) is written: rows at or beyond lens[b] and rows whose q-tile has
 * no k-tile receive 0 (the reference leaves them at the adapter's zero-fill, chill.py:96 and
 * chill_fwd.py:70-71), so the caller may pass uninitialised memory.
 * `lse` may be NULL (return_lse = False). */
int chill_fwd(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
              const ChillTensor4* o,
              float* lse, const int64_t lse_stride[3],
              const int32_t* lens, int64_t lens_stride,
              int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
              int32_t dtype, float sm_scale,
              const ChillMaskDesc* mask, void* stream);

/* Backward preprocessing: delta[b,h,t] = sum_d float(O[b,h,t,d]) * float(dO[b,h,t,d]).
 * Replaces the launch of _chill_attn_bwd_precompute (utils.py:94-217) at chill.py:278-290. */
int chill_bwd_delta(const ChillTensor4* o, const ChillTensor4* d_o,
                    float* delta, const int64_t delta_stride[3],
                    int32_t B, int32_t H, int32_t T, int32_t D,
                    int32_t dtype, void* stream);

/* dQ: replaces the dq branch of _chill_attn_bwd (chill_bwd.py:93-129 ->
 * chill_bwd_dq.py:15-397), launched at chill.py:442.  Every row of `dq` is written; rows at or
 * beyond lens[b] receive 0 (the reference relies on the adapter's zero-fill, chill.py:292). */
int chill_bwd_dq(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                 const ChillTensor4* d_o, const ChillTensor4* dq,
                 const float* lse, const int64_t lse_stride[3],
                 const float* delta, const int64_t delta_stride[3],
                 const int32_t* lens, int64_t lens_stride,
                 int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
                 int32_t dtype, float sm_scale,
                 const ChillMaskDesc* mask, void* stream);

/* dQ with the backward preprocessing fused into it: the launches of _chill_attn_bwd_precompute
 * (utils.py:94-217, at chill.py:278-290) and of the dq branch of _chill_attn_bwd (chill_bwd_dq.py:15-397)
 * in one.  Every workgroup computes delta = rowsum(O * dO) of its own query rows from the dO rows it
 * loads anyway and the same rows of `o`, uses them, and WRITES them to `delta` (every row, zeros at and
 * beyond lens[b]) for the chill_bwd_dkdv launch that must follow on the same stream.  One pass over O and
 * one kernel boundary less than chill_bwd_delta + chill_bwd_dq; dq as from chill_bwd_dq up to the
 * rounding of delta's sum (a different order of additions). */
int chill_bwd_dq_delta(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                       const ChillTensor4* o, const ChillTensor4* d_o, const ChillTensor4* dq,
                       const float* lse, const int64_t lse_stride[3],
                       float* delta, const int64_t delta_stride[3],
                       const int32_t* lens, int64_t lens_stride,
                       int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
                       int32_t dtype, float sm_scale,
                       const ChillMaskDesc* mask, void* stream);

/* dK, dV: replaces the dkdv branch of _chill_attn_bwd (chill_bwd.py:130-167 ->
 * chill_bwd_dkdv.py:15-509), launched at chill.py:442.  One workgroup per (batch, kv head,
 * k-tile); the GQA group loop (chill_bwd_dkdv.py:156) runs inside it.  Every row of `dk` and `dv`
 * is written; rows at or beyond lens[b] receive 0 (the reference relies on the adapter's
 * zero-fill, chill.py:293-294). */
int chill_bwd_dkdv(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                   const ChillTensor4* d_o, const ChillTensor4* dk, const ChillTensor4* dv,
                   const float* lse, const int64_t lse_stride[3],
                   const float* delta, const int64_t delta_stride[3],
                   const int32_t* lens, int64_t lens_stride,
                   int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
                   int32_t dtype, float sm_scale,
                   const ChillMaskDesc* mask, void* stream);

/* The whole backward (dQ with delta on its way, then dK/dV: chill_bwd_dq_delta + chill_bwd_dkdv with the same
 * arguments) WITHOUT a delta workspace from the caller.  It has no counterpart in the
 * reference: it is for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid it).  The fp32 delta rows live in an array inside the library,
 * CHILL_BWD_NOALLOC_MAX_ROWS floats (16 MiB) that every GPU the library runs on holds until the process
 * ends; B * H * T beyond that returns CHILL_ERR_TOO_LARGE.  The call allocates and frees nothing.  All
 * calls on one GPU share that array: calls that overlap on one GPU (two streams, two threads) race on
 * it; calls on one stream are ordered and need nothing more.  The FIRST call on a device looks the
 * array's address up (hipGetSymbolAddress, under a lock), which may load the code object: make that call
 * outside any stream capture; every later call on that device only launches kernels and may be captured. */
#define CHILL_BWD_NOALLOC_MAX_ROWS (4 * 1024 * 1024)
int chill_bwd_noalloc(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                      const ChillTensor4* o, const ChillTensor4* d_o,
                      const ChillTensor4* dq, const ChillTensor4* dk, const ChillTensor4* dv,
                      const float* lse, const int64_t lse_stride[3],
                      const int32_t* lens, int64_t lens_stride,
                      int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
                      int32_t dtype, float sm_scale,
                      const ChillMaskDesc* mask, void* stream);

/* Device-side evaluation of the mask functors, used to prove that the code the kernels run
 * agrees bit-for-bit with the host enumeration (the role ChillMask._mask_infer, mask.py:282-330,
 * plays for the Triton functions).  Writes `n*n` bytes (row = q, col = k) of
 * pred(q,k) && q < n && k < n into device memory `out`. */
int chill_mask_eval_device(const ChillMaskDesc* mask, int32_t n, uint8_t* out, void* stream);

/* Device-side dump of the tile decisions of one pass for sequence length `seq_len` (<= T):
 * for every row tile i (of `tile_in` positions) writes int32 out[i*4 + {0,1,2,3}] =
 * {start_tile, end_tile, full_start_tile, full_end_tile} over tiles of `tile_out` positions,
 * exactly as the kernels compute them (utils.py:221-272 and chill_fwd.py:161-185,
 * chill_bwd_dq.py:279-293, chill_bwd_dkdv.py:329-344).  `out` is device memory,
 * 4 * ceil(T / tile_in) int32. */
int chill_tile_ranges_device(const ChillMaskDesc* mask, int32_t pass, int32_t T, int32_t seq_len,
                             int32_t tile_in, int32_t tile_out, int32_t* out, void* stream);

/* ------------------------------------------------------------------------------------------
 * Host entry points (no GPU needed)
 * ---------------------------------------------------------------------------------------- */

/* Dense mask, host memory: out[q*n + k] = pred(q,k) && q < n && k < n  (ChillMask.make_mask,
 * mask.py:379-412). */
int chill_mask_eval(const ChillMaskDesc* mask, int32_t n, uint8_t* out);

/* Per-position inclusive limits (ChillMask._calc_limits, mask.py:414-454, without its clamp):
 * which = 0 -> k_range_for_q(i), which = 1 -> q_range_for_k(i), for i in [0, n), evaluated with
 * the given seq_len.  out[i*2 + {0,1}] = {lo, hi}. */
int chill_mask_limits(const ChillMaskDesc* mask, int32_t which, int32_t n, int32_t seq_len,
                      int32_t* out);

/* The work item (tile index within the launch, longest tiles of a head first) that workgroup `workgroup` of a launch of
 * `total` work items takes, or -1 when it has none: the XCD-contiguous order of the kernels, compiled for the host.
 * `resident` = workgroups of the kernel that share a CU (1-3); a grid that the chip holds at once is dealt out
 * with every second pass over an XCD's CUs in reverse.  Over the workgroups of a grid (total rounded up to a multiple
 * of 8) the items are a permutation of 0 .. total-1.  Counterpart of the program-id -> tile arithmetic at the top of
 * the reference's kernels (chill_fwd.py:58-61, chill_bwd.py:71-84). */
int chill_work_item(int32_t workgroup, int32_t total, int32_t resident);

/* Host twin of chill_tile_ranges_device (same functors compiled for the host). */
int chill_tile_ranges(const ChillMaskDesc* mask, int32_t pass, int32_t T, int32_t seq_len,
                      int32_t tile_in, int32_t tile_out, int32_t* out);

/* is_full_block(q, k, tile_q, tile_k, seq_len) and has_full_blocks(tile_q, tile_k, seq_len) of
 * the mask (e.g. mask.py:963-976).  Return 0/1 or a negative ChillStatus. */
int chill_mask_is_full_block(const ChillMaskDesc* mask, int32_t q, int32_t k, int32_t tile_q,
                             int32_t tile_k, int32_t seq_len);
int chill_mask_has_full_blocks(const ChillMaskDesc* mask, int32_t tile_q, int32_t tile_k,
                               int32_t seq_len);

/* Static MI355X tile table, replacing autotune.py:11-119: out = {tile_rows, tile_streamed,
 * waves_per_workgroup, lds_bytes} for (mask id, head dim, dtype, pass). */
int chill_tile_config(int32_t mask_id, int32_t D, int32_t dtype, int32_t pass, int32_t out[4]);

/* The same for one launch, batch_heads = B * H sequences of length T: at head dim 128 the forward and dQ
 * rows of 16-bit inputs use a smaller workgroup for short sequences and for grids that would not fill
 * the chip (the reference's tables, autotune.py:11-119, do not depend on the shape; its autotuner's key
 * does, autotune.py:129-240), and the dK/dV row one that covers half as many key rows for such grids
 * (batch_heads = B * H_kv for that pass).  Launches far too small for the chip (a few hundred 32-row
 * blocks in all; fp32, whose ordinary kernels are slow per block, up to a few thousand, depending on the
 * mask) take kernels of their own, in which four waves own 32 rows and split the streamed axis: reported
 * as {32, 32, 4, lds_bytes}, lds_bytes being the workgroup's, which in the forward and dQ holds two such
 * blocks of eight waves in all when the launch has more blocks than the chip has CUs.  chill_tile_config reports the row of long
 * sequences on a full chip. */
int chill_tile_config_for_shape(int32_t mask_id, int32_t D, int32_t dtype, int32_t pass, int64_t batch_heads,
                                int32_t T, int32_t out[4]);

/* The same for one launch with its mask: the dK/dV row of a chunkwise mask depends on the chunk size (with
 * chunks of a multiple of 64 rows a wave's key rows lie in one chunk, no block inside its band is partly
 * masked, and the launch takes the kernel with the generated loop at head dim 128;
 * chill_tile_config_for_shape reports the row of the other chunk sizes), and the forward and dK/dV rows of
 * a banded mask on the most keys a row sees (from 1024 keys on the forward at head dim 128 takes the row of
 * the masks that are not banded, from 4096 keys on so does dK/dV under a sliding window;
 * chill_tile_config_for_shape reports the rows of a narrow band).
 * Counterpart of the autotuner's key, which includes the mask's constants (autotune.py:129-240). */
int chill_tile_config_for_launch(const ChillMaskDesc* mask, int32_t D, int32_t dtype, int32_t pass,
                                 int64_t batch_heads, int32_t T, int32_t out[4]);

/* Number of unmasked (q, k) pairs with q, k < T, closed form per mask — the numerator of the
 * effective-FLOP metric (benchmark/benchmark.py:271-276 takes it from the dense mask). */
int64_t chill_mask_nnz(const ChillMaskDesc* mask, int32_t T);

const char* chill_status_string(int32_t status);
int32_t chill_abi_version(void);

/* 1 if this library was built around a user-written functor (it then serves CHILL_MASK_USER and
 * nothing else), 0 for the stock library.  No counterpart in the reference, where a user mask is
 * a Python class whose Triton methods are compiled on first use (chill.py:27-58). */
int32_t chill_has_user_mask(void);

#ifdef __cplusplus
}
#endif

#endif /* CHILL_ATTENTION_H */
