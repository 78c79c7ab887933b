// Device entry points of the C ABI: argument validation, lowering to plain kernel parameters and
// dispatch to the per-(dtype, head dim) launchers.  Nothing is allocated here and no state is
// kept; every launch goes to the caller's stream.
#include <hip/hip_runtime.h>

#include <mutex>

#include "chill_mask.h"
#include "chill_params.h"

namespace chill {

#define CHILL_FOR_EACH_INST(X)                                                              \
    X(f32, 16) X(f32, 32) X(f32, 64) X(f32, 128) X(f32, 256)                                \
    X(f16, 16) X(f16, 32) X(f16, 64) X(f16, 128) X(f16, 256)                                \
    X(bf16, 16) X(bf16, 32) X(bf16, 64) X(bf16, 128) X(bf16, 256)

#define CHILL_DECLARE(name, d)                                                              \
    int launch_fwd_##name##_##d(const FwdParams&, int, hipStream_t);                        \
    int launch_delta_##name##_##d(const DeltaParams&, hipStream_t);                         \
    int launch_dq_##name##_##d(const BwdParams&, int, hipStream_t);                         \
    int launch_dkdv_##name##_##d(const BwdParams&, int, hipStream_t);
CHILL_FOR_EACH_INST(CHILL_DECLARE)
#undef CHILL_DECLARE

typedef int (*FwdLauncher)(const FwdParams&, int, hipStream_t);
typedef int (*DeltaLauncher)(const DeltaParams&, hipStream_t);
typedef int (*BwdLauncher)(const BwdParams&, int, hipStream_t);

static int dim_index(int D) {
    switch (D) {
        case 16: return 0;
        case 32: return 1;
        case 64: return 2;
        case 128: return 3;
        case 256: return 4;
        default: return -1;
    }
}

// tables indexed [dtype][dim_index]; dtype order matches ChillDType (f32, f16, bf16)
#define CHILL_ROW(kind, name) \
    {launch_##kind##_##name##_16, launch_##kind##_##name##_32, launch_##kind##_##name##_64, launch_##kind##_##name##_128, launch_##kind##_##name##_256}
static const FwdLauncher kFwd[3][5] = {CHILL_ROW(fwd, f32), CHILL_ROW(fwd, f16), CHILL_ROW(fwd, bf16)};
static const DeltaLauncher kDelta[3][5] = {CHILL_ROW(delta, f32), CHILL_ROW(delta, f16), CHILL_ROW(delta, bf16)};
static const BwdLauncher kDq[3][5] = {CHILL_ROW(dq, f32), CHILL_ROW(dq, f16), CHILL_ROW(dq, bf16)};
static const BwdLauncher kDkdv[3][5] = {CHILL_ROW(dkdv, f32), CHILL_ROW(dkdv, f16), CHILL_ROW(dkdv, bf16)};
#undef CHILL_ROW

static int check_dtype_dim(int dtype, int D, int* es) {
    if (dtype != CHILL_F32 && dtype != CHILL_F16 && dtype != CHILL_BF16) return CHILL_ERR_BAD_DTYPE;
    if (dim_index(D) < 0) return CHILL_ERR_BAD_HEAD_DIM;
    *es = dtype == CHILL_F32 ? 4 : 2;
    return CHILL_OK;
}

// The exponent's factor sm_scale * log2(e).  The kernels multiply it into raw scores of which the
// masked ones are -inf, so it must not be zero: a zero scale (uniform attention over the visible keys,
// chill_fwd.py:213-214 scales first and masks afterwards) becomes one so small that every finite score
// still rounds to exponent 0.  Non-finite scales are refused.
static int lower_scale(float sm_scale, float* scale_log2) {
    if (!(sm_scale - sm_scale == 0.f)) return CHILL_ERR_BAD_ARGUMENT;
    float s = sm_scale * 1.4426950408889634f;
    if (s == 0.f) s = 1e-30f;
    *scale_log2 = s;
    return CHILL_OK;
}

static int check_shape(int B, int H, int H_kv, int T) {
    if (B <= 0 || H <= 0 || H_kv <= 0 || T <= 0) return CHILL_ERR_BAD_SHAPE;
    if (H % H_kv != 0) return CHILL_ERR_BAD_SHAPE;
    if (T > (1 << 29)) return CHILL_ERR_TOO_LARGE;
    return CHILL_OK;
}

// A [*, *, T, D] view the kernels can address: unit inner stride, 16-byte aligned rows.
static int lower_tensor(const ChillTensor4* t, int es, Strides3* out) {
    if (t == nullptr || t->ptr == nullptr) return CHILL_ERR_NULL_POINTER;
    if (t->stride[3] != 1) return CHILL_ERR_BAD_STRIDE;
    for (int i = 0; i < 3; i++) {
        if (t->stride[i] < 0) return CHILL_ERR_BAD_STRIDE;
        if ((t->stride[i] * es) % 16 != 0) return CHILL_ERR_BAD_STRIDE;
    }
    if (reinterpret_cast<uintptr_t>(t->ptr) % 16 != 0) return CHILL_ERR_BAD_STRIDE;
    out->b = t->stride[0];
    out->h = t->stride[1];
    out->t = t->stride[2];
    return CHILL_OK;
}

static int lower_vec3(const void* ptr, const int64_t stride[3], int64_t* sb, int64_t* sh) {
    if (ptr == nullptr || stride == nullptr) return CHILL_ERR_NULL_POINTER;
    if (stride[2] != 1 || stride[0] < 0 || stride[1] < 0) return CHILL_ERR_BAD_STRIDE;
    *sb = stride[0];
    *sh = stride[1];
    return CHILL_OK;
}

#define CHILL_TRY(expr)             \
    do {                            \
        int st_ = (expr);           \
        if (st_ != CHILL_OK) return st_; \
    } while (0)

}  // namespace chill

using namespace chill;

extern "C" {

int chill_fwd(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
              const ChillTensor4* o, float* lse, const int64_t lse_stride[3],
              const int32_t* lens, int64_t lens_stride,
              int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
              int32_t dtype, float sm_scale, const ChillMaskDesc* mask, void* stream) {
    int es = 0;
    FwdParams p = {};
    CHILL_TRY(check_dtype_dim(dtype, D, &es));
    CHILL_TRY(check_shape(B, H, H_kv, T));
    CHILL_TRY(lower_mask(mask, &p.margs));
    CHILL_TRY(lower_tensor(q, es, &p.sq));
    CHILL_TRY(lower_tensor(k, es, &p.sk));
    CHILL_TRY(lower_tensor(v, es, &p.sv));
    CHILL_TRY(lower_tensor(o, es, &p.so));
    if (lse != nullptr) CHILL_TRY(lower_vec3(lse, lse_stride, &p.lse_b, &p.lse_h));
    if (lens != nullptr && lens_stride < 0) return CHILL_ERR_BAD_STRIDE;
    p.q = q->ptr;
    p.k = k->ptr;
    p.v = v->ptr;
    p.o = o->ptr;
    p.lse = lse;
    p.lens = lens;
    p.lens_stride = lens_stride;
    p.B = B;
    p.H = H;
    p.H_kv = H_kv;
    p.T = T;
    p.group = H / H_kv;
    CHILL_TRY(lower_scale(sm_scale, &p.scale_log2));
    return kFwd[dtype][dim_index(D)](p, mask->id, static_cast<hipStream_t>(stream));
}

int chill_bwd_delta(const ChillTensor4* o, const ChillTensor4* d_o, float* delta,
                    const int64_t delta_stride[3], int32_t B, int32_t H, int32_t T, int32_t D,
                    int32_t dtype, void* stream) {
    int es = 0;
    DeltaParams p = {};
    CHILL_TRY(check_dtype_dim(dtype, D, &es));
    CHILL_TRY(check_shape(B, H, H, T));
    CHILL_TRY(lower_tensor(o, es, &p.so));
    CHILL_TRY(lower_tensor(d_o, es, &p.sdo));
    CHILL_TRY(lower_vec3(delta, delta_stride, &p.delta_b, &p.delta_h));
    p.o = o->ptr;
    p.d_o = d_o->ptr;
    p.delta = delta;
    p.B = B;
    p.H = H;
    p.T = T;
    return kDelta[dtype][dim_index(D)](p, static_cast<hipStream_t>(stream));
}

static int lower_bwd(BwdParams* p, const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                     const ChillTensor4* d_o, const float* lse, const int64_t lse_stride[3],
                     const float* delta, const int64_t delta_stride[3], const int32_t* lens,
                     int64_t lens_stride, int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
                     int32_t dtype, float sm_scale, const ChillMaskDesc* mask, int* es) {
    CHILL_TRY(check_dtype_dim(dtype, D, es));
    CHILL_TRY(check_shape(B, H, H_kv, T));
    CHILL_TRY(lower_mask(mask, &p->margs));
    CHILL_TRY(lower_tensor(q, *es, &p->sq));
    CHILL_TRY(lower_tensor(k, *es, &p->sk));
    CHILL_TRY(lower_tensor(v, *es, &p->sv));
    CHILL_TRY(lower_tensor(d_o, *es, &p->sdo));
    CHILL_TRY(lower_vec3(lse, lse_stride, &p->lse_b, &p->lse_h));
    CHILL_TRY(lower_vec3(delta, delta_stride, &p->delta_b, &p->delta_h));
    if (lens != nullptr && lens_stride < 0) return CHILL_ERR_BAD_STRIDE;
    p->q = q->ptr;
    p->k = k->ptr;
    p->v = v->ptr;
    p->d_o = d_o->ptr;
    p->lse = lse;
    p->delta = delta;
    p->lens = lens;
    p->lens_stride = lens_stride;
    p->B = B;
    p->H = H;
    p->H_kv = H_kv;
    p->T = T;
    p->group = H / H_kv;
    p->sm_scale = sm_scale;
    CHILL_TRY(lower_scale(sm_scale, &p->scale_log2));
    return CHILL_OK;
}

int chill_bwd_dq(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                 const ChillTensor4* d_o, const ChillTensor4* dq, const float* lse,
                 const int64_t lse_stride[3], const float* delta, const int64_t delta_stride[3],
                 const int32_t* lens, int64_t lens_stride, int32_t B, int32_t H, int32_t H_kv,
                 int32_t T, int32_t D, int32_t dtype, float sm_scale, const ChillMaskDesc* mask,
                 void* stream) {
    int es = 0;
    BwdParams p = {};
    CHILL_TRY(lower_bwd(&p, q, k, v, d_o, lse, lse_stride, delta, delta_stride, lens, lens_stride,
                        B, H, H_kv, T, D, dtype, sm_scale, mask, &es));
    CHILL_TRY(lower_tensor(dq, es, &p.sdq));
    p.dq = dq->ptr;
    return kDq[dtype][dim_index(D)](p, mask->id, static_cast<hipStream_t>(stream));
}

int chill_bwd_dq_delta(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                       const ChillTensor4* o, const ChillTensor4* d_o, const ChillTensor4* dq,
                       const float* lse, const int64_t lse_stride[3], float* delta,
                       const int64_t delta_stride[3], const int32_t* lens, int64_t lens_stride,
                       int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D, int32_t dtype,
                       float sm_scale, const ChillMaskDesc* mask, void* stream) {
    int es = 0;
    BwdParams p = {};
    CHILL_TRY(lower_bwd(&p, q, k, v, d_o, lse, lse_stride, delta, delta_stride, lens, lens_stride,
                        B, H, H_kv, T, D, dtype, sm_scale, mask, &es));
    CHILL_TRY(lower_tensor(dq, es, &p.sdq));
    CHILL_TRY(lower_tensor(o, es, &p.so));
    p.dq = dq->ptr;
    p.o = o->ptr;
    p.delta_out = delta;
    return kDq[dtype][dim_index(D)](p, mask->id, static_cast<hipStream_t>(stream));
}

int chill_bwd_dkdv(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                   const ChillTensor4* d_o, const ChillTensor4* dk, const ChillTensor4* dv,
                   const float* lse, const int64_t lse_stride[3], const float* delta,
                   const int64_t delta_stride[3], const int32_t* lens, int64_t lens_stride,
                   int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D, int32_t dtype,
                   float sm_scale, const ChillMaskDesc* mask, void* stream) {
    int es = 0;
    BwdParams p = {};
    CHILL_TRY(lower_bwd(&p, q, k, v, d_o, lse, lse_stride, delta, delta_stride, lens, lens_stride,
                        B, H, H_kv, T, D, dtype, sm_scale, mask, &es));
    CHILL_TRY(lower_tensor(dk, es, &p.sdk));
    CHILL_TRY(lower_tensor(dv, es, &p.sdv));
    p.dk = dk->ptr;
    p.dv = dv->ptr;
    return kDkdv[dtype][dim_index(D)](p, mask->id, static_cast<hipStream_t>(stream));
}

// ---------------------------------------------------------------------------------------------
// The whole backward without a workspace from the caller.  The fp32 delta rows, which chill_bwd_dq_delta
// writes and chill_bwd_dkdv reads, live in a device array of this library: each GPU the
// library runs on holds its own copy of `scratch` until the process ends.  In host code the array's
// name is a stand-in, not a device address: the address comes from hipGetSymbolAddress, once per
// device with that device current, and only that pointer is handed to kernels.
// ---------------------------------------------------------------------------------------------
constexpr int64_t kNoAllocMaxRows = (int64_t)CHILL_BWD_NOALLOC_MAX_ROWS;
static __device__ __align__(256) float scratch[kNoAllocMaxRows];

constexpr int kMaxDevices = 64;
static float* g_scratch_address[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

// the current device's copy of `scratch`
static int scratch_of_current_device(float** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return CHILL_ERR_HIP;
    std::lock_guard<std::mutex> guard(g_scratch_mutex);
    if (g_scratch_address[dev] == nullptr) {
        float* ptr = nullptr;
        if (hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr)
            return CHILL_ERR_HIP;
        g_scratch_address[dev] = ptr;
    }
    *out = g_scratch_address[dev];
    return CHILL_OK;
}

int chill_bwd_noalloc(const ChillTensor4* q, const ChillTensor4* k, const ChillTensor4* v,
                      const ChillTensor4* o, const ChillTensor4* d_o,
                      const ChillTensor4* dq, const ChillTensor4* dk, const ChillTensor4* dv,
                      const float* lse, const int64_t lse_stride[3],
                      const int32_t* lens, int64_t lens_stride,
                      int32_t B, int32_t H, int32_t H_kv, int32_t T, int32_t D,
                      int32_t dtype, float sm_scale, const ChillMaskDesc* mask, void* stream) {
    CHILL_TRY(check_shape(B, H, H_kv, T));
    // delta is [B, H, T] fp32, contiguous, in the library's array: sizes beyond it are refused
    if ((int64_t)B * H * T > kNoAllocMaxRows) return CHILL_ERR_TOO_LARGE;
    float* delta = nullptr;
    CHILL_TRY(scratch_of_current_device(&delta));
    const int64_t delta_stride[3] = {(int64_t)H * T, (int64_t)T, 1};
    // every row of delta is written by the first launch before the second reads it: nothing to clear
    CHILL_TRY(chill_bwd_dq_delta(q, k, v, o, d_o, dq, lse, lse_stride, delta, delta_stride, lens, lens_stride, B, H,
                                 H_kv, T, D, dtype, sm_scale, mask, stream));
    return chill_bwd_dkdv(q, k, v, d_o, dk, dv, lse, lse_stride, delta, delta_stride, lens, lens_stride, B, H, H_kv, T,
                          D, dtype, sm_scale, mask, stream);
}

}  // extern "C"
