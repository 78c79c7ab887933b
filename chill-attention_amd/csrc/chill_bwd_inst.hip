// One translation unit per (element type, head dim): compile with
//   -DCHILL_ELEM=bf16_t -DCHILL_ELEM_NAME=bf16 -DCHILL_HEAD_DIM=128
#include "chill_bwd_kernels.h"

#define CHILL_CAT3_(a, b, c) a##b##_##c
#define CHILL_CAT3(a, b, c) CHILL_CAT3_(a, b, c)

namespace chill {
int CHILL_CAT3(launch_delta_, CHILL_ELEM_NAME, CHILL_HEAD_DIM)(const DeltaParams& p, hipStream_t stream) {
    return launch_delta<CHILL_ELEM, CHILL_HEAD_DIM>(p, stream);
}
int CHILL_CAT3(launch_dq_, CHILL_ELEM_NAME, CHILL_HEAD_DIM)(const BwdParams& p, int mask_id, hipStream_t stream) {
    return launch_dq<CHILL_ELEM, CHILL_HEAD_DIM>(p, mask_id, stream);
}
int CHILL_CAT3(launch_dkdv_, CHILL_ELEM_NAME, CHILL_HEAD_DIM)(const BwdParams& p, int mask_id, hipStream_t stream) {
    return launch_dkdv<CHILL_ELEM, CHILL_HEAD_DIM>(p, mask_id, stream);
}
}  // namespace chill
