// One translation unit per (element type, head dim): compile with
//   -DCHILL_ELEM=bf16_t -DCHILL_ELEM_NAME=bf16 -DCHILL_HEAD_DIM=128
#include "chill_fwd_kernel.h"

#define CHILL_CAT3_(a, b, c) a##b##_##c
#define CHILL_CAT3(a, b, c) CHILL_CAT3_(a, b, c)

namespace chill {
int CHILL_CAT3(launch_fwd_, CHILL_ELEM_NAME, CHILL_HEAD_DIM)(const FwdParams& p, int mask_id, hipStream_t stream) {
    return launch_fwd<CHILL_ELEM, CHILL_HEAD_DIM>(p, mask_id, stream);
}
}  // namespace chill
