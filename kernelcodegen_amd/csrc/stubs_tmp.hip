#include "kcg_common.h"
extern "C" {
int kcg_fmha_f32(const float *, const float *, const float *, float *, int32_t, int32_t, int32_t, int32_t, float, int, const kcg_fmha_sched *, void *) { return KCG_ERR_UNSUPPORTED_SHAPE; }
int kcg_fmha_bf16(const uint16_t *, const uint16_t *, const uint16_t *, void *, int, int32_t, int32_t, int32_t, int32_t, float, int, const kcg_fmha_sched *, void *) { return KCG_ERR_UNSUPPORTED_SHAPE; }
int kcg_fmha_query(int, int32_t, int32_t, int32_t, int32_t, int, const kcg_fmha_sched *, kcg_launch_info *) { return KCG_ERR_UNSUPPORTED_SHAPE; }
int kcg_batched_matmul_f32(const float *, int, const float *, int, float *, int64_t, int64_t, int64_t, int64_t, void *) { return KCG_ERR_UNSUPPORTED_SHAPE; }
int kcg_softmax_f32(float *, int64_t, int64_t, void *) { return KCG_ERR_UNSUPPORTED_SHAPE; }
}
