// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "kcg.h"

namespace kcg {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef short bf16x8_t __attribute__((ext_vector_type(8)));
typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8_t __attribute__((ext_vector_type(8)));

constexpr int kWaveSize = 64;
constexpr int kNumXcd = 8;  // MI355X: 8 XCDs, workgroups are dealt to them round-robin

// Workgroup id -> logical tile id such that every XCD (which owns a private L2)
// walks one contiguous range of logical ids.  The dispatcher hands workgroup w
// to XCD (w % 8); XCD x therefore sees w = x, x+8, x+16, ...  Those are
// renumbered x*per + min(x, rem) + w/8, a bijection on [0, n).
__device__ __forceinline__ int xcd_contiguous_id(int w, int n) {
  const int xcd = w % kNumXcd;
  const int idx = w / kNumXcd;
  const int per = n / kNumXcd;
  const int rem = n % kNumXcd;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

// arith.maxf(0, x): NaN propagates, -0 -> +0 (src/Frontend/Operators.cc:238-242).
__device__ __forceinline__ float relu_maxf(float x) {
  return (x > 0.0f || x != x) ? x : 0.0f;
}

inline int launch_status() {
  return hipGetLastError() == hipSuccess ? KCG_OK : KCG_ERR_LAUNCH;
}

// Defined in fmha_f32.hip / fmha_bf16.hip; `info` != nullptr only fills the launch geometry.
int dispatch_fmha_f32(const float *Q, const float *K, const float *V, float *O, int B, int H, int S,
                      int D, float scale, int causal, const kcg_fmha_sched *sched,
                      hipStream_t stream, kcg_launch_info *info);
int dispatch_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O,
                       int o_dtype, int B, int H, int S, int D, float scale, int causal,
                       const kcg_fmha_sched *sched, hipStream_t stream, kcg_launch_info *info);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace kcg
