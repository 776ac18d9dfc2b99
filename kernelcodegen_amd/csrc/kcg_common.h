// Shared device/host helpers for the gfx950 kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <tuple>
#include <utility>

#include "kcg.h"

namespace kcg {

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef short bf16x8_t __attribute__((ext_vector_type(8)));
typedef short bf16x4_t __attribute__((ext_vector_type(4)));
typedef unsigned short u16x8_t __attribute__((ext_vector_type(8)));

constexpr int kWaveSize = 64;
constexpr int kNumCu = 256;  // MI355X compute units
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

// v_max3_f32 without the canonicalising self-max the compiler puts in front of fmaxf on
// MFMA results (NaN operands are ignored like in fmaxf; a NaN score still reaches the
// output through its own exponential).
__device__ __forceinline__ float max3(float a, float b, float c) {
#if defined(__HIP_DEVICE_COMPILE__)
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
#else
  return fmaxf(fmaxf(a, b), c);
#endif
}

// max(x of lane l, x of lane l ^ 32): one v_permlane32_swap (the upper half of the first
// register changes places with the lower half of the second) and one v_max.  Issued from
// assembly: the compiler's builtin for this instruction hands back its first result
// register for both results, which turns the maximum into "the lower half's value".
__device__ __forceinline__ float max_across_halves(float x) {
#if defined(__HIP_DEVICE_COMPILE__)
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return fmaxf(a, b);
#else
  return x;
#endif
}

// One wave-wide direct load: lane l's 16 bytes at (uniform base + off) go to LDS byte
// address lds_addr + 16 * l.  Issued from assembly so that the address is formed by the
// instruction itself (scalar base + 32-bit lane offset); the intrinsic materialises a
// 64-bit address per lane with VALU work, which on this chip comes out of fp32 MFMA time.
// M0 (the LDS base of the load) is saved and restored around the instruction.
__device__ __forceinline__ void direct_load_16B(const void *base, unsigned off, unsigned lds_addr) {
#if defined(__HIP_DEVICE_COMPILE__)
  unsigned saved_m0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %2, %3\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0)
      : "s"(lds_addr), "v"(off), "s"(base)
      : "memory");
#endif
}

// Launches `kern` and reports the launch's own status.  hipLaunchKernel returns
// the error of this launch; hipGetLastError would also surface a stale error
// left behind by an unrelated earlier runtime call of the host program.
template <typename... KArgs, size_t... I>
inline int launch_impl(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes,
                       hipStream_t stream, std::tuple<KArgs...> &args, std::index_sequence<I...>) {
  void *ptrs[] = {static_cast<void *>(&std::get<I>(args))...};
  const hipError_t e =
      hipLaunchKernel(reinterpret_cast<const void *>(kern), grid, block, ptrs, lds_bytes, stream);
  return e == hipSuccess ? KCG_OK : KCG_ERR_LAUNCH;
}

template <typename... KArgs, typename... Args>
inline int launch(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t lds_bytes,
                  hipStream_t stream, Args... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "kernel argument count");
  std::tuple<KArgs...> packed{static_cast<KArgs>(args)...};
  return launch_impl(kern, grid, block, lds_bytes, stream, packed, std::index_sequence_for<KArgs...>{});
}

// Kernels that need more than 48 KiB of dynamic LDS must opt in, once per function and
// device.  The opt-in is a runtime call of a few microseconds -- as long as the smallest
// matmuls run -- so it is made on a kernel's first launch only and remembered in a small
// lock-free table (thread safe; a lost race merely repeats the call).
inline bool lds_opt_in_once(const void *kern, int lds_bytes) {
  constexpr int kSlots = 256;
  static std::atomic<uintptr_t> seen[kSlots];  // zero-initialised: empty
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess) return false;
  // kernel addresses are at least 4-byte aligned code addresses well below 2^56
  const uintptr_t key = reinterpret_cast<uintptr_t>(kern) ^ (static_cast<uintptr_t>(device + 1) << 56);
  for (int i = 0; i < kSlots; ++i) {
    const uintptr_t v = seen[i].load(std::memory_order_acquire);
    if (v == key) return true;
    if (v == 0) break;
  }
  if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes) != hipSuccess) return false;
  for (int i = 0; i < kSlots; ++i) {
    uintptr_t expected = 0;
    if (seen[i].compare_exchange_strong(expected, key, std::memory_order_acq_rel) || expected == key) break;
  }
  return true;  // (a full table only means the call is repeated next time)
}

template <typename... KArgs>
inline bool allow_lds(void (*kern)(KArgs...), int lds_bytes) {
  if (lds_bytes <= 48 * 1024) return true;
  return lds_opt_in_once(reinterpret_cast<const void *>(kern), lds_bytes);
}

// Defined in gemm_f32.hip: BatchedMatmul with A as [batch][M][K] and B as [batch][K][N] or
// (trans_b) [batch][N][K] on the direct-load matmul kernel; KCG_ERR_UNSUPPORTED_SHAPE when
// the problem needs the generic kernel instead.
int dispatch_bmm_dl(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N,
                    int64_t K, bool trans_b, hipStream_t stream);

// Defined in fmha_f32.hip / fmha_bf16.hip; `info` != nullptr only fills the launch geometry.
int dispatch_fmha_f32(const float *Q, const float *K, const float *V, float *O, int B, int H, int S,
                      int D, float scale, int causal, const kcg_fmha_sched *sched,
                      hipStream_t stream, kcg_launch_info *info);
int dispatch_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O,
                       int o_dtype, int B, int H, int S, int D, float scale, int causal,
                       const kcg_fmha_sched *sched, hipStream_t stream, kcg_launch_info *info);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace kcg
