// What an MI355X sustains on the instruction mix of the bf16 attention kernel when nothing
// ever stalls: a loop of v_mfma_f32_32x32x16_bf16 on random operands, 8 waves per CU, run
// for some seconds so that the clock and power management settle.
//
//   mfma_mix_ceiling <mode> [seconds]
//   mode 0: MFMA only, operands in registers
//   mode 1: the A operand of every MFMA comes from LDS (one ds_read_b128 = 1 KiB per MFMA,
//           the K / V fragment traffic of the attention kernel)
//   mode 2: mode 1 plus 5.5 VALU instructions per MFMA, one of them v_exp_f32 (the softmax
//           arithmetic per MFMA that the attention kernel's counters show)
//   mode 3: mode 0 plus the VALU mix, no LDS
//
// Prints sustained TFLOP/s (MFMA FLOPs only).  Sample `rocm-smi --showclocks` and
// `amd-smi metric -p` from another shell while it runs to see clock and socket power.
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <chrono>
typedef float f16v __attribute__((ext_vector_type(16)));
typedef __bf16 bf8 __attribute__((ext_vector_type(8)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));

template <int MODE>
__global__ __launch_bounds__(512, 2) void k(float *out, const unsigned *rnd, int iters) {
  __shared__ __attribute__((aligned(16))) unsigned lds[16384];  // 64 KiB
  for (int i = threadIdx.x; i < 16384; i += 512) lds[i] = rnd[i];
  __syncthreads();
  const int lane = threadIdx.x & 63;
  u4 areg[4], breg[4];
  for (int j = 0; j < 4; ++j) {
    areg[j] = *(const u4 *)(rnd + 16384 + (threadIdx.x * 8 + j) * 4);
    breg[j] = *(const u4 *)(rnd + 16384 + (threadIdx.x * 8 + 4 + j) * 4);
  }
  f16v acc[4];
  for (int i = 0; i < 4; ++i) for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
  float v[4] = {0.3f, -0.2f, 0.7f, 0.1f};
  const float c = __builtin_bit_cast(float, rnd[threadIdx.x] & 0x3fffffff | 0x3f000000);  // [0.5, 2)
  const u4 *lp = (const u4 *)lds + lane;
  float sink = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 32; ++m) {
      u4 a = areg[m & 3];
      if (MODE == 1 || MODE == 2) a = lp[((it * 32 + m) & 63) * 64];
      // accumulators restart every 8 MFMAs like the S tile of the attention kernel
      if ((m & 31) < 4)
        acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, breg[(m >> 2) & 3]), f16v{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, 0, 0, 0);
      else
        acc[m & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8, a), __builtin_bit_cast(bf8, breg[(m >> 2) & 3]), acc[m & 3], 0, 0, 0);
      if (MODE == 2 || MODE == 3) {
        // 5.5 VALU instructions per MFMA, one of them an exponential, fed from an accumulator
        // that finished long ago (like the softmax of the previous tile)
        const float s = acc[(m + 2) & 3][m & 15];
        v[1] = fmaxf(v[1], s);                                       // v_max
        v[0] = __builtin_fmaf(s, c, v[1]);                           // v_fma
        v[2] = __builtin_amdgcn_exp2f(v[0]);                         // v_exp
        v[3] = __builtin_fmaf(v[2], c, v[3]);                        // v_fma
        sink += v[3];                                                // v_add
        if (m & 1) v[1] = v[1] * 0.5f;                               // v_mul every other slot
      }
    }
  }
  float s = sink;
  for (int i = 0; i < 4; ++i) for (int e = 0; e < 16; ++e) s += acc[i][e];
  out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

template <int MODE> void run(float *d, const unsigned *rnd, double secs) {
  const int iters = 20000;
  k<MODE><<<512, 512>>>(d, rnd, 2000);
  (void)hipDeviceSynchronize();
  auto t0 = std::chrono::steady_clock::now();
  int n = 0;
  double el = 0;
  do {
    for (int r = 0; r < 4; ++r) k<MODE><<<512, 512>>>(d, rnd, iters);
    (void)hipDeviceSynchronize();
    n += 4;
    el = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  } while (el < secs);
  const double flops = 512.0 * 8 * iters * 32 * 32768.0 * n;
  printf("mode %d: %d launches in %.2f s -> %.1f TFLOP/s sustained (%.1f%% of 2500)\n", MODE, n, el, flops / el / 1e12, flops / el / 1e12 / 25.0);
  fflush(stdout);
}
int main(int argc, char **argv) {
  const int mode = argc > 1 ? atoi(argv[1]) : 0;
  const double secs = argc > 2 ? atof(argv[2]) : 5.0;
  float *d; unsigned *rnd;
  const size_t nr = 16384 + 512 * 8 * 4 + 1024;
  (void)hipMalloc(&d, 512 * 512 * 4); (void)hipMalloc(&rnd, nr * 4);
  unsigned *h = (unsigned *)malloc(nr * 4);
  unsigned s = 12345;
  for (size_t i = 0; i < nr; ++i) {
    // two bf16 values ~ N(0,1)-like: random sign, exponent around 2^-2..2^1, random mantissa
    unsigned w = 0;
    for (int hlf = 0; hlf < 2; ++hlf) {
      s = s * 1664525u + 1013904223u;
      const unsigned sign = (s >> 31) << 15, ex = (125 + ((s >> 20) & 3)) << 7, man = (s >> 8) & 0x7f;
      w |= (sign | ex | man) << (16 * hlf);
    }
    h[i] = w;
  }
  (void)hipMemcpy(rnd, h, nr * 4, hipMemcpyHostToDevice);
  if (mode == 0) run<0>(d, rnd, secs);
  if (mode == 1) run<1>(d, rnd, secs);
  if (mode == 2) run<2>(d, rnd, secs);
  if (mode == 3) run<3>(d, rnd, secs);
  printf("%s\n", hipGetErrorString(hipGetLastError()));
  return 0;
}
