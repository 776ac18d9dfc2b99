// fp32 matmul on a 96 x 96 or 96 x 64 tile: the tiles for problems whose count of such tiles
// fills the 256 CUs in whole rounds where the power-of-two tiles do not (1536^3 is 256 tiles
// of 96 x 96, but 576 = 2.25 x 256 tiles of 64 x 64; 1152^2 is 216 tiles of 96 x 64).
//
// Same schedule as gemm_f32_dl_kernel (MatmulOptimizer's, src/Optimizer/Optimizer.cc:383-548:
// a tile of C per workgroup, K in BLOCK_SIZE_K slices through a ring of LDS stages, later
// slices in flight during compute, one barrier per slice); what differs is the wave tile.  96
// is not a multiple of 32 x 2 waves, so the four waves own 48 x 48 (or 48 x 32) each as 3 x 3
// (3 x 2) blocks of v_mfma_f32_16x16x4_f32 (lane l, r = l % 16, g = l / 16):
//   A operand: A[row r][k = g]      B operand: B[k = g][col r]
//   D: 4 floats, element e is C[4 * g + e][r].
// One ds_read_b128 of A gives lane (r, g) the four k = 4g .. 4g+3 of a 16-wide half of the
// slice; the j-th MFMA of that half consumes k = 4g + j from both operands, so the products
// summed into an element of C are those of the reference nest in a different order.
//
// K is a multiple of 32 and N of 4 (rows keep 16-byte alignment).  RAGGED: M and N need not
// divide the tile.  Rows of A at and beyond M and 16-byte column chunks of B at and beyond N
// only feed elements of C that are never stored, so their lanes fetch the last valid row /
// chunk instead (a loop-invariant change of the lane offsets), and the stores are bounds-checked.
#pragma once

#include <type_traits>

#include "gemm_dl_tile.h"
#include "kcg_common.h"

namespace kcg {

template <int BM, int BN, bool RELU, bool RAGGED>
__global__ __launch_bounds__(256, 2) void gemm_f32_t96_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N, int K,
    int tiles_m, int tiles_n, int group_m) {
  using G = GemmT96Tile<BM, BN>;
  static_assert(G::kThreads == 256, "launch bounds");
  extern __shared__ __align__(16) float lds[];

  const int logical = xcd_contiguous_id(blockIdx.x, tiles_m * tiles_n);
  const int width = group_m * tiles_n;
  const int group = logical / width;
  const int first_m = group * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int in_group = logical - group * width;
  const int m0 = (first_m + in_group % gsz) * G::kBM;
  const int n0 = (in_group / gsz) * G::kBN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / G::kWavesN;
  const int wn = wave % G::kWavesN;
  const int r16 = lane & 15;
  const int g = lane >> 4;

  float4_t acc[G::kBlocksM][G::kBlocksN];
#pragma unroll
  for (int i = 0; i < G::kBlocksM; ++i)
#pragma unroll
    for (int n = 0; n < G::kBlocksN; ++n) acc[i][n] = float4_t{0.f, 0.f, 0.f, 0.f};

  // ---- direct loads: uniform slice base + per-lane 32-bit byte offsets ----
  const int lds_base = static_cast<int>(reinterpret_cast<uintptr_t>(lds));
  unsigned oa[G::kLoadsA];
  unsigned ob[G::kLoadsB];
#pragma unroll
  for (int i = 0; i < G::kLoadsA; ++i) {
    const int idx = (wave * G::kLoadsA + i) * 256 + lane * 4;  // float index in the LDS A tile
    const int row = idx / G::kBK;
    const int c_log = ((idx % G::kBK) / 4) ^ G::fa(row);
    const int grow = RAGGED ? (row < M - m0 ? row : M - m0 - 1) : row;
    oa[i] = static_cast<unsigned>(grow * K + 4 * c_log) * 4u;
  }
#pragma unroll
  for (int i = 0; i < G::kLoadsB; ++i) {
    const int idx = (wave * G::kLoadsB + i) * 256 + lane * 4;  // float index in the LDS B tile
    const int col = G::b_col(idx);
    const int gcol = RAGGED ? (col < N - n0 ? col : N - n0 - 4) : col;
    ob[i] = static_cast<unsigned>(G::b_row(idx) * N + gcol) * 4u;
  }
  const char *ga = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0) * K);
  const char *gb = reinterpret_cast<const char *>(B + n0);
  const int64_t b_step = static_cast<int64_t>(G::kBK) * N * 4;
  constexpr int kLoadsPerSlice = G::kLoadsA + G::kLoadsB;
  auto issue_one = [&](int stage_off, int l) {
    if (l < G::kLoadsA) {
      direct_load_16B(ga, oa[l], static_cast<unsigned>(lds_base + (stage_off + (wave * G::kLoadsA + l) * 256) * 4));
    } else {
      const int i = l - G::kLoadsA;
      direct_load_16B(gb, ob[i],
                      static_cast<unsigned>(lds_base + (stage_off + G::kFloatsA + (wave * G::kLoadsB + i) * 256) * 4));
    }
  };
  // no branch in the slice loop: past the last slice the pointers stop advancing and the
  // final slice is fetched again into a stage nobody reads any more
  auto advance_if = [&](bool cond) {
    ga += cond ? G::kBK * 4 : 0;
    gb += cond ? b_step : 0;
  };

  // ---- operand reads (inline assembly with hand-counted waits, as in gemm_f32_dl_kernel:
  // while a direct load is in flight the compiler would drain every LDS read before each
  // MFMA group) ----
  int a_addr[G::kStages][2];
  int b_addr[G::kStages];
#pragma unroll
  for (int st = 0; st < G::kStages; ++st) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
      a_addr[st][h] = lds_base + (st * G::kStageFloats + (wm * G::kWaveM + r16) * G::kBK +
                                  4 * ((g + 4 * h) ^ G::fa(r16))) * 4;
    b_addr[st] = lds_base + (st * G::kStageFloats + G::kFloatsA + wn * G::kBlocksN * 64 + g * 16 + r16) * 4;
  }
  static_assert(G::fa(16) == G::fa(0) && G::kWaveM % 16 == 0, "the swizzle repeats every 16 rows");
  float4_t fa[2][G::kBlocksM];
  float fb[2][G::kBlocksN];
  float4_t na[G::kBlocksM];
  float nb[G::kBlocksN];
  auto read_a = [&](int stage, int h, float4_t(&dst)[G::kBlocksM]) {
    const int addr = a_addr[stage][h];
#pragma unroll
    for (int i = 0; i < G::kBlocksM; ++i)
      asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst[i]) : "v"(addr), "n"(i * 16 * G::kBK * 4) : "memory");
  };
  auto read_b = [&](int stage, int s, float(&dst)[G::kBlocksN]) {
    const int addr = b_addr[stage];
#pragma unroll
    for (int n = 0; n < G::kBlocksN; ++n)
      asm volatile("ds_read_b32 %0, %1 offset:%2"
                   : "=v"(dst[n])
                   : "v"(addr), "n"((s * G::kQuartetFloats + n * 64) * 4)
                   : "memory");
  };
  constexpr int kReadsA = G::kBlocksM, kReadsB = G::kBlocksN;  // LDS instructions per read_a / read_b

  // Publishes the slice requested before the newest one (see gemm_f32_dl_kernel).
  auto publish = [&]() {
    static_assert(kLoadsPerSlice < 16, "vmcnt immediate");
    __builtin_amdgcn_s_waitcnt(kLoadsPerSlice | 0x70);  // vmcnt(kLoadsPerSlice) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  const int ktiles = K / G::kBK;
  const int peeled = ktiles % 3;
  const int first_stage = (3 - peeled) % 3;
  const int second_stage = (first_stage + 1) % 3;
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(first_stage * G::kStageFloats, l);
  advance_if(ktiles > 1);
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(second_stage * G::kStageFloats, l);
  advance_if(ktiles > 2);
  publish();
  // Outstanding LDS reads must not cross a control-flow join: the compiler may copy their
  // destination registers there, before the data has arrived.
  auto drain_reads = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < G::kBlocksM; ++i) asm volatile("" : "+v"(na[i]));
#pragma unroll
    for (int n = 0; n < G::kBlocksN; ++n) asm volatile("" : "+v"(nb[n]));
  };
  if (first_stage == 0) {
    read_a(0, 0, na);
    read_b(0, 0, nb);
    drain_reads();
  } else if (first_stage == 1) {
    read_a(1, 0, na);
    read_b(1, 0, nb);
    drain_reads();
  } else {
    read_a(2, 0, na);
    read_b(2, 0, nb);
    drain_reads();
  }

  auto slice = [&](auto stage_c, int kt) {
    constexpr int ST = decltype(stage_c)::value;
    constexpr int ST1 = (ST + 1) % G::kStages;
    constexpr int ST2 = (ST + 2) % G::kStages;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < G::kBlocksM; ++i) fa[0][i] = na[i];
#pragma unroll
    for (int n = 0; n < G::kBlocksN; ++n) fb[0][n] = nb[n];
#pragma unroll
    for (int s = 0; s < G::kSteps; ++s) {
      // the loads of slice kt+2, one per step
#pragma unroll
      for (int l = 0; l < kLoadsPerSlice; ++l)
        if (s == 1 + l) issue_one(ST2 * G::kStageFloats, l);
      if (s + 1 < G::kSteps) {
        const bool with_a = (s + 1) % 4 == 0;
        if (with_a) read_a(ST, (s + 1) / 4, fa[((s + 1) / 4) & 1]);
        read_b(ST, s + 1, fb[(s + 1) & 1]);
        // the operands of step s were requested a step ago: all but this step's reads
        if (with_a) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsA + kReadsB) : "memory");
        else asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsB) : "memory");
      } else {
        publish();  // includes lgkmcnt(0)
        read_a(ST1, 0, na);
        read_b(ST1, 0, nb);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < G::kBlocksM; ++i)
#pragma unroll
        for (int n = 0; n < G::kBlocksN; ++n)
          acc[i][n] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[(s / 4) & 1][i][s % 4], fb[s & 1][n], acc[i][n], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    advance_if(kt + 3 < ktiles);
  };
  static_assert(G::kStages == 3 && G::kSteps == 8 && 1 + kLoadsPerSlice < G::kSteps, "slice loop layout");
  if (peeled == 2) {
    slice(std::integral_constant<int, 1>{}, 0);
    drain_reads();
  }
  if (peeled >= 1) {
    slice(std::integral_constant<int, 2>{}, peeled - 1);
    drain_reads();
  }
  for (int kt = peeled; kt < ktiles; kt += 3) {
    slice(std::integral_constant<int, 0>{}, kt);
    slice(std::integral_constant<int, 1>{}, kt + 1);
    slice(std::integral_constant<int, 2>{}, kt + 2);
  }
  // LDS may be handed to another workgroup once this one retires: drain the loads.
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)

  // 16 lanes write 64 consecutive bytes of a row of C
  const int row0 = m0 + wm * G::kWaveM + 4 * g, col0 = n0 + wn * G::kWaveN + r16;
  float *c_lane = C + static_cast<int64_t>(row0) * N + col0;
#pragma unroll
  for (int i = 0; i < G::kBlocksM; ++i)
#pragma unroll
    for (int n = 0; n < G::kBlocksN; ++n)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float v = acc[i][n][e];
        if (RELU) v = relu_maxf(v);
        if (!RAGGED || (row0 + i * 16 + e < M && col0 + n * 16 < N))
          c_lane[static_cast<int64_t>(i * 16 + e) * N + n * 16] = v;
      }
}

}  // namespace kcg
