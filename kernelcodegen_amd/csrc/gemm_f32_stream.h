// Streaming variant of the direct-load matmul kernel for products with a short K and many
// tiles -- the attention scores of BatchedMatmul, S = Q.K^T with K = head dim
// (src/Frontend/Operators.cc:253-420, test/test.cc:71-90).
//
// With K = 128 a 256 x 128 tile is eight K slices of matrix work between a prologue (the
// first slices have to arrive) and 128 KiB of C to write.  One workgroup per tile pays both
// per tile, and workgroups that share a CU do not hide them for each other.  Here one
// workgroup per CU stays resident and walks a list of tiles as ONE stream of K slices:
//   * the LDS ring (four stages) runs on across tile boundaries: the loads of slice kt+3
//     are requested during slice kt, whichever tile kt+3 belongs to, so a tile's first
//     slices are already in LDS when its matrix work starts;
//   * two accumulator sets alternate between tiles: while tile t accumulates into one, the
//     other still holds tile t-1, whose C is written out a few stores per MFMA step during
//     the first slices of tile t, so neither the stores nor their latency ever stop the
//     matrix pipe, and the chip writes C at an even rate instead of in bursts;
//   * stores carry no address arithmetic: a scalar base per row residue (tile origin +
//     r * row, r < 4), a per-lane offset per group of eight rows (invariant over tiles),
//     and an immediate for the column block.
// Same tile geometry, LDS layout, swizzle and MFMA operand mapping as gemm_f32_dl_kernel
// (GemmDlTile<256, 128, 16, 4, 2>), so the products summed into an element of C and their
// order are the same as there.
//
// Requirements (checked by the launcher): M % 256 == 0, N % 128 == 0, K % 64 == 0,
// N <= 2^21, 16-byte aligned operands.  KT = 8 (K >= 128) or 4 (K = 64): the number of
// leading slices of a tile that carry the previous tile's stores.
#pragma once

#include <type_traits>

#include "gemm_dl_tile.h"
#include "kcg_common.h"

namespace kcg {

template <bool TRANS_B, int KT, bool STREAM_C, bool RELU = false>
__global__ __launch_bounds__(512, 2) void gemm_f32_stream_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N, int K,
    int tiles_m, int tiles_n, int group_m, int batch, int64_t batch_a, int64_t batch_b, int64_t batch_c) {
  using G = GemmStreamGeometry;
  constexpr int BM = G::kBM, BN = G::kBN, BK = G::kBK, WAVES_N = G::kWavesN;
  using T = GemmDlTile<BM, BN, BK, G::kWavesM, WAVES_N, TRANS_B>;
  constexpr int NS = G::kStages;
  constexpr int kStageBytes = T::kStageFloats * 4;
  static_assert(T::kTilesM == 2 && T::kTilesN == 2 && T::kSteps == 8, "wave tile of 64 x 64, 8 steps per slice");
  static_assert(KT == 4 || KT == 8, "slices that carry stores");
  static_assert(2 * kStageBytes < 65536, "two stages within reach of a ds_read offset");
  constexpr int kStoresPerSlice = G::kAccPerLane / KT;
  constexpr int kStoresPerStep = kStoresPerSlice / T::kSteps;
  constexpr int kLoadsPerSlice = T::kInstrA + T::kInstrB;
  static_assert(kLoadsPerSlice == 3, "load positions in the slice");
  extern __shared__ __align__(16) float lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;
  const int r32 = lane & 31;
  const int half = lane >> 5;
  const int ktiles = K / BK;

  // ---- the workgroup's list of tiles: every XCD owns a contiguous range of (matrix, tile)
  // items, its workgroups take them round robin, so that the tiles in flight on one XCD are
  // neighbours and share rows of A and B in its L2.
  const GemmStreamItems items = gemm_stream_items(blockIdx.x, gridDim.x, tiles_m * tiles_n * batch, kNumXcd);
  const int item_step = items.step, item_end = items.end, item_first = items.first;
  if (item_first >= item_end) return;
  using Origin = GemmStreamOrigin;
  auto decode = [&](int item) { return gemm_stream_decode(item, tiles_m, tiles_n, group_m); };

  // ---- direct loads: lane offsets are the same for every tile ----
  const int lds_base = static_cast<int>(reinterpret_cast<uintptr_t>(lds));
  unsigned oa[T::kInstrA];
  unsigned ob[T::kInstrB];
#pragma unroll
  for (int i = 0; i < T::kInstrA; ++i) {
    const int idx = (wave * T::kInstrA + i) * 256 + lane * 4;
    const int row = idx / BK;
    oa[i] = static_cast<unsigned>(row * K + 4 * (((idx % BK) / 4) ^ T::fa(row))) * 4u;
  }
#pragma unroll
  for (int i = 0; i < T::kInstrB; ++i) {
    const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;
    if (TRANS_B) {
      const int row = idx / BK;
      ob[i] = static_cast<unsigned>(row * K + 4 * (((idx % BK) / 4) ^ T::fa(row))) * 4u;
    } else {
      ob[i] = static_cast<unsigned>((idx / BN) * N + idx % BN) * 4u;
    }
  }
  const int64_t b_step = TRANS_B ? BK * 4 : static_cast<int64_t>(BK) * N * 4;

  // The load cursor: the slice the next requests fetch.  It runs kAhead slices in front of
  // the matrix work and crosses into the next tile on its own.
  const char *lga, *lgb;
  int l_item = item_first;
  int l_left = ktiles;      // slices of the cursor's tile not requested yet, the one it points at included
  Origin next_origin = decode(item_first);
  auto point_cursor = [&](const Origin &o) {
    lga = reinterpret_cast<const char *>(A + o.bz * batch_a + static_cast<int64_t>(o.m0) * K);
    lgb = reinterpret_cast<const char *>(TRANS_B ? B + o.bz * batch_b + static_cast<int64_t>(o.n0) * K
                                                 : B + o.bz * batch_b + o.n0);
  };
  point_cursor(next_origin);
  // Steps the cursor past the slice just requested.  Holds control flow: only called where no
  // LDS read is outstanding.  Past the last tile the cursor stays on its last slice, which is
  // then fetched again into stages nobody reads any more.
  auto advance_cursor = [&]() {
    if (l_left > 1) {
      --l_left;
      lga += BK * 4;
      lgb += b_step;
    } else if (l_item + item_step < item_end) {
      l_item += item_step;
      next_origin = decode(l_item);
      point_cursor(next_origin);
      l_left = ktiles;
    }
  };
  auto issue_one = [&](int stage, int l) {
    if (l < T::kInstrA) {
      const int sa = lds_base + stage * kStageBytes + (wave * T::kInstrA + l) * 1024;
      direct_load_16B(lga, oa[l], static_cast<unsigned>(sa));
    } else {
      const int i = l - T::kInstrA;
      const int sb = lds_base + stage * kStageBytes + (T::kFloatsA + (wave * T::kInstrB + i) * (TRANS_B ? 256 : T::kRunB)) * 4;
      direct_load_16B(lgb, ob[i], static_cast<unsigned>(sb));
    }
  };

  // ---- operand reads: per-lane LDS addresses for stages 0 and 2; stages 1 and 3 are reached
  // through the offset field ----
  int a_addr[2][BK / 8];
  int b_addr[2][TRANS_B ? BK / 8 : 1];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
#pragma unroll
    for (int kk = 0; kk < BK / 8; ++kk)
      a_addr[p][kk] = lds_base + 2 * p * kStageBytes +
                      ((wm * T::kWaveM + r32) * BK + 4 * ((2 * kk) ^ half ^ T::fa(r32))) * 4;
    if (TRANS_B) {
#pragma unroll
      for (int kk = 0; kk < BK / 8; ++kk)
        b_addr[p][TRANS_B ? kk : 0] = lds_base + 2 * p * kStageBytes +
                                      (T::kFloatsA + (wn * T::kWaveN + r32) * BK + 4 * ((2 * kk) ^ half ^ T::fa(r32))) * 4;
    } else {
      b_addr[p][0] = lds_base + 2 * p * kStageBytes + (T::kFloatsA + half * T::brow(4) + wn * T::kWaveN + r32) * 4;
    }
  }
  using BFrag = std::conditional_t<TRANS_B, float4_t, float>;
  float4_t fa[2][T::kTilesM];
  BFrag fb[2][T::kTilesN];
  float4_t na[T::kTilesM];
  BFrag nb[T::kTilesN];
  auto read_a = [&](auto stage_c, int kk, float4_t(&dst)[T::kTilesM]) {
    constexpr int ST = decltype(stage_c)::value;
    const int addr = a_addr[ST / 2][kk];
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i)
      asm volatile("ds_read_b128 %0, %1 offset:%2"
                   : "=v"(dst[i])
                   : "v"(addr), "n"((ST % 2) * kStageBytes + i * 32 * BK * 4)
                   : "memory");
  };
  auto read_b = [&](auto stage_c, auto step_c, BFrag(&dst)[T::kTilesN]) {
    constexpr int ST = decltype(stage_c)::value;
    constexpr int s = decltype(step_c)::value;
    if constexpr (TRANS_B) {
      const int addr = b_addr[ST / 2][s / 4];
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n)
        asm volatile("ds_read_b128 %0, %1 offset:%2"
                     : "=v"(dst[n])
                     : "v"(addr), "n"((ST % 2) * kStageBytes + n * 32 * BK * 4)
                     : "memory");
    } else {
      const int addr = b_addr[ST / 2][0];
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n)
        asm volatile("ds_read_b32 %0, %1 offset:%2"
                     : "=v"(dst[n])
                     : "v"(addr), "n"((ST % 2) * kStageBytes + (T::brow((s / 4) * 8 + s % 4) + n * 32) * 4)
                     : "memory");
    }
  };
  auto b_operand = [&](const BFrag &f, int s) {
    if constexpr (TRANS_B) return f[s % 4];
    else return f;
  };
  constexpr int kReadsA = T::kTilesM;
  constexpr int kReadsB = T::kTilesN;
  // Outstanding LDS reads must not cross a control-flow join: the compiler may copy their
  // destination registers there, before the data has arrived.
  auto drain_reads = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i) asm volatile("" : "+v"(na[i]));
#pragma unroll
    for (int n = 0; n < T::kTilesN; ++n) asm volatile("" : "+v"(nb[n]));
  };

  // ---- C stores of the previous tile ----
  // Element e of block (i, n) is C[i*32 + 8*(e/4) + 4*half + e%4][n*32 + r32] of the wave's
  // 64 x 64 sub-tile.  Address = c_row[e%4] (scalar: sub-tile row residue) + c_off[i*4 + e/4]
  // (lane: 8-row group and column) + n * 128 (immediate).
  const unsigned row_bytes = static_cast<unsigned>(N) * 4u;
  unsigned c_off[8];
#pragma unroll
  for (int g = 0; g < 8; ++g)
    c_off[g] = static_cast<unsigned>(wm * T::kWaveM + (g / 4) * 32 + 8 * (g % 4) + 4 * half) * row_bytes +
               static_cast<unsigned>(wn * T::kWaveN + r32) * 4u;
  char *c_row[4];
  auto point_stores = [&](const Origin &o) {
    char *t = reinterpret_cast<char *>(C + o.bz * batch_c + static_cast<int64_t>(o.m0) * N + o.n0);
#pragma unroll
    for (int r = 0; r < 4; ++r) c_row[r] = t + static_cast<int64_t>(r) * row_bytes;
  };
  float16_t acc[2][T::kTilesM][T::kTilesN];
  // store q (0..63) of the accumulator set P
  auto store_one = [&](auto par_c, auto q_c) {
    constexpr int P = decltype(par_c)::value;
    constexpr int q = decltype(q_c)::value;
    constexpr int i = q / 32, g = (q / 8) % 4, r = (q / 2) % 4, n = q % 2;
    // (RELU, the epilogue of the plain matmul: two VALU instructions per store in the slice
    // loop, 128 per tile and wave against the tile's K / 2 x 4 MFMAs)
    const float v = RELU ? relu_maxf(acc[P][i][n][4 * g + r]) : acc[P][i][n][4 * g + r];
    const unsigned off = c_off[i * 4 + g];
    char *const base = c_row[r];
    if (STREAM_C)
      asm volatile("global_store_dword %0, %1, %2 offset:%3 nt" ::"v"(off), "v"(v), "s"(base), "n"(n * 128) : "memory");
    else
      asm volatile("global_store_dword %0, %1, %2 offset:%3" ::"v"(off), "v"(v), "s"(base), "n"(n * 128) : "memory");
  };

  // One K slice in stage ST, accumulated into set P.  PART >= 0: the slice also issues stores
  // PART * kStoresPerSlice ... of the other set.  The barrier at its end publishes slice kt+1:
  // the wave first waits for its own loads of that slice (requested at steps 1, 3, 5 of slice
  // kt-2), which are followed in its queue by the loads of slices kt+2 and kt+3, by the
  // stores of this slice and of slice kt-1 and by those of steps 6 and 7 of slice kt-2.
  // Stores of slices that belong to the previous tile are left out of the count: waiting for
  // more than needed is safe, for less is not.
  auto slice = [&](auto stage_c, auto par_c, auto part_c) {
    constexpr int ST = decltype(stage_c)::value;
    constexpr int P = decltype(par_c)::value;
    constexpr int PART = decltype(part_c)::value;
    constexpr int ST1 = (ST + 1) % NS;
    constexpr int ST3 = (ST + G::kAhead) % NS;
    constexpr int kYounger = 2 * kLoadsPerSlice + (PART >= 0 ? kStoresPerSlice : 0) +
                             (PART >= 1 ? kStoresPerSlice : 0) + (PART >= 2 ? 2 * kStoresPerStep : 0);
    static_assert(kYounger < 64, "vmcnt immediate");
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i) fa[0][i] = na[i];
#pragma unroll
    for (int n = 0; n < T::kTilesN; ++n) fb[0][n] = nb[n];
    // (no LDS read is outstanding here: a safe place for control flow)
    advance_cursor();
    auto step = [&](auto s_c) {
      constexpr int s = decltype(s_c)::value;
      if constexpr (PART >= 0) {
        store_one(std::integral_constant<int, 1 - P>{}, std::integral_constant<int, PART * kStoresPerSlice + s * kStoresPerStep>{});
        if constexpr (kStoresPerStep == 2)
          store_one(std::integral_constant<int, 1 - P>{}, std::integral_constant<int, PART * kStoresPerSlice + s * kStoresPerStep + 1>{});
      }
      if constexpr (s == 1) issue_one(ST3, 0);
      if constexpr (s == 3) issue_one(ST3, 1);
      if constexpr (s == 5) issue_one(ST3, 2);
      if constexpr (s + 1 < T::kSteps) {
        constexpr bool with_a = (s + 1) % 4 == 0;
        if constexpr (with_a) read_a(stage_c, (s + 1) / 4, fa[((s + 1) / 4) & 1]);
        if constexpr (TRANS_B) {
          if constexpr (with_a) read_b(stage_c, std::integral_constant<int, s + 1>{}, fb[((s + 1) / 4) & 1]);
          if constexpr (s % 4 == 0 && s > 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        } else {
          read_b(stage_c, std::integral_constant<int, s + 1>{}, fb[(s + 1) & 1]);
          if constexpr (with_a) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsA + kReadsB) : "memory");
          else asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsB) : "memory");
        }
      } else {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(kYounger) : "memory");
        read_a(std::integral_constant<int, ST1>{}, 0, na);
        read_b(std::integral_constant<int, ST1>{}, std::integral_constant<int, 0>{}, nb);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
        for (int n = 0; n < T::kTilesN; ++n)
          acc[P][i][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              fa[(s / 4) & 1][i][s % 4], b_operand(fb[TRANS_B ? (s / 4) & 1 : s & 1][n], s), acc[P][i][n], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    };
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
    step(std::integral_constant<int, 2>{});
    step(std::integral_constant<int, 3>{});
    step(std::integral_constant<int, 4>{});
    step(std::integral_constant<int, 5>{});
    step(std::integral_constant<int, 6>{});
    step(std::integral_constant<int, 7>{});
  };

  // One tile into accumulator set P; HAS_PREV: the other set holds the previous tile, whose
  // stores ride on the first KT slices.
  auto tile = [&](auto par_c, auto has_prev_c) {
    constexpr int P = decltype(par_c)::value;
    constexpr bool HAS_PREV = decltype(has_prev_c)::value;
    using S0 = std::integral_constant<int, 0>;
    using S1 = std::integral_constant<int, 1>;
    using S2 = std::integral_constant<int, 2>;
    using S3 = std::integral_constant<int, 3>;
    using None = std::integral_constant<int, -1>;
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[P][i][n][e] = 0.0f;
    slice(S0{}, par_c, std::integral_constant<int, HAS_PREV ? 0 : -1>{});
    slice(S1{}, par_c, std::integral_constant<int, HAS_PREV ? 1 : -1>{});
    slice(S2{}, par_c, std::integral_constant<int, HAS_PREV ? 2 : -1>{});
    slice(S3{}, par_c, std::integral_constant<int, HAS_PREV ? 3 : -1>{});
    if constexpr (KT == 8) {
      slice(S0{}, par_c, std::integral_constant<int, HAS_PREV ? 4 : -1>{});
      slice(S1{}, par_c, std::integral_constant<int, HAS_PREV ? 5 : -1>{});
      slice(S2{}, par_c, std::integral_constant<int, HAS_PREV ? 6 : -1>{});
      slice(S3{}, par_c, std::integral_constant<int, HAS_PREV ? 7 : -1>{});
    }
    drain_reads();
    for (int kt = KT; kt < ktiles; kt += NS) {
      slice(S0{}, par_c, None{});
      slice(S1{}, par_c, None{});
      slice(S2{}, par_c, None{});
      slice(S3{}, par_c, None{});
      drain_reads();
    }
  };

  // ---- prologue: the first kAhead slices of the first tile ----
  Origin cur = next_origin;
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(0, l);
  advance_cursor();
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(1, l);
  advance_cursor();
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(2, l);
  // (the cursor is advanced past this slice by the first slice of the stream)
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" ::"n"(2 * kLoadsPerSlice) : "memory");
  read_a(std::integral_constant<int, 0>{}, 0, na);
  read_b(std::integral_constant<int, 0>{}, std::integral_constant<int, 0>{}, nb);
  drain_reads();

  // ---- the stream of tiles, two per round (one per accumulator set) ----
  int c_item = item_first;
  tile(std::integral_constant<int, 0>{}, std::false_type{});
  int last_set = 0;
  for (;;) {
    point_stores(cur);
    c_item += item_step;
    if (c_item >= item_end) break;
    cur = next_origin;   // the cursor entered this tile during the previous one and cannot leave it before the tile starts
    tile(std::integral_constant<int, 1>{}, std::true_type{});
    last_set = 1;
    point_stores(cur);
    c_item += item_step;
    if (c_item >= item_end) break;
    cur = next_origin;
    tile(std::integral_constant<int, 0>{}, std::true_type{});
    last_set = 0;
  }
  // LDS may be handed to another workgroup once this one retires: drain the loads.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  // ---- the last tile's C ----
  auto flush = [&](auto par_c) {
    auto go = [&](auto q_c, auto &&self) {
      constexpr int q = decltype(q_c)::value;
      if constexpr (q < G::kAccPerLane) {
        store_one(par_c, q_c);
        self(std::integral_constant<int, q + 1>{}, self);
      }
    };
    go(std::integral_constant<int, 0>{}, go);
  };
  if (last_set == 0) flush(std::integral_constant<int, 0>{});
  else flush(std::integral_constant<int, 1>{});
}

}  // namespace kcg
