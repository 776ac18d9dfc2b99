// Tiled fp32 matmul for gfx950 (MI355X), with an optional fused ReLU epilogue.
//
// Stands in for the kernel the reference generates from
// MatmulOptimizer::applyOptimzer (src/Optimizer/Optimizer.cc:383-548): a
// BLOCK_SIZE_M x BLOCK_SIZE_N tile of C per workgroup, K walked in BLOCK_SIZE_K
// slices that are staged in double-buffered shared memory, the next slice
// prefetched from global memory into registers while the current one is
// consumed (Rewriter::pipeline, src/Optimizer/Rewriter.cc:809-1180).  What is
// different is everything below the schedule: wave64, the per-thread 8x8 FMA
// tile is replaced by a per-wave tile of v_mfma_f32_32x32x2_f32 blocks, the
// rasterisation is XCD aware and uses GROUP_SIZE_M (which the reference sets,
// include/KernelCodeGen.h:35, and never reads).
//
// Data layout in LDS (floats):
//   As[buf][BM][BK+4]   A tile as in global memory (row = m, k contiguous); the
//                       +4 pad keeps 16-byte alignment and makes the per-lane
//                       ds_read_b128 of 16 consecutive rows hit 64 distinct banks.
//   Bs[buf][BK][BN+8]   B tile as in global memory (row = k, n contiguous); the
//                       +8 pad shifts rows 4 apart by 32 banks so the two halves
//                       of a wave (which read rows k and k+4) do not collide.
//
// MFMA operand mapping (v_mfma_f32_32x32x2_f32, lane l, r = l % 32, h = l / 32):
//   A operand: A[row r][k = h]      B operand: B[k = h][col r]
//   D: 16 floats, element e is C[8*(e/4) + 4*h + e%4][r].
// Within an 8-wide K group half h of the wave takes k = 4h..4h+3 (one b128 LDS
// read of A) and the j-th MFMA of the group consumes k = 4h + j from both
// operands.  The set of products summed into each C element is unchanged; only
// their order differs from the ascending-k order of the reference nest.
#include <cstring>
#include <type_traits>

#include "gemm_dl_tile.h"
#include "gemm_f32_stream.h"
#include "gemm_f32_t96.h"
#include "kcg_common.h"

namespace kcg {

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
struct GemmTile {
  static constexpr int kThreads = WAVES_M * WAVES_N * kWaveSize;
  static constexpr int kWaveM = BM / WAVES_M;
  static constexpr int kWaveN = BN / WAVES_N;
  static constexpr int kTilesM = kWaveM / 32;
  static constexpr int kTilesN = kWaveN / 32;
  static constexpr int kPitchA = BK + 4;
  static constexpr int kPitchB = BN + 8;
  static constexpr int kFloatsA = BM * kPitchA;
  static constexpr int kFloatsB = BK * kPitchB;
  static constexpr int kLdsBytes = 2 * (kFloatsA + kFloatsB) * 4;
  static constexpr int kLoadsA = BM * BK / 4 / kThreads;  // float4 per thread
  static constexpr int kLoadsB = BK * BN / 4 / kThreads;
  static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile");
  static_assert(BK % 8 == 0, "K slice is consumed in groups of 8");
  static_assert((BM * BK / 4) % kThreads == 0 && (BK * BN / 4) % kThreads == 0, "load split");
};

// Four consecutive floats from an address that is only known to be 4-byte aligned.
__device__ __forceinline__ float4_t load4_dword_aligned(const float *p) {
  struct __attribute__((packed, aligned(4))) Quad {
    float v[4];
  };
  const Quad q = *reinterpret_cast<const Quad *>(p);
  return float4_t{q.v[0], q.v[1], q.v[2], q.v[3]};
}

// FULL: M % BM == 0, N % BN == 0, K % BK == 0 and 16-byte aligned rows, so that
// no bounds checks are needed and every global access is a dwordx4.  Otherwise
// tiles inside C still take vector loads for all but the last, partial K slice.

// BUFS: copies of the K-slice tiles in LDS.  2: the pipelined schedule described below.  1: the
// staged schedule that precedes Rewriter::pipeline in the reference's recipe (one copy of each
// shared tile: the next slice waits in registers until every wave has finished the current one,
// two barriers per slice) -- built so that a nest staged that far runs as it is written.

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RELU, bool FULL, int MIN_WAVES, int BUFS = 2>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWaveSize, MIN_WAVES) void gemm_f32_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N,
    int K, int tiles_m, int tiles_n, int group_m) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N>;
  static_assert(BUFS == 1 || BUFS == 2, "LDS copies");
  extern __shared__ __align__(16) float lds[];
  float *As = lds;                        // [BUFS][BM][kPitchA]
  float *Bs = lds + BUFS * T::kFloatsA;   // [BUFS][BK][kPitchB]

  // ---- workgroup -> C tile (XCD-contiguous, then GROUP_SIZE_M swizzle) ----
  const int logical = xcd_contiguous_id(blockIdx.x, tiles_m * tiles_n);
  const int width = group_m * tiles_n;
  const int group = logical / width;
  const int first_m = group * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int in_group = logical - group * width;
  const int tile_m = first_m + in_group % gsz;
  const int tile_n = in_group / gsz;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;
  const int r32 = lane & 31;
  const int half = lane >> 5;

  float16_t acc[T::kTilesM][T::kTilesN];
#pragma unroll
  for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
    for (int j = 0; j < T::kTilesN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  float4_t ra[T::kLoadsA];
  float4_t rb[T::kLoadsB];
  // ragged problems: a tile that lies wholly inside C needs bounds checks only in the
  // last, partial K slice
  const bool tile_inside = (m0 + BM <= M) && (n0 + BN <= N);

  // Transfer g of a K slice: g < kLoadsA moves one float4 of A per thread, the
  // rest one float4 of B.  load_one: global -> registers; store_one: registers -> LDS.
  constexpr int kTransfers = T::kLoadsA + T::kLoadsB;
  auto load_one = [&](int g, int k0) {
    if (g < T::kLoadsA) {
      const int idx = tid + g * T::kThreads;
      const int row = idx / (BK / 4);
      const int c4 = idx % (BK / 4);
      const int64_t gr = m0 + row;
      const int gk = k0 + c4 * 4;
      if (FULL) {
        ra[g] = *reinterpret_cast<const float4_t *>(A + gr * K + gk);
      } else if (tile_inside && k0 + BK <= K) {
        // interior tile of a ragged problem: no element is out of range, but rows need
        // not start on a 16-byte boundary
        ra[g] = load4_dword_aligned(A + gr * K + gk);
      } else {
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (gr < M) {
          const float *p = A + gr * K;
          if (gk + 3 < K) {
            v = load4_dword_aligned(p + gk);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (gk + e < K) v[e] = p[gk + e];
          }
        }
        ra[g] = v;
      }
    } else {
      const int i = g - T::kLoadsA;
      const int idx = tid + i * T::kThreads;
      const int row = idx / (BN / 4);
      const int c4 = idx % (BN / 4);
      const int64_t gk = k0 + row;
      const int gn = n0 + c4 * 4;
      if (FULL) {
        rb[i] = *reinterpret_cast<const float4_t *>(B + gk * N + gn);
      } else if (tile_inside && k0 + BK <= K) {
        rb[i] = load4_dword_aligned(B + gk * N + gn);
      } else {
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (gk < K) {
          const float *p = B + gk * N;
          if (gn + 3 < N) {
            v = load4_dword_aligned(p + gn);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (gn + e < N) v[e] = p[gn + e];
          }
        }
        rb[i] = v;
      }
    }
  };
  auto store_one = [&](int g, int buf) {
    if (g < T::kLoadsA) {
      const int idx = tid + g * T::kThreads;
      const int row = idx / (BK / 4);
      const int c4 = idx % (BK / 4);
      *reinterpret_cast<float4_t *>(As + buf * T::kFloatsA + row * T::kPitchA + c4 * 4) = ra[g];
    } else {
      const int i = g - T::kLoadsA;
      const int idx = tid + i * T::kThreads;
      const int row = idx / (BN / 4);
      const int c4 = idx % (BN / 4);
      *reinterpret_cast<float4_t *>(Bs + buf * T::kFloatsB + row * T::kPitchB + c4 * 4) = rb[i];
    }
  };
  // ---- main loop --------------------------------------------------------
  // One K slice is consumed in kSteps steps of kTilesM*kTilesN MFMAs; step s
  // takes k = 8*(s/4) + 4*half + s%4.  The operands of step s+1 are read from
  // LDS before the MFMAs of step s are issued, so the LDS latency sits under
  // the matrix pipe.  Slice kt+1, which arrived in registers during slice
  // kt-1, is written to the other LDS buffer at the top of slice kt and the
  // registers are refilled with slice kt+2.  The one barrier per slice comes
  // before the LAST step of slice kt: at that point every wave holds its last
  // operands of slice kt in registers, so the barrier both publishes slice
  // kt+1 and releases buffer `cur` for the writes of the next iteration, and
  // the first operands of slice kt+1 are read while the last MFMAs of slice kt
  // still run.
  constexpr int kSteps = BK / 2;
  const float *a_base = As + (wm * T::kWaveM + r32) * T::kPitchA + 4 * half;
  const float *b_base = Bs + (4 * half) * T::kPitchB + wn * T::kWaveN + r32;
  float4_t fa[2][T::kTilesM];
  float fb[2][T::kTilesN];
  float4_t na[T::kTilesM];
  float nb[T::kTilesN];

  const int ktiles = (K + BK - 1) / BK;
#pragma unroll
  for (int g = 0; g < kTransfers; ++g) load_one(g, 0);
#pragma unroll
  for (int g = 0; g < kTransfers; ++g) store_one(g, 0);
  if (BUFS == 2 && ktiles > 1) {
#pragma unroll
    for (int g = 0; g < kTransfers; ++g) load_one(g, BK);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < T::kTilesM; ++i)
    na[i] = *reinterpret_cast<const float4_t *>(a_base + i * 32 * T::kPitchA);
#pragma unroll
  for (int n = 0; n < T::kTilesN; ++n) nb[n] = b_base[n * 32];

  for (int kt = 0; kt < ktiles; ++kt) {
    const int cur = BUFS == 2 ? (kt & 1) : 0;
    const float *as = a_base + cur * T::kFloatsA;
    const float *bs = b_base + cur * T::kFloatsB;
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i) fa[0][i] = na[i];
#pragma unroll
    for (int n = 0; n < T::kTilesN; ++n) fb[0][n] = nb[n];
    if (BUFS == 2) {
      if (kt + 1 < ktiles) {
#pragma unroll
        for (int g = 0; g < kTransfers; ++g) store_one(g, cur ^ 1);
      }
      if (kt + 2 < ktiles) {
#pragma unroll
        for (int g = 0; g < kTransfers; ++g) load_one(g, (kt + 2) * BK);
      }
    } else if (kt + 1 < ktiles) {
      // one copy: the next slice travels to registers while this one is consumed
#pragma unroll
      for (int g = 0; g < kTransfers; ++g) load_one(g, (kt + 1) * BK);
    }
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      if (s + 1 < kSteps) {
        const int s1 = s + 1;
        if (s1 % 4 == 0) {
#pragma unroll
          for (int i = 0; i < T::kTilesM; ++i)
            fa[(s1 / 4) & 1][i] =
                *reinterpret_cast<const float4_t *>(as + i * 32 * T::kPitchA + (s1 / 4) * 8);
        }
#pragma unroll
        for (int n = 0; n < T::kTilesN; ++n)
          fb[s1 & 1][n] = bs[((s1 / 4) * 8 + s1 % 4) * T::kPitchB + n * 32];
      } else if (BUFS == 2) {
        __syncthreads();
        if (kt + 1 < ktiles) {
          const float *as1 = a_base + (cur ^ 1) * T::kFloatsA;
          const float *bs1 = b_base + (cur ^ 1) * T::kFloatsB;
#pragma unroll
          for (int i = 0; i < T::kTilesM; ++i)
            na[i] = *reinterpret_cast<const float4_t *>(as1 + i * 32 * T::kPitchA);
#pragma unroll
          for (int n = 0; n < T::kTilesN; ++n) nb[n] = bs1[n * 32];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
        for (int n = 0; n < T::kTilesN; ++n)
          acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[(s / 4) & 1][i][s % 4], fb[s & 1][n],
                                                           acc[i][n], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (BUFS == 1 && kt + 1 < ktiles) {
      __syncthreads();   // every wave holds its last operands of slice kt
#pragma unroll
      for (int g = 0; g < kTransfers; ++g) store_one(g, 0);
      __syncthreads();   // slice kt+1 is published
#pragma unroll
      for (int i = 0; i < T::kTilesM; ++i)
        na[i] = *reinterpret_cast<const float4_t *>(a_base + i * 32 * T::kPitchA);
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n) nb[n] = b_base[n * 32];
    }
  }

  // ---- epilogue + writeback: per store, lanes 0-31 and 32-63 each cover one
  // 128-byte row segment of C ----
#pragma unroll
  for (int i = 0; i < T::kTilesM; ++i) {
#pragma unroll
    for (int n = 0; n < T::kTilesN; ++n) {
      const int col = n0 + wn * T::kWaveN + n * 32 + r32;
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int row = m0 + wm * T::kWaveM + i * 32 + 8 * (e / 4) + 4 * half + (e % 4);
        float v = acc[i][n][e];
        if (RELU) v = relu_maxf(v);
        if (FULL || (row < M && col < N)) C[static_cast<int64_t>(row) * N + col] = v;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Full-tile kernel with direct global->LDS loads.
//
// For problems whose sizes divide the tile the K slices never pass through
// registers: global_load_lds_dwordx4 writes lane l's 16 bytes at (wave-uniform
// LDS base) + 16*l, so each instruction fills a 1 KiB run of LDS and each lane
// is free to fetch whichever global chunk belongs there.  Rows inside a run
// cannot be padded; bank conflicts are avoided like this instead:
//   As[stage][BM][BK]   16-byte chunk c of row m is stored at chunk c ^ fa(m),
//                       fa(m) = ((m / rows-per-128B) % chunks-per-row) ^ ((m/8) & 1):
//                       any 8 consecutive rows fill a 128-byte window and any 16
//                       a 256-byte window without sharing a slot, so the
//                       ds_read_b128 of one chunk column is conflict free.
//   Bs[stage][BK][BN]   rows as in global memory, 1 KiB runs (256/BN rows each)
//                       spaced 1 KiB + 8192/BN bytes apart, which puts rows k and
//                       k+4 (read together by the two halves of a wave) 128 bytes
//                       apart modulo 256.
// Three LDS stages: slice kt+2 is requested at the top of slice kt and has two
// slices of MFMA time to arrive; a wave only waits for its own loads of slice
// kt+1 (vmcnt) right before the barrier that publishes them.
// TRANS_B: B is given as [N][K] (the 'T' operand of BatchedMatmul, Q.K^T): its tile then
// has the shape and the LDS layout of the A tile, rows = n.
// RAGGED: M, N need not divide the tile and K need not divide BK (K and N are multiples of
// 4 and K >= BK).  Rows of A at and beyond M and 16-byte column chunks of B at and beyond N
// only feed elements of C that are never stored, so their lanes simply fetch the last
// valid row / chunk instead (a loop-invariant change of the lane offsets).  The last,
// partial K slice is the one place that needs zeros: its direct loads re-fetch the last
// full slice (never out of range) and the stage is then rewritten through registers, once
// per tile.
// blockIdx.y is the batch index of BatchedMatmul (src/Frontend/Operators.cc:253-420); the
// three strides are 0 for the plain matmul.
// SPLIT (K in whole slices): the launch holds split_full whole tiles followed by the remaining
// tiles cut along K into split_parts pieces, one workgroup per piece.  A piece accumulates its
// K / split_parts slices and writes the raw 64-byte-aligned BM x BN partial tile to
// ws[(tile - split_full) * split_parts + piece] (no epilogue); gemm_split_reduce_kernel adds
// the pieces up.  Whole tiles run exactly as without SPLIT.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RELU, bool RAGGED, bool TRANS_B, bool SPLIT>
__device__ __forceinline__ void gemm_dl_body(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N,
    int K, int tiles_m, int tiles_n, int group_m, int64_t batch_a, int64_t batch_b, int64_t batch_c,
    int split_full, int split_parts, float *__restrict__ ws) {
  using T = GemmDlTile<BM, BN, BK, WAVES_M, WAVES_N, TRANS_B>;
  static_assert(!(SPLIT && TRANS_B), "K-split pieces exist for row-major B only");
  extern __shared__ __align__(16) float lds[];
  A += blockIdx.y * batch_a;
  B += blockIdx.y * batch_b;
  C += blockIdx.y * batch_c;

  // (SPLIT: the whole tiles come first in the grid and the pieces after them, each set
  // spread over the XCDs by itself -- split_full is a multiple of the XCD count -- so that
  // every XCD, and every CU of it, gets the same mix)
  int logical, piece = 0;
  bool partial = false;
  if (SPLIT && static_cast<int>(blockIdx.x) >= split_full) {
    const int q = xcd_contiguous_id(blockIdx.x - split_full, static_cast<int>(gridDim.x) - split_full);
    logical = split_full + q / split_parts;
    piece = q - (q / split_parts) * split_parts;
    partial = true;
  } else {
    logical = xcd_contiguous_id(blockIdx.x, SPLIT ? split_full : tiles_m * tiles_n);
  }
  const int width = group_m * tiles_n;
  const int group = logical / width;
  const int first_m = group * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int in_group = logical - group * width;
  const int tile_m = first_m + in_group % gsz;
  const int tile_n = in_group / gsz;
  const int m0 = tile_m * BM;
  const int n0 = tile_n * BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N;
  const int wn = wave % WAVES_N;
  const int r32 = lane & 31;
  const int half = lane >> 5;

  float16_t acc[T::kTilesM][T::kTilesN];
#pragma unroll
  for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
    for (int j = 0; j < T::kTilesN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // ---- direct loads: uniform slice base + per-lane 32-bit byte offsets ----
  const int lds_base = static_cast<int>(reinterpret_cast<uintptr_t>(lds));  // LDS byte address
  unsigned oa[T::kInstrA];
  unsigned ob[T::kInstrB];
#pragma unroll
  for (int i = 0; i < T::kInstrA; ++i) {
    const int idx = (wave * T::kInstrA + i) * 256 + lane * 4;  // float index in the LDS A tile
    const int row = idx / BK;
    const int c_log = ((idx % BK) / 4) ^ T::fa(row);
    const int grow = RAGGED ? (row < M - m0 ? row : M - m0 - 1) : row;
    oa[i] = static_cast<unsigned>(grow * K + 4 * c_log) * 4u;
  }
#pragma unroll
  for (int i = 0; i < T::kInstrB; ++i) {
    const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;  // float index in the unpadded B tile
    if (TRANS_B) {
      const int row = idx / BK;
      const int c_log = ((idx % BK) / 4) ^ T::fa(row);
      const int grow = RAGGED ? (row < N - n0 ? row : N - n0 - 1) : row;
      ob[i] = static_cast<unsigned>(grow * K + 4 * c_log) * 4u;
    } else {
      const int col = idx % BN;
      const int gcol = RAGGED ? (col < N - n0 ? col : N - n0 - 4) : col;
      ob[i] = static_cast<unsigned>((idx / BN) * N + gcol) * 4u;
    }
  }
  const char *ga = reinterpret_cast<const char *>(A + static_cast<int64_t>(m0) * K);
  const char *gb = reinterpret_cast<const char *>(TRANS_B ? B + static_cast<int64_t>(n0) * K : B + n0);
  const int64_t b_step = TRANS_B ? BK * 4 : static_cast<int64_t>(BK) * N * 4;
  // slices of this workgroup: all of K, or one piece of it
  const int my_slices = (SPLIT && partial) ? (K / BK) / split_parts : K / BK;
  if (SPLIT && partial) {
    ga += static_cast<int64_t>(piece) * my_slices * (BK * 4);
    gb += static_cast<int64_t>(piece) * my_slices * b_step;
  }
  constexpr int kLoadsPerSlice = T::kInstrA + T::kInstrB;
  // load l of the slice at (ga, gb) into the stage at float offset stage_off
  auto issue_one = [&](int stage_off, int l) {
    if (l < T::kInstrA) {
      const int sa = lds_base + (stage_off + (wave * T::kInstrA + l) * 256) * 4;
      direct_load_16B(ga, oa[l], static_cast<unsigned>(sa));
    } else {
      const int i = l - T::kInstrA;
      const int sb = lds_base + (stage_off + T::kFloatsA + (wave * T::kInstrB + i) * (TRANS_B ? 256 : T::kRunB)) * 4;
      direct_load_16B(gb, ob[i], static_cast<unsigned>(sb));
    }
  };
  // The loop body is kept free of branches (after a join the compiler's wait-count
  // tracking turns imprecise and drains the operand prefetch): past the last
  // slice the pointers simply stop advancing and the final slice is fetched again
  // into a stage nobody reads any more.
  auto advance_if = [&](bool cond) {
    ga += cond ? BK * 4 : 0;
    gb += cond ? b_step : 0;
  };

  // ---- operand reads ----
  // While a direct load is in flight the compiler treats the LDS counter as
  // unordered and would wait for ALL outstanding LDS reads (lgkmcnt(0)) before
  // every MFMA group, which undoes the operand prefetch.  The reads are therefore
  // issued from inline assembly, invisible to that bookkeeping, and waited for by
  // hand: LDS reads return in order, so "all but the newest n" is lgkmcnt(n).
  // Per-lane LDS byte addresses, one set per stage (swizzle folded in): the slice loop is
  // unrolled over the three stages so that no address arithmetic is left in it -- on this
  // chip every VALU instruction between fp32 MFMAs is paid for in matrix time.
  int a_addr[T::kStages][BK / 8];
  int b_addr[T::kStages][TRANS_B ? BK / 8 : 1];
#pragma unroll
  for (int st = 0; st < T::kStages; ++st) {
#pragma unroll
    for (int kk = 0; kk < BK / 8; ++kk)
      a_addr[st][kk] = lds_base + (st * T::kStageFloats + (wm * T::kWaveM + r32) * BK +
                                   4 * ((2 * kk) ^ half ^ T::fa(r32))) * 4;
    if (TRANS_B) {
#pragma unroll
      for (int kk = 0; kk < BK / 8; ++kk)
        b_addr[st][TRANS_B ? kk : 0] = lds_base + (st * T::kStageFloats + T::kFloatsA + (wn * T::kWaveN + r32) * BK +
                                                   4 * ((2 * kk) ^ half ^ T::fa(r32))) * 4;
    } else {
      b_addr[st][0] = lds_base + (st * T::kStageFloats + T::kFloatsA + half * T::brow(4) + wn * T::kWaveN + r32) * 4;
    }
  }

  // B operand registers: one float per step, or (TRANS_B) one float4 per group of four steps
  using BFrag = std::conditional_t<TRANS_B, float4_t, float>;
  float4_t fa[2][T::kTilesM];
  BFrag fb[2][T::kTilesN];
  float4_t na[T::kTilesM];
  BFrag nb[T::kTilesN];
  auto read_a = [&](int stage, int kk, float4_t(&dst)[T::kTilesM]) {
    const int addr = a_addr[stage][kk];
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i)
      asm volatile("ds_read_b128 %0, %1 offset:%2"
                   : "=v"(dst[i])
                   : "v"(addr), "n"(i * 32 * BK * 4)
                   : "memory");
  };
  // operands of step s; with TRANS_B only every fourth step reads (the whole group of four)
  auto read_b = [&](int stage, int s, BFrag(&dst)[T::kTilesN]) {
    if constexpr (TRANS_B) {
      const int addr = b_addr[stage][s / 4];
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n)
        asm volatile("ds_read_b128 %0, %1 offset:%2"
                     : "=v"(dst[n])
                     : "v"(addr), "n"(n * 32 * BK * 4)
                     : "memory");
    } else {
      const int addr = b_addr[stage][0];
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n)
        asm volatile("ds_read_b32 %0, %1 offset:%2"
                     : "=v"(dst[n])
                     : "v"(addr), "n"((T::brow((s / 4) * 8 + s % 4) + n * 32) * 4)
                     : "memory");
    }
  };
  auto b_operand = [&](const BFrag &f, int s) {
    if constexpr (TRANS_B) return f[s % 4];
    else return f;
  };
  constexpr int kReadsA = T::kTilesM;  // LDS instructions per read_a / read_b
  constexpr int kReadsB = T::kTilesN;
  static_assert((T::brow(BK - 1) + BN) * 4 < 65536 && BM * BK * 4 < 65536 && BN * BK * 4 < 65536,
                "ds_read offset field");

  // Publishes the slice requested before the newest one: the wave waits for its
  // own loads of that slice and for its LDS reads, then joins the barrier.  A bare
  // s_barrier is used because __syncthreads() carries a release fence for which
  // the compiler drains every outstanding load (vmcnt(0)), including the slice
  // that was only just requested.
  auto publish = [&]() {
    // s_waitcnt vmcnt(kLoadsPerSlice) lgkmcnt(0), as the builtin so that the compiler's
    // own wait-count bookkeeping sees it (encoding: vmcnt [3:0], expcnt [6:4], lgkmcnt [11:8])
    static_assert(kLoadsPerSlice < 16, "vmcnt immediate");
    __builtin_amdgcn_s_waitcnt(kLoadsPerSlice | 0x70);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };

  const int kfull = my_slices;                   // slices the direct loads may fetch
  // (SPLIT: K is a whole number of slices, the host sees to that; RAGGED then means edges
  // in M and N only)
  const int ktiles = (RAGGED && !SPLIT) ? (K + BK - 1) / BK : kfull;
  // The last, partial slice (RAGGED): rewritten through registers with zeros beyond K.
  // Lane L of load l owns the same 16 bytes of the stage as in the direct load.
  auto rewrite_tail = [&](int stage_off) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the stage's own direct loads have landed
    const int k0 = kfull * BK;
#pragma unroll
    for (int l = 0; l < kLoadsPerSlice; ++l) {
      float4_t v = {0.f, 0.f, 0.f, 0.f};
      if (l < T::kInstrA) {
        const int idx = (wave * T::kInstrA + l) * 256 + lane * 4;
        const int row = idx / BK;
        const int k = k0 + 4 * (((idx % BK) / 4) ^ T::fa(row));
        const int grow = m0 + (row < M - m0 ? row : M - m0 - 1);
        if (k < K) v = *reinterpret_cast<const float4_t *>(A + static_cast<int64_t>(grow) * K + k);
        *reinterpret_cast<float4_t *>(lds + stage_off + idx) = v;
      } else {
        const int i = l - T::kInstrA;
        const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;
        if (TRANS_B) {
          const int row = idx / BK;
          const int k = k0 + 4 * (((idx % BK) / 4) ^ T::fa(row));
          const int grow = n0 + (row < N - n0 ? row : N - n0 - 1);
          if (k < K) v = *reinterpret_cast<const float4_t *>(B + static_cast<int64_t>(grow) * K + k);
          *reinterpret_cast<float4_t *>(lds + stage_off + T::kFloatsA + idx) = v;
        } else {
          const int krow = k0 + idx / BN;
          const int col = idx % BN;
          const int gcol = n0 + (col < N - n0 ? col : N - n0 - 4);
          if (krow < K) v = *reinterpret_cast<const float4_t *>(B + static_cast<int64_t>(krow) * N + gcol);
          *reinterpret_cast<float4_t *>(lds + stage_off + T::kFloatsA + (wave * T::kInstrB + i) * T::kRunB +
                                        lane * 4) = v;
        }
      }
    }
  };
  // The slice loop runs whole groups of three slices (stages 0, 1, 2); the ktiles % 3
  // slices in front of the first group use the last stages of the ring, so that the
  // first group starts at stage 0.
  const int peeled = ktiles % 3;
  const int first_stage = (3 - peeled) % 3;
  const int second_stage = (first_stage + 1) % 3;
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(first_stage * T::kStageFloats, l);
  advance_if(kfull > 1);
#pragma unroll
  for (int l = 0; l < kLoadsPerSlice; ++l) issue_one(second_stage * T::kStageFloats, l);
  advance_if(kfull > 2);
  publish();
  // Outstanding LDS reads must not cross a control-flow join: the compiler may copy their
  // destination registers there, before the data has arrived.
  auto drain_reads = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i) asm volatile("" : "+v"(na[i]));
#pragma unroll
    for (int n = 0; n < T::kTilesN; ++n) asm volatile("" : "+v"(nb[n]));
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

  // One K slice held in stage ST (a compile-time constant: all LDS addresses and the
  // direct-load targets are immediates or loop-invariant registers).
  auto slice = [&](auto stage_c, int kt) {
    constexpr int ST = decltype(stage_c)::value;
    constexpr int ST1 = (ST + 1) % T::kStages;
    constexpr int ST2 = (ST + 2) % T::kStages;
    // the reads of step 0, issued after the previous barrier, are the newest in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i) fa[0][i] = na[i];
#pragma unroll
    for (int n = 0; n < T::kTilesN; ++n) fb[0][n] = nb[n];
    // (no LDS read is outstanding here: a safe place for control flow)
    if (RAGGED && kfull != ktiles && kt == ktiles - 2) rewrite_tail(ST1 * T::kStageFloats);
#pragma unroll
    for (int s = 0; s < T::kSteps; ++s) {
      // The loads of slice kt+2 are spread over the steps: requests issued in one
      // burst by every wave of the CU queue up at the address unit.
#pragma unroll
      for (int l = 0; l < kLoadsPerSlice; ++l)
        if (s == 1 + l * (T::kSteps - 2) / kLoadsPerSlice) issue_one(ST2 * T::kStageFloats, l);
      if (s + 1 < T::kSteps) {
        const bool with_a = (s + 1) % 4 == 0;
        if (with_a) read_a(ST, (s + 1) / 4, fa[((s + 1) / 4) & 1]);
        if constexpr (TRANS_B) {
          // both operands come in groups of four steps, requested one step before the group
          if (with_a) read_b(ST, s + 1, fb[((s + 1) / 4) & 1]);
          if (s % 4 == 0 && s > 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        } else {
          read_b(ST, s + 1, fb[(s + 1) & 1]);
          // operands of step s were requested one step ago: all but this step's reads
          if (with_a) asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsA + kReadsB) : "memory");
          else asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(kReadsB) : "memory");
        }
      } else {
        publish();  // includes lgkmcnt(0): the operands of the last step are in
        read_a(ST1, 0, na);
        read_b(ST1, 0, nb);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
        for (int n = 0; n < T::kTilesN; ++n)
          acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(
              fa[(s / 4) & 1][i][s % 4], b_operand(fb[TRANS_B ? (s / 4) & 1 : s & 1][n], s), acc[i][n], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    advance_if(kt + 3 < kfull);
  };
  static_assert(T::kStages == 3, "the slice loop is unrolled over three stages");
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
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0), lgkmcnt/expcnt untouched

  // A C that does not fit the 256 MiB last-level cache is streamed past it (non-temporal
  // stores): with a short K the write of C is a large part of the run time.
  // Addresses are (uniform 64-bit tile origin) + (32-bit byte offset inside the tile): one
  // 32-bit add per store instead of a 64-bit multiply-add -- VALU work that the short-K
  // problems (attention scores: K = 128) would otherwise pay for in matrix time.  The
  // offset stays below 2^32 because N < 2^22 on this path.
  const bool to_ws = SPLIT && partial;
  char *c_tile = to_ws ? reinterpret_cast<char *>(ws + (static_cast<int64_t>(logical - split_full) * split_parts + piece) * (BM * BN))
                       : reinterpret_cast<char *>(C + static_cast<int64_t>(m0) * N + n0);
  const unsigned ldc = to_ws ? static_cast<unsigned>(BN) : static_cast<unsigned>(N);
  const unsigned lane_off = (static_cast<unsigned>(wm * T::kWaveM + 4 * half) * ldc +
                             static_cast<unsigned>(wn * T::kWaveN + r32)) * 4u;
  const unsigned row_bytes = ldc * 4u;
  auto store_c = [&](auto stream_c) {
#pragma unroll
    for (int i = 0; i < T::kTilesM; ++i) {
#pragma unroll
      for (int n = 0; n < T::kTilesN; ++n) {
        const int col = n0 + wn * T::kWaveN + n * 32 + r32;
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int local_row = i * 32 + 8 * (e / 4) + (e % 4);
          const int row = m0 + wm * T::kWaveM + 4 * half + local_row;
          float v = acc[i][n][e];
          if (RELU && !to_ws) v = relu_maxf(v);
          if (!RAGGED || to_ws || (row < M && col < N)) {   // a partial tile is stored whole
            float *p = reinterpret_cast<float *>(c_tile + (lane_off + static_cast<unsigned>(local_row) * row_bytes +
                                                           static_cast<unsigned>(n * 32 * 4)));
            if (decltype(stream_c)::value) __builtin_nontemporal_store(v, p);
            else *p = v;
          }
        }
      }
    }
  };
  if (static_cast<int64_t>(M) * N * gridDim.y > (int64_t{48} << 20)) store_c(std::true_type{});
  else store_c(std::false_type{});
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RELU, bool RAGGED, int MIN_WAVES,
          bool TRANS_B = false>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWaveSize, MIN_WAVES) void gemm_f32_dl_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N,
    int K, int tiles_m, int tiles_n, int group_m, int64_t batch_a, int64_t batch_b, int64_t batch_c) {
  gemm_dl_body<BM, BN, BK, WAVES_M, WAVES_N, RELU, RAGGED, TRANS_B, false>(A, B, C, M, N, K, tiles_m, tiles_n, group_m,
                                                                           batch_a, batch_b, batch_c, 0, 1, nullptr);
}

// The launch with K-split tail tiles (see gemm_dl_body).
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RELU, bool RAGGED, int MIN_WAVES>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWaveSize, MIN_WAVES) void gemm_f32_dl_split_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N,
    int K, int tiles_m, int tiles_n, int group_m, int split_full, int split_parts, float *__restrict__ ws) {
  gemm_dl_body<BM, BN, BK, WAVES_M, WAVES_N, RELU, RAGGED, false, true>(A, B, C, M, N, K, tiles_m, tiles_n, group_m, 0, 0,
                                                                        0, split_full, split_parts, ws);
}

// C tile = epilogue(sum of the split_parts partial tiles).  A tile is shared by
// kSplitReduceSlabs workgroups (one float4 per thread each), so that the launch spreads over
// the chip; a thread requests its float4 of every piece before the first add (pieces beyond
// split_parts re-read piece 0 and are left out of the sum) and adds them in piece order.
constexpr int kSplitMaxParts = 8;
template <int BM, int BN>
constexpr int kSplitReduceSlabs = BM * BN / 4 / 256;
template <int BM, int BN, bool RELU>
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(const float *__restrict__ ws, float *__restrict__ C,
                                                                int M, int N, int tiles_m, int tiles_n, int group_m,
                                                                int split_full, int split_parts) {
  constexpr int kSlabs = kSplitReduceSlabs<BM, BN>;
  static_assert(kSlabs * 256 * 4 == BM * BN, "one float4 per thread");
  const int tile = blockIdx.x / kSlabs, slab = blockIdx.x % kSlabs;
  const int logical = split_full + tile;
  const int width = group_m * tiles_n;
  const int group = logical / width;
  const int first_m = group * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int in_group = logical - group * width;
  const int m0 = (first_m + in_group % gsz) * BM;
  const int n0 = (in_group / gsz) * BN;
  const int idx = slab * 256 + threadIdx.x;
  const float *src = ws + static_cast<int64_t>(tile) * split_parts * (BM * BN) + idx * 4;
  float4_t v[kSplitMaxParts];
#pragma unroll
  for (int p = 0; p < kSplitMaxParts; ++p)
    v[p] = *reinterpret_cast<const float4_t *>(src + (p < split_parts ? p : 0) * (BM * BN));
  float4_t sum = v[0];
#pragma unroll
  for (int p = 1; p < kSplitMaxParts; ++p)
    if (p < split_parts) {
#pragma unroll
      for (int j = 0; j < 4; ++j) sum[j] += v[p][j];
    }
  if (RELU) {
#pragma unroll
    for (int j = 0; j < 4; ++j) sum[j] = relu_maxf(sum[j]);
  }
  // (N is a multiple of 4: a float4 lies inside the matrix or outside it)
  const int row = m0 + idx / (BN / 4), col = n0 + (idx % (BN / 4)) * 4;
  if (row < M && col < N) *reinterpret_cast<float4_t *>(C + static_cast<int64_t>(row) * N + col) = sum;
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int MIN_WAVES>
static int launch_gemm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                       int epilogue, int group_m, int lds_stages, hipStream_t stream, kcg_launch_info *info) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N>;
  const int64_t tiles_m = (M + BM - 1) / BM;
  const int64_t tiles_n = (N + BN - 1) / BN;
  if (tiles_m * tiles_n > 0x7fffffffLL || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL)
    return KCG_ERR_BAD_SHAPE;
  const bool full = (M % BM == 0) && (N % BN == 0) && (K % BK == 0) && aligned16(A) && aligned16(B);
  // the direct-load kernel also takes ragged problems whose rows keep 16-byte alignment
  const bool ragged_dl = !full && (K % 4 == 0) && (N % 4 == 0) && K >= BK && aligned16(A) && aligned16(B);
  const bool relu = epilogue == KCG_EPILOGUE_RELU;
  // lds_stages (the schedule's buffer count): 3 = the direct-load ring, 2 = slices staged
  // through registers into double-buffered LDS, 1 = the same with one copy of each tile (built
  // for the two tiles the host layer stages: 128 x 128 x 8 and 256 x 128 x 16), 0 = the ring
  // where the shape allows it
  constexpr bool kHasSingle = (BM == 128 && BN == 128 && BK == 8) || (BM == 256 && BN == 128 && BK == 16);
  const bool dl_shape = (full || ragged_dl) && K < (1 << 22) && N < (1 << 22);
  const bool use_dl = dl_shape && lds_stages != 2 && lds_stages != 1;
  if (lds_stages == 3 && !dl_shape) return KCG_ERR_BAD_SCHEDULE;
  if (lds_stages == 1 && !kHasSingle) return KCG_ERR_BAD_SCHEDULE;
  if (info) {
    *info = kcg_launch_info{};
    info->launches = 1;
    info->main_rows = static_cast<int>(M);
    info->grid[0] = static_cast<int>(tiles_m * tiles_n);
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = T::kThreads;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = T::kLdsBytes;
    info->waves_per_block = WAVES_M * WAVES_N;
    const char *kind = "";
    if constexpr (BK == 8 || BK == 16 || BK == 32) {
      if (use_dl) {
        info->lds_bytes = GemmDlTile<BM, BN, BK, WAVES_M, WAVES_N>::kLdsBytes;
        kind = full ? "_dl" : "_dl_ragged";
      }
    }
    if (lds_stages == 1) {
      info->lds_bytes = T::kLdsBytes / 2;
      kind = "_single";
    }
    snprintf(info->kernel, sizeof info->kernel, "gemm_f32_%dx%dx%d_w%dx%d%s", BM, BN, BK, WAVES_M,
             WAVES_N, kind);
    return KCG_OK;
  }
  dim3 grid(static_cast<unsigned>(tiles_m * tiles_n));
  dim3 block(T::kThreads);
  if constexpr (BK == 8 || BK == 16 || BK == 32) {
    using TD = GemmDlTile<BM, BN, BK, WAVES_M, WAVES_N>;
    // the direct-load kernel addresses a slice with 32-bit byte offsets
    if (use_dl) {
      auto launch_dl = [&](auto kern) {
        if (!allow_lds(kern, TD::kLdsBytes)) return static_cast<int>(KCG_ERR_LAUNCH);
        return launch(kern, grid, block, TD::kLdsBytes, stream, A, B, C, static_cast<int>(M),
                      static_cast<int>(N), static_cast<int>(K), static_cast<int>(tiles_m),
                      static_cast<int>(tiles_n), group_m, int64_t{0}, int64_t{0}, int64_t{0});
      };
      if (full)
        return relu ? launch_dl(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, true, false, MIN_WAVES>)
                    : launch_dl(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, false, MIN_WAVES>);
      return relu ? launch_dl(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, true, true, MIN_WAVES>)
                  : launch_dl(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, true, MIN_WAVES>);
    }
  }
  if constexpr (kHasSingle) {
    if (lds_stages == 1) {
      auto launch_single = [&](auto kern) {
        if (!allow_lds(kern, T::kLdsBytes / 2)) return static_cast<int>(KCG_ERR_LAUNCH);
        return launch(kern, grid, block, T::kLdsBytes / 2, stream, A, B, C, static_cast<int>(M), static_cast<int>(N),
                      static_cast<int>(K), static_cast<int>(tiles_m), static_cast<int>(tiles_n), group_m);
      };
      if (relu)
        return full ? launch_single(gemm_f32_kernel<BM, BN, BK, WAVES_M, WAVES_N, true, true, MIN_WAVES, 1>)
                    : launch_single(gemm_f32_kernel<BM, BN, BK, WAVES_M, WAVES_N, true, false, MIN_WAVES, 1>);
      return full ? launch_single(gemm_f32_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, true, MIN_WAVES, 1>)
                  : launch_single(gemm_f32_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, false, MIN_WAVES, 1>);
    }
  }
#define KCG_LAUNCH(RELU_, FULL_)                                                                 \
  do {                                                                                           \
    auto kern = gemm_f32_kernel<BM, BN, BK, WAVES_M, WAVES_N, RELU_, FULL_, MIN_WAVES>;          \
    if (!allow_lds(kern, T::kLdsBytes)) return KCG_ERR_LAUNCH;                                   \
    return launch(kern, grid, block, T::kLdsBytes, stream, A, B, C, static_cast<int>(M),         \
                  static_cast<int>(N), static_cast<int>(K), static_cast<int>(tiles_m),           \
                  static_cast<int>(tiles_n), group_m);                                           \
  } while (0)
  if (relu) {
    if (full) KCG_LAUNCH(true, true);
    else KCG_LAUNCH(true, false);
  } else {
    if (full) KCG_LAUNCH(false, true);
    else KCG_LAUNCH(false, false);
  }
#undef KCG_LAUNCH
}

// Default tile by problem size.  Workgroups are spread over 256 CUs and the CU
// with the most workgroups sets the run time, so a tile is priced at
//   (tile area) x (max tiles per CU) / (its measured large-problem efficiency);
// small or awkwardly sized problems thereby get smaller tiles instead of leaving
// most of the chip idle (the reference's fixed 128x128 tile does the latter).
struct TileCand {
  int bm, bn, bk, wm, wn;
  double eff;        // fraction of MFMA peak on problems that fill the chip evenly
  double max_tiles;  // small tiles re-read A and B too often once the problem outgrows the L2s
};
static constexpr TileCand kTileCands[] = {{256, 128, 16, 64, 64, 0.91, 1e30},
                                          {128, 128, 32, 64, 64, 0.885, 1e30},  // BLOCK_K 16 is 10 % slower at 4096^3
                                          {128, 64, 32, 64, 32, 0.85, 4096},
                                          {64, 64, 32, 32, 32, 0.84, 6400}};

// Cost of `batch` M x N problems on tile c, in tile-area units per CU (proportional to run
// time for a given K); negative when the tile is not a candidate for this size.
static double tile_cost(const TileCand &c, int64_t M, int64_t N, int64_t batch) {
  const double per_matrix = static_cast<double>((M + c.bm - 1) / c.bm) * static_cast<double>((N + c.bn - 1) / c.bn);
  if (per_matrix > c.max_tiles) return -1.0;
  const double tiles = per_matrix * static_cast<double>(batch);
  const double per_cu = static_cast<double>((static_cast<int64_t>(tiles) + kNumCu - 1) / kNumCu);
  // a CU left with a single 4-wave workgroup has one wave per SIMD to hide latency with
  const double lonely = (c.bm * c.bn <= 128 * 128 && tiles <= kNumCu) ? 0.95 : 1.0;
  return per_cu * c.bm * c.bn / (c.eff * lonely);
}

static kcg_gemm_sched sched_of(const TileCand &c) { return {c.bm, c.bn, c.bk, 8, c.wm, c.wn, 4, 64, 0}; }

static kcg_gemm_sched default_tile(int64_t M, int64_t N, int64_t batch, double *cost_out = nullptr) {
  kcg_gemm_sched d = sched_of(kTileCands[0]);
  double best = -1.0;
  for (const TileCand &c : kTileCands) {
    const double cost = tile_cost(c, M, N, batch);
    if (cost < 0.0) continue;
    if (best < 0.0 || cost < best) {
      best = cost;
      d = sched_of(c);
    }
  }
  if (cost_out) *cost_out = best;
  return d;
}

// A large problem whose tile count leaves the last round of workgroups mostly empty is cut
// in two along M: the first `main_rows` rows run on the 256 x 128 tile in whole rounds, the
// rest on a small tile in a second launch on the same stream (rows of a row-major matrix are
// contiguous, so both are ordinary matmuls on sub-matrices).  7168^3: 140 -> 149 TFLOP/s,
// 9216^3: 144 -> 152, 14336^3: 147 -> 153.  main_rows == M: one launch.
struct GemmPlan {
  kcg_gemm_sched main;
  int64_t main_rows;
  kcg_gemm_sched tail;
};
static GemmPlan default_plan(int64_t M, int64_t N, double *cost_out = nullptr) {
  GemmPlan plan;
  double single = 0.0;
  plan.main = default_tile(M, N, 1, &single);
  plan.main_rows = M;
  plan.tail = plan.main;
  const TileCand &big = kTileCands[0];
  const int64_t rows_of_tiles = (M + big.bm - 1) / big.bm;
  // Worth it only when a few tiles spill into one more round (tiles per CU = n + a small
  // fraction): workgroups of a launch run nearly in step, so those few hold the whole chip
  // for a round.  With a fraction around one half the measured loss is nil at 6144^3 (152
  // TFLOP/s either way) but grows with the size (14336^3: 145 as one launch, 150 cut).
  const int64_t tiles = rows_of_tiles * ((N + big.bn - 1) / big.bn);
  const int64_t spill = tiles % kNumCu;
  const int64_t max_spill = tiles >= 10 * kNumCu ? kNumCu * 11 / 20 : kNumCu * 7 / 20;
  if (cost_out) *cost_out = single;
  if (tiles <= kNumCu || spill == 0 || spill > max_spill) return plan;
  double best = single;
  for (int64_t k = 1; k <= 8 && k < rows_of_tiles; ++k) {
    const int64_t m1 = (rows_of_tiles - k) * big.bm;
    const double c1 = tile_cost(big, m1, N, 1);
    double c2 = 0.0;
    const kcg_gemm_sched t = default_tile(M - m1, N, 1, &c2);
    const double cost = c1 + c2;
    if (cost < best) {
      best = cost;
      plan.main = sched_of(big);
      plan.main_rows = m1;
      plan.tail = t;
    }
  }
  if (cost_out) *cost_out = best;
  return plan;
}

// The tiles on 16 x 16 x 4 MFMA blocks (gemm_f32_t96.h: 96 x 96 and 96 x 64): K in whole slices,
// rows 16-byte aligned.
static bool t96_shape(int64_t M, int64_t N, int64_t K) {
  return M > 0 && N > 0 && K > 0 && N % 4 == 0 && K % 32 == 0 && K < (1 << 22) && N < (1 << 22) &&
         M <= 0x7fffffffLL && ((M + 63) / 64) * ((N + 63) / 64) <= 0x7fffffffLL;
}
// Their cost in the units of tile_cost; negative where a tile is no candidate.  Measured
// fraction of MFMA peak with the CUs holding R whole rounds of tiles, 96 x 96: 0.83 (R = 1: one
// wave per SIMD), 0.89 (2), 0.935 (4), 0.95 (9 and more), i.e. about 0.96 - 0.13 / R; 96 x 64:
// 0.78 (1), 0.90 (2), 0.945 (6), about 0.955 - 0.175 / R; scaled by 0.94 like the entries of
// kTileCands (whose 0.91 for 256 x 128 stands for a measured 0.97).
// Short K is left to the other tiles: these store C in 64-byte row segments.
struct T96Cand {
  int bn;
  double eff_many, eff_drop;   // fraction of peak = eff_many - eff_drop / R
};
static constexpr T96Cand kT96Cands[] = {{96, 0.96, 0.13}, {64, 0.955, 0.175}};
static double t96_cost(const T96Cand &c, int64_t M, int64_t N, int64_t K) {
  if (!t96_shape(M, N, K) || K < 512) return -1.0;
  const int64_t tiles = ((M + 95) / 96) * ((N + c.bn - 1) / c.bn);
  if (tiles > 4096) return -1.0;
  const double rounds = static_cast<double>((tiles + kNumCu - 1) / kNumCu);
  return rounds * 96 * c.bn / (0.94 * (c.eff_many - c.eff_drop / rounds));
}
// the cheaper of the two; *bn_out its BLOCK_SIZE_N
static double t96_cost(int64_t M, int64_t N, int64_t K, int *bn_out = nullptr) {
  double best = -1.0;
  for (const T96Cand &c : kT96Cands) {
    const double cost = t96_cost(c, M, N, K);
    if (cost > 0.0 && (best < 0.0 || cost < best)) {
      best = cost;
      if (bn_out) *bn_out = c.bn;
    }
  }
  return best;
}
// The model is good to a few per cent: a 96-wide tile must win by that much.
constexpr double kT96Margin = 0.97;
template <int BM, int BN>
static int launch_t96(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int epilogue,
                      int group_m, hipStream_t stream, kcg_launch_info *info) {
  using G = GemmT96Tile<BM, BN>;
  if (!t96_shape(M, N, K) || !aligned16(A) || !aligned16(B)) return KCG_ERR_BAD_SCHEDULE;
  const int tiles_m = static_cast<int>((M + G::kBM - 1) / G::kBM), tiles_n = static_cast<int>((N + G::kBN - 1) / G::kBN);
  const bool ragged = M % G::kBM != 0 || N % G::kBN != 0;
  if (info) {
    *info = kcg_launch_info{};
    info->launches = 1;
    info->main_rows = static_cast<int>(M);
    info->grid[0] = tiles_m * tiles_n;
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = G::kThreads;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = G::kLdsBytes;
    info->waves_per_block = G::kWavesM * G::kWavesN;
    snprintf(info->kernel, sizeof info->kernel, "gemm_f32_%dx%dx32_w2x2_dl%s", BM, BN, ragged ? "_ragged" : "");
    return KCG_OK;
  }
  const dim3 grid(static_cast<unsigned>(tiles_m * tiles_n)), block(G::kThreads);
  auto go = [&](auto kern) {
    if (!allow_lds(kern, G::kLdsBytes)) return static_cast<int>(KCG_ERR_LAUNCH);
    return launch(kern, grid, block, G::kLdsBytes, stream, A, B, C, static_cast<int>(M), static_cast<int>(N),
                  static_cast<int>(K), tiles_m, tiles_n, group_m);
  };
  const bool relu = epilogue == KCG_EPILOGUE_RELU;
  if (ragged) return relu ? go(gemm_f32_t96_kernel<BM, BN, true, true>) : go(gemm_f32_t96_kernel<BM, BN, false, true>);
  return relu ? go(gemm_f32_t96_kernel<BM, BN, true, false>) : go(gemm_f32_t96_kernel<BM, BN, false, false>);
}

// Resolves a schedule (NULL / zero fields = defaults) to one of the built tile
// shapes and either launches it or fills `info`.
static int launch_sched(const kcg_gemm_sched &d, const float *A, const float *B, float *C, int64_t M, int64_t N,
                        int64_t K, int epilogue, hipStream_t stream, kcg_launch_info *info) {
  if (d.wave_size != 64 || d.vec_width != 4 || d.group_m < 1) return KCG_ERR_BAD_SCHEDULE;
  if (d.lds_stages < 0 || d.lds_stages > 3) return KCG_ERR_BAD_SCHEDULE;
#define KCG_TRY(BM, BN, BK, WM, WN, MINW)                                                         \
  if (d.block_m == BM && d.block_n == BN && d.block_k == BK && d.wave_m == BM / WM &&             \
      d.wave_n == BN / WN)                                                                        \
    return launch_gemm<BM, BN, BK, WM, WN, MINW>(A, B, C, M, N, K, epilogue, d.group_m,           \
                                                  d.lds_stages, stream, info);
  if (d.block_m == 96 && (d.block_n == 96 || d.block_n == 64) && d.block_k == 32 && d.wave_m == 48 &&
      d.wave_n == d.block_n / 2) {
    if (d.lds_stages == 1 || d.lds_stages == 2) return KCG_ERR_BAD_SCHEDULE;   // built as the direct-load ring only
    return d.block_n == 96 ? launch_t96<96, 96>(A, B, C, M, N, K, epilogue, d.group_m, stream, info)
                           : launch_t96<96, 64>(A, B, C, M, N, K, epilogue, d.group_m, stream, info);
  }
  KCG_TRY(128, 128, 32, 2, 2, 2)
  KCG_TRY(128, 128, 16, 2, 2, 2)
  KCG_TRY(128, 128, 8, 2, 2, 2)
  KCG_TRY(256, 128, 16, 4, 2, 2)
  KCG_TRY(256, 128, 32, 4, 2, 1)
  KCG_TRY(64, 64, 32, 2, 2, 2)
  KCG_TRY(128, 64, 32, 2, 2, 2)
#undef KCG_TRY
  return KCG_ERR_BAD_SCHEDULE;
}

// (defined with the BatchedMatmul launchers below)
static bool stream_shape(int64_t batch, int64_t M, int64_t N, int64_t K, const float *A, const float *B,
                         const float *C);
static int launch_bmm_stream(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N,
                             int64_t K, bool trans_b, bool relu, int group_m, hipStream_t stream,
                             kcg_launch_info *info);

static int dispatch_gemm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                         int epilogue, const kcg_gemm_sched *s, hipStream_t stream,
                         kcg_launch_info *info) {
  kcg_gemm_sched d = {256, 128, 16, 8, 64, 64, 4, 64, 0};
  if (!s || (s->block_m == 0 && s->block_n == 0)) {
    double plan_cost = 0.0;
    const GemmPlan plan = default_plan(M, N, &plan_cost);
    d = plan.main;
    // a caller who fixes any tile field gets one launch with that field honoured
    const bool free_choice = !s || (s->block_k == 0 && s->wave_m == 0 && s->wave_n == 0 && s->lds_stages == 0);
    if (!free_choice) d = default_tile(M, N, 1);
    const bool plain_rest = !s || ((s->wave_size == 0 || s->wave_size == 64) && (s->vec_width == 0 || s->vec_width == 4));
    // A short K (512 to 1024) with at least two whole 256 x 128 tiles per CU: the streaming
    // kernel of BatchedMatmul, one matrix -- a tile's prologue and its C stores run under the
    // neighbouring tiles' slices (without an epilogue 8192 x 8192 x 1024: 140 -> 151 TFLOP/s,
    // 8192 x 4096 x 512: 142 -> 147, 32768 x 768 x 768: 146 -> 148; same tile, slice order and
    // MFMA mapping: the same bits).  The ReLU epilogue puts two VALU instructions per stored
    // element into that kernel's slice loop, which costs most of the gain (K = 512: +1 to +4 %,
    // K = 1024: +-1 %) and more than the gain below K = 512 (-2 % at K = 256): shorter K stays
    // on the tiled kernel, so that the choice does not depend on the epilogue.
    // (its workgroups take whole tiles, ceil(tiles / 256) on the busiest CU: only where that
    // leaves less than 6 % of the last round empty -- the plans below handle the rest better)
    const int64_t stream_tiles = (M / GemmStreamGeometry::kBM) * (N / GemmStreamGeometry::kBN);
    const int64_t stream_rounds = (stream_tiles + kNumCu - 1) / kNumCu;
    if (free_choice && plain_rest && K >= 512 && stream_shape(1, M, N, K, A, B, C) &&
        stream_tiles * 100 >= stream_rounds * kNumCu * 94) {
      if (s && s->group_m < 0) return KCG_ERR_BAD_SCHEDULE;
      return launch_bmm_stream(A, B, C, 1, M, N, K, false, epilogue == KCG_EPILOGUE_RELU, s && s->group_m ? s->group_m : 8,
                               stream, info);
    }
    // extents that 96 divides, where that tile fills the rounds of the CUs better
    int bn96 = 96;
    const double c96 = t96_cost(M, N, K, &bn96);
    if (free_choice && c96 > 0.0 && c96 < kT96Margin * plan_cost && aligned16(A) && aligned16(B) && plain_rest) {
      if (s && s->group_m < 0) return KCG_ERR_BAD_SCHEDULE;
      const int gm = s && s->group_m ? s->group_m : 8;
      return bn96 == 96 ? launch_t96<96, 96>(A, B, C, M, N, K, epilogue, gm, stream, info)
                        : launch_t96<96, 64>(A, B, C, M, N, K, epilogue, gm, stream, info);
    }
    if (free_choice && plan.main_rows < M) {
      // caller's remaining fields (GROUP_SIZE_M) apply to both launches
      kcg_gemm_sched t = plan.tail;
      if (s && s->group_m) d.group_m = t.group_m = s->group_m;
      if (s && ((s->wave_size && s->wave_size != 64) || (s->vec_width && s->vec_width != 4)))
        return KCG_ERR_BAD_SCHEDULE;
      const int64_t m1 = plan.main_rows;
      if (info) {
        // both launches: the main one in the leading fields, the second in tail_*; the
        // kernel name also carries the cut
        kcg_launch_info tail_info;
        int st = launch_sched(t, A, B, C, M - m1, N, K, epilogue, stream, &tail_info);
        if (st != KCG_OK) return st;
        st = launch_sched(d, A, B, C, m1, N, K, epilogue, stream, info);
        if (st != KCG_OK) return st;
        const size_t used = strlen(info->kernel);
        snprintf(info->kernel + used, sizeof info->kernel - used, "+%lldrows_%dx%dx%d", static_cast<long long>(M - m1),
                 t.block_m, t.block_n, t.block_k);
        info->launches = 2;
        info->main_rows = static_cast<int>(m1);
        info->tail_rows = static_cast<int>(M - m1);
        for (int i = 0; i < 3; ++i) {
          info->tail_grid[i] = tail_info.grid[i];
          info->tail_block[i] = tail_info.block[i];
        }
        info->tail_lds_bytes = tail_info.lds_bytes;
        memcpy(info->tail_kernel, tail_info.kernel, sizeof info->tail_kernel);
        return KCG_OK;
      }
      const int st = launch_sched(d, A, B, C, m1, N, K, epilogue, stream, nullptr);
      if (st != KCG_OK) return st;
      return launch_sched(t, A + m1 * K, B, C + m1 * N, M - m1, N, K, epilogue, stream, nullptr);
    }
  }
  if (s) {
    if (s->block_m) d.block_m = s->block_m;
    if (s->block_n) d.block_n = s->block_n;
    if (s->block_k) d.block_k = s->block_k;
    if (s->group_m) d.group_m = s->group_m;
    if (s->wave_m) d.wave_m = s->wave_m;
    if (s->wave_n) d.wave_n = s->wave_n;
    if (s->vec_width) d.vec_width = s->vec_width;
    if (s->wave_size) d.wave_size = s->wave_size;
    d.lds_stages = s->lds_stages;
  }
  return launch_sched(d, A, B, C, M, N, K, epilogue, stream, info);
}

// ---- K-split tail (the one plan that needs device memory beyond the operands) ----
// A problem whose 64 x 64 tiles (K in whole slices of 32, N a multiple of 4; edge tiles in M
// and N allowed) come to a few rounds of the CUs plus a small rest (1536^3: 576 = 2 x 256 +
// 64) holds every CU for one more round on behalf of a quarter of them.  With a workspace the rest is cut along K instead: the launch holds the whole
// tiles of the full rounds plus `parts` pieces of each remaining tile, so that every CU gets
// the same share; the pieces go to the workspace as raw partial tiles and a second, small
// launch adds them up and applies the epilogue.  The sums are taken in a fixed order: the
// result does not vary from run to run (it differs from the unsplit sum in the last bits).
struct SplitPlan {
  int full = 0, rest = 0, parts = 0;
  int64_t ws_bytes = 0;
};
// Picks the number of pieces per remaining tile.  Times in steps of K of one 64 x 64 tile: a
// whole tile costs K, a piece K / parts plus a fixed part (its prologue and its 16 KiB of
// partial sums, measured at about 100 steps); pieces beyond one per CU run as further waves
// of pieces.  The plan competes with the default plan of kcg_gemm_f32 (any tile, one launch
// or two), priced by the same model as default_tile.  `max_bytes` bounds the workspace the
// plan may need.
constexpr int64_t kSplitPieceBytes = 64 * 64 * 4;
constexpr int64_t kSplitMaxPieces = 2048;   // 32 MiB of partial sums at most
static bool split_tail_plan(int64_t M, int64_t N, int64_t K, int64_t max_bytes, SplitPlan *out) {
  if (N % 4 || K % 32 || N >= (1 << 22) || K >= (1 << 22)) return false;
  const TileCand &small = kTileCands[3];
  static_assert(kTileCands[3].bm == 64 && kTileCands[3].bn == 64 && kTileCands[3].bk == 32, "the tile of the split kernel");
  const int64_t tiles = ((M + 63) / 64) * ((N + 63) / 64);
  if (static_cast<double>(tiles) > small.max_tiles) return false;
  const int64_t rounds = tiles / kNumCu, rest = tiles % kNumCu;
  if (rest == 0) return false;
  // the default plan in steps of K of a 64 x 64 tile at that tile's efficiency
  double default_area = 0.0;
  default_plan(M, N, &default_area);
  // (the 96-wide tile competes only where it beats the split plan itself by the margin)
  const double c96 = t96_cost(M, N, K);
  const double plain96 = c96 > 0.0 ? c96 * small.eff / (64.0 * 64.0) * K : -1.0;
  const double plain = default_area * small.eff / (64.0 * 64.0) * K;
  const int64_t slices = K / 32;
  const int64_t max_pieces = std::min(max_bytes / kSplitPieceBytes, kSplitMaxPieces);
  constexpr double kPieceOverhead = 100.0;
  double best = plain;
  int parts = 0;
  static_assert(kSplitMaxParts == 8, "the candidates below");
  for (int cand : {2, 3, 4, 5, 6, 8}) {
    if (slices % cand != 0 || slices / cand < 4 || rest * cand > max_pieces) continue;
    const int64_t waves = (rest * cand + kNumCu - 1) / kNumCu;
    const double cost = static_cast<double>(rounds) * K + waves * (static_cast<double>(K) / cand + kPieceOverhead);
    if (cost < best) {
      best = cost;
      parts = cand;
    }
  }
  // worth a second launch when the model's saving outweighs that launch; the bounds are
  // measured ones (768 x 768 x 1536 at 312 steps saved still gains 10 %, 1536 x 1536 x 512 at
  // 284 loses; 1344 x 1344 x 4096 at 5 % of the run gains 4 %).  The first launch must also
  // run long enough for the second to be queued behind it: calls shorter than that are
  // bound by the host's launch rate, and two launches take twice as long as one
  // (512 x 512 x 768, 292 steps: 5 % slower; 512 x 512 x 1024, 356 steps: 30 % faster).
  if (parts == 0 || best > 0.95 * plain || plain - best < 300.0 || best < 330.0) return false;
  if (plain96 > 0.0 && plain96 < kT96Margin * best) return false;
  out->full = static_cast<int>(rounds * kNumCu);
  out->rest = static_cast<int>(rest);
  out->parts = parts;
  out->ws_bytes = rest * parts * kSplitPieceBytes;
  return true;
}

static int launch_split(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int epilogue,
                        int group_m, const SplitPlan &sp, float *ws, hipStream_t stream) {
  using TD = GemmDlTile<64, 64, 32, 2, 2>;
  const int tiles_m = static_cast<int>((M + 63) / 64), tiles_n = static_cast<int>((N + 63) / 64);
  const bool relu = epilogue == KCG_EPILOGUE_RELU;
  const bool ragged = M % 64 != 0 || N % 64 != 0;
  const dim3 grid(static_cast<unsigned>(sp.full + sp.rest * sp.parts)), block(256);
  auto main_launch = [&](auto kern) {
    if (!allow_lds(kern, TD::kLdsBytes)) return static_cast<int>(KCG_ERR_LAUNCH);
    return launch(kern, grid, block, TD::kLdsBytes, stream, A, B, C, static_cast<int>(M), static_cast<int>(N),
                  static_cast<int>(K), tiles_m, tiles_n, group_m, sp.full, sp.parts, ws);
  };
  const int st = ragged ? (relu ? main_launch(gemm_f32_dl_split_kernel<64, 64, 32, 2, 2, true, true, 2>)
                                : main_launch(gemm_f32_dl_split_kernel<64, 64, 32, 2, 2, false, true, 2>))
                        : (relu ? main_launch(gemm_f32_dl_split_kernel<64, 64, 32, 2, 2, true, false, 2>)
                                : main_launch(gemm_f32_dl_split_kernel<64, 64, 32, 2, 2, false, false, 2>));
  if (st != KCG_OK) return st;
  const float *cws = ws;
  const dim3 reduce_grid(static_cast<unsigned>(sp.rest * kSplitReduceSlabs<64, 64>));
  return relu ? launch(gemm_split_reduce_kernel<64, 64, true>, reduce_grid, dim3(256), 0, stream, cws, C,
                       static_cast<int>(M), static_cast<int>(N), tiles_m, tiles_n, group_m, sp.full, sp.parts)
              : launch(gemm_split_reduce_kernel<64, 64, false>, reduce_grid, dim3(256), 0, stream, cws, C,
                       static_cast<int>(M), static_cast<int>(N), tiles_m, tiles_n, group_m, sp.full, sp.parts);
}

// The schedule leaves the tile to the library (only GROUP_SIZE_M may be set).
static bool tile_is_free(const kcg_gemm_sched *s) {
  return !s || (s->block_m == 0 && s->block_n == 0 && s->block_k == 0 && s->wave_m == 0 && s->wave_n == 0 &&
                s->lds_stages == 0 && (s->wave_size == 0 || s->wave_size == 64) &&
                (s->vec_width == 0 || s->vec_width == 4));
}

// kcg_gemm_f32 with a workspace the caller lends: runs the K-split plan where there is one
// and the workspace holds it, the plain plan otherwise.
static int dispatch_gemm_ws(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int epilogue,
                            const kcg_gemm_sched *s, float *ws, int64_t ws_bytes, hipStream_t stream) {
  // (the plain path refuses a GROUP_SIZE_M below 1 in launch_sched; the split launch numbers
  // its tiles with the same value and must refuse it too: a negative one turns the tile
  // origins negative)
  if (s && s->group_m < 0) return KCG_ERR_BAD_SCHEDULE;
  SplitPlan sp;
  if (ws && tile_is_free(s) && split_tail_plan(M, N, K, ws_bytes, &sp) && aligned16(A) &&
      aligned16(B) && aligned16(C) && aligned16(ws))
    return launch_split(A, B, C, M, N, K, epilogue, s && s->group_m ? s->group_m : 8, sp, ws, stream);
  return dispatch_gemm(A, B, C, M, N, K, epilogue, s, stream, nullptr);
}

// BatchedMatmul (src/Frontend/Operators.cc:253-420) on the direct-load kernel: A row-major
// [batch][M][K]; B [batch][K][N] or, trans_b, [batch][N][K].  Returns
// KCG_ERR_UNSUPPORTED_SHAPE for problems this kernel does not take (rows that are not
// 16-byte aligned, K shorter than one slice, more than 65535 matrices).
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int MIN_WAVES>
static int launch_bmm_dl(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N,
                         int64_t K, bool trans_b, hipStream_t stream) {
  const int64_t tiles_m = (M + BM - 1) / BM;
  const int64_t tiles_n = (N + BN - 1) / BN;
  if (tiles_m * tiles_n > 0x7fffffffLL || M > 0x7fffffffLL || N >= (1 << 22) || K >= (1 << 22) || batch > 65535)
    return KCG_ERR_UNSUPPORTED_SHAPE;
  if (K % 4 != 0 || K < BK || (!trans_b && N % 4 != 0) || !aligned16(A) || !aligned16(B))
    return KCG_ERR_UNSUPPORTED_SHAPE;
  const bool full = (M % BM == 0) && (N % BN == 0) && (K % BK == 0);
  dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(batch));
  dim3 block(WAVES_M * WAVES_N * kWaveSize);
  auto go = [&](auto kern, int lds_bytes) {
    if (!allow_lds(kern, lds_bytes)) return static_cast<int>(KCG_ERR_LAUNCH);
    return launch(kern, grid, block, lds_bytes, stream, A, B, C, static_cast<int>(M), static_cast<int>(N),
                  static_cast<int>(K), static_cast<int>(tiles_m), static_cast<int>(tiles_n), 8, M * K, K * N,
                  M * N);
  };
  if (trans_b) {
    constexpr int lds_bytes = GemmDlTile<BM, BN, BK, WAVES_M, WAVES_N, true>::kLdsBytes;
    return full ? go(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, false, MIN_WAVES, true>, lds_bytes)
                : go(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, true, MIN_WAVES, true>, lds_bytes);
  }
  constexpr int lds_bytes = GemmDlTile<BM, BN, BK, WAVES_M, WAVES_N, false>::kLdsBytes;
  return full ? go(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, false, MIN_WAVES, false>, lds_bytes)
              : go(gemm_f32_dl_kernel<BM, BN, BK, WAVES_M, WAVES_N, false, true, MIN_WAVES, false>, lds_bytes);
}

// The streaming kernel (gemm_f32_stream.h): one resident workgroup per CU walks its share of
// the (matrix, tile) list.  Taken when every workgroup has at least two tiles to chain.
// `relu`: the fused epilogue of the plain matmul (row-major B only).  `info` != nullptr only
// fills the launch geometry.
static int launch_bmm_stream(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N,
                             int64_t K, bool trans_b, bool relu, int group_m, hipStream_t stream,
                             kcg_launch_info *info) {
  if (relu && trans_b) return KCG_ERR_BAD_SCHEDULE;
  using G = GemmStreamGeometry;
  const int64_t tiles_m = M / G::kBM, tiles_n = N / G::kBN;
  const int64_t items = tiles_m * tiles_n * batch;
  const int ctas = static_cast<int>(items < kNumCu ? items : kNumCu);
  const bool stream_c = M * N * batch > (int64_t{48} << 20);   // C beyond the last-level cache: non-temporal stores
  if (info) {
    *info = kcg_launch_info{};
    info->launches = 1;
    info->main_rows = static_cast<int>(M);
    info->grid[0] = ctas;
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = 512;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = G::kStages * GemmDlTile<G::kBM, G::kBN, G::kBK, G::kWavesM, G::kWavesN, false>::kStageFloats * 4;
    info->waves_per_block = G::kWavesM * G::kWavesN;
    snprintf(info->kernel, sizeof info->kernel, "gemm_f32_%dx%dx%d_w%dx%d_stream", G::kBM, G::kBN, G::kBK, G::kWavesM,
             G::kWavesN);
    return KCG_OK;
  }
  auto go = [&](auto kern, int lds_bytes) {
    if (!allow_lds(kern, lds_bytes)) return static_cast<int>(KCG_ERR_LAUNCH);
    return launch(kern, dim3(ctas), dim3(512), lds_bytes, stream, A, B, C, static_cast<int>(M), static_cast<int>(N),
                  static_cast<int>(K), static_cast<int>(tiles_m), static_cast<int>(tiles_n), group_m,
                  static_cast<int>(batch), M * K, K * N, M * N);
  };
  auto pick = [&](auto trans_c, auto kt_c, auto relu_c) {
    constexpr bool TB = decltype(trans_c)::value;
    constexpr int KT = decltype(kt_c)::value;
    constexpr bool RL = decltype(relu_c)::value;
    constexpr int lds_bytes =
        G::kStages * GemmDlTile<G::kBM, G::kBN, G::kBK, G::kWavesM, G::kWavesN, TB>::kStageFloats * 4;
    return stream_c ? go(gemm_f32_stream_kernel<TB, KT, true, RL>, lds_bytes)
                    : go(gemm_f32_stream_kernel<TB, KT, false, RL>, lds_bytes);
  };
  using K4 = std::integral_constant<int, 4>;
  using K8 = std::integral_constant<int, 8>;
  using No = std::false_type;
  if (trans_b) return K >= 128 ? pick(std::true_type{}, K8{}, No{}) : pick(std::true_type{}, K4{}, No{});
  if (relu) return pick(No{}, K8{}, std::true_type{});   // (the plain matmul only streams from K = 512)
  return K >= 128 ? pick(No{}, K8{}, No{}) : pick(No{}, K4{}, No{});
}

static bool stream_shape(int64_t batch, int64_t M, int64_t N, int64_t K, const float *A, const float *B,
                         const float *C) {
  using G = GemmStreamGeometry;
  if (M % G::kBM || N % G::kBN || K % (4 * G::kBK) || K < 4 * G::kBK) return false;
  if (N > (1 << 21) || K >= (1 << 22) || M > 0x7fffffffLL) return false;
  const int64_t items = (M / G::kBM) * (N / G::kBN) * batch;
  if (items < 2 * kNumCu || items > 0x7fffffffLL) return false;
  // a long K hides the per-tile prologue and epilogue by itself
  if (K > 1024) return false;
  return aligned16(A) && aligned16(B) && aligned16(C);
}

int dispatch_bmm_dl(const float *A, const float *B, float *C, int64_t batch, int64_t M, int64_t N, int64_t K,
                    bool trans_b, hipStream_t stream) {
  if (stream_shape(batch, M, N, K, A, B, C))
    return launch_bmm_stream(A, B, C, batch, M, N, K, trans_b, false, 8, stream, nullptr);
  const kcg_gemm_sched d = default_tile(M, N, batch);
  if (d.block_m == 256) return launch_bmm_dl<256, 128, 16, 4, 2, 2>(A, B, C, batch, M, N, K, trans_b, stream);
  // 128 x 128: the shallow slice has the shorter prologue, which is what counts for the short K
  // of attention products (K = 128: 116 against 107 TFLOP/s); from K = 4096 on the deep one wins
  if (d.block_m == 128 && d.block_n == 128)
    return K <= 1024 ? launch_bmm_dl<128, 128, 16, 2, 2, 2>(A, B, C, batch, M, N, K, trans_b, stream)
                     : launch_bmm_dl<128, 128, 32, 2, 2, 2>(A, B, C, batch, M, N, K, trans_b, stream);
  if (d.block_m == 128) return launch_bmm_dl<128, 64, 32, 2, 2, 2>(A, B, C, batch, M, N, K, trans_b, stream);
  return launch_bmm_dl<64, 64, 32, 2, 2, 2>(A, B, C, batch, M, N, K, trans_b, stream);
}

}  // namespace kcg

// ---- the partial-sum buffer of kcg_gemm_f32_noalloc ----
// One array per GPU, part of the loaded code object: it exists from the moment the library is
// loaded on a device until the process ends, and no call allocates or frees anything.  Every
// call on a GPU uses that GPU's array (the K-split plan overwrites the pieces it reads, so
// nothing has to be cleared between calls); calls that overlap in time on one GPU would
// write each other's partial sums.
namespace kcg_noalloc {
constexpr int64_t kScratchBytes = int64_t{4} << 20;   // 256 partial tiles of 64 x 64 floats: the largest plan
}
static __device__ __align__(256) unsigned char scratch[kcg_noalloc::kScratchBytes];
namespace kcg_noalloc {
// Device address of `scratch` on the current device, looked up on the first call on that
// device (in host code the array's name is only a handle for this lookup).
static float *scratch_of_current_device() {
  constexpr int kMaxDevices = 64;
  static std::atomic<void *> ptrs[kMaxDevices];   // zero-initialised: not looked up yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  void *p = ptrs[dev].load(std::memory_order_acquire);
  if (p) return static_cast<float *>(p);
  if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
  ptrs[dev].store(p, std::memory_order_release);
  return static_cast<float *>(p);
}
}  // namespace kcg_noalloc

extern "C" {

// Shape checks shared by the launch and the query entry point.
static int gemm_shape_status(int64_t M, int64_t N, int64_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return KCG_ERR_BAD_SHAPE;
  // Operands of 2^31 elements and more are refused: a 66000 x 33000 A faulted the GPU in its
  // one test run.  A host replay of the kernel's address arithmetic for the launches of that
  // call (tests/gemm_dl_address_model.cc) finds every access inside its tensor, so the cause
  // lies elsewhere and is not known; the size class stays switched off.
  constexpr int64_t kMaxElements = 0x7fffffffLL;
  if (M > kMaxElements / K || K > kMaxElements / N || M > kMaxElements / N) return KCG_ERR_UNSUPPORTED_SHAPE;
  return KCG_OK;
}

int kcg_gemm_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                 int epilogue, const kcg_gemm_sched *sched, void *stream) {
  if (!A || !B || !C) return KCG_ERR_NULL_POINTER;
  if (const int st = gemm_shape_status(M, N, K)) return st;
  if (epilogue != KCG_EPILOGUE_NONE && epilogue != KCG_EPILOGUE_RELU) return KCG_ERR_BAD_ARGUMENT;
  return kcg::dispatch_gemm(A, B, C, M, N, K, epilogue, sched, static_cast<hipStream_t>(stream),
                            nullptr);
}

int64_t kcg_gemm_f32_ws_bytes(int64_t M, int64_t N, int64_t K, const kcg_gemm_sched *sched) {
  if (gemm_shape_status(M, N, K) != KCG_OK || !kcg::tile_is_free(sched)) return 0;
  kcg::SplitPlan sp;
  return kcg::split_tail_plan(M, N, K, INT64_MAX, &sp) ? sp.ws_bytes : 0;
}

int kcg_gemm_f32_ws(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int epilogue,
                    const kcg_gemm_sched *sched, void *workspace, int64_t workspace_bytes, void *stream) {
  if (!A || !B || !C) return KCG_ERR_NULL_POINTER;
  if (const int st = gemm_shape_status(M, N, K)) return st;
  if (epilogue != KCG_EPILOGUE_NONE && epilogue != KCG_EPILOGUE_RELU) return KCG_ERR_BAD_ARGUMENT;
  if (workspace_bytes < 0) return KCG_ERR_BAD_ARGUMENT;
  return kcg::dispatch_gemm_ws(A, B, C, M, N, K, epilogue, sched, static_cast<float *>(workspace), workspace_bytes,
                               static_cast<hipStream_t>(stream));
}

int kcg_gemm_f32_ws_query(int64_t M, int64_t N, int64_t K, const kcg_gemm_sched *sched, int64_t workspace_bytes,
                          kcg_launch_info *out) {
  if (!out) return KCG_ERR_NULL_POINTER;
  if (const int st = gemm_shape_status(M, N, K)) return st;
  if (workspace_bytes < 0) return KCG_ERR_BAD_ARGUMENT;
  if (sched && sched->group_m < 0) return KCG_ERR_BAD_SCHEDULE;
  kcg::SplitPlan sp;
  if (!kcg::tile_is_free(sched) || !kcg::split_tail_plan(M, N, K, workspace_bytes, &sp))
    return kcg::dispatch_gemm(nullptr, nullptr, nullptr, M, N, K, KCG_EPILOGUE_NONE, sched, nullptr, out);
  // the two launches of kcg::launch_split: whole tiles and pieces, then the adding launch
  using TD = kcg::GemmDlTile<64, 64, 32, 2, 2>;
  *out = kcg_launch_info{};
  out->launches = 2;
  out->grid[0] = sp.full + sp.rest * sp.parts;
  out->grid[1] = out->grid[2] = 1;
  out->block[0] = 256;
  out->block[1] = out->block[2] = 1;
  out->lds_bytes = TD::kLdsBytes;
  out->waves_per_block = 4;
  snprintf(out->kernel, sizeof out->kernel, "gemm_f32_dl_split_64x64x32_full%d_rest%dx%d", sp.full, sp.rest, sp.parts);
  out->main_rows = static_cast<int32_t>(M);
  out->tail_rows = 0;
  out->tail_grid[0] = sp.rest * kcg::kSplitReduceSlabs<64, 64>;
  out->tail_grid[1] = out->tail_grid[2] = 1;
  out->tail_block[0] = 256;
  out->tail_block[1] = out->tail_block[2] = 1;
  out->tail_lds_bytes = 0;
  snprintf(out->tail_kernel, sizeof out->tail_kernel, "gemm_split_reduce_64x64_parts%d", sp.parts);
  return KCG_OK;
}

int kcg_gemm_f32_noalloc(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K, int epilogue,
                         const kcg_gemm_sched *sched, void *stream) {
  if (!A || !B || !C) return KCG_ERR_NULL_POINTER;
  if (const int st = gemm_shape_status(M, N, K)) return st;
  if (epilogue != KCG_EPILOGUE_NONE && epilogue != KCG_EPILOGUE_RELU) return KCG_ERR_BAD_ARGUMENT;
  if (sched && sched->group_m < 0) return KCG_ERR_BAD_SCHEDULE;
  // the plan is looked for among those whose partial sums fit the array; where there is none
  // the call is the plain one, which uses no memory of its own
  kcg::SplitPlan sp;
  if (!kcg::tile_is_free(sched) || !kcg::split_tail_plan(M, N, K, kcg_noalloc::kScratchBytes, &sp))
    return kcg::dispatch_gemm(A, B, C, M, N, K, epilogue, sched, static_cast<hipStream_t>(stream), nullptr);
  if (sp.ws_bytes > kcg_noalloc::kScratchBytes) return KCG_ERR_UNSUPPORTED_SHAPE;
  float *ws = kcg_noalloc::scratch_of_current_device();
  if (!ws) return KCG_ERR_LAUNCH;
  return kcg::dispatch_gemm_ws(A, B, C, M, N, K, epilogue, sched, ws, kcg_noalloc::kScratchBytes,
                               static_cast<hipStream_t>(stream));
}

int kcg_gemm_f32_query(int64_t M, int64_t N, int64_t K, const kcg_gemm_sched *sched,
                       kcg_launch_info *out) {
  if (!out) return KCG_ERR_NULL_POINTER;
  if (const int st = gemm_shape_status(M, N, K)) return st;
  return kcg::dispatch_gemm(nullptr, nullptr, nullptr, M, N, K, KCG_EPILOGUE_NONE, sched, nullptr,
                            out);
}

}  // extern "C"
