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

// FULL: M % BM == 0, N % BN == 0, K % BK == 0 and 16-byte aligned rows, so that
// no bounds checks are needed and every global access is a dwordx4.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RELU, bool FULL, int MIN_WAVES>
__global__ __launch_bounds__(WAVES_M *WAVES_N *kWaveSize, MIN_WAVES) void gemm_f32_kernel(
    const float *__restrict__ A, const float *__restrict__ B, float *__restrict__ C, int M, int N,
    int K, int tiles_m, int tiles_n, int group_m) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N>;
  extern __shared__ __align__(16) float lds[];
  float *As = lds;                     // [2][BM][kPitchA]
  float *Bs = lds + 2 * T::kFloatsA;   // [2][BK][kPitchB]

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

  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < T::kLoadsA; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (BK / 4);
      const int c4 = idx % (BK / 4);
      const int64_t gr = m0 + row;
      const int gk = k0 + c4 * 4;
      if (FULL) {
        ra[i] = *reinterpret_cast<const float4_t *>(A + gr * K + gk);
      } else {
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (gr < M) {
          const float *p = A + gr * K;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (gk + e < K) v[e] = p[gk + e];
        }
        ra[i] = v;
      }
    }
#pragma unroll
    for (int i = 0; i < T::kLoadsB; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (BN / 4);
      const int c4 = idx % (BN / 4);
      const int64_t gk = k0 + row;
      const int gn = n0 + c4 * 4;
      if (FULL) {
        rb[i] = *reinterpret_cast<const float4_t *>(B + gk * N + gn);
      } else {
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (gk < K) {
          const float *p = B + gk * N;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (gn + e < N) v[e] = p[gn + e];
        }
        rb[i] = v;
      }
    }
  };

  auto store_lds = [&](int buf) {
    float *as = As + buf * T::kFloatsA;
    float *bs = Bs + buf * T::kFloatsB;
#pragma unroll
    for (int i = 0; i < T::kLoadsA; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (BK / 4);
      const int c4 = idx % (BK / 4);
      *reinterpret_cast<float4_t *>(as + row * T::kPitchA + c4 * 4) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < T::kLoadsB; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (BN / 4);
      const int c4 = idx % (BN / 4);
      *reinterpret_cast<float4_t *>(bs + row * T::kPitchB + c4 * 4) = rb[i];
    }
  };

  auto compute = [&](int buf) {
    const float *as = As + buf * T::kFloatsA + (wm * T::kWaveM + r32) * T::kPitchA + 4 * half;
    const float *bs = Bs + buf * T::kFloatsB + (4 * half) * T::kPitchB + wn * T::kWaveN + r32;
#pragma unroll
    for (int kk = 0; kk < BK / 8; ++kk) {
      float4_t a[T::kTilesM];
#pragma unroll
      for (int i = 0; i < T::kTilesM; ++i)
        a[i] = *reinterpret_cast<const float4_t *>(as + i * 32 * T::kPitchA + kk * 8);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float b[T::kTilesN];
#pragma unroll
        for (int n = 0; n < T::kTilesN; ++n) b[n] = bs[(kk * 8 + j) * T::kPitchB + n * 32];
#pragma unroll
        for (int i = 0; i < T::kTilesM; ++i)
#pragma unroll
          for (int n = 0; n < T::kTilesN; ++n)
            acc[i][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i][j], b[n], acc[i][n], 0, 0, 0);
      }
    }
  };

  const int ktiles = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int kt = 0; kt < ktiles; ++kt) {
    const int cur = kt & 1;
    const bool more = (kt + 1) < ktiles;
    if (more) load_global((kt + 1) * BK);
    compute(cur);
    if (more) store_lds(cur ^ 1);
    __syncthreads();
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

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int MIN_WAVES>
static int launch_gemm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                       int epilogue, int group_m, hipStream_t stream, kcg_launch_info *info) {
  using T = GemmTile<BM, BN, BK, WAVES_M, WAVES_N>;
  const int64_t tiles_m = (M + BM - 1) / BM;
  const int64_t tiles_n = (N + BN - 1) / BN;
  if (tiles_m * tiles_n > 0x7fffffffLL || M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL)
    return KCG_ERR_BAD_SHAPE;
  const bool full = (M % BM == 0) && (N % BN == 0) && (K % BK == 0) && aligned16(A) && aligned16(B);
  const bool relu = epilogue == KCG_EPILOGUE_RELU;
  if (info) {
    info->grid[0] = static_cast<int>(tiles_m * tiles_n);
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = T::kThreads;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = T::kLdsBytes;
    info->waves_per_block = WAVES_M * WAVES_N;
    snprintf(info->kernel, sizeof info->kernel, "gemm_f32_%dx%dx%d_w%dx%d", BM, BN, BK, WAVES_M,
             WAVES_N);
    return KCG_OK;
  }
  dim3 grid(static_cast<unsigned>(tiles_m * tiles_n));
  dim3 block(T::kThreads);
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

// Resolves a schedule (NULL / zero fields = defaults) to one of the built tile
// shapes and either launches it or fills `info`.
static int dispatch_gemm(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                         int epilogue, const kcg_gemm_sched *s, hipStream_t stream,
                         kcg_launch_info *info) {
  // Default tile by problem size.  Workgroups are spread over 256 CUs and the CU
  // with the most workgroups sets the run time, so a tile is scored by
  //   (its measured large-problem efficiency) x (tiles / (256 * max tiles per CU));
  // small or awkwardly sized problems thereby get smaller tiles instead of leaving
  // most of the chip idle (the reference's fixed 128x128 tile does the latter).
  kcg_gemm_sched d = {256, 128, 16, 8, 64, 64, 4, 64};
  if (!s || (s->block_m == 0 && s->block_n == 0)) {
    struct Cand {
      int bm, bn, bk, wm, wn;
      double eff;
    };
    const Cand cands[] = {{256, 128, 16, 64, 64, 0.88}, {128, 128, 16, 64, 64, 0.86}, {64, 64, 32, 32, 32, 0.77}};
    double best = -1.0;
    for (const Cand &c : cands) {
      const double tiles = static_cast<double>((M + c.bm - 1) / c.bm) * static_cast<double>((N + c.bn - 1) / c.bn);
      const double per_cu = static_cast<double>((static_cast<int64_t>(tiles) + kNumCu - 1) / kNumCu);
      // padding waste of ragged edges counts against a large tile too
      const double useful = (static_cast<double>(M) * N) / (tiles * c.bm * c.bn);
      const double score = c.eff * useful * tiles / (per_cu * kNumCu);
      if (score > best) {
        best = score;
        d = {c.bm, c.bn, c.bk, 8, c.wm, c.wn, 4, 64};
      }
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
  }
  if (d.wave_size != 64 || d.vec_width != 4 || d.group_m < 1) return KCG_ERR_BAD_SCHEDULE;
#define KCG_TRY(BM, BN, BK, WM, WN, MINW)                                                         \
  if (d.block_m == BM && d.block_n == BN && d.block_k == BK && d.wave_m == BM / WM &&             \
      d.wave_n == BN / WN)                                                                        \
    return launch_gemm<BM, BN, BK, WM, WN, MINW>(A, B, C, M, N, K, epilogue, d.group_m, stream,   \
                                                  info);
  KCG_TRY(128, 128, 32, 2, 2, 2)
  KCG_TRY(128, 128, 16, 2, 2, 2)
  KCG_TRY(128, 128, 8, 2, 2, 2)
  KCG_TRY(256, 128, 16, 4, 2, 2)
  KCG_TRY(256, 128, 32, 4, 2, 1)
  KCG_TRY(256, 256, 16, 2, 2, 1)
  KCG_TRY(64, 64, 32, 2, 2, 2)
#undef KCG_TRY
  return KCG_ERR_BAD_SCHEDULE;
}

}  // namespace kcg

extern "C" {

int kcg_gemm_f32(const float *A, const float *B, float *C, int64_t M, int64_t N, int64_t K,
                 int epilogue, const kcg_gemm_sched *sched, void *stream) {
  if (!A || !B || !C) return KCG_ERR_NULL_POINTER;
  if (M <= 0 || N <= 0 || K <= 0) return KCG_ERR_BAD_SHAPE;
  if (epilogue != KCG_EPILOGUE_NONE && epilogue != KCG_EPILOGUE_RELU) return KCG_ERR_BAD_ARGUMENT;
  return kcg::dispatch_gemm(A, B, C, M, N, K, epilogue, sched, static_cast<hipStream_t>(stream),
                            nullptr);
}

int kcg_gemm_f32_query(int64_t M, int64_t N, int64_t K, const kcg_gemm_sched *sched,
                       kcg_launch_info *out) {
  if (!out) return KCG_ERR_NULL_POINTER;
  if (M <= 0 || N <= 0 || K <= 0) return KCG_ERR_BAD_SHAPE;
  return kcg::dispatch_gemm(nullptr, nullptr, nullptr, M, N, K, KCG_EPILOGUE_NONE, sched, nullptr,
                            out);
}

}  // extern "C"
