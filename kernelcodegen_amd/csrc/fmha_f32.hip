// Fused multi-head attention, fp32, for gfx950 (MI355X).
//
// Semantics: the Frontend graph BatchedMatmul(Q, K^T) -> Softmax(axis -1) ->
// BatchedMatmul(P, V) (test/test.cc:88-90; src/Frontend/Operators.cc:253-420,
// 425-542), which FMHAOptimizer matches (src/Optimizer/Optimizer.cc:586-672) and
// replaces by one kernel Fused_Multi_Head_Attention_<b>_<h>_SL<S>_HD<D>(Q,K,V,O)
// (:1101-1118) tiled Br x Bc with an online softmax (:948-1077, 1191-1331).
// The tiling idea is kept (a workgroup owns Br query rows and sweeps K/V in Bc
// row tiles, running max / sum / rescale).  Everything else is gfx950 specific:
//
//  * 4 (or 8) waves per workgroup, 32 query rows per wave, Br = 128 (256), Bc = 32 (or 64).
//  * The first product is computed transposed, S^T = K . Q^T, with
//    v_mfma_f32_32x32x2_f32: lane (r = l%32, h = l/32) then holds, for query r,
//    the 16 keys {8g + 4h + i}.  That is exactly the B-operand layout the second
//    product O^T = V^T . P^T needs, so P never leaves registers and the running
//    max / sum / rescale factor are per-lane scalars (one cross-half exchange
//    per tile for the max, one at the end for the sum).
//  * Q (pre-multiplied by scale * log2 e) stays in registers for the whole sweep
//    (the reference re-reads it per K/V tile, src/Optimizer/Optimizer.cc:1206).
//  * K and V tiles are fetched directly into LDS before the MFMA phase that hides them
//    (V_t during S = K_t.Q, K_{t+1} during O += P.V_t).
//  * The running maximum is a lazily raised reference (see kTau): VALU work between
//    the two MFMA phases costs matrix time, so the rescale of O is skipped whenever
//    the mathematics allows it.
//  * Causal: a workgroup runs the query-block pair (n-1-i, i), so all workgroups
//    sweep the same number of tiles.
//
// K and V tiles go from global memory straight into LDS (global_load_lds_dwordx4 with a
// scalar base and a 32-bit lane offset: no staging registers, no LDS stores and no address
// arithmetic on the vector ALU, whose time comes out of the fp32 MFMA's).  An instruction
// fills 1 KiB of consecutive LDS, lane L supplying the 16 bytes at position L, so rows
// cannot be padded; each lane fetches whichever global chunk belongs at its position:
//   Ks: D/32 panels, panel g = [Bc rows][32 floats d = 32g..32g+31]; the 16-byte chunk c
//       of row r sits at position c ^ ((r >> 1) & 7): the ds_read_b128 of 16 consecutive
//       rows of one chunk column then hits 16 distinct 16-byte slots of a 256-byte window.
//   Vs: [Bc rows][D floats]; the 32-float group i of row r sits at group i ^ ((r >> 2) & 1):
//       rows k and k+4, read together by the two halves of a wave, use different halves
//       of the 256-byte window.
#include "kcg_common.h"

namespace kcg {

template <int D, int BC, int WAVES>
struct FmhaF32Tile {
  static constexpr int kThreads = 64 * WAVES;
  static constexpr int kBr = 32 * WAVES;
  static constexpr int kTileBytes = BC * D * 4;              // one K (or V) tile, unpadded
  static constexpr int kLdsBytes = 2 * kTileBytes;
  static constexpr int kRuns = kTileBytes / 1024;            // 1 KiB direct loads per tile
  static constexpr int kRunsPerWave = kRuns / WAVES;
  static constexpr int kPanelBytes = BC * 128;               // K: BC rows x 32 floats of one d-group
  static constexpr int kRunsPerPanel = BC / 8;
  static constexpr int kRowsPerRunV = 256 / D;               // V: whole rows per 1 KiB
  static constexpr int kKeyTiles = BC / 32;
  static constexpr int kDTiles = D / 32;
  static_assert(BC % 32 == 0 && D % 32 == 0 && D <= 256, "tile extents");
  static_assert(kRuns % WAVES == 0, "load split");
};

// How far (in log2 units) a tile's row maximum may exceed the running reference before
// the accumulators are rescaled.
constexpr float kTau = 8.0f;

template <int D, int BC, int WAVES, bool CAUSAL>
__global__ __launch_bounds__(64 * WAVES, WAVES == 2 ? 1 : 8 / WAVES) void fmha_f32_kernel(const float *__restrict__ Q,
                                                          const float *__restrict__ K,
                                                          const float *__restrict__ V,
                                                          float *__restrict__ O, int S,
                                                          int q_blocks, int q_items, float scale_log2e) {
  using T = FmhaF32Tile<D, BC, WAVES>;
  extern __shared__ __align__(16) float lds[];
  const char *Ks = reinterpret_cast<const char *>(lds);
  const char *Vs = Ks + T::kTileBytes;
  const unsigned lds_k = static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds));  // LDS byte address
  const unsigned lds_v = lds_k + T::kTileBytes;

  // Every XCD walks a contiguous range of (head, work item) ids, head-major, so the
  // K/V of a head are fetched into one XCD's L2 only.  Causal: a work item is the pair
  // of query blocks (n-1-i, i), so every workgroup sweeps the same number of K/V tiles.
  const int bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int bh = bid / q_items;
  const int item = bid - bh * q_items;
  const int hi_block = q_blocks - 1 - item;
  const int npass = CAUSAL ? (hi_block != item ? 2 : 1) : 1;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31;
  const int half = lane >> 5;

  const int64_t base = static_cast<int64_t>(bh) * S * D;
  const float *Qb = Q + base;
  const float *Kb = K + base;
  const float *Vb = V + base;
  float *Ob = O + base;


  // ---- direct tile loads ----
  // Run rho = wave * kRunsPerWave + i of a tile.  K: panel g = rho / kRunsPerPanel, rows
  // 8q .. 8q+7 (q = rho % kRunsPerPanel); lane L is row 8q + L/8, position L%8.  V: rows
  // rho * kRowsPerRunV ..; lane L is row + L / (D/4), position L % (D/4).
  int k_row[T::kRunsPerWave], v_row[T::kRunsPerWave];      // tile row this lane fetches
  unsigned k_col[T::kRunsPerWave], v_col[T::kRunsPerWave];  // byte offset inside the global row
#pragma unroll
  for (int i = 0; i < T::kRunsPerWave; ++i) {
    const int rho = wave * T::kRunsPerWave + i;
    const int g = rho / T::kRunsPerPanel, q = rho % T::kRunsPerPanel;
    k_row[i] = 8 * q + lane / 8;
    k_col[i] = static_cast<unsigned>(g * 8 + ((lane % 8) ^ ((k_row[i] >> 1) & 7))) * 16u;
    v_row[i] = rho * T::kRowsPerRunV + lane / (D / 4);
    const int pc = lane % (D / 4);
    v_col[i] = static_cast<unsigned>((((pc >> 3) ^ ((v_row[i] >> 2) & 1)) << 3) + (pc & 7)) * 16u;
  }
  // A tile that sticks out beyond S fetches row S-1 in place of the rows that do not exist
  // (K: those scores are masked; V: those rows are zeroed below before anybody reads them).
  auto load_k = [&](int kv0) {
    const char *g = reinterpret_cast<const char *>(Kb + static_cast<int64_t>(kv0) * D);
    const int last = S - 1 - kv0;
#pragma unroll
    for (int i = 0; i < T::kRunsPerWave; ++i) {
      const int row = k_row[i] < last ? k_row[i] : last;
      direct_load_16B(g, static_cast<unsigned>(row) * (D * 4u) + k_col[i],
                      lds_k + (wave * T::kRunsPerWave + i) * 1024u);
    }
  };
  auto load_v = [&](int kv0) {
    const char *g = reinterpret_cast<const char *>(Vb + static_cast<int64_t>(kv0) * D);
    const int last = S - 1 - kv0;
#pragma unroll
    for (int i = 0; i < T::kRunsPerWave; ++i) {
      const int row = v_row[i] < last ? v_row[i] : last;
      direct_load_16B(g, static_cast<unsigned>(row) * (D * 4u) + v_col[i],
                      lds_v + (wave * T::kRunsPerWave + i) * 1024u);
    }
  };
  // Waits for this wave's direct loads; V rows at and beyond S become zeros (P is 0 there,
  // but 0 * inf would not be).
  auto v_landed = [&](int kv0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (kv0 + BC > S) {
#pragma unroll
      for (int i = 0; i < T::kRunsPerWave; ++i)
        if (kv0 + v_row[i] >= S)
          *reinterpret_cast<float4_t *>(lds + T::kTileBytes / 4 + (wave * T::kRunsPerWave + i) * 256 + lane * 4) =
              float4_t{0.f, 0.f, 0.f, 0.f};
    }
  };
  // per-lane read addresses (bytes inside a tile), swizzles folded in
  int ka[4];  // K chunk 2j + half of row r32, j = kk % 4 (panel kk / 4 and key tile by offset)
#pragma unroll
  for (int j = 0; j < 4; ++j) ka[j] = r32 * 128 + 16 * ((2 * j + half) ^ ((r32 >> 1) & 7));
  // V[key][32 i + r32] with key = 4 half + (compile-time part): group i ^ half
  const int va_even = half * (4 * D * 4) + half * 128 + r32 * 4;   // even i: (i ^ half) = i + half
  const int va_odd = half * (4 * D * 4) - half * 128 + r32 * 4;    // odd i:  (i ^ half) = i - half

#pragma unroll 1
  for (int pass = 0; pass < npass; ++pass) {
  const int qb = CAUSAL ? (pass == 0 ? hi_block : item) : item;  // the long block first
  const int q0 = qb * T::kBr;
  const int qrow = q0 + wave * 32 + r32;  // this lane's query
  const bool qvalid = qrow < S;

  // the first K tile is requested before the Q rows so that both are in flight together
  // (Ks is free: every wave passed the last barrier of the previous pass)
  load_k(0);

  // ---- Q fragment: q[kk][j] = Q[qrow][8*kk + 4*half + j] * scale * log2(e) ----
  float4_t q[D / 8];
#pragma unroll
  for (int kk = 0; kk < D / 8; ++kk) {
    float4_t v = {0.f, 0.f, 0.f, 0.f};
    if (qvalid)
      v = *reinterpret_cast<const float4_t *>(Qb + static_cast<int64_t>(qrow) * D + 8 * kk + 4 * half);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= scale_log2e;
    q[kk] = v;
  }

  float16_t acc_o[T::kDTiles];
#pragma unroll
  for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc_o[i][e] = 0.0f;
  float m_run = -INFINITY;  // reference max of this query (both halves agree)
  float l_run = 0.0f;       // running sum over this lane's keys only

  const int kv_end = CAUSAL ? ((q0 + T::kBr) < S ? (q0 + T::kBr) : S) : S;
  const int n_tiles = (kv_end + BC - 1) / BC;

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // Causal: the tiles that lie wholly above this wave's 32 query rows contribute nothing
  // (every P is 0).  The wave computes the first n_own tiles and, in a second loop that
  // does not touch the accumulators, only moves its share of the remaining tiles and keeps
  // the barriers; the matrix pipe of its SIMD is then free for the other workgroup of the CU.
  const int last_row_tile = (q0 + wave * 32 + 31) / BC;
  const int n_own = (CAUSAL && last_row_tile + 1 < n_tiles) ? last_row_tile + 1 : n_tiles;

  for (int t = 0; t < n_own; ++t) {
    const int kv0 = t * BC;
    load_v(kv0);

    // ---- S^T = K . Q^T  (rows = keys, columns = queries) ----
    float16_t s[T::kKeyTiles];
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kt][e] = 0.0f;
      // the K fragment of the next 8 d-columns is requested before the four MFMAs of the
      // current one are issued
      auto k_frag = [&](int kk) {
        return *reinterpret_cast<const float4_t *>(Ks + ka[kk % 4] + (kk / 4) * T::kPanelBytes + kt * 32 * 128);
      };
      float4_t kf[2];
      kf[0] = k_frag(0);
#pragma unroll
      for (int kk = 0; kk < D / 8; ++kk) {
        if (kk + 1 < D / 8) kf[(kk + 1) & 1] = k_frag(kk + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[kk & 1][j], q[kk][j], s[kt], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    // ---- mask (sequence end, causal diagonal) ----
    const bool need_mask = (kv0 + BC > S) || (CAUSAL && (kv0 + BC - 1 > q0 + wave * 32));
    if (need_mask) {
#pragma unroll
      for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = kv0 + kt * 32 + 8 * (e / 4) + 4 * half + (e % 4);
          const bool dead = (key >= S) || (CAUSAL && key > qrow);
          if (dead) s[kt][e] = -INFINITY;
        }
    }

    // ---- online softmax (base 2; Q carries scale * log2 e), lazy rescale ----
    // m_run is a reference maximum, not the exact one: it is raised (and O, l rescaled)
    // only when the tile maximum exceeds it by more than kTau, so that after the first
    // tiles almost no tile pays the 16 * kDTiles multiplications.  Between rescales
    // P <= 2^kTau; the final O / l is exact for any reference.  The decision is per
    // query row (both lanes of a row see the same m_loc and m_run).
    float m_loc = max3(s[0][0], s[0][1], s[0][2]);
#pragma unroll
    for (int x = 3; x + 1 < T::kKeyTiles * 16; x += 2) m_loc = max3(m_loc, s[x / 16][x % 16], s[(x + 1) / 16][(x + 1) % 16]);
    m_loc = max_across_halves(fmaxf(m_loc, s[T::kKeyTiles - 1][15]));
    const bool raise = m_loc > m_run + kTau;  // false for NaN and for rows masked so far
    if (__builtin_amdgcn_ballot_w64(raise) != 0) {
      const float alpha = raise ? __builtin_amdgcn_exp2f(m_run - m_loc) : 1.0f;  // m_run = -inf -> 0
      if (raise) m_run = m_loc;
      l_run *= alpha;
#pragma unroll
      for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc_o[i][e] *= alpha;
    }
    const float m_use = (m_run == -INFINITY) ? 0.0f : m_run;  // fully masked so far
    float psum = 0.0f;
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = __builtin_amdgcn_exp2f(s[kt][e] - m_use);
        s[kt][e] = p;
        psum += p;
      }
    l_run += psum;

    v_landed(kv0);
    __syncthreads();  // V tile visible; every wave is done reading Ks

    const bool more = (t + 1) < n_tiles;
    if (more) load_k(kv0 + BC);

    // ---- O^T += V^T . P^T  (rows = d, columns = queries, contraction over keys) ----
    // The matrix phase with the longer dependency chains gets the higher wave priority:
    // two workgroups sharing a CU then take turns instead of the older one always winning.
    __builtin_amdgcn_s_setprio(1);
    {
      // step x = (kt, e): key 32*kt + 8*(e/4) + 4*half + e%4; its kDTiles V values are
      // requested one step (kDTiles MFMAs) ahead
      constexpr int kPvSteps = T::kKeyTiles * 16;
      float vf[2][T::kDTiles];
      auto vfetch = [&](int x) {
        const int kt = x / 16, e = x % 16;
        const int row_off = (kt * 32 + 8 * (e / 4) + (e % 4)) * (D * 4);  // + 4 * half rows, in va_*
#pragma unroll
        for (int i = 0; i < T::kDTiles; ++i)
          vf[x & 1][i] = *reinterpret_cast<const float *>(Vs + ((i & 1) ? va_odd : va_even) + row_off + i * 128);
      };
      vfetch(0);
#pragma unroll
      for (int x = 0; x < kPvSteps; ++x) {
        if (x + 1 < kPvSteps) vfetch(x + 1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < T::kDTiles; ++i)
          acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[x & 1][i], s[x / 16][x % 16], acc_o[i], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    __builtin_amdgcn_s_setprio(0);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();  // next K tile visible; every wave is done reading Vs
  }
  if (CAUSAL) {
    for (int t = n_own; t < n_tiles; ++t) {
      const int kv0 = t * BC;
      load_v(kv0);
      v_landed(kv0);
      __syncthreads();
      if ((t + 1) < n_tiles) load_k(kv0 + BC);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
  }

  // ---- normalise and store: lane holds O[qrow][32*i + 8*g + 4*half + 0..3] ----
  const float l_tot = l_run + __shfl_xor(l_run, 32);
  const float inv = 1.0f / l_tot;
  if (qvalid) {
#pragma unroll
    for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        float4_t v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = acc_o[i][4 * g + e] * inv;
        *reinterpret_cast<float4_t *>(Ob + static_cast<int64_t>(qrow) * D + 32 * i + 8 * g + 4 * half) = v;
      }
  }
  }  // pass
}

template <int D, int BC, int WAVES>
static int launch_fmha_f32(const float *Q, const float *K, const float *V, float *O, int B, int H,
                           int S, float scale, int causal, hipStream_t stream,
                           kcg_launch_info *info) {
  using T = FmhaF32Tile<D, BC, WAVES>;
  const int64_t q_blocks = (static_cast<int64_t>(S) + T::kBr - 1) / T::kBr;
  const int64_t q_items = causal ? (q_blocks + 1) / 2 : q_blocks;
  const int64_t blocks = q_items * B * H;
  if (blocks > 0x7fffffffLL) return KCG_ERR_BAD_SHAPE;
  if (info) {
    *info = kcg_launch_info{};
    info->launches = 1;
    info->grid[0] = static_cast<int>(blocks);
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = T::kThreads;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = T::kLdsBytes;
    info->waves_per_block = WAVES;
    snprintf(info->kernel, sizeof info->kernel, "fmha_f32_d%d_br%d_bc%d%s", D, T::kBr, BC,
             causal ? "_causal_paired" : "");
    return KCG_OK;
  }
  const float scale_log2e = scale * 1.4426950408889634f;
#define KCG_LAUNCH(CAUSAL_)                                                                       \
  do {                                                                                            \
    auto kern = fmha_f32_kernel<D, BC, WAVES, CAUSAL_>;                                                  \
    if (!allow_lds(kern, T::kLdsBytes)) return KCG_ERR_LAUNCH;                                    \
    return launch(kern, dim3(static_cast<unsigned>(blocks)), dim3(T::kThreads), T::kLdsBytes,     \
                  stream, Q, K, V, O, S, static_cast<int>(q_blocks), static_cast<int>(q_items),     \
                  scale_log2e);                \
  } while (0)
  if (causal) KCG_LAUNCH(true);
  else KCG_LAUNCH(false);
#undef KCG_LAUNCH
}

int dispatch_fmha_f32(const float *Q, const float *K, const float *V, float *O, int B, int H, int S,
                      int D, float scale, int causal, const kcg_fmha_sched *sched,
                      hipStream_t stream, kcg_launch_info *info) {
  // Default block: 128 query rows (two workgroups per CU).  On a short non-causal sweep that
  // puts exactly one or two such workgroups on every CU for the whole launch, the older
  // workgroup of a CU outruns the younger and the launch waits for the stragglers: one
  // 256-row workgroup per CU is faster there (configs[3]: 139 against 134 TFLOP/s).  On
  // longer sweeps and on causal launches the small block measures 1-3 % faster, and far
  // faster whenever the large one would leave CUs idle.
  int br = 128, bc = 32;
  if (!causal && S <= 2048) {
    const auto items = [&](int rows) { return (static_cast<int64_t>(S) + rows - 1) / rows * B * H; };
    if (items(128) <= 2 * kNumCu && items(256) >= kNumCu) br = 256;
  }
  if (sched) {
    if (sched->br) br = sched->br;
    if (sched->bc) bc = sched->bc;
  }
  // (Br 64 x Bc 128 is the tile the reference's own table gives at Hd = 128: Br = 8192 / Hd,
  // Bc = 8192 / Br, include/KernelCodeGen.h:38-41, src/Optimizer/Optimizer.cc:1136-1144;
  // at Hd = 64 that table gives 128 x 64)
  const bool reference_tile = D == 128 && br == 64 && bc == 128;
  if (br != 128 && br != 256 && !reference_tile) return KCG_ERR_BAD_SCHEDULE;
  if (bc != 32 && bc != 64 && !reference_tile) return KCG_ERR_BAD_SCHEDULE;
#define KCG_PICK(D_, BC_, WAVES_)                \
  if (D == D_ && bc == BC_ && br == 32 * WAVES_) \
    return launch_fmha_f32<D_, BC_, WAVES_>(Q, K, V, O, B, H, S, scale, causal, stream, info);
  KCG_PICK(128, 32, 4)
  KCG_PICK(128, 32, 8)
  KCG_PICK(128, 64, 4)
  KCG_PICK(128, 128, 2)
  KCG_PICK(64, 32, 4)
  KCG_PICK(64, 32, 8)
  KCG_PICK(64, 64, 4)
  KCG_PICK(64, 64, 8)
#undef KCG_PICK
  if (D == 128 || D == 64) return KCG_ERR_BAD_SCHEDULE;
  return KCG_ERR_UNSUPPORTED_SHAPE;
}

}  // namespace kcg

extern "C" {

int kcg_fmha_f32(const float *Q, const float *K, const float *V, float *O, int32_t B, int32_t H,
                 int32_t S, int32_t D, float scale, int causal, const kcg_fmha_sched *sched,
                 void *stream) {
  if (!Q || !K || !V || !O) return KCG_ERR_NULL_POINTER;
  if (B <= 0 || H <= 0 || S <= 0 || D <= 0) return KCG_ERR_BAD_SHAPE;
  if (causal != 0 && causal != 1) return KCG_ERR_BAD_ARGUMENT;
  if (!(scale == scale)) return KCG_ERR_BAD_ARGUMENT;
  if (!kcg::aligned16(Q) || !kcg::aligned16(K) || !kcg::aligned16(V) || !kcg::aligned16(O))
    return KCG_ERR_BAD_ARGUMENT;
  // tensors of 2^31 elements and more: not verified on the GPU (see kcg_gemm_f32)
  if (static_cast<int64_t>(B) * H > 0x7fffffffLL / (static_cast<int64_t>(S) * D)) return KCG_ERR_UNSUPPORTED_SHAPE;
  return kcg::dispatch_fmha_f32(Q, K, V, O, B, H, S, D, scale, causal, sched,
                                static_cast<hipStream_t>(stream), nullptr);
}

}  // extern "C"
