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
//  * K and V tiles are staged in padded LDS in their global layout; the next
//    tile's global loads are issued before the MFMA phase that hides them
//    (V_t during S = K_t.Q, K_{t+1} during O += P.V_t).
//  * The running maximum is a lazily raised reference (see kTau): VALU work between
//    the two MFMA phases costs matrix time, so the rescale of O is skipped whenever
//    the mathematics allows it.
//  * Causal: a workgroup runs the query-block pair (n-1-i, i), so all workgroups
//    sweep the same number of tiles.
//
// LDS (floats): Ks[Bc][D+4]  (b128 reads of 16 consecutive rows hit 64 banks)
//               Vs[Bc][D+8]  (rows 4 apart are 32 banks apart: the two halves of
//                             a wave read rows k and k+4 of one column block)
#include "kcg_common.h"

namespace kcg {

template <int D, int BC, int WAVES>
struct FmhaF32Tile {
  static constexpr int kThreads = 64 * WAVES;
  static constexpr int kBr = 32 * WAVES;
  static constexpr int kPitchK = D + 4;
  static constexpr int kPitchV = D + 8;
  static constexpr int kLdsBytes = (BC * kPitchK + BC * kPitchV) * 4;
  static constexpr int kLoads = BC * D / 4 / kThreads;  // float4 per thread per tile
  static constexpr int kKeyTiles = BC / 32;
  static constexpr int kDTiles = D / 32;
  static_assert(BC % 32 == 0 && D % 32 == 0, "tile extents");
  static_assert((BC * D / 4) % kThreads == 0, "load split");
};

// How far (in log2 units) a tile's row maximum may exceed the running reference before
// the accumulators are rescaled.
constexpr float kTau = 8.0f;

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

// max over both halves of the wave for the same lane%32 (one v_permlane32_swap)
__device__ __forceinline__ float max_across_halves(float x) {
  const unsigned u = __builtin_bit_cast(unsigned, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, r[0]), __builtin_bit_cast(float, r[1]));
}

template <int D, int BC, int WAVES, bool CAUSAL>
__global__ __launch_bounds__(64 * WAVES, 8 / WAVES) void fmha_f32_kernel(const float *__restrict__ Q,
                                                          const float *__restrict__ K,
                                                          const float *__restrict__ V,
                                                          float *__restrict__ O, int S,
                                                          int q_blocks, int q_items, float scale_log2e) {
  using T = FmhaF32Tile<D, BC, WAVES>;
  extern __shared__ __align__(16) float lds[];
  float *Ks = lds;
  float *Vs = lds + BC * T::kPitchK;

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
  const int wave = tid >> 6;
  const int r32 = lane & 31;
  const int half = lane >> 5;

  const int64_t base = static_cast<int64_t>(bh) * S * D;
  const float *Qb = Q + base;
  const float *Kb = K + base;
  const float *Vb = V + base;
  float *Ob = O + base;


  // Tile transfer: thread -> (row ld_row + i * kRowsPerIter, 16-byte column ld_c4).  A full
  // tile is fetched with a uniform base (scalar registers) plus one per-lane byte offset;
  // only the ragged last tile pays for per-row predicates (rows at and beyond S read as 0).
  constexpr int kRowsPerIter = T::kThreads / (D / 4);
  const int ld_row = tid / (D / 4);
  const int ld_c4 = tid % (D / 4);
  const unsigned ld_off = static_cast<unsigned>(ld_row * D + ld_c4 * 4) * 4u;
  float4_t stage[T::kLoads];
  auto load_tile = [&](const float *src, int kv0) {
    const char *g = reinterpret_cast<const char *>(src + static_cast<int64_t>(kv0) * D);
    if (kv0 + BC <= S) {
#pragma unroll
      for (int i = 0; i < T::kLoads; ++i)
        stage[i] = *reinterpret_cast<const float4_t *>(g + i * (kRowsPerIter * D * 4) + ld_off);
    } else {
#pragma unroll
      for (int i = 0; i < T::kLoads; ++i) {
        float4_t v = {0.f, 0.f, 0.f, 0.f};
        if (kv0 + ld_row + i * kRowsPerIter < S)
          v = *reinterpret_cast<const float4_t *>(g + i * (kRowsPerIter * D * 4) + ld_off);
        stage[i] = v;
      }
    }
  };
  auto store_tile = [&](float *dst, int pitch) {
    float *d = dst + ld_row * pitch + ld_c4 * 4;
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i)
      *reinterpret_cast<float4_t *>(d + i * kRowsPerIter * pitch) = stage[i];
  };

#pragma unroll 1
  for (int pass = 0; pass < npass; ++pass) {
  const int qb = CAUSAL ? (pass == 0 ? hi_block : item) : item;  // the long block first
  const int q0 = qb * T::kBr;
  const int qrow = q0 + wave * 32 + r32;  // this lane's query
  const bool qvalid = qrow < S;

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

  load_tile(Kb, 0);
  store_tile(Ks, T::kPitchK);
  __syncthreads();

  for (int t = 0; t < n_tiles; ++t) {
    const int kv0 = t * BC;
    load_tile(Vb, kv0);

    // ---- S^T = K . Q^T  (rows = keys, columns = queries) ----
    float16_t s[T::kKeyTiles];
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kt][e] = 0.0f;
      const float *kp = Ks + (kt * 32 + r32) * T::kPitchK + 4 * half;
      // the K fragment of the next 8 d-columns is requested before the four MFMAs of the
      // current one are issued
      float4_t kf[2];
      kf[0] = *reinterpret_cast<const float4_t *>(kp);
#pragma unroll
      for (int kk = 0; kk < D / 8; ++kk) {
        if (kk + 1 < D / 8) kf[(kk + 1) & 1] = *reinterpret_cast<const float4_t *>(kp + 8 * (kk + 1));
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

    store_tile(Vs, T::kPitchV);
    __syncthreads();  // V tile visible; every wave is done reading Ks

    const bool more = (t + 1) < n_tiles;
    if (more) load_tile(Kb, kv0 + BC);

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
        const float *vp = Vs + (kt * 32 + 8 * (e / 4) + 4 * half + (e % 4)) * T::kPitchV + r32;
#pragma unroll
        for (int i = 0; i < T::kDTiles; ++i) vf[x & 1][i] = vp[i * 32];
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
    if (more) store_tile(Ks, T::kPitchK);
    __syncthreads();  // next K tile visible; every wave is done reading Vs
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
  int br = 128, bc = 32;
  if (sched) {
    if (sched->br) br = sched->br;
    if (sched->bc) bc = sched->bc;
  }
  if (br != 128 && br != 256) return KCG_ERR_BAD_SCHEDULE;
  if (bc != 32 && bc != 64) return KCG_ERR_BAD_SCHEDULE;
#define KCG_PICK(D_, BC_, WAVES_)                \
  if (D == D_ && bc == BC_ && br == 32 * WAVES_) \
    return launch_fmha_f32<D_, BC_, WAVES_>(Q, K, V, O, B, H, S, scale, causal, stream, info);
  KCG_PICK(128, 32, 4)
  KCG_PICK(128, 32, 8)
  KCG_PICK(128, 64, 4)
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
  return kcg::dispatch_fmha_f32(Q, K, V, O, B, H, S, D, scale, causal, sched,
                                static_cast<hipStream_t>(stream), nullptr);
}

}  // extern "C"
