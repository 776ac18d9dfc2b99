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
//  * 4 waves per workgroup, 32 query rows per wave, Br = 128, Bc = 32 (or 64).
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
//
// LDS (floats): Ks[Bc][D+4]  (b128 reads of 16 consecutive rows hit 64 banks)
//               Vs[Bc][D+8]  (rows 4 apart are 32 banks apart: the two halves of
//                             a wave read rows k and k+4 of one column block)
#include "kcg_common.h"

namespace kcg {

template <int D, int BC>
struct FmhaF32Tile {
  static constexpr int kThreads = 256;
  static constexpr int kBr = 128;
  static constexpr int kPitchK = D + 4;
  static constexpr int kPitchV = D + 8;
  static constexpr int kLdsBytes = (BC * kPitchK + BC * kPitchV) * 4;
  static constexpr int kLoads = BC * D / 4 / kThreads;  // float4 per thread per tile
  static constexpr int kKeyTiles = BC / 32;
  static constexpr int kDTiles = D / 32;
  static_assert(BC % 32 == 0 && D % 32 == 0, "tile extents");
  static_assert((BC * D / 4) % kThreads == 0, "load split");
};

template <int D, int BC, bool CAUSAL>
__global__ __launch_bounds__(256, 2) void fmha_f32_kernel(const float *__restrict__ Q,
                                                          const float *__restrict__ K,
                                                          const float *__restrict__ V,
                                                          float *__restrict__ O, int S,
                                                          int q_blocks, float scale_log2e) {
  using T = FmhaF32Tile<D, BC>;
  extern __shared__ __align__(16) float lds[];
  float *Ks = lds;
  float *Vs = lds + BC * T::kPitchK;

  // Every XCD walks a contiguous range of (head, query block) ids, head-major, so
  // the K/V of a head are fetched into one XCD's L2 only.  Heavy (late) query
  // blocks first when causal, so the tail of the grid is cheap.
  const int bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int bh = bid / q_blocks;
  const int qb_raw = bid - bh * q_blocks;
  const int qb = CAUSAL ? (q_blocks - 1 - qb_raw) : qb_raw;
  const int q0 = qb * T::kBr;

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
  float m_run = -INFINITY;  // running max of this query (both halves agree)
  float l_run = 0.0f;       // running sum over this lane's keys only

  const int kv_end = CAUSAL ? ((q0 + T::kBr) < S ? (q0 + T::kBr) : S) : S;
  const int n_tiles = (kv_end + BC - 1) / BC;

  float4_t stage[T::kLoads];
  auto load_tile = [&](const float *src, int kv0) {
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (D / 4);
      const int c4 = idx % (D / 4);
      float4_t v = {0.f, 0.f, 0.f, 0.f};
      if (kv0 + row < S)
        v = *reinterpret_cast<const float4_t *>(src + static_cast<int64_t>(kv0 + row) * D + c4 * 4);
      stage[i] = v;
    }
  };
  auto store_tile = [&](float *dst, int pitch) {
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (D / 4);
      const int c4 = idx % (D / 4);
      *reinterpret_cast<float4_t *>(dst + row * pitch + c4 * 4) = stage[i];
    }
  };

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
#pragma unroll
      for (int kk = 0; kk < D / 8; ++kk) {
        const float4_t kf = *reinterpret_cast<const float4_t *>(kp + 8 * kk);
#pragma unroll
        for (int j = 0; j < 4; ++j)
          s[kt] = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[j], q[kk][j], s[kt], 0, 0, 0);
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

    // ---- online softmax (base 2; Q carries scale * log2 e) ----
    float m_loc = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) m_loc = fmaxf(m_loc, s[kt][e]);
    m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32));
    const float m_new = fmaxf(m_run, m_loc);
    const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;  // fully masked so far
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);                 // m_run = -inf -> 0
    float psum = 0.0f;
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = __builtin_amdgcn_exp2f(s[kt][e] - m_use);
        s[kt][e] = p;
        psum += p;
      }
    l_run = l_run * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_o[i][e] *= alpha;

    store_tile(Vs, T::kPitchV);
    __syncthreads();  // V tile visible; every wave is done reading Ks

    const bool more = (t + 1) < n_tiles;
    if (more) load_tile(Kb, kv0 + BC);

    // ---- O^T += V^T . P^T  (rows = d, columns = queries, contraction over keys) ----
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float *vp = Vs + (kt * 32 + 8 * (e / 4) + 4 * half + (e % 4)) * T::kPitchV + r32;
#pragma unroll
        for (int i = 0; i < T::kDTiles; ++i)
          acc_o[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(vp[i * 32], s[kt][e], acc_o[i], 0, 0, 0);
      }
    }

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
}

template <int D, int BC>
static int launch_fmha_f32(const float *Q, const float *K, const float *V, float *O, int B, int H,
                           int S, float scale, int causal, hipStream_t stream,
                           kcg_launch_info *info) {
  using T = FmhaF32Tile<D, BC>;
  const int64_t q_blocks = (static_cast<int64_t>(S) + T::kBr - 1) / T::kBr;
  const int64_t blocks = q_blocks * B * H;
  if (blocks > 0x7fffffffLL) return KCG_ERR_BAD_SHAPE;
  if (info) {
    info->grid[0] = static_cast<int>(blocks);
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = T::kThreads;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = T::kLdsBytes;
    info->waves_per_block = 4;
    snprintf(info->kernel, sizeof info->kernel, "fmha_f32_d%d_br%d_bc%d%s", D, T::kBr, BC,
             causal ? "_causal" : "");
    return KCG_OK;
  }
  const float scale_log2e = scale * 1.4426950408889634f;
#define KCG_LAUNCH(CAUSAL_)                                                                       \
  do {                                                                                            \
    auto kern = fmha_f32_kernel<D, BC, CAUSAL_>;                                                  \
    if (!allow_lds(kern, T::kLdsBytes)) return KCG_ERR_LAUNCH;                                    \
    return launch(kern, dim3(static_cast<unsigned>(blocks)), dim3(T::kThreads), T::kLdsBytes,     \
                  stream, Q, K, V, O, S, static_cast<int>(q_blocks), scale_log2e);                \
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
  if (br != 128) return KCG_ERR_BAD_SCHEDULE;
  if (D == 128) {
    if (bc == 64) return launch_fmha_f32<128, 64>(Q, K, V, O, B, H, S, scale, causal, stream, info);
    if (bc == 32) return launch_fmha_f32<128, 32>(Q, K, V, O, B, H, S, scale, causal, stream, info);
    return KCG_ERR_BAD_SCHEDULE;
  }
  if (D == 64) {
    if (bc == 64) return launch_fmha_f32<64, 64>(Q, K, V, O, B, H, S, scale, causal, stream, info);
    if (bc == 32) return launch_fmha_f32<64, 32>(Q, K, V, O, B, H, S, scale, causal, stream, info);
    return KCG_ERR_BAD_SCHEDULE;
  }
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
