// Fused multi-head attention with bf16 inputs for gfx950 (MI355X): bf16 x bf16
// products accumulated in fp32 (v_mfma_f32_32x32x16_bf16), softmax in fp32.
//
// The reference has no bf16 type (src/Frontend/Operators.cc:5-10); this kernel
// is the bf16 counterpart of the fused kernel FMHAOptimizer builds
// (src/Optimizer/Optimizer.cc:1079-1333) for the graph BatchedMatmul(Q, K^T) ->
// Softmax -> BatchedMatmul(P, V) (test/test.cc:88-90), with the optional scale
// and causal mask.
//
// Work split: 4 waves per workgroup, QT*32 query rows per wave (Br = 128*QT),
// K/V swept in tiles of BC rows.
//
//  * S^T = K . Q^T: A operand = K rows from LDS (one ds_read_b128 = 8 bf16 of d
//    per lane), B operand = Q, held in registers for the whole sweep.  Lane
//    (r = l%32, h = l/32) ends up with S for query r and keys {8g + 4h + i}.
//  * For the 16-key block b of a 32-key tile, P elements e = 8b .. 8b+7 of that
//    lane are keys 16b + 8u + 4h + j (u = e/4 % 2, j = e%4): packed to bf16 they
//    are the B operand of O^T += V^T . P^T as they stand.  P never leaves
//    registers; max / sum / rescale are per-lane scalars.
//  * The matching A operand (V^T: row = d, 8 keys per lane) is fetched from V in
//    its natural [key][d] LDS layout with two ds_read_b64_tr_b16 per MFMA: in
//    each group of 16 lanes, source lane L addresses V[k0 + L/4][d0 + 4*(L%4)..+3]
//    and destination lane i receives keys k0..k0+3 of column d0 + i.
//
// LDS (bf16 elements): Ks[BC][D+8]   pitch = 4 banks mod 64: b128 reads of 16
//                                    consecutive rows are conflict free
//                      Vs[BC][D+32]  pitch = 16 banks mod 64: the 4 rows x 32 B
//                                    touched by one 16-lane transpose group, and
//                                    the neighbouring group 32 B further, are
//                                    bank-disjoint
#include "kcg_common.h"

namespace kcg {

typedef __bf16 bf16x8_v __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_v __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

#define KCG_LDS_BF16X4 __attribute__((address_space(3))) bf16x4_v

template <int D, int BC, int QT>
struct FmhaBf16Tile {
  static constexpr int kThreads = 256;
  static constexpr int kBr = 128 * QT;
  static constexpr int kWaveRows = 32 * QT;
  static constexpr int kPitchK = D + 8;
  static constexpr int kPitchV = D + 32;
  static constexpr int kLdsBytes = (BC * kPitchK + BC * kPitchV) * 2;
  static constexpr int kLoads = BC * D / 8 / kThreads;  // 16-byte loads per thread per tile
  static constexpr int kKeyTiles = BC / 32;
  static constexpr int kDTiles = D / 32;
  static constexpr int kDSteps = D / 16;
  static_assert(BC % 32 == 0 && D % 32 == 0, "tile extents");
  static_assert((BC * D / 8) % kThreads == 0, "load split");
};

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
  bf16x2_v r;
  r[0] = static_cast<__bf16>(a);
  r[1] = static_cast<__bf16>(b);
  return __builtin_bit_cast(unsigned, r);
}

template <int D, int BC, int QT, bool CAUSAL, bool OUT_BF16>
__global__ __launch_bounds__(256, (QT == 1 ? 2 : 1)) void fmha_bf16_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    void *__restrict__ O, int S, int q_blocks, float scale_log2e) {
  using T = FmhaBf16Tile<D, BC, QT>;
  extern __shared__ __align__(16) uint16_t lds16[];
  uint16_t *Ks = lds16;
  uint16_t *Vs = lds16 + BC * T::kPitchK;

  // Every XCD walks a contiguous range of (head, query block) ids, head-major, so
  // the K/V of a head are fetched into one XCD's L2 only; heavy (late) query
  // blocks first when causal.
  const int bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int qb_raw = bid % q_blocks;
  const int bh = bid / q_blocks;
  const int qb = CAUSAL ? (q_blocks - 1 - qb_raw) : qb_raw;
  const int q0 = qb * T::kBr;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r32 = lane & 31;
  const int half = lane >> 5;

  const int64_t base = static_cast<int64_t>(bh) * S * D;
  const uint16_t *Qb = Q + base;
  const uint16_t *Kb = K + base;
  const uint16_t *Vb = V + base;

  const int wq0 = q0 + wave * T::kWaveRows;  // first query row of this wave

  // ---- Q fragments: q[qt][s] = Q[wq0 + 32*qt + r32][16*s + 8*half .. +7] ----
  bf16x8_v q[QT][T::kDSteps];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int row = wq0 + 32 * qt + r32;
#pragma unroll
    for (int s = 0; s < T::kDSteps; ++s) {
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (row < S)
        v = *reinterpret_cast<const u32x4_t *>(Qb + static_cast<int64_t>(row) * D + 16 * s + 8 * half);
      q[qt][s] = __builtin_bit_cast(bf16x8_v, v);
    }
  }

  float16_t acc_o[QT][T::kDTiles];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt)
#pragma unroll
    for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_o[qt][i][e] = 0.0f;
  float m_run[QT], l_run[QT];
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    m_run[qt] = -INFINITY;
    l_run[qt] = 0.0f;
  }

  const int kv_end = CAUSAL ? ((q0 + T::kBr) < S ? (q0 + T::kBr) : S) : S;
  const int n_tiles = (kv_end + BC - 1) / BC;

  u32x4_t stage[T::kLoads];
  auto load_tile = [&](const uint16_t *src, int kv0) {
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (D / 8);
      const int c8 = idx % (D / 8);
      u32x4_t v = {0u, 0u, 0u, 0u};
      if (kv0 + row < S)
        v = *reinterpret_cast<const u32x4_t *>(src + static_cast<int64_t>(kv0 + row) * D + c8 * 8);
      stage[i] = v;
    }
  };
  auto store_tile = [&](uint16_t *dst, int pitch) {
#pragma unroll
    for (int i = 0; i < T::kLoads; ++i) {
      const int idx = tid + i * T::kThreads;
      const int row = idx / (D / 8);
      const int c8 = idx % (D / 8);
      *reinterpret_cast<u32x4_t *>(dst + row * pitch + c8 * 8) = stage[i];
    }
  };

  // Per-lane constant part of the V transpose-read address (elements):
  // row offset 4*half + (lane%16)/4, column 16*((lane/16)%2) + 4*(lane%4).
  const int l16 = lane & 15;
  const int vtr_off = (4 * half + (l16 >> 2)) * T::kPitchV + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);

  load_tile(Kb, 0);
  store_tile(Ks, T::kPitchK);
  __syncthreads();

  for (int t = 0; t < n_tiles; ++t) {
    const int kv0 = t * BC;
    load_tile(Vb, kv0);

    // ---- S^T = K . Q^T ----
    float16_t s[QT][T::kKeyTiles];
#pragma unroll
    for (int qt = 0; qt < QT; ++qt)
#pragma unroll
      for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) s[qt][kt][e] = 0.0f;
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt) {
      const uint16_t *kp = Ks + (kt * 32 + r32) * T::kPitchK + 8 * half;
#pragma unroll
      for (int ds = 0; ds < T::kDSteps; ++ds) {
        const bf16x8_v kf =
            __builtin_bit_cast(bf16x8_v, *reinterpret_cast<const u32x4_t *>(kp + 16 * ds));
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
          s[qt][kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, q[qt][ds], s[qt][kt], 0, 0, 0);
      }
    }

    // ---- scale, mask, online softmax (base 2) ----
    unsigned p[QT][T::kKeyTiles][8];  // bf16 pairs: word w packs P elements 2w, 2w+1
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      const int qrow = wq0 + 32 * qt + r32;
      const bool need_mask = (kv0 + BC > S) || (CAUSAL && (kv0 + BC - 1 > wq0 + 32 * qt));
#pragma unroll
      for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) s[qt][kt][e] *= scale_log2e;
      if (need_mask) {
#pragma unroll
        for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = kv0 + kt * 32 + 8 * (e / 4) + 4 * half + (e % 4);
            const bool dead = (key >= S) || (CAUSAL && key > qrow);
            if (dead) s[qt][kt][e] = -INFINITY;
          }
      }
      float m_loc = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e) m_loc = fmaxf(m_loc, s[qt][kt][e]);
      m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32));
      const float m_new = fmaxf(m_run[qt], m_loc);
      const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_use);
      float psum = 0.0f;
#pragma unroll
      for (int kt = 0; kt < T::kKeyTiles; ++kt) {
#pragma unroll
        for (int e = 0; e < 16; e += 2) {
          const float p0 = __builtin_amdgcn_exp2f(s[qt][kt][e] - m_use);
          const float p1 = __builtin_amdgcn_exp2f(s[qt][kt][e + 1] - m_use);
          psum += p0 + p1;
          p[qt][kt][e / 2] = pack_bf16(p0, p1);
        }
      }
      l_run[qt] = l_run[qt] * alpha + psum;
      m_run[qt] = m_new;
#pragma unroll
      for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc_o[qt][i][e] *= alpha;
    }

    store_tile(Vs, T::kPitchV);
    __syncthreads();  // V tile visible; every wave is done reading Ks

    const bool more = (t + 1) < n_tiles;
    if (more) load_tile(Kb, kv0 + BC);

    // ---- O^T += V^T . P^T ----
#pragma unroll
    for (int kt = 0; kt < T::kKeyTiles; ++kt) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const uint16_t *vp = Vs + (kt * 32 + 16 * b) * T::kPitchV + vtr_off;
#pragma unroll
        for (int i = 0; i < T::kDTiles; ++i) {
          const bf16x4_v lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (KCG_LDS_BF16X4 *)(vp + 32 * i));
          const bf16x4_v hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (KCG_LDS_BF16X4 *)(vp + 8 * T::kPitchV + 32 * i));
          const bf16x8_v vf = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
          for (int qt = 0; qt < QT; ++qt) {
            const u32x4_t pw = {p[qt][kt][4 * b], p[qt][kt][4 * b + 1], p[qt][kt][4 * b + 2],
                                p[qt][kt][4 * b + 3]};
            acc_o[qt][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                vf, __builtin_bit_cast(bf16x8_v, pw), acc_o[qt][i], 0, 0, 0);
          }
        }
      }
    }

    if (more) store_tile(Ks, T::kPitchK);
    __syncthreads();  // next K tile visible; every wave is done reading Vs
  }

  // ---- normalise and store: lane holds O[qrow][32*i + 8*g + 4*half + 0..3] ----
#pragma unroll
  for (int qt = 0; qt < QT; ++qt) {
    const int qrow = wq0 + 32 * qt + r32;
    const float l_tot = l_run[qt] + __shfl_xor(l_run[qt], 32);
    const float inv = 1.0f / l_tot;
    if (qrow < S) {
      const int64_t off = base + static_cast<int64_t>(qrow) * D + 4 * half;
#pragma unroll
      for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float v0 = acc_o[qt][i][4 * g + 0] * inv;
          const float v1 = acc_o[qt][i][4 * g + 1] * inv;
          const float v2 = acc_o[qt][i][4 * g + 2] * inv;
          const float v3 = acc_o[qt][i][4 * g + 3] * inv;
          if (OUT_BF16) {
            u32x2_t w = {pack_bf16(v0, v1), pack_bf16(v2, v3)};
            *reinterpret_cast<u32x2_t *>(static_cast<uint16_t *>(O) + off + 32 * i + 8 * g) = w;
          } else {
            float4_t w = {v0, v1, v2, v3};
            *reinterpret_cast<float4_t *>(static_cast<float *>(O) + off + 32 * i + 8 * g) = w;
          }
        }
    }
  }
}

template <int D, int BC, int QT>
static int launch_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O,
                            int o_dtype, int B, int H, int S, float scale, int causal,
                            hipStream_t stream, kcg_launch_info *info) {
  using T = FmhaBf16Tile<D, BC, QT>;
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
    snprintf(info->kernel, sizeof info->kernel, "fmha_bf16_d%d_br%d_bc%d%s", D, T::kBr, BC,
             causal ? "_causal" : "");
    return KCG_OK;
  }
  const float scale_log2e = scale * 1.4426950408889634f;
#define KCG_LAUNCH(CAUSAL_, OBF_)                                                                 \
  do {                                                                                            \
    auto kern = fmha_bf16_kernel<D, BC, QT, CAUSAL_, OBF_>;                                       \
    if (!allow_lds(kern, T::kLdsBytes)) return KCG_ERR_LAUNCH;                                    \
    return launch(kern, dim3(static_cast<unsigned>(blocks)), dim3(T::kThreads), T::kLdsBytes,     \
                  stream, Q, K, V, O, S, static_cast<int>(q_blocks), scale_log2e);                \
  } while (0)
  const bool obf = o_dtype == KCG_BF16;
  if (causal) {
    if (obf) KCG_LAUNCH(true, true);
    else KCG_LAUNCH(true, false);
  } else {
    if (obf) KCG_LAUNCH(false, true);
    else KCG_LAUNCH(false, false);
  }
#undef KCG_LAUNCH
}

int dispatch_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O,
                       int o_dtype, int B, int H, int S, int D, float scale, int causal,
                       const kcg_fmha_sched *sched, hipStream_t stream, kcg_launch_info *info) {
  int br = 128, bc = 64;
  if (sched) {
    if (sched->br) br = sched->br;
    if (sched->bc) bc = sched->bc;
  }
  if (bc != 64) return KCG_ERR_BAD_SCHEDULE;
  if (D == 128) {
    if (br == 128)
      return launch_fmha_bf16<128, 64, 1>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);
    if (br == 256)
      return launch_fmha_bf16<128, 64, 2>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);
    return KCG_ERR_BAD_SCHEDULE;
  }
  if (D == 64) {
    if (br == 128)
      return launch_fmha_bf16<64, 64, 1>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);
    if (br == 256)
      return launch_fmha_bf16<64, 64, 2>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);
    return KCG_ERR_BAD_SCHEDULE;
  }
  return KCG_ERR_UNSUPPORTED_SHAPE;
}

}  // namespace kcg

extern "C" {

int kcg_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O, int o_dtype,
                  int32_t B, int32_t H, int32_t S, int32_t D, float scale, int causal,
                  const kcg_fmha_sched *sched, void *stream) {
  if (!Q || !K || !V || !O) return KCG_ERR_NULL_POINTER;
  if (B <= 0 || H <= 0 || S <= 0 || D <= 0) return KCG_ERR_BAD_SHAPE;
  if (causal != 0 && causal != 1) return KCG_ERR_BAD_ARGUMENT;
  if (o_dtype != KCG_BF16 && o_dtype != KCG_F32) return KCG_ERR_BAD_ARGUMENT;
  if (!(scale == scale)) return KCG_ERR_BAD_ARGUMENT;
  if (!kcg::aligned16(Q) || !kcg::aligned16(K) || !kcg::aligned16(V) || !kcg::aligned16(O))
    return KCG_ERR_BAD_ARGUMENT;
  return kcg::dispatch_fmha_bf16(Q, K, V, O, o_dtype, B, H, S, D, scale, causal, sched,
                                 static_cast<hipStream_t>(stream), nullptr);
}

}  // extern "C"
