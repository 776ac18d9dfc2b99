// Fused multi-head attention with bf16 inputs for gfx950 (MI355X): bf16 x bf16
// products accumulated in fp32 (v_mfma_f32_32x32x16_bf16), softmax in fp32.
//
// The reference has no bf16 type (src/Frontend/Operators.cc:5-10); this kernel
// is the bf16 counterpart of the fused kernel FMHAOptimizer builds
// (src/Optimizer/Optimizer.cc:1079-1333) for the graph BatchedMatmul(Q, K^T) ->
// Softmax -> BatchedMatmul(P, V) (test/test.cc:88-90), with the optional scale
// and causal mask.
//
// Two kernels: fmha_bf16_kernel (described first; 4 waves, 128 query rows, also the general
// softmax path for scale <= 0) and fmha_bf16_pp_kernel (8 waves, 256 query rows, its own
// header further down), which long sequences that fill the chip take.
//
// Work split: WAVES (4 or 8) waves per workgroup, 32 query rows per wave
// (Br = 128 or 256), K/V swept in tiles of BC = 64 rows.
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
//  * K/V tiles go from global memory straight into LDS (global_load_lds_dwordx4,
//    no staging registers, no LDS store instructions): one wave instruction fills
//    1024 consecutive LDS bytes, lane L supplying the 16-byte chunk that belongs
//    at position L.  Rows are therefore unpadded; bank conflicts are avoided by
//    an XOR swizzle of the 16-byte chunk index, applied to the *global* address
//    when loading and to the LDS address when reading:
//        K: chunk c of row r sits at c ^ fk(r)   (16 consecutive rows, same c,
//                                                  hit 16 distinct 16-byte slots)
//        V: chunk c of row r sits at c ^ fv(r)   (the 4 rows x 32 B of one
//                                                  16-lane transpose group, and
//                                                  the neighbouring group, are
//                                                  slot-disjoint)
//    The buffers are double-buffered: tile t+1 streams in while tile t is
//    consumed; each wave waits for its own loads (vmcnt) before the single
//    barrier that ends the step.
//  * Online softmax in base 2 with a lazy rescale: the running reference maximum
//    of a row is only raised (and O, l rescaled) when the tile maximum exceeds it
//    by more than kTau; exp2(s*c - m) is one FMA + v_exp_f32; row sums use
//    v_dot2c_f32_bf16 on the packed P.
//  * Causal: a workgroup runs the query-block pair (n-1-i, i), so all workgroups
//    sweep the same number of tiles; tiles above a wave's last row are skipped.
#include <type_traits>

#include "kcg_common.h"

namespace kcg {

typedef __bf16 bf16x8_v __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_v __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2_v __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));

#define KCG_LDS_BF16X4 __attribute__((address_space(3))) bf16x4_v
#define KCG_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define KCG_LDS_PTR(p) ((__attribute__((address_space(3))) void *)(p))

template <int D, int BC, int QT, int WAVES>
struct FmhaBf16Tile {
  static constexpr int kThreads = 64 * WAVES;
  static constexpr int kBr = 32 * QT * WAVES;
  static constexpr int kWaveRows = 32 * QT;
  static constexpr int kCpr = D / 8;            // 16-byte chunks per row
  static constexpr int kRowsPer256 = 16 / kCpr;  // rows that share one 256-byte bank window
  static constexpr int kRpi = 64 / kCpr;         // rows filled by one wave-wide direct load
  static constexpr int kIpw = BC / kRpi / WAVES;  // direct loads per wave per tile
  static constexpr int kTile = BC * D;           // elements per K (or V) buffer, unpadded
  // K/V tile buffers: a ring of 2 (tile t+1 streams in while tile t is consumed).  A ring
  // of 3 with loads two tiles ahead was measured slower for the 8-wave workgroup.
  static constexpr int kRing = 2;
  static constexpr int kAheadTiles = kRing - 1;
  static constexpr int kLdsBytes = kRing * 2 * kTile * 2;
  static constexpr int kKeyTiles = BC / 32;
  static constexpr int kDTiles = D / 32;
  static constexpr int kDSteps = D / 16;
  static_assert(D == 64 || D == 128, "head dim");
  static_assert(BC % (WAVES * kRpi) == 0 && BC % 32 == 0, "tile extents");
  // chunk-index swizzles (see the file header)
  __host__ __device__ static constexpr int fk(int row) { return (row / kRowsPer256) % kCpr; }
  __host__ __device__ static constexpr int fv(int row) { return 4 * ((row / kRowsPer256) & (kCpr / 4 - 1)); }
};

__device__ __forceinline__ unsigned pack_bf16(float a, float b) {
  bf16x2_v r;
  r[0] = static_cast<__bf16>(a);
  r[1] = static_cast<__bf16>(b);
  return __builtin_bit_cast(unsigned, r);
}

// a.x + a.y + acc for a packed bf16 pair (v_dot2c_f32_bf16 with a pair of ones).
__device__ __forceinline__ float add_bf16_pair(unsigned pair, float acc) {
  const bf16x2_v ones = {static_cast<__bf16>(1.0f), static_cast<__bf16>(1.0f)};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_v, pair), ones, acc, false);
}

// How far (in log2 units) a tile's row maximum may exceed the running reference
// before the accumulators are rescaled.  Between rescales P is at most 2^kTau,
// harmless for bf16 P (relative precision is scale free) and fp32 sums; the final
// O / l normalisation is exact for any reference.
constexpr float kTau = 8.0f;

// POS_SCALE: scale > 0, so exp2(s * c - m) is one FMA and the row maximum can be
// taken on the raw products.  The general variant scales first.
template <int D, int BC, int QT, int WAVES, bool CAUSAL, bool OUT_BF16, bool POS_SCALE>
__global__ __launch_bounds__(64 * WAVES, (QT == 1 && WAVES > 2 ? 2 : 1)) void fmha_bf16_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    void *__restrict__ O, int S, int q_blocks, int q_items, float scale_log2e) {
  using T = FmhaBf16Tile<D, BC, QT, WAVES>;
  extern __shared__ __align__(16) uint16_t lds16[];
  uint16_t *Ks = lds16;                  // [kRing][BC][D], chunk-swizzled
  uint16_t *Vs = lds16 + T::kRing * T::kTile;   // [kRing][BC][D], chunk-swizzled

  // Every XCD walks a contiguous range of (head, work item) ids, head-major, so
  // the K/V of a head are fetched into one XCD's L2 only.  Causal: a work item is
  // the pair of query blocks (n-1-i, i), so every workgroup sweeps the same
  // number of K/V tiles and the grid has no heavy tail.
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
  const uint16_t *Qb = Q + base;
  const uint16_t *Kb = K + base;
  const uint16_t *Vb = V + base;

  // ---- direct global -> LDS tile loads ----
  // Wave instruction j of this wave fills LDS rows ld_row0 + j*kRpi .. +kRpi-1; lane L
  // sits at row ld_row0 + j*kRpi + L / kCpr, chunk position L % kCpr, and fetches the
  // global chunk (position ^ swizzle(row)) of that row.
  const int ld_row0 = wave * T::kIpw * T::kRpi;
  const int ld_lrow = lane / T::kCpr;
  const int ld_pos = lane % T::kCpr;
  unsigned goff_k[T::kIpw], goff_v[T::kIpw];  // byte offsets inside a tile, per instruction
#pragma unroll
  for (int j = 0; j < T::kIpw; ++j) {
    const int row = ld_row0 + j * T::kRpi + ld_lrow;
    goff_k[j] = static_cast<unsigned>(row * D + (ld_pos ^ T::fk(row)) * 8) * 2u;
    goff_v[j] = static_cast<unsigned>(row * D + (ld_pos ^ T::fv(row)) * 8) * 2u;
  }
  // One direct load (K for even `which`, V for odd) of the tile at kv0 into buffer `buf`:
  // uniform 64-bit tile base + per-lane 32-bit byte offset.
  auto load_one = [&](int kv0, int buf, int which) {
    const int j = which >> 1;
    const char *g = reinterpret_cast<const char *>(((which & 1) ? Vb : Kb) + static_cast<int64_t>(kv0) * D);
    uint16_t *l = ((which & 1) ? Vs : Ks) + buf * T::kTile + (ld_row0 + j * T::kRpi) * D;
    const unsigned off = (which & 1) ? goff_v[j] : goff_k[j];
    __builtin_amdgcn_global_load_lds(KCG_GLOBAL_PTR(g + off), KCG_LDS_PTR(l), 16, 0, 0);
  };
  // Ragged last tile: rows at and beyond S are zero-filled, through registers.
  auto load_tiles_ragged = [&](int kv0, int buf) {
    const char *kg = reinterpret_cast<const char *>(Kb + static_cast<int64_t>(kv0) * D);
    const char *vg = reinterpret_cast<const char *>(Vb + static_cast<int64_t>(kv0) * D);
    uint16_t *kl = Ks + buf * T::kTile + ld_row0 * D;
    uint16_t *vl = Vs + buf * T::kTile + ld_row0 * D;
#pragma unroll
    for (int j = 0; j < T::kIpw; ++j) {
      const int row = ld_row0 + j * T::kRpi + ld_lrow;
      const bool ok = kv0 + row < S;
      const u32x4_t z = {0u, 0u, 0u, 0u};
      const u32x4_t kvq = ok ? *reinterpret_cast<const u32x4_t *>(kg + goff_k[j]) : z;
      const u32x4_t vvq = ok ? *reinterpret_cast<const u32x4_t *>(vg + goff_v[j]) : z;
      *reinterpret_cast<u32x4_t *>(kl + (j * T::kRpi + ld_lrow) * D + ld_pos * 8) = kvq;
      *reinterpret_cast<u32x4_t *>(vl + (j * T::kRpi + ld_lrow) * D + ld_pos * 8) = vvq;
    }
  };
  auto load_tiles = [&](int kv0, int buf) {
    if (kv0 + BC <= S) {
#pragma unroll
      for (int w = 0; w < 2 * T::kIpw; ++w) load_one(kv0, buf, w);
    } else {
      load_tiles_ragged(kv0, buf);
    }
  };
  // Every wave waits for its own direct loads; the barrier then publishes all of them.
  // `in_flight` = direct loads this wave may leave outstanding (those of tiles further
  // ahead than the next one).
  auto tiles_ready = [&](bool keep_newest) {
    if (keep_newest) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * T::kIpw) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };

  // ---- per-lane read addresses (elements), swizzle folded in ----
  // K fragment of d-step ds: row r32 (+32*kt), chunk (2*ds + half) ^ fk(row)
  const int k_row_off = r32 * D;
  const int k_swz = T::fk(r32) ^ half;  // chunk position = (2*ds) ^ k_swz
  // V transpose read: row 4*half + (lane%16)/4 (+8u + 16b + 32kt), column
  // 32*i + 16*((lane/16)%2) + 4*(lane%4): chunk 4*i + (v_c0 ^ ...), 8-byte half v_sub
  const int l16 = lane & 15;
  const int v_lrow = 4 * half + (l16 >> 2);
  const int v_c0 = (2 * ((lane >> 4) & 1) + ((l16 & 3) >> 1)) ^ T::fv(v_lrow);  // chunk = (4*i) ^ v_c0
  const int v_sub = 4 * (l16 & 1);
  const int v_row_off = v_lrow * D + v_sub;

#pragma unroll 1
  for (int pass = 0; pass < npass; ++pass) {
    // the long block goes first: the long sweeps of a head's workgroups then start together
    // and share each K/V tile in L2 (short-first was measured to fetch 26% more)
    const int qb = CAUSAL ? (pass == 0 ? hi_block : item) : item;
    const int q0 = qb * T::kBr;
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
    float m_ref[QT], l_run[QT];  // reference maximum (log2 units), this lane's share of the row sum
#pragma unroll
    for (int qt = 0; qt < QT; ++qt) {
      m_ref[qt] = -INFINITY;
      l_run[qt] = 0.0f;
    }

    const int kv_end = CAUSAL ? ((q0 + T::kBr) < S ? (q0 + T::kBr) : S) : S;
    const int n_tiles = (kv_end + BC - 1) / BC;

    load_tiles(0, 0);
    if (T::kAheadTiles > 1 && n_tiles > 1) load_tiles(BC, 1);
    tiles_ready(false);

    for (int t = 0; t < n_tiles; ++t) {
      const int kv0 = t * BC;
      const int cur = t % T::kRing;
      const int nxt = (t + T::kAheadTiles) % T::kRing;  // buffer of the tile fetched in this step
      // the next tile streams in while this one is computed; when it is a full tile its
      // direct loads are issued one per d-step, between the MFMAs of S = K.Q^T
      const bool more = t + T::kAheadTiles < n_tiles;
      const int kv_nxt = kv0 + T::kAheadTiles * BC;
      const bool spread = more && (kv_nxt + BC <= S);
      if (more && !spread) load_tiles(kv_nxt, nxt);

      // A wave whose last query precedes the tile has nothing to add (causal).
      const bool wave_active = !CAUSAL || (kv0 <= wq0 + T::kWaveRows - 1);
      if (spread && !wave_active) load_tiles(kv_nxt, nxt);
      if (wave_active) {
        const uint16_t *ks = Ks + cur * T::kTile + k_row_off;
        const uint16_t *vs = Vs + cur * T::kTile + v_row_off;

        // ---- S^T = K . Q^T ----
        float16_t s[QT][T::kKeyTiles];
#pragma unroll
        for (int qt = 0; qt < QT; ++qt)
#pragma unroll
          for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
            for (int e = 0; e < 16; ++e) s[qt][kt][e] = 0.0f;
        {
          // K fragments are requested two d-steps ahead of the MFMAs that use them
          constexpr int kAhead = 2;
          bf16x8_v kf[T::kDSteps][T::kKeyTiles];
          auto fetch = [&](int ds) {
#pragma unroll
            for (int kt = 0; kt < T::kKeyTiles; ++kt)
              kf[ds][kt] = __builtin_bit_cast(
                  bf16x8_v, *reinterpret_cast<const u32x4_t *>(ks + kt * 32 * D + ((2 * ds) ^ k_swz) * 8));
          };
#pragma unroll
          for (int ds = 0; ds < kAhead; ++ds) fetch(ds);
#pragma unroll
          for (int ds = 0; ds < T::kDSteps; ++ds) {
            if (ds + kAhead < T::kDSteps) fetch(ds + kAhead);
            // (one direct load per d-step in the 4- and 8-wave tiles; the two-wave 64 x 128
            // tile has four times as many loads per wave)
            constexpr int kLoadsPerDs = (2 * T::kIpw + T::kDSteps - 1) / T::kDSteps;
#pragma unroll
            for (int j = 0; j < kLoadsPerDs; ++j)
              if (ds * kLoadsPerDs + j < 2 * T::kIpw && spread) load_one(kv_nxt, nxt, ds * kLoadsPerDs + j);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
              for (int qt = 0; qt < QT; ++qt)
                s[qt][kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ds][kt], q[qt][ds], s[qt][kt], 0, 0, 0);
          }
        }

        // ---- mask, online softmax (base 2, lazy rescale) ----
        unsigned p[QT][T::kKeyTiles][8];  // bf16 pairs: word w packs P elements 2w, 2w+1
#pragma unroll
        for (int qt = 0; qt < QT; ++qt) {
          const int qrow = wq0 + 32 * qt + r32;
          const bool need_mask = (kv0 + BC > S) || (CAUSAL && (kv0 + BC - 1 > wq0 + 32 * qt));
          if (POS_SCALE) {
            // fast path: exp2(s * c - m) as one FMA; the maximum is taken on raw S
            if (need_mask) {
              // element (kt, e) is key kv0 + 4*half + off, off = 32*kt + 8*(e/4) + e%4;
              // it is dead when off > lim
              const int last = CAUSAL ? (qrow < S - 1 ? qrow : S - 1) : (S - 1);
              const int lim = last - kv0 - 4 * half;
#pragma unroll
              for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
                for (int e = 0; e < 16; ++e)
                  if (32 * kt + 8 * (e / 4) + (e % 4) > lim) s[qt][kt][e] = -INFINITY;
            }
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
              for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[qt][kt][e]);
            float m_loc = mx * scale_log2e;  // -inf stays -inf
            m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32));
            // per-row decision: a row's result never depends on what other rows do
            if (m_loc > m_ref[qt] + kTau) {
              const float m_new = fmaxf(m_ref[qt], m_loc);
              const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
              const float alpha = __builtin_amdgcn_exp2f(m_ref[qt] - m_use);  // m_ref = -inf -> 0
              l_run[qt] *= alpha;
              m_ref[qt] = m_new;
#pragma unroll
              for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
                for (int e = 0; e < 16; ++e) acc_o[qt][i][e] *= alpha;
            }
            const float neg_m = (m_ref[qt] == -INFINITY) ? 0.0f : -m_ref[qt];
            float psum = 0.0f;
#pragma unroll
            for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
              for (int w = 0; w < 8; ++w) {
                const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[qt][kt][2 * w], scale_log2e, neg_m));
                const float p1 =
                    __builtin_amdgcn_exp2f(__builtin_fmaf(s[qt][kt][2 * w + 1], scale_log2e, neg_m));
                const unsigned pk = pack_bf16(p0, p1);
                p[qt][kt][w] = pk;
                psum = add_bf16_pair(pk, psum);
              }
            l_run[qt] += psum;
          } else {
            // general path (scale <= 0): scale first, then mask and maximum
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
                  if ((key >= S) || (CAUSAL && key > qrow)) s[qt][kt][e] = -INFINITY;
                }
            }
            float m_loc = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
              for (int e = 0; e < 16; ++e) m_loc = fmaxf(m_loc, s[qt][kt][e]);
            m_loc = fmaxf(m_loc, __shfl_xor(m_loc, 32));
            const float m_new = fmaxf(m_ref[qt], m_loc);
            const float m_use = (m_new == -INFINITY) ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_ref[qt] - m_use);
            float psum = 0.0f;
#pragma unroll
            for (int kt = 0; kt < T::kKeyTiles; ++kt)
#pragma unroll
              for (int w = 0; w < 8; ++w) {
                const float p0 = __builtin_amdgcn_exp2f(s[qt][kt][2 * w] - m_use);
                const float p1 = __builtin_amdgcn_exp2f(s[qt][kt][2 * w + 1] - m_use);
                const unsigned pk = pack_bf16(p0, p1);
                p[qt][kt][w] = pk;
                psum = add_bf16_pair(pk, psum);
              }
            l_run[qt] = l_run[qt] * alpha + psum;
            m_ref[qt] = m_new;
#pragma unroll
            for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
              for (int e = 0; e < 16; ++e) acc_o[qt][i][e] *= alpha;
          }
        }

        // ---- O^T += V^T . P^T ----
#pragma unroll
        for (int kt = 0; kt < T::kKeyTiles; ++kt) {
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            const uint16_t *vp = vs + (kt * 32 + 16 * b) * D;
#pragma unroll
            for (int i = 0; i < T::kDTiles; ++i) {
              const int col = ((4 * i) ^ v_c0) * 8;
              const bf16x4_v lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((KCG_LDS_BF16X4 *)(vp + col));
              const bf16x4_v hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((KCG_LDS_BF16X4 *)(vp + 8 * D + col));
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
      }

      // the next tile is complete and visible after this; with a ring of 3 the loads of
      // the tile after it (issued in this step, when direct) stay in flight
      tiles_ready(T::kAheadTiles > 1 && spread);
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
}

// ---------------------------------------------------------------------------
// Ping-pong kernel: 8 waves, 256 query rows, two groups of four waves half a
// tile apart; one workgroup per CU walks its share of the launch as one stream
// of K/V tiles.
//
// A wave64 VALU instruction issued beside the MFMAs of the *other* wave of its SIMD
// costs that wave nothing (measured: the MFMA wave keeps one MFMA per 32 clocks), but
// two waves that are in the same phase only contend: both wait for the matrix pipe,
// then both for the vector ALU.  Waves w and w + 4 share a SIMD, so group 1 (waves
// 4-7) runs one interval behind group 0 (waves 0-3), and every workgroup barrier ends
// an interval:
//
//   interval     2t             2t+1           2t+2              2t+3
//   group 0      PV(t-1), S(t)  softmax(t)     PV(t), S(t+1)     softmax(t+1)
//   group 1      softmax(t-1)   PV(t-1), S(t)  softmax(t)        PV(t), S(t+1)
//
//  * In its matrix interval a wave is alone on the SIMD's matrix pipe, so nothing hides
//    the latency of its LDS operand reads but the wave itself: the 32 MFMAs of an
//    interval take their A operands from a queue of eight fragments that is refilled
//    eight MFMAs ahead; the first eight are requested at the start of the softmax
//    interval and arrive under its arithmetic.
//  * The kernel runs at the socket's power limit, and what it buys there is fewer
//    instructions per tile.  Softmax per tile and lane (32 scores): one FMA + v_exp per
//    score (exp2(s * c - m), c = scale * log2(e)), 16 v_cvt_pk, 16 v_dot2c for the row sum
//    and one half-wave exchange -- and no row maximum: the exponentials are taken
//    against the reference the row already has, and only when the row sum shows that
//    one of them exceeded 2^kTau (or on the row's first tile) is the maximum computed,
//    the reference raised and the tile redone.  Q stays unscaled: scaling it once and
//    rounding it to bf16 again would save the FMAs but more than doubles the error
//    against the fp32 evaluation.
//  * K tiles live in a ring of 4 LDS buffers, V tiles in a ring of 5; the tile three
//    steps ahead is requested at the start of the softmax interval (direct global -> LDS
//    loads issued from assembly), when both groups are done with the buffers it
//    replaces.  All vector memory waits are counted by hand (wait_vm): the compiler
//    would wait for every outstanding load before each LDS read or use of Q.
//  * The K/V tiles of all query blocks a workgroup handles -- both blocks of a causal
//    pair, then the next work item, possibly of another head -- follow each other in one
//    stream, so the pipeline is filled once per workgroup; the Q rows of the next block
//    are requested right after the last S of the current one.
//
// Build-time experiment switches (all off in the library; `make variants` builds one library
// per switch, `bench.py --sweep fmha-variants` times them against the default in one job).
// Each is a lever on the causal sweep that was built, measured and not adopted:
//   KCG_FMHA_EXP_ALL_PAIRS      waves also compute the diagonal tiles that lie wholly above
//                               their rows (every score masked) instead of skipping them:
//                               the tile loop then has no causal control flow at all.
//   KCG_FMHA_EXP_LO_DESCENDING  the short block of a causal pair sweeps its tiles from the
//                               diagonal down to tile 0, which puts all workgroups of a head
//                               on the same K/V tile at the same time during that pass.
//   KCG_FMHA_EXP_STAGE_O        the O rows of a pass leave through a 2 KiB LDS staging area per
//                               wave as 64-byte row pieces (16 cache lines per store
//                               instruction instead of 32 with 16 bytes each).
template <int D>
struct FmhaPpTile {
  static constexpr int kWaves = 8;
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int kBr = 32 * kWaves;
  static constexpr int kBc = 64;
  static constexpr int kCpr = D / 8;             // 16-byte chunks per row
  static constexpr int kRowsPer256 = 16 / kCpr;  // rows that share one 256-byte bank window
  static constexpr int kRpi = 64 / kCpr;         // rows filled by one wave-wide direct load
  static constexpr int kIpw = kBc / kRpi / kWaves;  // direct loads per wave per K (or V) tile
  static constexpr int kTile = kBc * D;          // elements per tile buffer
  static constexpr int kAhead = 3;               // tiles requested ahead of the one in use
  static constexpr int kRingK = 4;
  static constexpr int kRingV = 5;
  static constexpr int kRingBytes = (kRingK + kRingV) * kTile * 2;
#ifdef KCG_FMHA_EXP_STAGE_O
  static constexpr int kStageBytes = 2048;       // per wave
  static constexpr int kLdsBytes = kRingBytes + kWaves * kStageBytes;
#else
  static constexpr int kLdsBytes = kRingBytes;
#endif
  static constexpr int kDTiles = D / 32;
  static constexpr int kDSteps = D / 16;
  static constexpr int kPvMfmas = 4 * kDTiles;   // MFMAs of O += P.V per tile
  static constexpr int kSMfmas = 2 * kDSteps;    // MFMAs of S = K.Q^T per tile
  static constexpr int kQueue = 8;               // operand fragments read ahead of the MFMA that uses them
  static_assert(D == 64 || D == 128, "head dim");
  static_assert(kIpw >= 1 && kBc % (kWaves * kRpi) == 0, "tile extents");
  static_assert(kPvMfmas >= kQueue && kSMfmas >= kQueue, "operand queue");
  __host__ __device__ static constexpr int fk(int row) { return (row / kRowsPer256) % kCpr; }
  __host__ __device__ static constexpr int fv(int row) { return 4 * ((row / kRowsPer256) & (kCpr / 4 - 1)); }
};

template <int D, bool CAUSAL, bool OUT_BF16>
__global__ __launch_bounds__(512, 2) void fmha_bf16_pp_kernel(
    const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K, const uint16_t *__restrict__ V,
    void *__restrict__ O, int S, int q_blocks, int q_items, int total_items, float scale_log2e) {
  using T = FmhaPpTile<D>;
  constexpr int BC = T::kBc;
  extern __shared__ __align__(16) uint16_t lds16[];
  uint16_t *Ks = lds16;                         // [kRingK][BC][D], chunk-swizzled
  uint16_t *Vs = lds16 + T::kRingK * T::kTile;  // [kRingV][BC][D], chunk-swizzled

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int group = wave >> 2;
  const int r32 = lane & 31;
  const int half = lane >> 5;

  // Work items of this workgroup: an item is one (head, query block) or, causal, one (head,
  // pair of query blocks (n-1-i, i)); a pass is one query block of an item.  The dispatcher
  // deals workgroup w to XCD w % 8; every XCD owns a contiguous range of items (head-major,
  // so the K/V of a head are fetched into one XCD's L2 only) and its workgroups take them
  // round-robin: workgroups that run side by side then sweep the K/V of the same few heads
  // at the same time and share each tile in that L2.
  const int xcd = blockIdx.x % kNumXcd;
  const int xcd_wgs = gridDim.x / kNumXcd + (xcd < static_cast<int>(gridDim.x % kNumXcd) ? 1 : 0);
  // (a launch with one item per workgroup simply renumbers the workgroups XCD by XCD)
  const bool one_each = static_cast<int>(gridDim.x) == total_items;
  const int item_begin = one_each ? xcd_contiguous_id(blockIdx.x, gridDim.x)
                                  : static_cast<int>(static_cast<int64_t>(xcd) * total_items / kNumXcd) + blockIdx.x / kNumXcd;
  const int item_end = one_each ? item_begin + 1 : static_cast<int>(static_cast<int64_t>(xcd + 1) * total_items / kNumXcd);
  const int item_step = xcd_wgs;
  struct Pass {
    int item, pass, npass, bh, block, nt;
  };
  // K/V tile that step `idx` of a pass works on
#ifdef KCG_FMHA_EXP_LO_DESCENDING
  auto tile_of = [&](const Pass &c, int idx) { return (CAUSAL && c.pass == 1) ? c.nt - 1 - idx : idx; };
#else
  auto tile_of = [&](const Pass &, int idx) { return idx; };
#endif
  auto describe = [&](Pass &c) {
    c.bh = c.item / q_items;
    const int it = c.item - c.bh * q_items;
    const int hi = q_blocks - 1 - it;
    c.npass = CAUSAL ? (hi != it ? 2 : 1) : 1;
    c.block = CAUSAL ? (c.pass == 0 ? hi : it) : it;  // the long block of a causal pair goes first
    const int q0 = c.block * T::kBr;
    const int kv_end = CAUSAL ? ((q0 + T::kBr) < S ? (q0 + T::kBr) : S) : S;
    c.nt = (kv_end + BC - 1) / BC;
  };
  // steps to the next pass; false when the workgroup's list is exhausted
  auto next_pass = [&](Pass &c) {
    if (++c.pass == c.npass) {
      c.pass = 0;
      c.item += item_step;
      if (c.item >= item_end) return false;
    }
    describe(c);
    return true;
  };
  if (item_begin >= item_end) return;  // (uniform: before any barrier)

  // ---- direct global -> LDS tile loads (same lane mapping as fmha_bf16_kernel) ----
  const int ld_row0 = wave * T::kIpw * T::kRpi;
  const int ld_lrow = lane / T::kCpr;
  const int ld_pos = lane % T::kCpr;
  unsigned goff_k[T::kIpw], goff_v[T::kIpw];
#pragma unroll
  for (int j = 0; j < T::kIpw; ++j) {
    const int row = ld_row0 + j * T::kRpi + ld_lrow;
    goff_k[j] = static_cast<unsigned>(row * D + (ld_pos ^ T::fk(row)) * 8) * 2u;
    goff_v[j] = static_cast<unsigned>(row * D + (ld_pos ^ T::fv(row)) * 8) * 2u;
  }
  constexpr int kLoadsPerStep = 2 * T::kIpw;
#ifdef KCG_FMHA_EXP_STAGE_O
  constexpr int kStores = (OUT_BF16 ? 2 : 4) * T::kDTiles;  // vector stores of one pass's O rows
#else
  constexpr int kStores = 4 * T::kDTiles;  // vector stores of one pass's O rows
#endif
  constexpr int kQLoads = T::kDSteps;      // vector loads of one pass's Q rows
  const unsigned lds_k0 = static_cast<unsigned>(reinterpret_cast<uintptr_t>(Ks + ld_row0 * D));
  const unsigned lds_v0 = static_cast<unsigned>(reinterpret_cast<uintptr_t>(Vs + ld_row0 * D));
  // The K/V tiles of all passes of all items form one stream; the load cursor runs kAhead
  // tiles ahead of the tile being computed.
  Pass lc = {item_begin, 0, 0, 0, 0, 0};
  describe(lc);
  int ld_tile = 0;        // next tile of lc to request
  bool ld_valid = true;   // false once every tile of the list has been requested
  int ld_ks = 0, ld_vs = 0;  // ring slots of that tile
  // requests the next tile of the stream; returns the number of vector memory operations issued
  auto issue_next = [&]() {
    if (!ld_valid) return 0;
    const int kv0 = tile_of(lc, ld_tile) * BC;
    const int64_t row0 = static_cast<int64_t>(lc.bh) * S + kv0;
    const char *kg = reinterpret_cast<const char *>(K + row0 * D);
    const char *vg = reinterpret_cast<const char *>(V + row0 * D);
    int issued = kLoadsPerStep;
    if (kv0 + BC <= S) {
      // Issued from assembly (scalar base + 32-bit lane offset).  With the compiler's builtin
      // every later LDS read is preceded by a wait for ALL outstanding direct loads
      // (vmcnt(0)): it cannot tell which buffer they fill, and the tiles requested three
      // steps ahead would be waited for at once.
#pragma unroll
      for (int j = 0; j < T::kIpw; ++j)
        direct_load_16B(kg, goff_k[j], lds_k0 + static_cast<unsigned>((ld_ks * T::kTile + j * T::kRpi * D) * 2));
#pragma unroll
      for (int j = 0; j < T::kIpw; ++j)
        direct_load_16B(vg, goff_v[j], lds_v0 + static_cast<unsigned>((ld_vs * T::kTile + j * T::kRpi * D) * 2));
    } else {
      // ragged last tile: rows at and beyond S are zero-filled, through registers (the
      // compiler waits for these loads itself, with a count that ignores the direct loads,
      // i.e. a stricter one: counts are in issue order); nothing of it stays in flight
      uint16_t *kl = Ks + ld_ks * T::kTile + ld_row0 * D;
      uint16_t *vl = Vs + ld_vs * T::kTile + ld_row0 * D;
#pragma unroll
      for (int j = 0; j < T::kIpw; ++j) {
        const int row = ld_row0 + j * T::kRpi + ld_lrow;
        const bool ok = kv0 + row < S;
        const u32x4_t z = {0u, 0u, 0u, 0u};
        const u32x4_t kvq = ok ? *reinterpret_cast<const u32x4_t *>(kg + goff_k[j]) : z;
        const u32x4_t vvq = ok ? *reinterpret_cast<const u32x4_t *>(vg + goff_v[j]) : z;
        *reinterpret_cast<u32x4_t *>(kl + (j * T::kRpi + ld_lrow) * D + ld_pos * 8) = kvq;
        *reinterpret_cast<u32x4_t *>(vl + (j * T::kRpi + ld_lrow) * D + ld_pos * 8) = vvq;
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      issued = 0;
    }
    ld_ks = ld_ks == T::kRingK - 1 ? 0 : ld_ks + 1;
    ld_vs = ld_vs == T::kRingV - 1 ? 0 : ld_vs + 1;
    if (++ld_tile == lc.nt) {
      ld_tile = 0;
      ld_valid = next_pass(lc);
    }
    return issued;
  };
  // Ends an interval (LDS reads and writes of this wave are complete first).
  auto sync = [&]() {
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  // Waits until at most n (even, <= 62) of this wave's vector memory operations are in flight.
  auto wait_vm = [&](int n) {
    // the two counts that occur in nearly every step come first
    if (n == 2 * kLoadsPerStep) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kLoadsPerStep) : "memory");
      return;
    }
    if (n == kLoadsPerStep) {
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kLoadsPerStep) : "memory");
      return;
    }
    switch (n >> 1) {
#define KCG_VM_CASE(h) \
  case h: asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * (h)) : "memory"); break;
      KCG_VM_CASE(1) KCG_VM_CASE(2) KCG_VM_CASE(3) KCG_VM_CASE(4) KCG_VM_CASE(5) KCG_VM_CASE(6) KCG_VM_CASE(7)
      KCG_VM_CASE(8) KCG_VM_CASE(9) KCG_VM_CASE(10) KCG_VM_CASE(11) KCG_VM_CASE(12) KCG_VM_CASE(13)
      KCG_VM_CASE(14) KCG_VM_CASE(15) KCG_VM_CASE(16) KCG_VM_CASE(17) KCG_VM_CASE(18) KCG_VM_CASE(19)
      KCG_VM_CASE(20) KCG_VM_CASE(21) KCG_VM_CASE(22) KCG_VM_CASE(23) KCG_VM_CASE(24) KCG_VM_CASE(25)
      KCG_VM_CASE(26) KCG_VM_CASE(27) KCG_VM_CASE(28) KCG_VM_CASE(29) KCG_VM_CASE(30) KCG_VM_CASE(31)
#undef KCG_VM_CASE
      default: asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); break;
    }
  };
  static_assert(kLoadsPerStep % 2 == 0 && kStores % 2 == 0 && kQLoads % 2 == 0, "wait_vm takes even counts");
  static_assert(2 * kLoadsPerStep + 2 * (kStores + kQLoads) <= 62, "vmcnt range");

  // ---- per-lane LDS read offsets (elements), swizzle folded in ----
  const int k_row_off = r32 * D;
  const int k_swz = T::fk(r32) ^ half;
  const int l16 = lane & 15;
  const int v_lrow = 4 * half + (l16 >> 2);
  const int v_c0 = (2 * ((lane >> 4) & 1) + ((l16 & 3) >> 1)) ^ T::fv(v_lrow);
  const int v_sub = 4 * (l16 & 1);
  const int v_row_off = v_lrow * D + v_sub;

  // ---- state of the current pass ----
  Pass cc = {item_begin, 0, 0, 0, 0, 0};
  describe(cc);
  bf16x8_v q[T::kDSteps];         // Q[wq0 + r32][16*s + 8*half .. +7]
  float16_t acc_o[T::kDTiles];
  float16_t s[2];                 // raw products of the tile at hand
  unsigned p[2][8];               // bf16 pairs of P
  bf16x8_v oq[T::kQueue];         // A-operand fragments read ahead (V^T, then K)
  float m_ref = -INFINITY;        // reference maximum of the row (log2 units)
  float l_run = 0.0f;             // this lane's share of the row sum
  int wq0 = 0;

  // Q rows of a pass, straight into the operand registers.  Issued from assembly and waited
  // for by hand: a load the compiler knows about, in a branch of the tile loop, makes it
  // wait for every outstanding load (vmcnt(0)) before each later use of q, which would also
  // drain the tile loads requested three steps ahead.  Rows at and beyond S read row S - 1
  // (their results are never stored).
  auto load_q = [&](const Pass &c) {
    int row = c.block * T::kBr + wave * 32 + r32;
    row = row < S ? row : S - 1;
    const uint16_t *src = Q + (static_cast<int64_t>(c.bh) * S + row) * D + 8 * half;
    // (in-out operands: the new rows land in the very registers that hold the old ones, so
    // that no register copy can be placed between the request and the wait)
#pragma unroll
    for (int ds = 0; ds < T::kDSteps; ++ds)
      asm volatile("global_load_dwordx4 %0, %1, off offset:%2" : "+v"(q[ds]) : "v"(src), "n"(32 * ds) : "memory");
  };
  auto q_arrived = [&]() {
#pragma unroll
    for (int ds = 0; ds < T::kDSteps; ++ds) asm volatile("" : "+v"(q[ds]));
  };
  auto start_pass = [&]() {
    wq0 = cc.block * T::kBr + wave * 32;
#pragma unroll
    for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc_o[i][e] = 0.0f;
    m_ref = -INFINITY;
    l_run = 0.0f;
  };

  // A operand of PV MFMA m (key block m / kDTiles of 16 keys, d tile m % kDTiles): V^T from
  // the [key][d] tile with two transposing reads
  auto read_v = [&](int vslot, int m) {
    const int kb = m / T::kDTiles, i = m % T::kDTiles;
    const uint16_t *vp = Vs + vslot * T::kTile + v_row_off + kb * 16 * D + ((4 * i) ^ v_c0) * 8;
    const bf16x4_v lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((KCG_LDS_BF16X4 *)(vp));
    const bf16x4_v hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((KCG_LDS_BF16X4 *)(vp + 8 * D));
    return __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  // A operand of S MFMA m (d step m / 2, key half m % 2): 8 bf16 of one K row
  auto read_k = [&](int kslot, int m) {
    const int ds = m / 2, kt = m % 2;
    const uint16_t *kp = Ks + kslot * T::kTile + k_row_off + kt * 32 * D + ((2 * ds) ^ k_swz) * 8;
    return __builtin_bit_cast(bf16x8_v, *reinterpret_cast<const u32x4_t *>(kp));
  };
  // B operand of PV MFMA m: the 16-key block m / kDTiles of P
  auto p_block = [&](int m) {
    const int kb = m / T::kDTiles;
    const u32x4_t pw = {p[kb / 2][4 * (kb % 2)], p[kb / 2][4 * (kb % 2) + 1], p[kb / 2][4 * (kb % 2) + 2],
                        p[kb / 2][4 * (kb % 2) + 3]};
    return __builtin_bit_cast(bf16x8_v, pw);
  };

  // mask, P = exp2(s * c - m) packed to bf16, row sum; reference maximum only when needed
  auto softmax = [&](int kv0) {
    const int qrow = wq0 + r32;
    if ((kv0 + BC > S) || (CAUSAL && (kv0 + BC - 1 > wq0))) {
      // element (kt, e) is key kv0 + 4*half + off, off = 32*kt + 8*(e/4) + e%4; dead when off > lim
      const int last = CAUSAL ? (qrow < S - 1 ? qrow : S - 1) : (S - 1);
      const int lim = last - kv0 - 4 * half;
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          if (32 * kt + 8 * (e / 4) + (e % 4) > lim) s[kt][e] = -INFINITY;
    }
    // P = exp2(s * c - m) as bf16 pairs; returns this lane's share of the row sum
    auto exp_tile = [&](float neg_m) {
      float ps[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int w = 0; w < 8; ++w) {
          const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][2 * w], scale_log2e, neg_m));
          const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][2 * w + 1], scale_log2e, neg_m));
          p[kt][w] = pack_bf16(p0, p1);
          ps[w & 3] = add_bf16_pair(p[kt][w], ps[w & 3]);
        }
      return (ps[0] + ps[1]) + (ps[2] + ps[3]);
    };
    // Fast path: no row maximum at all.  The exponentials are taken against the reference
    // the row already has; if one of them came out larger than 2^kTau the sum shows it
    // (every term is >= 0), and only then -- and on a row's first tile -- is the maximum
    // computed, the reference raised and the tile's exponentials taken again.  Both halves
    // of the wave see the same sum and the same reference, so they decide alike.
    float psum = exp_tile((m_ref == -INFINITY) ? 0.0f : -m_ref);
    const float big = max_across_halves(psum);
    if (m_ref == -INFINITY || big > 256.0f /* 2^kTau */) {
      float mx0 = max3(s[0][0], s[0][1], s[0][2]), mx1 = max3(s[1][0], s[1][1], s[1][2]);
#pragma unroll
      for (int e = 3; e + 1 < 16; e += 2) {
        mx0 = max3(mx0, s[0][e], s[0][e + 1]);
        mx1 = max3(mx1, s[1][e], s[1][e + 1]);
      }
      // scale > 0: the maximum of the scaled scores is the scaled maximum (-inf stays -inf)
      const float m_loc = max_across_halves(max3(mx0, mx1, fmaxf(s[0][15], s[1][15]))) * scale_log2e;
      if (m_loc > m_ref) {
        const float alpha = __builtin_amdgcn_exp2f(m_ref - m_loc);  // m_ref = -inf -> 0
        m_ref = m_loc;
        l_run *= alpha;
#pragma unroll
        for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
          for (int e = 0; e < 16; ++e) acc_o[i][e] *= alpha;
      }
      psum = exp_tile((m_ref == -INFINITY) ? 0.0f : -m_ref);
    }
    l_run += psum;
  };

#ifdef KCG_FMHA_EXP_STAGE_O
  // normalise and store: lane holds O[wq0 + r32][32*i + 8*g + 4*half + 0..3]; 64 bytes of each
  // of the wave's 32 rows per round go through the staging area (16-byte chunks XOR-swizzled
  // against bank conflicts) and leave four lanes a row
  auto store_o = [&]() {
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.0f / l_tot;
    char *stage = reinterpret_cast<char *>(lds16) + T::kRingBytes + wave * T::kStageBytes;
    char *wr = stage + r32 * 64 + 8 * half;
    const int wswz = (r32 >> 1) & 3;
    constexpr int kRounds = OUT_BF16 ? T::kDTiles : 2 * T::kDTiles;
    constexpr int kRowBytes = OUT_BF16 ? 2 * D : 4 * D;
    char *obase = static_cast<char *>(O) + (static_cast<int64_t>(cc.bh) * S + wq0) * kRowBytes;
    const bool whole = wq0 + 32 <= S;
#pragma unroll
    for (int rd = 0; rd < kRounds; ++rd) {
      if (OUT_BF16) {
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          u32x2_t w = {pack_bf16(acc_o[rd][4 * g + 0] * inv, acc_o[rd][4 * g + 1] * inv),
                       pack_bf16(acc_o[rd][4 * g + 2] * inv, acc_o[rd][4 * g + 3] * inv)};
          *reinterpret_cast<u32x2_t *>(wr + ((g ^ wswz) * 16)) = w;
        }
      } else {
        // 16 columns of fp32 per round: g = 2*(rd%2) + gg, chunk = 2*gg + half
#pragma unroll
        for (int gg = 0; gg < 2; ++gg) {
          const int g = 2 * (rd % 2) + gg;
          float4_t w = {acc_o[rd / 2][4 * g + 0] * inv, acc_o[rd / 2][4 * g + 1] * inv,
                        acc_o[rd / 2][4 * g + 2] * inv, acc_o[rd / 2][4 * g + 3] * inv};
          *reinterpret_cast<float4_t *>(stage + r32 * 64 + (((2 * gg + half) ^ wswz) * 16)) = w;
        }
      }
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int row = 16 * k + (lane >> 2);
        const int chunk = lane & 3;
        const u32x4_t v = *reinterpret_cast<const u32x4_t *>(stage + row * 64 + ((chunk ^ ((row >> 1) & 3)) * 16));
        if (whole || wq0 + row < S)
          *reinterpret_cast<u32x4_t *>(obase + static_cast<int64_t>(row) * kRowBytes + rd * 64 + chunk * 16) = v;
      }
    }
  };
#else
  // normalise and store: lane holds O[qrow][32*i + 8*g + 4*half + 0..3]
  auto store_o = [&]() {
    const int qrow = wq0 + r32;
    const float l_tot = l_run + __shfl_xor(l_run, 32);
    const float inv = 1.0f / l_tot;
    if (qrow < S) {
      const int64_t off = (static_cast<int64_t>(cc.bh) * S + qrow) * D + 4 * half;
#pragma unroll
      for (int i = 0; i < T::kDTiles; ++i)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const float v0 = acc_o[i][4 * g + 0] * inv;
          const float v1 = acc_o[i][4 * g + 1] * inv;
          const float v2 = acc_o[i][4 * g + 2] * inv;
          const float v3 = acc_o[i][4 * g + 3] * inv;
          if (OUT_BF16) {
            u32x2_t w = {pack_bf16(v0, v1), pack_bf16(v2, v3)};
            *reinterpret_cast<u32x2_t *>(static_cast<uint16_t *>(O) + off + 32 * i + 8 * g) = w;
          } else {
            float4_t w = {v0, v1, v2, v3};
            *reinterpret_cast<float4_t *>(static_cast<float *>(O) + off + 32 * i + 8 * g) = w;
          }
        }
    }
  };
#endif
  // Stores a wave is known to issue for a pass: all of them when every row is inside the
  // sequence; a wave with rows beyond S may skip the instructions altogether, so it counts
  // none (the hand-counted waits then wait for more than they need, never for less).
  auto stores_of_pass = [&]() { return wq0 + 32 <= S ? kStores : 0; };

  // A wave whose last query precedes the tile has nothing to add (causal).
#ifdef KCG_FMHA_EXP_ALL_PAIRS
  auto active = [&](int) { return true; };
#else
  auto active = [&](int idx) { return !CAUSAL || (tile_of(cc, idx) * BC <= wq0 + 31); };
#endif
  const float16_t zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // the 2 * kDSteps MFMAs of S = K . Q^T from ring slot kslot; `primed`: the first kQueue
  // fragments are already in the queue
  auto s_phase = [&](int kslot, bool primed) {
    if (!primed) {
#pragma unroll
      for (int m = 0; m < T::kQueue; ++m) oq[m] = read_k(kslot, m);
    }
#pragma unroll
    for (int m = 0; m < T::kSMfmas; ++m) {
      s[m % 2] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(oq[m % T::kQueue], q[m / 2], m < 2 ? zero16 : s[m % 2], 0, 0, 0);
      if (m + T::kQueue < T::kSMfmas) oq[m % T::kQueue] = read_k(kslot, m + T::kQueue);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // the 4 * kDTiles MFMAs of O += P . V; the queue holds the first kQueue fragments of V and
  // is refilled kQueue MFMAs ahead, at the end with the first fragments of the next K tile
  // (always: a branch here makes the compiler keep two copies of the accumulators and
  // spill; when no S follows the fragments are simply not used)
  auto pv_phase = [&](int vslot, int kslot) {
#pragma unroll
    for (int m = 0; m < T::kPvMfmas; ++m) {
      acc_o[m % T::kDTiles] =
          __builtin_amdgcn_mfma_f32_32x32x16_bf16(oq[m % T::kQueue], p_block(m), acc_o[m % T::kDTiles], 0, 0, 0);
      if (m + T::kQueue < T::kPvMfmas) oq[m % T::kQueue] = read_v(vslot, m + T::kQueue);
      else oq[m % T::kQueue] = read_k(kslot, m + T::kQueue - T::kPvMfmas);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // Vector memory operations of this wave, newest first, as far back as the waits look:
  //   d_cur / d_prev: tile loads of this step / the step before (softmax interval)
  //   x_cur / x_prev / x_prev2: O stores and Q loads of this step's matrix interval / the
  //   two steps before
  int d_cur = 0, d_prev = 0, x_cur = 0, x_prev = 0, x_prev2 = 0;
  // The pass after the current one, if any (its Q rows are requested as soon as the last S
  // of the current pass has been issued).
  Pass np = cc;
  bool np_valid = next_pass(np);

  // ---- prologue: the first tiles of the stream, then group 1 falls one interval behind ----
  for (int jj = 0; jj < T::kAhead; ++jj) issue_next();
  load_q(cc);
  start_pass();
  wait_vm(0);
  q_arrived();
  sync();
  if (group == 1) sync();
  int t = 0;       // tile (of the current pass) whose products are in s
  int ks_next = 1; // ring slot of the K tile after that one
  int vs_cur = 0;  // ring slot of its V tile
  if (active(0)) s_phase(0, false);
  if (cc.nt == 1 && np_valid) {
    load_q(np);
    x_cur = kQLoads;
  }
  sync();
  x_prev = x_cur;
  x_cur = 0;

  for (bool running = true; running;) {
    // -- softmax interval, beside the other group's PV and S
    const bool act = active(t);
    // requested first, so that their latency passes under the softmax arithmetic: the tile
    // three steps ahead, and the first operands of PV (this V tile was published one barrier ago)
    d_cur = issue_next();
    if (act) {
#pragma unroll
      for (int m = 0; m < T::kQueue; ++m) oq[m] = read_v(vs_cur, m);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (act) softmax(tile_of(cc, t) * BC);
    // Still allowed in flight: the tile loads of this step and of the step before, and
    // whatever the two last matrix intervals issued after the older of them.  The K and V
    // tiles requested two steps ago are published by the coming barriers.
    wait_vm(d_cur + d_prev + x_prev + x_prev2);
    sync();
    // -- matrix interval: PV, then S of the next tile; alone on the matrix pipe
    __builtin_amdgcn_s_setprio(1);
    const bool last_of_pass = t + 1 == cc.nt;
    const bool has_next = !last_of_pass || np_valid;
    if (act) pv_phase(vs_cur, ks_next);
    vs_cur = vs_cur == T::kRingV - 1 ? 0 : vs_cur + 1;
    if (last_of_pass) {
      store_o();
      const int stores = stores_of_pass();
      x_cur += stores;
      if (np_valid) {
        // the Q rows were requested one step ago, after the last S of the pass that ends
        // here; newer than them: this step's tile loads and the stores just issued
        cc = np;
        np_valid = next_pass(np);
        t = -1;
        start_pass();
        wait_vm(d_cur + stores);
        q_arrived();
      }
    }
    ++t;
    if (has_next && active(t)) s_phase(ks_next, act);
    if (has_next && t + 1 == cc.nt && np_valid) {
      load_q(np);  // this was the pass's last S: the Q registers are free
      x_cur += kQLoads;
    }
    ks_next = ks_next == T::kRingK - 1 ? 0 : ks_next + 1;
    __builtin_amdgcn_s_setprio(0);
    // group 1 ends the interval in which group 0 reads ahead into the next V tile: its own
    // share of that tile and of the K tile after it (requested in its last softmax interval
    // but one) must be in
    if (group == 1) wait_vm(x_cur + d_cur + x_prev);
    sync();
    d_prev = d_cur;
    x_prev2 = x_prev;
    x_prev = x_cur;
    x_cur = 0;
    running = has_next;
  }
  if (group == 0) sync();
}

template <int D, int BC, int QT, int WAVES, bool POS>
static int launch_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O,
                            int o_dtype, int B, int H, int S, float scale, int causal,
                            hipStream_t stream, kcg_launch_info *info) {
  using T = FmhaBf16Tile<D, BC, QT, WAVES>;
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
    snprintf(info->kernel, sizeof info->kernel, "fmha_bf16_d%d_br%d_bc%d%s", D, T::kBr, BC,
             causal ? "_causal_paired" : "");
    return KCG_OK;
  }
  const float scale_log2e = scale * 1.4426950408889634f;
#define KCG_LAUNCH(CAUSAL_, OBF_, POS_)                                                                 \
  do {                                                                                            \
    auto kern = fmha_bf16_kernel<D, BC, QT, WAVES, CAUSAL_, OBF_, POS_>;                                       \
    if (!allow_lds(kern, T::kLdsBytes)) return KCG_ERR_LAUNCH;                                    \
    return launch(kern, dim3(static_cast<unsigned>(blocks)), dim3(T::kThreads), T::kLdsBytes,     \
                  stream, Q, K, V, O, S, static_cast<int>(q_blocks), static_cast<int>(q_items),   \
                  scale_log2e);                                                                   \
  } while (0)
  const bool obf = o_dtype == KCG_BF16;
  if (causal) {
    if (obf) KCG_LAUNCH(true, true, POS);
    else KCG_LAUNCH(true, false, POS);
  } else {
    if (obf) KCG_LAUNCH(false, true, POS);
    else KCG_LAUNCH(false, false, POS);
  }
#undef KCG_LAUNCH
}

template <int D>
static int launch_fmha_bf16_pp(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O, int o_dtype,
                               int B, int H, int S, float scale, int causal, hipStream_t stream,
                               kcg_launch_info *info) {
  using T = FmhaPpTile<D>;
  const int64_t q_blocks = (static_cast<int64_t>(S) + T::kBr - 1) / T::kBr;
  const int64_t q_items = causal ? (q_blocks + 1) / 2 : q_blocks;
  const int64_t items = q_items * B * H;
  if (items > 0x7fffffffLL) return KCG_ERR_BAD_SHAPE;
  // one workgroup per CU (the 144 KiB of LDS allow no second one); each walks its share of
  // the items as one stream of K/V tiles
  const int64_t blocks = items < kNumCu ? items : kNumCu;
  if (info) {
    *info = kcg_launch_info{};
    info->launches = 1;
    info->grid[0] = static_cast<int>(blocks);
    info->grid[1] = info->grid[2] = 1;
    info->block[0] = T::kThreads;
    info->block[1] = info->block[2] = 1;
    info->lds_bytes = T::kLdsBytes;
    info->waves_per_block = T::kWaves;
    snprintf(info->kernel, sizeof info->kernel, "fmha_bf16_d%d_br%d_bc%d_pingpong%s", D, T::kBr, T::kBc,
             causal ? "_causal_paired" : "");
    return KCG_OK;
  }
  const float scale_log2e = scale * 1.4426950408889634f;
  auto go = [&](auto kern) {
    if (!allow_lds(kern, T::kLdsBytes)) return static_cast<int>(KCG_ERR_LAUNCH);
    return launch(kern, dim3(static_cast<unsigned>(blocks)), dim3(T::kThreads), T::kLdsBytes, stream, Q, K, V, O, S,
                  static_cast<int>(q_blocks), static_cast<int>(q_items), static_cast<int>(items), scale_log2e);
  };
  const bool obf = o_dtype == KCG_BF16;
  if (causal) return obf ? go(fmha_bf16_pp_kernel<D, true, true>) : go(fmha_bf16_pp_kernel<D, true, false>);
  return obf ? go(fmha_bf16_pp_kernel<D, false, true>) : go(fmha_bf16_pp_kernel<D, false, false>);
}

int dispatch_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V, void *O,
                       int o_dtype, int B, int H, int S, int D, float scale, int causal,
                       const kcg_fmha_sched *sched, hipStream_t stream, kcg_launch_info *info) {
  // default, from a sweep of 38 shapes x {causal, not} x both block sizes on the box: at
  // D = 128 the 256-row ping-pong kernel when its work items (causal: pairs of blocks) give
  // every CU two or more, or exactly fill the CUs on a long or non-causal sweep (3-15 %
  // faster there; on half-filled launches the 128-row block is 30-40 % faster: B=1, H=32,
  // S=2048 causal 629 against 475 TFLOP/s).  At D = 64 a tile has half the matrix work for
  // the same softmax, the two wave groups no longer balance, and the 128-row kernel is
  // ahead on every shape of the sweep.
  const int64_t blocks256 = (static_cast<int64_t>(S) + 255) / 256;
  const int64_t items256 = (causal ? (blocks256 + 1) / 2 : blocks256) * B * H;
  const bool large = D == 128 && (items256 >= 2 * kNumCu || (items256 >= kNumCu && (S >= 2048 || !causal)));
  int br = large ? 256 : 128, bc = 64;
  if (sched) {
    if (sched->br) br = sched->br;
    if (sched->bc) bc = sched->bc;
  }
  // (Br 64 x Bc 128 is the tile the reference's own table gives at Hd = 128, include/
  // KernelCodeGen.h:38-41, src/Optimizer/Optimizer.cc:1136-1144: two waves on the 128-row
  // kernel's code, built so that the reference's literal configuration binds)
  const bool reference_tile = D == 128 && br == 64 && bc == 128;
  if (bc != 64 && !reference_tile) return KCG_ERR_BAD_SCHEDULE;
  if (br != 128 && br != 256 && !reference_tile) return KCG_ERR_BAD_SCHEDULE;
  // scale <= 0 takes the general softmax path, built for the 128-row block only
  const bool pos = scale > 0.0f;
  if (reference_tile) {
    if (pos) return launch_fmha_bf16<128, 128, 1, 2, true>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);
    return launch_fmha_bf16<128, 128, 1, 2, false>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);
  }
#define KCG_PICK(D_)                                                                              \
  if (D == D_) {                                                                                  \
    if (!pos)                                                                                     \
      return launch_fmha_bf16<D_, 64, 1, 4, false>(Q, K, V, O, o_dtype, B, H, S, scale, causal,      \
                                                stream, info);                                    \
    if (br == 128)                                                                                \
      return launch_fmha_bf16<D_, 64, 1, 4, true>(Q, K, V, O, o_dtype, B, H, S, scale, causal,       \
                                               stream, info);                                     \
    return launch_fmha_bf16_pp<D_>(Q, K, V, O, o_dtype, B, H, S, scale, causal, stream, info);      \
  }
  KCG_PICK(128)
  KCG_PICK(64)
#undef KCG_PICK
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
  // tensors of 2^31 elements and more: not verified on the GPU (see kcg_gemm_f32)
  if (static_cast<int64_t>(B) * H > 0x7fffffffLL / (static_cast<int64_t>(S) * D)) return KCG_ERR_UNSUPPORTED_SHAPE;
  return kcg::dispatch_fmha_bf16(Q, K, V, O, o_dtype, B, H, S, D, scale, causal, sched,
                                 static_cast<hipStream_t>(stream), nullptr);
}

}  // extern "C"
