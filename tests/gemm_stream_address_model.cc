// Host replay of the address arithmetic of gemm_f32_stream_kernel
// (kernelcodegen_amd/csrc/gemm_f32_stream.h): the resident workgroups of one launch are
// walked through their lists of (matrix, tile) items with the kernel's own item functions
// (gemm_stream_items, gemm_stream_decode of gemm_dl_tile.h) and, per tile, through the
// integer expressions of its loads and stores (same operand widths: 32-bit lane offsets,
// 64-bit scalar bases).  Checked:
//   * every tile of every matrix is taken by exactly one workgroup,
//   * every byte a direct load touches lies inside A or B (the load cursor included, which
//     runs three slices ahead and stays on its last slice past the end of the list),
//   * every store lies inside C, no 32-bit offset wraps, and the 64 stores per lane of the
//     8 waves cover the 256 x 128 tile exactly once,
//   * every LDS byte a direct load writes lies inside the four-stage ring.
// Exit status 0 = clean.
//
// Usage: gemm_stream_address_model TRANS_B BATCH M N K GRID
// Built and run by tests/test_gemm_dl_addresses.py with g++ (no GPU, no HIP).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "gemm_dl_tile.h"

namespace {

int g_errors = 0;
void fail(const char *what, long long a, long long b) {
  if (g_errors < 20) fprintf(stderr, "VIOLATION %s: %lld %lld\n", what, a, b);
  ++g_errors;
}
unsigned as_u32(int64_t v, const char *what) {
  if (v < 0 || v > static_cast<int64_t>(UINT32_MAX)) fail(what, v, 0);
  return static_cast<unsigned>(v);
}

template <bool TRANS_B>
int replay(int64_t batch, int64_t M64, int64_t N64, int64_t K64, int grid) {
  using G = kcg::GemmStreamGeometry;
  using T = kcg::GemmDlTile<G::kBM, G::kBN, G::kBK, G::kWavesM, G::kWavesN, TRANS_B>;
  constexpr int BM = G::kBM, BN = G::kBN, BK = G::kBK;
  constexpr int kStageBytes = T::kStageFloats * 4;
  constexpr int kLdsBytes = G::kStages * kStageBytes;
  if (M64 % BM || N64 % BN || K64 % (4 * BK) || K64 < 4 * BK || N64 > (1 << 21)) {
    fprintf(stderr, "shape not taken by the streaming kernel\n");
    return 2;
  }
  const int M = static_cast<int>(M64), N = static_cast<int>(N64), K = static_cast<int>(K64);
  const int tiles_m = M / BM, tiles_n = N / BN, group_m = 8;
  const int ktiles = K / BK;
  const int64_t total_items64 = static_cast<int64_t>(tiles_m) * tiles_n * batch;
  if (total_items64 > INT32_MAX) return 2;
  const int total_items = static_cast<int>(total_items64);
  const int64_t batch_a = M64 * K64, batch_b = K64 * N64, batch_c = M64 * N64;  // elements
  const int64_t bytes_a = batch * batch_a * 4, bytes_b = batch * batch_b * 4, bytes_c = batch * batch_c * 4;
  std::vector<unsigned char> taken(total_items, 0);
  int64_t hi_a = 0, hi_b = 0, hi_c = 0;

  // lane offsets, the same for every tile
  unsigned oa[8][T::kInstrA][64], ob[8][T::kInstrB][64];
  for (int wave = 0; wave < 8; ++wave)
    for (int lane = 0; lane < 64; ++lane) {
      for (int i = 0; i < T::kInstrA; ++i) {
        const int idx = (wave * T::kInstrA + i) * 256 + lane * 4;
        const int row = idx / BK;
        oa[wave][i][lane] = as_u32((static_cast<int64_t>(row) * K + 4 * (((idx % BK) / 4) ^ T::fa(row))) * 4, "oa");
        const int lds = (wave * T::kInstrA + i) * 1024 + lane * 16;
        if (lds + 16 > T::kFloatsA * 4) fail("lds A", lds, 0);
      }
      for (int i = 0; i < T::kInstrB; ++i) {
        const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;
        if (TRANS_B) {
          const int row = idx / BK;
          ob[wave][i][lane] = as_u32((static_cast<int64_t>(row) * K + 4 * (((idx % BK) / 4) ^ T::fa(row))) * 4, "ob");
        } else {
          ob[wave][i][lane] = as_u32((static_cast<int64_t>(idx / BN) * N + idx % BN) * 4, "ob");
        }
        const int lds = (T::kFloatsA + (wave * T::kInstrB + i) * (TRANS_B ? 256 : T::kRunB)) * 4 + lane * 16;
        if (lds + 16 > kStageBytes || (G::kStages - 1) * kStageBytes + lds + 16 > kLdsBytes) fail("lds B", lds, 0);
      }
    }
  // store offsets of a lane (c_off) and the coverage of one tile by the 8 x 64 x 64 stores
  {
    std::vector<unsigned char> cover(BM * BN, 0);
    for (int wave = 0; wave < 8; ++wave) {
      const int wm = wave / G::kWavesN, wn = wave % G::kWavesN;
      for (int lane = 0; lane < 64; ++lane) {
        const int r32 = lane & 31, half = lane >> 5;
        for (int q = 0; q < G::kAccPerLane; ++q) {
          const int i = q / 32, g = (q / 8) % 4, r = (q / 2) % 4, n = q % 2;
          const int64_t off = (static_cast<int64_t>(wm * T::kWaveM + i * 32 + 8 * g + 4 * half) * N + wn * T::kWaveN + r32) * 4;
          as_u32(off, "c_off");
          const int64_t byte = static_cast<int64_t>(r) * N * 4 + off + n * 128;   // relative to the tile origin
          const int row = static_cast<int>(byte / (static_cast<int64_t>(N) * 4));
          const int col = static_cast<int>(byte % (static_cast<int64_t>(N) * 4)) / 4;
          // the element the accumulator register holds: acc[i][n][4g + r] of the wave's sub-tile
          const int want_row = wm * T::kWaveM + i * 32 + 8 * g + 4 * half + r, want_col = wn * T::kWaveN + n * 32 + r32;
          if (row != want_row || col != want_col) fail("store target", row * 1000 + col, want_row * 1000 + want_col);
          if (row >= BM || col >= BN) fail("store outside the tile", row, col);
          else if (cover[row * BN + col]++) fail("element stored twice", row, col);
        }
      }
    }
    for (int e = 0; e < BM * BN; ++e)
      if (!cover[e]) { fail("element never stored", e / BN, e % BN); break; }
  }

  const int64_t b_step = TRANS_B ? BK * 4 : static_cast<int64_t>(BK) * N * 4;
  long long slices_requested = 0;
  for (int wg = 0; wg < grid; ++wg) {
    const kcg::GemmStreamItems it = kcg::gemm_stream_items(wg, grid, total_items, 8);
    if (it.first >= it.end) continue;
    // the matrix work: one tile per item
    for (int item = it.first; item < it.end; item += it.step) {
      if (item < 0 || item >= total_items) { fail("item", item, wg); continue; }
      if (taken[item]++) fail("item taken twice", item, wg);
      const kcg::GemmStreamOrigin o = kcg::gemm_stream_decode(item, tiles_m, tiles_n, group_m);
      if (o.bz < 0 || o.bz >= batch || o.m0 < 0 || o.m0 + BM > M || o.n0 < 0 || o.n0 + BN > N) fail("origin", item, o.bz);
      // C: highest byte any store of this tile reaches
      const int64_t c0 = (o.bz * batch_c + static_cast<int64_t>(o.m0) * N + o.n0) * 4;
      const int64_t last = c0 + (static_cast<int64_t>(BM - 1) * N + BN - 1) * 4 + 4;
      if (c0 < 0 || last > bytes_c) fail("C range", c0, last);
      if (last > hi_c) hi_c = last;
    }
    // the load cursor: every slice of every item in order, then parked on the last slice
    int l_item = it.first, l_left = ktiles;
    kcg::GemmStreamOrigin o = kcg::gemm_stream_decode(l_item, tiles_m, tiles_n, group_m);
    int64_t lga = (o.bz * batch_a + static_cast<int64_t>(o.m0) * K) * 4;
    int64_t lgb = TRANS_B ? (o.bz * batch_b + static_cast<int64_t>(o.n0) * K) * 4 : (o.bz * batch_b + o.n0) * 4;
    const long long my_items = (it.end - it.first + it.step - 1) / it.step;
    const long long requests = my_items * ktiles + 8;   // a few more than the kernel can issue
    for (long long s = 0; s < requests; ++s) {
      for (int wave = 0; wave < 8; wave += 7)           // first and last wave reach the extremes
        for (int lane = 0; lane < 64; ++lane) {
          for (int i = 0; i < T::kInstrA; ++i) {
            const int64_t b = lga + oa[wave][i][lane];
            if (b < 0 || b + 16 > bytes_a) fail("A load", b, wg);
            if (b + 16 > hi_a) hi_a = b + 16;
          }
          for (int i = 0; i < T::kInstrB; ++i) {
            const int64_t b = lgb + ob[wave][i][lane];
            if (b < 0 || b + 16 > bytes_b) fail("B load", b, wg);
            if (b + 16 > hi_b) hi_b = b + 16;
          }
        }
      ++slices_requested;
      // advance_cursor()
      if (l_left > 1) {
        --l_left;
        lga += BK * 4;
        lgb += b_step;
      } else if (l_item + it.step < it.end) {
        l_item += it.step;
        o = kcg::gemm_stream_decode(l_item, tiles_m, tiles_n, group_m);
        lga = (o.bz * batch_a + static_cast<int64_t>(o.m0) * K) * 4;
        lgb = TRANS_B ? (o.bz * batch_b + static_cast<int64_t>(o.n0) * K) * 4 : (o.bz * batch_b + o.n0) * 4;
        l_left = ktiles;
      }
    }
  }
  for (int item = 0; item < total_items; ++item)
    if (!taken[item]) { fail("item never taken", item, 0); break; }
  printf("items %d, slices requested %lld, highest byte A %lld of %lld, B %lld of %lld, C %lld of %lld: %d violations\n",
         total_items, slices_requested, static_cast<long long>(hi_a), static_cast<long long>(bytes_a),
         static_cast<long long>(hi_b), static_cast<long long>(bytes_b), static_cast<long long>(hi_c),
         static_cast<long long>(bytes_c), g_errors);
  if (hi_a != bytes_a || hi_b != bytes_b || hi_c != bytes_c) fail("a tensor's last byte is never reached", hi_a, hi_c);
  return g_errors ? 1 : 0;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc != 7) {
    fprintf(stderr, "usage: %s TRANS_B BATCH M N K GRID\n", argv[0]);
    return 2;
  }
  const int tb = atoi(argv[1]);
  const int64_t batch = atoll(argv[2]), M = atoll(argv[3]), N = atoll(argv[4]), K = atoll(argv[5]);
  const int grid = atoi(argv[6]);
  return tb ? replay<true>(batch, M, N, K, grid) : replay<false>(batch, M, N, K, grid);
}
