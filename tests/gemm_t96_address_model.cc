// Host replay of gemm_f32_t96_kernel's address arithmetic (kernelcodegen_amd/csrc/gemm_f32_t96.h)
// with the kernel's own geometry (gemm_dl_tile.h).  For every workgroup on the rim of the grid
// and a sample inside, every wave and lane:
//   * the global bytes of each direct load lie inside A / B, the 32-bit lane offsets do not
//     overflow, and the loads of a slice fill the stage's A and B tiles exactly once;
//   * the element an operand read fetches from the filled stage is the one the MFMA step
//     multiplies: A[m0 + row][k] and B[k][n0 + col] with the same k for both operands, each k
//     of the slice exactly once per (row, col);
//   * the stores cover the part of the C tile that lies inside C exactly once (M and N need
//     not divide the tile: lanes beyond an edge load the last valid row / chunk).
// usage: gemm_t96_address_model BLOCK_N M N K GROUP_M   (BLOCK_N 96 or 64; prints "... N violations")
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "gemm_dl_tile.h"


static long violations = 0;
static void fail(const char *what, long a, long b, long c) {
  if (violations < 20) std::printf("VIOLATION %s (%ld, %ld, %ld)\n", what, a, b, c);
  ++violations;
}

static int xcd_contiguous_id(int w, int n) {
  const int xcd = w % 8, idx = w / 8, per = n / 8, rem = n % 8;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

template <class G>
static int replay(int64_t M, int64_t N, int64_t K, int group_m) {
  if (N % 4 || K % G::kBK) return 2;
  const int tiles_m = static_cast<int>((M + G::kBM - 1) / G::kBM), tiles_n = static_cast<int>((N + G::kBN - 1) / G::kBN);
  const int grid = tiles_m * tiles_n;
  const int64_t a_bytes = M * K * 4, b_bytes = K * N * 4, c_elems = M * N;
  std::vector<int> seen_tile(grid, 0);
  long checked = 0;
  for (int block = 0; block < grid; ++block) {
    const int logical = xcd_contiguous_id(block, grid);
    const int width = group_m * tiles_n;
    const int group = logical / width;
    const int first_m = group * group_m;
    const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
    const int in_group = logical - group * width;
    const int tile_m = first_m + in_group % gsz, tile_n = in_group / gsz;
    if (tile_m < 0 || tile_m >= tiles_m || tile_n < 0 || tile_n >= tiles_n) {
      fail("tile origin", block, tile_m, tile_n);
      continue;
    }
    ++seen_tile[tile_m * tiles_n + tile_n];
    const bool rim = tile_m == 0 || tile_n == 0 || tile_m == tiles_m - 1 || tile_n == tiles_n - 1;
    if (!rim && block % 37 != 0) continue;
    ++checked;
    const int64_t m0 = int64_t{tile_m} * G::kBM, n0 = int64_t{tile_n} * G::kBN;
    // stage image: which (row, k) / (k, col) of the slice each LDS float holds
    std::vector<int> a_img(G::kFloatsA, -1), b_img(G::kFloatsB, -1);
    for (int wave = 0; wave < 4; ++wave)
      for (int lane = 0; lane < 64; ++lane) {
        for (int i = 0; i < G::kLoadsA; ++i) {
          const int idx = (wave * G::kLoadsA + i) * 256 + lane * 4;
          const int row = idx / G::kBK;
          const int c_log = ((idx % G::kBK) / 4) ^ G::fa(row);
          // (rows at and beyond M: the last valid row instead)
          const int64_t grow = row < M - m0 ? row : M - m0 - 1;
          const uint64_t off64 = (static_cast<uint64_t>(grow) * K + 4 * c_log) * 4u;
          if (off64 > 0xffffffffull) fail("A lane offset overflows 32 bits", row, c_log, 0);
          for (int64_t kt = 0; kt < K / G::kBK; kt += (K / G::kBK > 2 ? K / G::kBK - 1 : 1)) {
            const int64_t byte = (m0 * K + kt * G::kBK) * 4 + static_cast<int64_t>(off64);
            if (byte < 0 || byte + 16 > a_bytes) fail("A load outside A", block, row, kt);
          }
          for (int e = 0; e < 4; ++e) {
            if (a_img[idx + e] != -1) fail("A stage float written twice", idx + e, 0, 0);
            a_img[idx + e] = row * G::kBK + 4 * c_log + e;
          }
        }
        for (int i = 0; i < G::kLoadsB; ++i) {
          const int idx = (wave * G::kLoadsB + i) * 256 + lane * 4;
          const int row = G::b_row(idx), col = G::b_col(idx);
          // (column chunks at and beyond N: the last valid chunk instead)
          const int64_t gcol = col < N - n0 ? col : N - n0 - 4;
          const uint64_t off64 = (static_cast<uint64_t>(row) * N + gcol) * 4u;
          if (off64 > 0xffffffffull) fail("B lane offset overflows 32 bits", row, col, 0);
          if (gcol < 0) fail("B chunk clamped below the tile", block, col, 0);
          if (row < 0 || row >= G::kBK || col < 0 || col + 4 > G::kBN) fail("B chunk outside the slice", idx, row, col);
          for (int64_t kt = 0; kt < K / G::kBK; kt += (K / G::kBK > 2 ? K / G::kBK - 1 : 1)) {
            const int64_t byte = (kt * G::kBK * N + n0) * 4 + static_cast<int64_t>(off64);
            if (byte < 0 || byte + 16 > b_bytes) fail("B load outside B", block, row, kt);
          }
          for (int e = 0; e < 4; ++e) {
            if (b_img[idx + e] != -1) fail("B stage float written twice", idx + e, 0, 0);
            b_img[idx + e] = row * G::kBN + col + e;
          }
        }
      }
    for (int v : a_img)
      if (v < 0) fail("A stage float never written", 0, 0, 0);
    for (int v : b_img)
      if (v < 0) fail("B stage float never written", 0, 0, 0);
    // operand reads and stores
    std::vector<int> c_cover(G::kBM * G::kBN, 0);
    for (int wave = 0; wave < 4; ++wave) {
      const int wm = wave / G::kWavesN, wn = wave % G::kWavesN;
      for (int lane = 0; lane < 64; ++lane) {
        const int r16 = lane & 15, g = lane >> 4;
        for (int s = 0; s < G::kSteps; ++s) {
          const int h = s / 4, j = s % 4;
          for (int i = 0; i < G::kBlocksM; ++i) {
            // ds_read_b128 at a_addr[h] + i * 16 rows, element j
            const int fo = (wm * G::kWaveM + r16) * G::kBK + 4 * ((g + 4 * h) ^ G::fa(r16)) + i * 16 * G::kBK + j;
            const int want_row = wm * G::kWaveM + i * 16 + r16, want_k = 16 * h + 4 * g + j;
            if (fo < 0 || fo >= G::kFloatsA || a_img[fo] != want_row * G::kBK + want_k)
              fail("A operand", wave, lane, s);
          }
          for (int n = 0; n < G::kBlocksN; ++n) {
            // ds_read_b32 at b_addr + s quartets + n windows
            const int fo = wn * G::kBlocksN * 64 + g * 16 + r16 + s * G::kQuartetFloats + n * 64;
            const int want_col = wn * G::kWaveN + n * 16 + r16, want_k = 16 * h + 4 * g + j;
            if (fo < 0 || fo >= G::kFloatsB || b_img[fo] != want_k * G::kBN + want_col)
              fail("B operand", wave, lane, s);
          }
        }
        // D of a block: element e of lane (r16, g) is C[4 * g + e][r16]
        for (int i = 0; i < G::kBlocksM; ++i)
          for (int n = 0; n < G::kBlocksN; ++n)
            for (int e = 0; e < 4; ++e) {
              const int row = wm * G::kWaveM + i * 16 + 4 * g + e, col = wn * G::kWaveN + n * 16 + r16;
              if (m0 + row >= M || n0 + col >= N) continue;   // the kernel's bounds check
              ++c_cover[row * G::kBN + col];
              const int64_t elem = (m0 + row) * N + n0 + col;
              if (elem < 0 || elem >= c_elems) fail("store outside C", block, row, col);
            }
      }
    }
    // the k an MFMA step sums over (lane group g supplies k = 16h + 4g + j): every k of the slice once
    uint32_t kmask = 0u;
    for (int s = 0; s < G::kSteps; ++s)
      for (int g = 0; g < 4; ++g) {
        const uint32_t bit = 1u << (16 * (s / 4) + 4 * g + s % 4);
        if (kmask & bit) fail("a k of the slice is summed twice", s, g, 0);
        kmask |= bit;
      }
    if (kmask != 0xffffffffu) fail("the steps of a slice do not cover its 32 k", kmask, 0, 0);
    for (int row = 0; row < G::kBM; ++row)
      for (int col = 0; col < G::kBN; ++col)
        if (c_cover[row * G::kBN + col] != ((m0 + row < M && n0 + col < N) ? 1 : 0))
          fail("C element of the tile stored other than once / outside C", block, row, col);
  }
  for (int t = 0; t < grid; ++t)
    if (seen_tile[t] != 1) fail("tile computed other than once", t, seen_tile[t], 0);
  std::printf("gemm_f32_t96 tile %dx%d, %lldx%lldx%lld group_m %d: %d workgroups, %ld replayed, %ld violations\n", G::kBM,
              G::kBN, static_cast<long long>(M), static_cast<long long>(N), static_cast<long long>(K), group_m, grid,
              checked, violations);
  return violations ? 1 : 0;
}

int main(int argc, char **argv) {
  if (argc != 6) return 2;
  const int bn = atoi(argv[1]);
  const int64_t M = atoll(argv[2]), N = atoll(argv[3]), K = atoll(argv[4]);
  const int group_m = atoi(argv[5]);
  if (bn == 96) return replay<kcg::GemmT96Tile<96, 96>>(M, N, K, group_m);
  if (bn == 64) return replay<kcg::GemmT96Tile<96, 64>>(M, N, K, group_m);
  return 2;
}
