// Host replay of the address arithmetic of gemm_f32_dl_kernel
// (kernelcodegen_amd/csrc/gemm_f32.hip): for one launch it walks every workgroup, wave and
// lane through the same integer expressions the kernel evaluates (same operand widths:
// 32-bit lane offsets, 64-bit tile bases) and checks that
//   * no 32-bit intermediate overflows,
//   * every byte a direct load, a tail re-load or a C store touches lies inside A, B or C,
//   * every LDS byte a direct load writes lies inside the workgroup's allocation.
// Prints the lowest and highest byte offset reached in each tensor.  Exit status 0 = clean.
//
// Usage: gemm_dl_address_model BM BN BK WAVES_M WAVES_N M N K GROUP_M
//        gemm_dl_address_model split M N K GROUP_M FULL PARTS   (the launch with K-split tail tiles)
// Built and run by tests/test_gemm_dl_addresses.py with g++ (no GPU, no HIP).
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <initializer_list>
#include <string>
#include <vector>

#include "gemm_dl_tile.h"

namespace {

struct Range {
  int64_t lo = INT64_MAX, hi = INT64_MIN;  // [lo, hi): bytes touched
  void add(int64_t first, int64_t bytes) {
    if (first < lo) lo = first;
    if (first + bytes > hi) hi = first + bytes;
  }
};

int g_errors = 0;
void fail(const char *what, int wg, int wave, int lane, int64_t value) {
  if (g_errors < 20)
    fprintf(stderr, "VIOLATION %s: workgroup %d wave %d lane %d value %lld\n", what, wg, wave, lane,
            static_cast<long long>(value));
  ++g_errors;
}

// a 32-bit signed intermediate of the kernel: the value it should have, checked for overflow
int as_int(int64_t v, const char *what, int wg, int wave, int lane) {
  if (v > INT32_MAX || v < INT32_MIN) fail(what, wg, wave, lane, v);
  return static_cast<int>(v);
}
// unsigned 32-bit byte offset: must not wrap
unsigned as_u32(int64_t v, const char *what, int wg, int wave, int lane) {
  if (v < 0 || v > static_cast<int64_t>(UINT32_MAX)) fail(what, wg, wave, lane, v);
  return static_cast<unsigned>(v);
}

int xcd_contiguous_id(int w, int n) {
  const int xcd = w % 8, idx = w / 8, per = n / 8, rem = n % 8;
  return xcd * per + (xcd < rem ? xcd : rem) + idx;
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
int replay(int64_t M64, int64_t N64, int64_t K64, int group_m) {
  using T = kcg::GemmDlTile<BM, BN, BK, WAVES_M, WAVES_N, false>;
  const int M = static_cast<int>(M64), N = static_cast<int>(N64), K = static_cast<int>(K64);
  const int64_t bytes_a = M64 * K64 * 4, bytes_b = K64 * N64 * 4, bytes_c = M64 * N64 * 4;
  const int tiles_m = static_cast<int>((M64 + BM - 1) / BM), tiles_n = static_cast<int>((N64 + BN - 1) / BN);
  const bool ragged = (M % BM) || (N % BN) || (K % BK);
  if (K % 4 || N % 4 || K < BK) {
    fprintf(stderr, "not a direct-load problem (K %% 4, N %% 4, K >= BK)\n");
    return 2;
  }
  Range ra, rb, rc, rl;
  int64_t loads = 0, stores = 0;
  const int grid = tiles_m * tiles_n;
  for (int wg = 0; wg < grid; ++wg) {
    const int logical = xcd_contiguous_id(wg, grid);
    const int width = group_m * tiles_n;
    const int group = logical / width;
    const int first_m = group * group_m;
    const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
    const int in_group = logical - group * width;
    const int tile_m = first_m + in_group % gsz;
    const int tile_n = in_group / gsz;
    if (tile_m < 0 || tile_m >= tiles_m || tile_n < 0 || tile_n >= tiles_n) fail("tile index", wg, 0, 0, tile_m);
    const int m0 = as_int(static_cast<int64_t>(tile_m) * BM, "m0", wg, 0, 0);
    const int n0 = as_int(static_cast<int64_t>(tile_n) * BN, "n0", wg, 0, 0);

    // slice bases (bytes from the start of A / B), as the kernel advances them
    const int kfull = K / BK;
    const int ktiles = ragged ? (K + BK - 1) / BK : kfull;
    const int64_t b_step = static_cast<int64_t>(BK) * N * 4;
    int64_t ga = static_cast<int64_t>(m0) * K * 4, gb = static_cast<int64_t>(n0) * 4;
    int64_t ga_lo = ga, ga_hi = ga, gb_lo = gb, gb_hi = gb;
    auto advance_if = [&](bool cond) {
      ga += cond ? BK * 4 : 0;
      gb += cond ? b_step : 0;
      if (ga > ga_hi) ga_hi = ga;
      if (gb > gb_hi) gb_hi = gb;
    };
    advance_if(kfull > 1);
    advance_if(kfull > 2);
    for (int kt = 0; kt < ktiles; ++kt) advance_if(kt + 3 < kfull);
    // the highest base must still be a full slice
    if (ga_hi - static_cast<int64_t>(m0) * K * 4 > static_cast<int64_t>(kfull - 1) * BK * 4)
      fail("A slice base beyond the last full slice", wg, 0, 0, ga_hi);

    for (int wave = 0; wave < T::kWaves; ++wave) {
      const int wm = wave / WAVES_N, wn = wave % WAVES_N;
      for (int lane = 0; lane < 64; ++lane) {
        const int r32 = lane & 31, half = lane >> 5;
        // ---- direct loads of A ----
        for (int i = 0; i < T::kInstrA; ++i) {
          const int idx = (wave * T::kInstrA + i) * 256 + lane * 4;
          const int row = idx / BK;
          const int c_log = ((idx % BK) / 4) ^ T::fa(row);
          const int grow = ragged ? (row < M - m0 ? row : M - m0 - 1) : row;
          const int el = as_int(static_cast<int64_t>(grow) * K + 4 * c_log, "oa element index", wg, wave, lane);
          const unsigned oa = as_u32(static_cast<int64_t>(static_cast<unsigned>(el)) * 4, "oa bytes", wg, wave, lane);
          for (int64_t basep : {ga_lo, ga_hi}) {
            const int64_t addr = basep + oa;  // scalar base + zero-extended lane offset
            if (addr < 0 || addr + 16 > bytes_a) fail("A direct load out of range", wg, wave, lane, addr);
            ra.add(addr, 16);
            ++loads;
          }
          for (int st = 0; st < T::kStages; ++st) {
            const int64_t sa = (static_cast<int64_t>(st) * T::kStageFloats + (wave * T::kInstrA + i) * 256) * 4 + 16 * lane;
            if (sa < 0 || sa + 16 > T::kLdsBytes) fail("A direct load LDS target", wg, wave, lane, sa);
            rl.add(sa, 16);
          }
          // the chunk must be inside the slice: columns 4*c_log .. +3 < BK
          if (c_log < 0 || 4 * c_log + 4 > BK) fail("A chunk outside the slice", wg, wave, lane, c_log);
        }
        // ---- direct loads of B ----
        for (int i = 0; i < T::kInstrB; ++i) {
          const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;
          const int col = idx % BN;
          const int gcol = ragged ? (col < N - n0 ? col : N - n0 - 4) : col;
          const int el = as_int(static_cast<int64_t>(idx / BN) * N + gcol, "ob element index", wg, wave, lane);
          const unsigned ob = as_u32(static_cast<int64_t>(static_cast<unsigned>(el)) * 4, "ob bytes", wg, wave, lane);
          if (gcol < 0) fail("B column clamp below zero", wg, wave, lane, gcol);
          for (int64_t basep : {gb_lo, gb_hi}) {
            const int64_t addr = basep + ob;
            if (addr < 0 || addr + 16 > bytes_b) fail("B direct load out of range", wg, wave, lane, addr);
            rb.add(addr, 16);
            ++loads;
          }
          for (int st = 0; st < T::kStages; ++st) {
            const int64_t sb =
                (static_cast<int64_t>(st) * T::kStageFloats + T::kFloatsA + (wave * T::kInstrB + i) * T::kRunB) * 4 + 16 * lane;
            if (sb < 0 || sb + 16 > T::kLdsBytes) fail("B direct load LDS target", wg, wave, lane, sb);
            rl.add(sb, 16);
          }
        }
        // ---- the partial last slice, re-read through registers ----
        if (ragged && kfull != ktiles) {
          const int k0 = kfull * BK;
          for (int l = 0; l < T::kInstrA + T::kInstrB; ++l) {
            if (l < T::kInstrA) {
              const int idx = (wave * T::kInstrA + l) * 256 + lane * 4;
              const int row = idx / BK;
              const int k = k0 + 4 * (((idx % BK) / 4) ^ T::fa(row));
              const int grow = m0 + (row < M - m0 ? row : M - m0 - 1);
              if (k < K) {
                const int64_t addr = (static_cast<int64_t>(grow) * K + k) * 4;
                if (addr < 0 || addr + 16 > bytes_a) fail("A tail load out of range", wg, wave, lane, addr);
                ra.add(addr, 16);
                ++loads;
              }
              const int64_t la = static_cast<int64_t>(idx) * 4;  // + stage offset
              if (la + 16 > T::kFloatsA * 4) fail("A tail LDS store", wg, wave, lane, la);
            } else {
              const int i = l - T::kInstrA;
              const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;
              const int krow = k0 + idx / BN;
              const int col = idx % BN;
              const int gcol = n0 + (col < N - n0 ? col : N - n0 - 4);
              if (krow < K) {
                const int64_t addr = (static_cast<int64_t>(krow) * N + gcol) * 4;
                if (addr < 0 || addr + 16 > bytes_b) fail("B tail load out of range", wg, wave, lane, addr);
                rb.add(addr, 16);
                ++loads;
              }
              const int64_t lb = (static_cast<int64_t>(T::kFloatsA) + (wave * T::kInstrB + i) * T::kRunB + lane * 4) * 4;
              if (lb + 16 > T::kStageFloats * 4) fail("B tail LDS store", wg, wave, lane, lb);
            }
          }
        }
        // ---- C stores: uniform 64-bit tile origin + 32-bit lane offset ----
        const int64_t c_tile = (static_cast<int64_t>(m0) * N + n0) * 4;
        const unsigned lane_off =
            (static_cast<unsigned>(wm * T::kWaveM + 4 * half) * static_cast<unsigned>(N) +
             static_cast<unsigned>(wn * T::kWaveN + r32)) * 4u;
        const unsigned row_bytes = static_cast<unsigned>(N) * 4u;
        for (int i = 0; i < T::kTilesM; ++i)
          for (int n = 0; n < T::kTilesN; ++n) {
            const int col = n0 + wn * T::kWaveN + n * 32 + r32;
            for (int e = 0; e < 16; ++e) {
              const int local_row = i * 32 + 8 * (e / 4) + (e % 4);
              const int row = m0 + wm * T::kWaveM + 4 * half + local_row;
              if (ragged && !(row < M && col < N)) continue;
              const unsigned off32 = lane_off + static_cast<unsigned>(local_row) * row_bytes + static_cast<unsigned>(n * 32 * 4);
              const int64_t addr = c_tile + off32;
              const int64_t want = (static_cast<int64_t>(row) * N + col) * 4;
              if (addr != want) fail("C store address differs from (row, col)", wg, wave, lane, addr - want);
              if (addr < 0 || addr + 4 > bytes_c) fail("C store out of range", wg, wave, lane, addr);
              rc.add(addr, 4);
              ++stores;
            }
          }
      }
    }
  }
  printf("tile %dx%dx%d waves %dx%d  M %d N %d K %d  %s  grid %d\n", BM, BN, BK, WAVES_M, WAVES_N, M, N, K,
         ragged ? "ragged" : "full", grid);
  printf("A bytes [%lld, %lld) of %lld\n", (long long)ra.lo, (long long)ra.hi, (long long)bytes_a);
  printf("B bytes [%lld, %lld) of %lld\n", (long long)rb.lo, (long long)rb.hi, (long long)bytes_b);
  printf("C bytes [%lld, %lld) of %lld\n", (long long)rc.lo, (long long)rc.hi, (long long)bytes_c);
  printf("LDS bytes [%lld, %lld) of %d\n", (long long)rl.lo, (long long)rl.hi, T::kLdsBytes);
  printf("checked %lld load addresses, %lld store addresses, %d violations\n", (long long)loads, (long long)stores, g_errors);
  // every byte of C must have been written exactly by the union of the stores
  if (rc.lo != 0 || rc.hi != bytes_c) {
    fprintf(stderr, "C not covered\n");
    return 1;
  }
  return g_errors ? 1 : 0;
}

// The launch with K-split tail tiles (gemm_f32_dl_split_kernel<64, 64, 32, 2, 2> followed by
// gemm_split_reduce_kernel): `full` whole tiles, then every remaining tile in `parts` pieces.
// Checks the two-set numbering (every whole tile and every (tile, piece) exactly once), the K
// range every piece loads, that the pieces fill the workspace exactly, and that whole tiles
// plus reduced tiles write every element of C exactly once.  M and N need not be multiples of
// the tile (edge tiles clamp their loads and bound their stores to C; partial tiles go to
// the workspace whole); K is a whole number of slices and N a multiple of 4.
int replay_split(int64_t M64, int64_t N64, int64_t K64, int group_m, int full, int parts) {
  constexpr int BM = 64, BN = 64, BK = 32, WAVES_N = 2;
  using T = kcg::GemmDlTile<BM, BN, BK, 2, 2, false>;
  const int M = static_cast<int>(M64), N = static_cast<int>(N64), K = static_cast<int>(K64);
  if (N % 4 || K % BK) return 2;
  const int64_t bytes_a = M64 * K64 * 4, bytes_b = K64 * N64 * 4;
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN, tiles = tiles_m * tiles_n;
  const int rest = tiles - full;
  if (full % 8 || rest <= 0 || parts < 2 || (K / BK) % parts) return 2;
  const int grid = full + rest * parts;
  const int64_t ws_floats = static_cast<int64_t>(rest) * parts * BM * BN;
  std::vector<unsigned char> c_written(static_cast<size_t>(M) * N, 0), ws_written(static_cast<size_t>(ws_floats), 0);
  std::vector<unsigned char> whole_seen(full, 0), piece_seen(static_cast<size_t>(rest) * parts, 0);
  auto origin = [&](int logical, int *m0, int *n0) {
    const int width = group_m * tiles_n;
    const int group = logical / width;
    const int first_m = group * group_m;
    const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
    const int in_group = logical - group * width;
    *m0 = (first_m + in_group % gsz) * BM;
    *n0 = (in_group / gsz) * BN;
  };
  for (int wg = 0; wg < grid; ++wg) {
    int logical, piece = 0;
    bool partial = false;
    if (wg >= full) {
      const int q = xcd_contiguous_id(wg - full, grid - full);
      logical = full + q / parts;
      piece = q - (q / parts) * parts;
      partial = true;
      if (logical < full || logical >= tiles || piece_seen[static_cast<size_t>(logical - full) * parts + piece]++)
        fail("piece numbering", wg, 0, 0, logical);
    } else {
      logical = xcd_contiguous_id(wg, full);
      if (logical < 0 || logical >= full || whole_seen[logical]++) fail("whole tile numbering", wg, 0, 0, logical);
    }
    int m0, n0;
    origin(logical, &m0, &n0);
    if (m0 < 0 || m0 >= M || n0 < 0 || n0 >= N) fail("tile origin", wg, 0, 0, m0);
    const int my_slices = partial ? (K / BK) / parts : K / BK;
    const int64_t b_step = static_cast<int64_t>(BK) * N * 4;
    const int64_t ga0 = static_cast<int64_t>(m0) * K * 4 + static_cast<int64_t>(piece) * my_slices * (BK * 4);
    const int64_t gb0 = static_cast<int64_t>(n0) * 4 + static_cast<int64_t>(piece) * my_slices * b_step;
    // the slice bases run from the first to the last slice of the range and then stay
    const int64_t ga1 = ga0 + static_cast<int64_t>(my_slices - 1) * BK * 4, gb1 = gb0 + static_cast<int64_t>(my_slices - 1) * b_step;
    // the K columns / rows this workgroup may touch
    const int k_lo = partial ? piece * my_slices * BK : 0, k_hi = k_lo + my_slices * BK;
    for (int wave = 0; wave < T::kWaves; ++wave) {
      const int wm = wave / WAVES_N, wn = wave % WAVES_N;
      for (int lane = 0; lane < 64; ++lane) {
        const int r32 = lane & 31, half = lane >> 5;
        for (int i = 0; i < T::kInstrA; ++i) {
          const int idx = (wave * T::kInstrA + i) * 256 + lane * 4;
          const int row = idx / BK;
          const int grow = row < M - m0 ? row : M - m0 - 1;   // rows at and beyond M fetch the last valid row
          const unsigned oa = as_u32((static_cast<int64_t>(grow) * K + 4 * (((idx % BK) / 4) ^ T::fa(row))) * 4, "oa", wg, wave, lane);
          for (int64_t basep : {ga0, ga1}) {
            const int64_t addr = basep + oa;
            if (addr < 0 || addr + 16 > bytes_a) fail("A load out of range", wg, wave, lane, addr);
            const int64_t col = (addr / 4) % K;
            if (col < k_lo || col + 4 > k_hi) fail("A load outside the piece's K range", wg, wave, lane, col);
          }
        }
        for (int i = 0; i < T::kInstrB; ++i) {
          const int idx = (wave * T::kInstrB + i) * 256 + lane * 4;
          const int col = idx % BN;
          const int gcol = col < N - n0 ? col : N - n0 - 4;   // column chunks at and beyond N fetch the last valid chunk
          const unsigned ob = as_u32((static_cast<int64_t>(idx / BN) * N + gcol) * 4, "ob", wg, wave, lane);
          for (int64_t basep : {gb0, gb1}) {
            const int64_t addr = basep + ob;
            if (addr < 0 || addr + 16 > bytes_b) fail("B load out of range", wg, wave, lane, addr);
            const int64_t krow = (addr / 4) / N;
            if (krow < k_lo || krow >= k_hi) fail("B load outside the piece's K range", wg, wave, lane, krow);
          }
        }
        // stores: to the workspace (leading dimension BN) or to C
        const unsigned ldc = partial ? BN : static_cast<unsigned>(N);
        const unsigned lane_off = (static_cast<unsigned>(wm * T::kWaveM + 4 * half) * ldc + static_cast<unsigned>(wn * T::kWaveN + r32)) * 4u;
        for (int i = 0; i < T::kTilesM; ++i)
          for (int n = 0; n < T::kTilesN; ++n)
            for (int e = 0; e < 16; ++e) {
              const int local_row = i * 32 + 8 * (e / 4) + (e % 4);
              const unsigned off32 = lane_off + static_cast<unsigned>(local_row) * (ldc * 4u) + static_cast<unsigned>(n * 32 * 4);
              if (partial) {
                const int64_t fl = (static_cast<int64_t>(logical - full) * parts + piece) * (BM * BN) + off32 / 4;
                if (fl < 0 || fl >= ws_floats) fail("workspace store out of range", wg, wave, lane, fl);
                else if (ws_written[static_cast<size_t>(fl)]++) fail("workspace float written twice", wg, wave, lane, fl);
                // position inside the partial tile = (row, column) of the tile
                const int row = wm * T::kWaveM + 4 * half + local_row, col = wn * T::kWaveN + n * 32 + r32;
                if (static_cast<int64_t>(off32 / 4) != static_cast<int64_t>(row) * BN + col) fail("partial tile layout", wg, wave, lane, off32);
              } else {
                // whole tiles at the edges of C store only what lies inside it
                const int grow = m0 + wm * T::kWaveM + 4 * half + local_row, gcol = n0 + wn * T::kWaveN + n * 32 + r32;
                if (grow >= M || gcol >= N) continue;
                const int64_t el = (static_cast<int64_t>(m0) * N + n0) + off32 / 4;
                if (el != static_cast<int64_t>(grow) * N + gcol) fail("C store target", wg, wave, lane, el);
                if (el < 0 || el >= static_cast<int64_t>(M) * N) fail("C store out of range", wg, wave, lane, el);
                else if (c_written[static_cast<size_t>(el)]++) fail("C element written twice", wg, wave, lane, el);
              }
            }
      }
    }
  }
  // the second launch: four workgroups per remaining tile, one float4 per thread; a thread
  // reads its float4 of all eight piece slots (slots beyond `parts` re-read piece 0)
  constexpr int kSlabs = BM * BN / 4 / 256;
  for (int wg = 0; wg < rest * kSlabs; ++wg) {
    const int j = wg / kSlabs, slab = wg % kSlabs;
    int m0, n0;
    origin(full + j, &m0, &n0);
    for (int tid = 0; tid < 256; ++tid) {
      const int idx = slab * 256 + tid;
      for (int p = 0; p < 8; ++p) {
        const int64_t fl = static_cast<int64_t>(j) * parts * (BM * BN) + idx * 4 + static_cast<int64_t>(p < parts ? p : 0) * (BM * BN);
        if (fl < 0 || fl + 4 > ws_floats) fail("reduce read out of range", j, 0, 0, fl);
      }
      const int row = m0 + idx / (BN / 4), col = n0 + (idx % (BN / 4)) * 4;
      if (row >= M || col >= N) continue;   // the float4 lies outside C (N is a multiple of 4)
      for (int x = 0; x < 4; ++x) {
        const int64_t el = static_cast<int64_t>(row) * N + col + x;
        if (col + x >= N || el < 0 || el >= static_cast<int64_t>(M) * N) fail("reduce store out of range", j, 0, 0, el);
        else if (c_written[static_cast<size_t>(el)]++) fail("C element written twice (reduce)", j, 0, 0, el);
      }
    }
  }
  for (size_t e = 0; e < c_written.size(); ++e)
    if (!c_written[e]) { fail("C element never written", 0, 0, 0, static_cast<int64_t>(e)); break; }
  for (size_t e = 0; e < ws_written.size(); ++e)
    if (!ws_written[e]) { fail("workspace float never written", 0, 0, 0, static_cast<int64_t>(e)); break; }
  printf("split launch: %d whole tiles + %d tiles in %d pieces, grid %d, workspace %lld bytes: %d violations\n", full, rest,
         parts, grid, static_cast<long long>(ws_floats * 4), g_errors);
  return g_errors ? 1 : 0;
}

}  // namespace

int main(int argc, char **argv) {
  if (argc == 8 && std::string(argv[1]) == "split")
    return replay_split(atoll(argv[2]), atoll(argv[3]), atoll(argv[4]), atoi(argv[5]), atoi(argv[6]), atoi(argv[7]));
  if (argc != 10) {
    fprintf(stderr, "usage: %s BM BN BK WAVES_M WAVES_N M N K GROUP_M\n", argv[0]);
    return 2;
  }
  const int bm = atoi(argv[1]), bn = atoi(argv[2]), bk = atoi(argv[3]), wm = atoi(argv[4]), wn = atoi(argv[5]);
  const int64_t M = atoll(argv[6]), N = atoll(argv[7]), K = atoll(argv[8]);
  const int group_m = atoi(argv[9]);
#define TRY(BM, BN, BK, WM, WN) \
  if (bm == BM && bn == BN && bk == BK && wm == WM && wn == WN) return replay<BM, BN, BK, WM, WN>(M, N, K, group_m);
  TRY(128, 128, 32, 2, 2)
  TRY(128, 128, 16, 2, 2)
  TRY(128, 128, 8, 2, 2)
  TRY(256, 128, 16, 4, 2)
  TRY(256, 128, 32, 4, 2)
  TRY(64, 64, 32, 2, 2)
  TRY(128, 64, 32, 2, 2)
#undef TRY
  fprintf(stderr, "tile not built\n");
  return 2;
}
