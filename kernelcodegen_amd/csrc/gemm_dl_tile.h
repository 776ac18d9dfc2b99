// Tile geometry of the direct-load matmul kernels (gemm_f32_dl_kernel, gemm_f32_stream_kernel):
// LDS layout, swizzle, the split of the tile loads over waves, and the streaming kernel's
// work-item arithmetic.  Kept free of HIP headers so that a host program can include it and
// replay the kernels' address arithmetic with the same constants and functions
// (tests/gemm_dl_address_model.cc, tests/gemm_stream_address_model.cc).
#pragma once

#if defined(__HIPCC__)
#define KCG_HD __host__ __device__
#else
#define KCG_HD
#endif

namespace kcg {

// TRANS_B: B is given as [N][K] (the 'T' operand of BatchedMatmul, Q.K^T): its tile then
// has the shape and the LDS layout of the A tile, rows = n.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool TRANS_B = false>
struct GemmDlTile {
  static constexpr int kWaves = WAVES_M * WAVES_N;
  static constexpr int kThreads = kWaves * 64;
  static constexpr int kWaveM = BM / WAVES_M;
  static constexpr int kWaveN = BN / WAVES_N;
  static constexpr int kTilesM = kWaveM / 32;
  static constexpr int kTilesN = kWaveN / 32;
  static constexpr int kCprA = BK / 4;        // 16-byte chunks per A row
  static constexpr int kRp128A = 8 / kCprA;   // A rows per 128 bytes
  static constexpr int kFloatsA = BM * BK;
  static constexpr int kRowsPerRunB = 256 / BN;      // B rows per 1 KiB run (BN <= 256)
  static constexpr int kRunB = 256 + 2048 / BN;      // floats between runs
  static constexpr int kRunsB = BK * BN / 256;
  static constexpr int kFloatsB = TRANS_B ? BN * BK : kRunsB * kRunB;
  static constexpr int kStageFloats = kFloatsA + kFloatsB;
  static constexpr int kStages = 3;
  static constexpr int kLdsBytes = kStages * kStageFloats * 4;
  static constexpr int kInstrA = kFloatsA / 256 / kWaves;  // 1 KiB loads per wave and slice
  static constexpr int kInstrB = kRunsB / kWaves;
  static constexpr int kSteps = BK / 2;
  static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tile");
  static_assert(BK == 8 || BK == 16 || BK == 32, "K slice");
  static_assert(BN == 64 || BN == 128 || BN == 256, "B rows per run");
  static_assert(kFloatsA % (256 * kWaves) == 0 && kRunsB % kWaves == 0, "load split");
  KCG_HD static constexpr int fa(int row) {
    return ((row / kRp128A) % kCprA) ^ ((row / (kRp128A * kCprA)) & 1);
  }
  // float offset of B row k inside a stage's B region
  KCG_HD static constexpr int brow(int k) {
    return (k / kRowsPerRunB) * kRunB + (k % kRowsPerRunB) * BN;
  }
};

// ---- tiles on 16 x 16 x 4 MFMA blocks: 96 x 96 and 96 x 64 (gemm_f32_t96.h) ----
// Four waves (2 x 2) of BM/2 x BN/2, i.e. BM/32 x BN/32 blocks each; K slices of 32.  The A
// tile has rows of 32 floats with their 16-byte chunks swizzled by fa.  The B tile is stored
// by "row quartets": the k-step s of a slice multiplies rows {4g + s : g = 0..3} of its
// 16-row half at once (lane group g of a wave supplies row 4g + s), so those four rows are
// interleaved in LDS: quartet q = 4 * half + s holds, for every window w of 16 columns, the
// 16 floats of row 4g + s at float offset q * 4 * BN + w * 64 + g * 16, and a wave's
// ds_read_b32 of one operand touches 256 consecutive bytes.
template <int BM, int BN>
struct GemmT96Tile {
  static constexpr int kBM = BM, kBN = BN, kBK = 32, kWavesM = 2, kWavesN = 2;
  static constexpr int kWaveM = BM / 2, kWaveN = BN / 2;
  static constexpr int kBlocksM = kWaveM / 16, kBlocksN = kWaveN / 16;   // 16-wide blocks per wave
  static constexpr int kThreads = 256, kStages = 3;
  static constexpr int kFloatsA = kBM * kBK, kFloatsB = kBK * kBN;
  static constexpr int kStageFloats = kFloatsA + kFloatsB;
  static constexpr int kLdsBytes = kStages * kStageFloats * 4;
  static constexpr int kLoadsA = kFloatsA / 256 / 4, kLoadsB = kFloatsB / 256 / 4;  // 1 KiB loads per wave and slice
  static constexpr int kSteps = kBK / 4;
  static constexpr int kQuartetFloats = 4 * kBN;
  static_assert(BM % 32 == 0 && BN % 32 == 0, "whole 1 KiB loads per wave, whole blocks per wave");
  // Chunk swizzle of the A tile (row r holds its logical 16-byte chunk c at position c ^ fa(r)).
  // A ds_read_b128 is served in four groups of 16 lanes -- lanes {0-3, 12-15, 20-23, 24-27},
  // {4-7, 8-11, 16-19, 28-31} and the same two sets + 32 -- and lane l reads row l % 16, chunk
  // l / 16 of a k-half here, so a group holds all 16 rows, rows 0-3 and 12-15 with one chunk and
  // rows 4-11 with its neighbour (chunk ^ 1).  With r / 2, flipped in its lowest bit for rows
  // 4-11, the eight even rows of a group land in the eight 16-byte slots of one 128-byte half of
  // the 256-byte bank window and the eight odd rows in those of the other.
  KCG_HD static constexpr int fa(int row) {
    const int r = row % 16;
    return (r >> 1) ^ ((r >= 4 && r < 12) ? 1 : 0);
  }
  // float offset inside a slice's B tile -> (row k of the slice, first column) of that 16-byte chunk
  KCG_HD static constexpr int b_row(int idx) {
    const int q = idx / kQuartetFloats, in_q = idx % kQuartetFloats;
    return 16 * (q / 4) + 4 * ((in_q % 64) / 16) + q % 4;
  }
  KCG_HD static constexpr int b_col(int idx) {
    const int in_q = idx % kQuartetFloats;
    return 16 * (in_q / 64) + in_q % 16;
  }
};
using GemmT96Geometry = GemmT96Tile<96, 96>;

// ---- streaming kernel (gemm_f32_stream.h) ----
struct GemmStreamGeometry {
  static constexpr int kBM = 256, kBN = 128, kBK = 16, kWavesM = 4, kWavesN = 2;
  static constexpr int kStages = 4;
  static constexpr int kAhead = 3;           // slices between a load request and its use
  static constexpr int kAccPerLane = 64;     // floats of C per lane and tile
};

// The (matrix, tile) items of workgroup `block` of a grid of `grid` workgroups: every XCD
// (workgroup w runs on XCD w mod xcds) owns a contiguous range of the items, its
// workgroups take them round robin: first, first + step, ... below end.
struct GemmStreamItems {
  int first, end, step;
};
KCG_HD inline GemmStreamItems gemm_stream_items(int block, int grid, int total_items, int xcds) {
  const int xcd = block % xcds;
  GemmStreamItems r;
  r.step = (grid - xcd + xcds - 1) / xcds;   // workgroups on this XCD
  r.end = static_cast<int>(static_cast<long long>(total_items) * (xcd + 1) / xcds);
  r.first = static_cast<int>(static_cast<long long>(total_items) * xcd / xcds) + block / xcds;
  return r;
}

// Matrix index and tile origin of an item; tiles of a matrix in group_m-wide column-major
// groups, as in gemm_f32_dl_kernel.
struct GemmStreamOrigin {
  int bz, m0, n0;
};
KCG_HD inline GemmStreamOrigin gemm_stream_decode(int item, int tiles_m, int tiles_n, int group_m) {
  const int per_mat = tiles_m * tiles_n;
  const int bz = item / per_mat;
  const int logical = item - bz * per_mat;
  const int width = group_m * tiles_n;
  const int group = logical / width;
  const int first_m = group * group_m;
  const int gsz = (tiles_m - first_m) < group_m ? (tiles_m - first_m) : group_m;
  const int in_group = logical - group * width;
  return GemmStreamOrigin{bz, (first_m + in_group % gsz) * GemmStreamGeometry::kBM,
                          (in_group / gsz) * GemmStreamGeometry::kBN};
}

}  // namespace kcg
