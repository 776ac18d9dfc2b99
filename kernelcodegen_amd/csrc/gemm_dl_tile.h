// Tile geometry of the direct-load matmul kernel (gemm_f32_dl_kernel): LDS layout, swizzle
// and the split of the tile loads over waves.  Kept free of HIP headers so that a host
// program can include it and replay the kernel's address arithmetic with the same
// constants (tests/gemm_dl_address_model.cc does).
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

}  // namespace kcg
