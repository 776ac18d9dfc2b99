// Un-fused fp32 operators for graphs that neither the matmul nor the FMHA
// pattern matches: BatchedMatmul (src/Frontend/Operators.cc:253-420) in its four
// layout combinations, and the in-place last-axis Softmax (:425-542).
#include "kcg_common.h"

namespace kcg {

// ---------------------------------------------------------------------------
// Batched matmul: one 64x64 tile of C[b] per workgroup, 4 waves of one
// v_mfma_f32_32x32x2_f32 block each, K walked in slices of 16 through LDS held
// K-major ([k][m] and [k][n]) so both MFMA operands are read along M / N.
// Loads are element-wise and bounds-checked, which makes every layout
// ('N'/'T' for A and for B) and every extent legal.
// ---------------------------------------------------------------------------
template <bool TA, bool TB>
__global__ __launch_bounds__(256) void bmm_f32_kernel(const float *__restrict__ A,
                                                      const float *__restrict__ B,
                                                      float *__restrict__ C, int M, int N, int K,
                                                      int tiles_n) {
  constexpr int BT = 64, BK = 16, PITCH = BT + 8;
  __shared__ float As[BK * PITCH];
  __shared__ float Bs[BK * PITCH];
  const int64_t b = blockIdx.y;
  const float *Ab = A + b * M * K;
  const float *Bb = B + b * K * N;
  float *Cb = C + b * M * N;
  const int tile_m = blockIdx.x / tiles_n;
  const int tile_n = blockIdx.x % tiles_n;
  const int m0 = tile_m * BT, n0 = tile_n * BT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r32 = lane & 31, half = lane >> 5;
  const int wm = wave >> 1, wn = wave & 1;

  float16_t acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0.0f;

  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      // A: walk the contiguous global axis with the fastest thread index.
      const int am = TA ? (idx % BT) : (idx / BK);
      const int ak = TA ? (idx / BT) : (idx % BK);
      const int gm = m0 + am, gk = k0 + ak;
      float av = 0.0f;
      if (gm < M && gk < K) av = TA ? Ab[static_cast<int64_t>(gk) * M + gm] : Ab[static_cast<int64_t>(gm) * K + gk];
      As[ak * PITCH + am] = av;
      const int bn = TB ? (idx / BK) : (idx % BT);
      const int bk = TB ? (idx % BK) : (idx / BT);
      const int gn = n0 + bn, gk2 = k0 + bk;
      float bv = 0.0f;
      if (gn < N && gk2 < K) bv = TB ? Bb[static_cast<int64_t>(gn) * K + gk2] : Bb[static_cast<int64_t>(gk2) * N + gn];
      Bs[bk * PITCH + bn] = bv;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; kk += 2) {
      const float a = As[(kk + half) * PITCH + wm * 32 + r32];
      const float bb = Bs[(kk + half) * PITCH + wn * 32 + r32];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, bb, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  const int col = n0 + wn * 32 + r32;
#pragma unroll
  for (int e = 0; e < 16; ++e) {
    const int row = m0 + wm * 32 + 8 * (e / 4) + 4 * half + (e % 4);
    if (row < M && col < N) Cb[static_cast<int64_t>(row) * N + col] = acc[e];
  }
}

// ---------------------------------------------------------------------------
// Softmax over the last axis, in place, one workgroup per row.
// x = exp(x - max) / sum(exp(x - max)): equal to the reference's
// exp(x) / sum(exp(x)) by shift invariance, without its overflow for x > 88.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

// Generic rows (any length, any alignment): three sweeps over the row, the second and
// third served by the caches.
__global__ __launch_bounds__(256) void softmax_f32_kernel(float *__restrict__ x, int64_t n) {
  __shared__ float red[4];
  float *row = x + static_cast<int64_t>(blockIdx.x) * n;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr float kLog2e = 1.4426950408889634f;

  float m = -INFINITY;
  for (int64_t i = tid; i < n; i += 256) m = fmaxf(m, row[i]);
  m = wave_max(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  const float m_use = (m == -INFINITY) ? 0.0f : m;

  float sum = 0.0f;
  for (int64_t i = tid; i < n; i += 256) sum += exp2f((row[i] - m_use) * kLog2e);
  sum = wave_sum(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = 1.0f / sum;
  for (int64_t i = tid; i < n; i += 256) row[i] = exp2f((row[i] - m_use) * kLog2e) * inv;
}

// Short rows, up to 256 * NV floats (a multiple of 4, 16-byte aligned): one wave per row, the
// whole row in registers -- every element is read once and written once, all loads of a
// row are in flight together, and there is neither LDS nor a barrier.  STREAM marks the
// accesses non-temporal for tensors that are larger than the last-level cache anyway.
template <int NV, bool STREAM>
__global__ __launch_bounds__(256) void softmax_f32_wave_rows_kernel(float *__restrict__ x,
                                                                    int64_t rows, int n4) {
  const int lane = threadIdx.x & 63;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  float4_t *p = reinterpret_cast<float4_t *>(x) + row * n4;
  constexpr float kLog2e = 1.4426950408889634f;
  float4_t v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + 64 * i;
    v[i] = float4_t{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    if (c < n4) v[i] = STREAM ? __builtin_nontemporal_load(p + c) : p[c];
  }
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) m = fmaxf(fmaxf(m, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
  m = wave_max(m);
  const float m_use = (m == -INFINITY) ? 0.0f : m;
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[i][e] = __builtin_amdgcn_exp2f((v[i][e] - m_use) * kLog2e);
      sum += v[i][e];
    }
  sum = wave_sum(sum);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = lane + 64 * i;
    const float4_t r = v[i] * inv;
    if (c < n4) {
      if (STREAM) __builtin_nontemporal_store(r, p + c);
      else p[c] = r;
    }
  }
}

// Rows of up to 1024 * NV floats (NV up to 32: 32768 floats, 128 registers): one workgroup
// per row, the row in registers, maximum and sum combined through LDS.
template <int NV, bool STREAM>
__global__ __launch_bounds__(256) void softmax_f32_block_row_kernel(float *__restrict__ x, int n4) {
  __shared__ float red[8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float4_t *p = reinterpret_cast<float4_t *>(x) + static_cast<int64_t>(blockIdx.x) * n4;
  constexpr float kLog2e = 1.4426950408889634f;
  float4_t v[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = tid + 256 * i;
    v[i] = float4_t{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    if (c < n4) v[i] = STREAM ? __builtin_nontemporal_load(p + c) : p[c];
  }
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) m = fmaxf(fmaxf(m, fmaxf(v[i][0], v[i][1])), fmaxf(v[i][2], v[i][3]));
  m = wave_max(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float m_use = (m == -INFINITY) ? 0.0f : m;
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[i][e] = __builtin_amdgcn_exp2f((v[i][e] - m_use) * kLog2e);
      sum += v[i][e];
    }
  sum = wave_sum(sum);
  if (lane == 0) red[4 + wave] = sum;
  __syncthreads();
  sum = (red[4] + red[5]) + (red[6] + red[7]);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = tid + 256 * i;
    const float4_t r = v[i] * inv;
    if (c < n4) {
      if (STREAM) __builtin_nontemporal_store(r, p + c);
      else p[c] = r;
    }
  }
}

// Rows of up to 256 * NV floats with no alignment to rely on (row length not a multiple of
// 4): the same register-resident scheme with one float per access; consecutive lanes read
// consecutive floats, so a wave still moves whole 256-byte segments.
template <int NV>
__global__ __launch_bounds__(256) void softmax_f32_block_row_scalar_kernel(float *__restrict__ x, int n) {
  __shared__ float red[8];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  float *p = x + static_cast<int64_t>(blockIdx.x) * n;
  constexpr float kLog2e = 1.4426950408889634f;
  float v[NV];
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = tid + 256 * i;
    v[i] = c < n ? p[c] : -INFINITY;
    m = fmaxf(m, v[i]);
  }
  m = wave_max(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  const float m_use = (m == -INFINITY) ? 0.0f : m;
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    v[i] = __builtin_amdgcn_exp2f((v[i] - m_use) * kLog2e);
    sum += v[i];
  }
  sum = wave_sum(sum);
  if (lane == 0) red[4 + wave] = sum;
  __syncthreads();
  sum = (red[4] + red[5]) + (red[6] + red[7]);
  const float inv = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int c = tid + 256 * i;
    if (c < n) p[c] = v[i] * inv;
  }
}

}  // namespace kcg

extern "C" {

// At most 65535 matrices per launch (grid.y).
static int batched_matmul_chunk(const float *A, int transA, const float *B, int transB, float *C,
                                int64_t batch, int64_t M, int64_t N, int64_t K, hipStream_t s) {
  const int64_t tiles_m = (M + 63) / 64, tiles_n = (N + 63) / 64;
  // the two layouts of the attention graph (Q.K^T is NT, P.V is NN: test/test.cc:71-90) run
  // on the direct-load matmul kernel when their rows are 16-byte aligned
  if (!transA) {
    const int st = kcg::dispatch_bmm_dl(A, B, C, batch, M, N, K, transB != 0, s);
    if (st != KCG_ERR_UNSUPPORTED_SHAPE) return st;
  }
  dim3 grid(static_cast<unsigned>(tiles_m * tiles_n), static_cast<unsigned>(batch));
  const int m = static_cast<int>(M), n = static_cast<int>(N), k = static_cast<int>(K);
  const int tn = static_cast<int>(tiles_n);
  if (!transA && !transB) return kcg::launch(kcg::bmm_f32_kernel<false, false>, grid, dim3(256), 0, s, A, B, C, m, n, k, tn);
  if (!transA && transB) return kcg::launch(kcg::bmm_f32_kernel<false, true>, grid, dim3(256), 0, s, A, B, C, m, n, k, tn);
  if (transA && !transB) return kcg::launch(kcg::bmm_f32_kernel<true, false>, grid, dim3(256), 0, s, A, B, C, m, n, k, tn);
  return kcg::launch(kcg::bmm_f32_kernel<true, true>, grid, dim3(256), 0, s, A, B, C, m, n, k, tn);
}

int kcg_batched_matmul_f32(const float *A, int transA, const float *B, int transB, float *C,
                           int64_t batch, int64_t M, int64_t N, int64_t K, void *stream) {
  if (!A || !B || !C) return KCG_ERR_NULL_POINTER;
  if (batch <= 0 || M <= 0 || N <= 0 || K <= 0) return KCG_ERR_BAD_SHAPE;
  if ((transA != 0 && transA != 1) || (transB != 0 && transB != 1)) return KCG_ERR_BAD_ARGUMENT;
  if (M > 0x7fffffffLL || N > 0x7fffffffLL || K > 0x7fffffffLL ||
      ((M + 63) / 64) * ((N + 63) / 64) > 0x7fffffffLL)
    return KCG_ERR_BAD_SHAPE;
  // tensors of 2^31 elements and more: not verified on the GPU (see kcg_gemm_f32)
  {
    const int64_t mk = M * K, kn = K * N, mn = M * N;  // each below 2^62
    const int64_t largest = mk > kn ? (mk > mn ? mk : mn) : (kn > mn ? kn : mn);
    if (batch > 0x7fffffffLL / largest) return KCG_ERR_UNSUPPORTED_SHAPE;
  }
  constexpr int64_t kMaxPerLaunch = 65535;
  for (int64_t b0 = 0; b0 < batch; b0 += kMaxPerLaunch) {
    const int64_t nb = batch - b0 < kMaxPerLaunch ? batch - b0 : kMaxPerLaunch;
    const int st = batched_matmul_chunk(A + b0 * M * K, transA, B + b0 * K * N, transB, C + b0 * M * N, nb,
                                        M, N, K, static_cast<hipStream_t>(stream));
    if (st != KCG_OK) return st;
  }
  return KCG_OK;
}

int kcg_softmax_f32(float *x, int64_t rows, int64_t n, void *stream) {
  if (!x) return KCG_ERR_NULL_POINTER;
  if (rows <= 0 || n <= 0 || rows > 0x7fffffffLL) return KCG_ERR_BAD_SHAPE;
  if (rows > 0x7fffffffLL / n) return KCG_ERR_UNSUPPORTED_SHAPE;  // same limit as every entry point
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (n % 4 == 0 && n <= 32768 && kcg::aligned16(x)) {
    const int n4 = static_cast<int>(n / 4);
    // a tensor that does not fit the 256 MiB last-level cache is streamed past it
    const bool stream_past = rows * n * 4 > (int64_t{192} << 20);
    const dim3 wave_grid(static_cast<unsigned>((rows + 3) / 4)), row_grid(static_cast<unsigned>(rows));
#define KCG_WAVE_ROWS(NV)                                                                          \
  return stream_past ? kcg::launch(kcg::softmax_f32_wave_rows_kernel<NV, true>, wave_grid,         \
                                   dim3(256), 0, s, x, rows, n4)                                   \
                     : kcg::launch(kcg::softmax_f32_wave_rows_kernel<NV, false>, wave_grid,        \
                                   dim3(256), 0, s, x, rows, n4)
#define KCG_BLOCK_ROW(NV)                                                                          \
  return stream_past ? kcg::launch(kcg::softmax_f32_block_row_kernel<NV, true>, row_grid,          \
                                   dim3(256), 0, s, x, n4)                                         \
                     : kcg::launch(kcg::softmax_f32_block_row_kernel<NV, false>, row_grid,         \
                                   dim3(256), 0, s, x, n4)
    if (n4 <= 64) KCG_WAVE_ROWS(1);
    if (n4 <= 128) KCG_WAVE_ROWS(2);
    if (n4 <= 256) KCG_WAVE_ROWS(4);
    if (n4 <= 512) KCG_BLOCK_ROW(2);
    if (n4 <= 1024) KCG_BLOCK_ROW(4);
    if (n4 <= 2048) KCG_BLOCK_ROW(8);
    if (n4 <= 4096) KCG_BLOCK_ROW(16);
    KCG_BLOCK_ROW(32);
#undef KCG_WAVE_ROWS
#undef KCG_BLOCK_ROW
  }
  if (n <= 8192) {
    const dim3 row_grid(static_cast<unsigned>(rows));
    const int ni = static_cast<int>(n);
    if (n <= 1024) return kcg::launch(kcg::softmax_f32_block_row_scalar_kernel<4>, row_grid, dim3(256), 0, s, x, ni);
    if (n <= 2048) return kcg::launch(kcg::softmax_f32_block_row_scalar_kernel<8>, row_grid, dim3(256), 0, s, x, ni);
    if (n <= 4096) return kcg::launch(kcg::softmax_f32_block_row_scalar_kernel<16>, row_grid, dim3(256), 0, s, x, ni);
    return kcg::launch(kcg::softmax_f32_block_row_scalar_kernel<32>, row_grid, dim3(256), 0, s, x, ni);
  }
  return kcg::launch(kcg::softmax_f32_kernel, dim3(static_cast<unsigned>(rows)), dim3(256), 0, s, x, n);
}

}  // extern "C"
