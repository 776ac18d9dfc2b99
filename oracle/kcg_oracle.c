/*
 * CPU oracle for the KernelCodeGen hot path (matmul + ReLU, batched matmul,
 * softmax, fused multi-head attention).
 *
 * THIS IS TEST INFRASTRUCTURE.  It is the checker the HIP kernels are compared
 * against and the timed CPU baseline; it is never linked into, loaded by or
 * called from the product library.  Only tests/, __graft_entry__.smoke() and
 * the cpu_baseline leg of bench.py may use it.
 *
 * Every function restates, in plain C, the affine loop nest that the
 * reference's Frontend builds for the same operator.  The reference has no CPU
 * execution path of its own (Rewriter::loweringAffineDialect is declared at
 * include/Optimizer/Rewriter.h:221 and its body is commented out at
 * src/Optimizer/Rewriter.cc:1605-1612), and it cannot be compiled here (it
 * needs MLIR/LLVM 15 and nvcc), so the semantics of the affine module are the
 * specification.  The reference ships no numeric golden vectors; each function
 * below is pinned instead by closed forms, invariants and brute force in
 * tests/test_oracle.py (identity / all-ones / small-integer / rank-1 products,
 * fp64 brute force, softmax shift invariance and row sums, V=1, K=0, causal
 * prefix means, one-hot key selection, the literal three-operator graph).
 *
 * Arithmetic rules kept from the reference:
 *   - fp32 throughout; the accumulator starts at 0.0f and is updated as
 *     acc = a*b + acc with k ascending, multiply and add as two separate
 *     roundings (arith.mulf then arith.addf, src/Frontend/Operators.cc:163-164;
 *     compile with -ffp-contract=off).
 *   - OpenMP is applied to the outer (parallel) loops only, so the order of
 *     operations that produce any one output element never changes.
 *
 * Extensions that the reference graph does not have (explicit opt-ins; with
 * scale = 1, causal = 0 the fmha functions reduce to the reference graph):
 *   - a multiplicative scale applied to S = Q.K^T before the softmax,
 *   - a causal mask (key j > query i contributes nothing),
 *   - bf16 inputs (widened exactly to fp32, then the fp32 algorithm).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define KCG_ORACLE_API __attribute__((visibility("default")))

KCG_ORACLE_API int kcg_oracle_num_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* ------------------------------------------------------------------------ */
/* Matmul  --  src/Frontend/Operators.cc:140-173                              */
/*   for i in [0,M) for j in [0,N) { acc = 0; for k: acc = A[i,k]*B[k,j]+acc; */
/*                                   C[i,j] = acc }                          */
/* Row-major A[M,K], B[K,N], C[M,N] (test/test.cc:16-19, README.md:9-27).     */
/* ------------------------------------------------------------------------ */

/* Literal loop order (i, j, k).  Slow (strided B); used on small shapes to
 * pin the reordered variant below. */
KCG_ORACLE_API void kcg_oracle_matmul_f32_literal(const float *A, const float *B,
                                                  float *C, int64_t M, int64_t N,
                                                  int64_t K) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < M; ++i) {
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        float mul = A[i * K + k] * B[k * N + j];
        acc = mul + acc;
      }
      C[i * N + j] = acc;
    }
  }
}

/* Same arithmetic, loop order (i, k, j) with row i of C as the accumulator:
 * every C[i,j] still starts at 0 and receives a*b + acc for k = 0,1,...,K-1 in
 * that order, so the result is bit-identical to the literal nest while the
 * inner loop streams B rows and vectorises.  Rows [row_begin, row_end) only,
 * so that a bounded sample of a large problem can be computed. */
KCG_ORACLE_API void kcg_oracle_matmul_f32_rows(const float *A, const float *B,
                                               float *C, int64_t M, int64_t N,
                                               int64_t K, int64_t row_begin,
                                               int64_t row_end) {
  (void)M;
#pragma omp parallel for schedule(static)
  for (int64_t i = row_begin; i < row_end; ++i) {
    float *restrict c = C + i * N;
    for (int64_t j = 0; j < N; ++j) c[j] = 0.0f;
    for (int64_t k = 0; k < K; ++k) {
      const float a = A[i * K + k];
      const float *restrict b = B + k * N;
      for (int64_t j = 0; j < N; ++j) {
        float mul = a * b[j];
        c[j] = mul + c[j];
      }
    }
  }
}

KCG_ORACLE_API void kcg_oracle_matmul_f32(const float *A, const float *B, float *C,
                                          int64_t M, int64_t N, int64_t K) {
  kcg_oracle_matmul_f32_rows(A, B, C, M, N, K, 0, M);
}

/* ------------------------------------------------------------------------ */
/* Relu  --  src/Frontend/Operators.cc:229-244                                */
/*   y = arith.maxf(0.0, x): NaN propagates, maxf(+0,-0) = +0.                */
/* In place when y == x (MemorySpace::inplace, Operators.cc:221-227).         */
/* ------------------------------------------------------------------------ */
static inline float kcg_maxf_zero(float x) {
  if (x != x) return x; /* arith.maxf returns NaN if either operand is NaN */
  return x > 0.0f ? x : 0.0f;
}

KCG_ORACLE_API void kcg_oracle_relu_f32(const float *x, float *y, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) y[i] = kcg_maxf_zero(x[i]);
}

/* ------------------------------------------------------------------------ */
/* BatchedMatmul  --  src/Frontend/Operators.cc:353-414                       */
/* Contiguous [batch, rows, cols] operands.  Layout::rowMajor ('N') A is      */
/* [batch, M, K]; Layout::colMajor ('T') A is [batch, K, M]; rowMajor B is    */
/* [batch, K, N]; colMajor B is [batch, N, K] (shape rules Operators.cc:       */
/* 276-308).  The col-major-A index bug at Operators.cc:390-392 (it pushes    */
/* (k, j) instead of (k, i)) is not reproduced: A^T means A[b, k, i].         */
/* ------------------------------------------------------------------------ */
KCG_ORACLE_API void kcg_oracle_batched_matmul_f32(const float *A, int transA,
                                                  const float *B, int transB,
                                                  float *C, int64_t batch,
                                                  int64_t M, int64_t N,
                                                  int64_t K) {
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t b = 0; b < batch; ++b) {
    for (int64_t i = 0; i < M; ++i) {
      const float *Ab = A + b * M * K;
      const float *Bb = B + b * K * N;
      float *Cb = C + b * M * N;
      for (int64_t j = 0; j < N; ++j) {
        float acc = 0.0f;
        for (int64_t k = 0; k < K; ++k) {
          float a = transA ? Ab[k * M + i] : Ab[i * K + k];
          float bv = transB ? Bb[j * K + k] : Bb[k * N + j];
          float mul = a * bv;
          acc = mul + acc;
        }
        Cb[i * N + j] = acc;
      }
    }
  }
}

/* ------------------------------------------------------------------------ */
/* Softmax over the last axis, in place  --  src/Frontend/Operators.cc:471-536*/
/*   sum = 0; for k: sum = exp(x[k]) + sum;   for k: x[k] = exp(x[k]) / sum   */
/* No max subtraction, no scale, no mask (that is what the reference builds). */
/* math.exp has no pinned lowering in the reference; libm expf is used.       */
/* ------------------------------------------------------------------------ */
KCG_ORACLE_API void kcg_oracle_softmax_f32(float *x, int64_t rows, int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < rows; ++r) {
    float *row = x + r * n;
    float sum = 0.0f;
    for (int64_t k = 0; k < n; ++k) sum = expf(row[k]) + sum;
    for (int64_t k = 0; k < n; ++k) row[k] = expf(row[k]) / sum;
  }
}

/* ------------------------------------------------------------------------ */
/* FMHA = BatchedMatmul(Q 'N', K 'T') -> Softmax(axis -1, in place) ->        */
/*        BatchedMatmul(P 'N', V 'N')      (test/test.cc:88-90)               */
/* Q, K, V, O are [B, H, S, D] contiguous fp32.  One row of S is formed at a  */
/* time so the [B,H,S,S] tensor is never allocated; the operations producing  */
/* each output element and their order are those of the three-operator graph. */
/*                                                                            */
/*   s[j] = (sum_d Q[i,d]*K[j,d]) * scale           scale: extension          */
/*   j > i dropped when causal                      causal: extension         */
/*   sum  = sum_j exp(s[j]);  p[j] = exp(s[j]) / sum                          */
/*   O[i,d] = sum_j p[j]*V[j,d]   (j ascending, acc = p*v + acc)              */
/*                                                                            */
/* stable != 0 subtracts the row maximum before exp (mathematically the same  */
/* by shift invariance; avoids overflow for |s| > 88).  The reference form is */
/* stable = 0.                                                                */
/* Query rows [row_begin,row_end) of every (b,h) are computed (bounded        */
/* samples of a large problem); O rows outside the range are left untouched.  */
/* ------------------------------------------------------------------------ */
static void fmha_rows(const float *Q, const float *K, const float *V, float *O,
                      int64_t BH, int64_t S, int64_t D, float scale, int causal,
                      int stable, int64_t row_begin, int64_t row_end) {
  const int64_t nrows = row_end - row_begin;
#pragma omp parallel
  {
    float *s = (float *)malloc((size_t)S * sizeof(float));
    float *acc = (float *)malloc((size_t)D * sizeof(float));
#pragma omp for collapse(2) schedule(dynamic, 8)
    for (int64_t bh = 0; bh < BH; ++bh) {
      for (int64_t r = 0; r < nrows; ++r) {
        const int64_t i = row_begin + r;
        const float *q = Q + (bh * S + i) * D;
        const float *Kb = K + bh * S * D;
        const float *Vb = V + bh * S * D;
        const int64_t jn = causal ? (i + 1) : S;
        float mx = -INFINITY;
        for (int64_t j = 0; j < jn; ++j) {
          const float *kr = Kb + j * D;
          float a = 0.0f;
          for (int64_t d = 0; d < D; ++d) {
            float mul = q[d] * kr[d];
            a = mul + a;
          }
          a = a * scale;
          s[j] = a;
          if (a > mx) mx = a;
        }
        const float shift = stable ? mx : 0.0f;
        float sum = 0.0f;
        for (int64_t j = 0; j < jn; ++j) sum = expf(s[j] - shift) + sum;
        for (int64_t j = 0; j < jn; ++j) s[j] = expf(s[j] - shift) / sum;
        for (int64_t d = 0; d < D; ++d) acc[d] = 0.0f;
        for (int64_t j = 0; j < jn; ++j) {
          const float p = s[j];
          const float *vr = Vb + j * D;
          for (int64_t d = 0; d < D; ++d) {
            float mul = p * vr[d];
            acc[d] = mul + acc[d];
          }
        }
        float *o = O + (bh * S + i) * D;
        for (int64_t d = 0; d < D; ++d) o[d] = acc[d];
      }
    }
    free(s);
    free(acc);
  }
}

KCG_ORACLE_API void kcg_oracle_fmha_f32_rows(const float *Q, const float *K,
                                             const float *V, float *O, int64_t B,
                                             int64_t H, int64_t S, int64_t D,
                                             float scale, int causal, int stable,
                                             int64_t row_begin, int64_t row_end) {
  fmha_rows(Q, K, V, O, B * H, S, D, scale, causal, stable, row_begin, row_end);
}

KCG_ORACLE_API void kcg_oracle_fmha_f32(const float *Q, const float *K,
                                        const float *V, float *O, int64_t B,
                                        int64_t H, int64_t S, int64_t D,
                                        float scale, int causal, int stable) {
  fmha_rows(Q, K, V, O, B * H, S, D, scale, causal, stable, 0, S);
}

/* bf16 <-> fp32.  Widening is exact (bf16 is the top 16 bits of an fp32).
 * Narrowing rounds to nearest even; NaN stays NaN (quiet bit forced). */
static inline float bf16_to_f32(uint16_t h) {
  uint32_t u = (uint32_t)h << 16;
  float f;
  memcpy(&f, &u, sizeof f);
  return f;
}

KCG_ORACLE_API void kcg_oracle_bf16_to_f32(const uint16_t *src, float *dst,
                                           int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) dst[i] = bf16_to_f32(src[i]);
}

KCG_ORACLE_API void kcg_oracle_f32_to_bf16(const float *src, uint16_t *dst,
                                           int64_t n) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    uint32_t u;
    memcpy(&u, &src[i], sizeof u);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
      dst[i] = (uint16_t)((u >> 16) | 0x0040u);
    } else {
      uint32_t lsb = (u >> 16) & 1u;
      u += 0x7fffu + lsb;
      dst[i] = (uint16_t)(u >> 16);
    }
  }
}

/* bf16-input FMHA (extension): Q, K, V hold bf16 bit patterns; they are widened
 * exactly to fp32 and the fp32 algorithm above runs on those values.  The
 * output stays fp32 (a caller comparing against a bf16 result narrows it). */
KCG_ORACLE_API void kcg_oracle_fmha_bf16_rows(const uint16_t *Q, const uint16_t *K,
                                              const uint16_t *V, float *O,
                                              int64_t B, int64_t H, int64_t S,
                                              int64_t D, float scale, int causal,
                                              int stable, int64_t row_begin,
                                              int64_t row_end) {
  const int64_t n = B * H * S * D;
  float *q = (float *)malloc((size_t)n * sizeof(float));
  float *k = (float *)malloc((size_t)n * sizeof(float));
  float *v = (float *)malloc((size_t)n * sizeof(float));
  kcg_oracle_bf16_to_f32(Q, q, n);
  kcg_oracle_bf16_to_f32(K, k, n);
  kcg_oracle_bf16_to_f32(V, v, n);
  fmha_rows(q, k, v, O, B * H, S, D, scale, causal, stable, row_begin, row_end);
  free(q);
  free(k);
  free(v);
}
