/*
 * kcg.h -- C-ABI of the MI355X (gfx950) kernels that stand in for the text the
 * reference's CUDA emitter prints.
 *
 * The reference's backend entry is `std::string CUDAGen(mlir::ModuleOp&)`
 * (include/Backend/CUDA.h:6, src/Backend/CUDA.cc:878-890).  It prints one
 *     namespace <graph> { __global__ void kernelN(float* arg0, float* arg1, ...) }
 * per optimised function (src/Backend/CUDA.cc:793-801), with raw device
 * pointers in first-use order (A,B,C / Q,K,V,O), every size baked in, and the
 * launch geometry only in a comment (src/Backend/CUDA.cc:786-791).  A harness
 * outside the reference tree allocates, copies, launches and times
 * (test/test.cc:27-34).  The entry points below are what such a harness binds
 * instead: same operand order, caller-owned device pointers, row-major
 * contiguous tensors, no hidden allocation, no implicit synchronisation; the
 * launch is asynchronous on the given HIP stream (0 = the null stream).
 *
 * Unlike the reference (assert(false) / exit(EXIT_FAILURE), e.g.
 * src/Frontend/Operators.cc:271, include/KernelCodeGen.h:78-81) nothing here
 * aborts: every entry point returns a kcg_status.
 *
 * All entry points are thread-safe and hold no state between calls.  A call may
 * issue more than one kernel on the stream.  No tensor may have 2^31 elements
 * or more (KCG_ERR_UNSUPPORTED_SHAPE): the one run with a larger operand ended in a GPU
 * memory fault whose cause is not known (a host replay of the matmul kernel's address
 * arithmetic, tests/gemm_dl_address_model.cc, finds every access of that call inside its
 * tensor).  The largest operand that has been run on the GPU is 1 GiB; operands between
 * 1 GiB and the limit are accepted but unverified.
 */
#ifndef KCG_H
#define KCG_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define KCG_API __attribute__((visibility("default")))

typedef enum kcg_status {
  KCG_OK = 0,
  KCG_ERR_NULL_POINTER = 1,      /* a required pointer argument is NULL        */
  KCG_ERR_BAD_SHAPE = 2,         /* non-positive or overflowing extent         */
  KCG_ERR_UNSUPPORTED_SHAPE = 3, /* extent not handled by the selected kernel  */
  KCG_ERR_BAD_SCHEDULE = 4,      /* tile sizes that no kernel is built for     */
  KCG_ERR_BAD_ARGUMENT = 5,      /* unknown epilogue / dtype / flag            */
  KCG_ERR_LAUNCH = 6,            /* HIP reported an error at launch            */
  KCG_ERR_NO_DEVICE = 7          /* no usable gfx950 device                    */
} kcg_status;

/* Human-readable text for a status (never NULL). */
KCG_API const char *kcg_status_str(int status);

/* Library version "major.minor.patch". */
KCG_API const char *kcg_version(void);

/* ---- tiled fp32 matmul (+ fused ReLU epilogue) ---------------------------- */

/* Epilogue applied to each C element before it is stored.  KCG_EPILOGUE_RELU is
 * arith.maxf(0, x) as the reference's Relu operator defines it
 * (src/Frontend/Operators.cc:238-242): NaN propagates, -0 becomes +0.  The
 * reference never fuses it (its emitter skips the Relu function,
 * src/Backend/CUDA.cc:859-866); the fusion is an extension. */
typedef enum kcg_epilogue { KCG_EPILOGUE_NONE = 0, KCG_EPILOGUE_RELU = 1 } kcg_epilogue;

/* Schedule of the matmul kernel: the string-keyed tile table of the reference
 * (include/KernelCodeGen.h:34-37: BLOCK_SIZE_M/N/K, GROUP_SIZE_M, THREAD_SIZE_M/N,
 * VECTORIZE_WIDTH, WARP_SIZE) as a plain struct.  A NULL schedule, or a field
 * set to 0, selects the built-in default for gfx950 (256 x 128 x 16 block tile,
 * wave64, 64 x 64 per-wave tile of 32x32x2 fp32 MFMA blocks, group_m 8; with no tile
 * given the library picks among its tiles by problem size).  Built tiles (block_m x
 * block_n x block_k, wave_m x wave_n): 256x128x{16,32} and 128x128x{8,16,32} in waves of
 * 64x64, 128x64x32 in 64x32, 64x64x32 in 32x32, and 96x96x32 / 96x64x32 in waves of 48x48 /
 * 48x32 (16x16x4 MFMA blocks; K a multiple of 32 and N of 4, else KCG_ERR_BAD_SCHEDULE). */
typedef struct kcg_gemm_sched {
  int32_t block_m;   /* BLOCK_SIZE_M: rows of C per workgroup                  */
  int32_t block_n;   /* BLOCK_SIZE_N: columns of C per workgroup               */
  int32_t block_k;   /* BLOCK_SIZE_K: K-slice staged in LDS per step           */
  int32_t group_m;   /* GROUP_SIZE_M: M-tiles per rasterisation group          */
  int32_t wave_m;    /* rows of C per wavefront (the THREAD_SIZE_M analogue)   */
  int32_t wave_n;    /* columns of C per wavefront (THREAD_SIZE_N analogue)    */
  int32_t vec_width; /* VECTORIZE_WIDTH: floats per global/LDS access (4)      */
  int32_t wave_size; /* WARP_SIZE: must be 64 (or 0) on gfx950                 */
  int32_t lds_stages;/* copies of the K-slice tiles held in LDS, i.e. the leading
                      * dimension Rewriter::pipeline gives the shared buffers
                      * (src/Optimizer/Rewriter.cc:809-1180; the reference's
                      * schedule has 2).  2: slices staged through registers into
                      * double-buffered LDS; 3: ring of three filled by direct
                      * global->LDS loads (needs 16-byte aligned rows, K >= block_k);
                      * 1: one copy, the staged schedule that precedes pipeline in the
                      * reference's recipe (two barriers per slice; built for the
                      * 128x128x8 and 256x128x16 tiles); 0: the library chooses
                      * (3 where the shape allows, else 2). */
} kcg_gemm_sched;

/* C[M,N] = epilogue(A[M,K] . B[K,N]); fp32, row-major, contiguous.
 * Replaces `<graph>::kernel0(float* A, float* B, float* C)` as generated for
 * Matmul_m<M>n<N>k<K> (src/Optimizer/Optimizer.cc:383-548; prototype
 * src/Backend/CUDA.cc:793-801; adaptor contract test/test.cc:27-33).
 * Any M, N, K >= 1 is accepted (the reference requires M, N % 128 == 0 and
 * K % 8 == 0, src/Optimizer/Rewriter.cc:124-128); ragged edges take a
 * bounds-checked path.  A, B, C must not alias.  Each of A, B and C is limited to
 * 2^31 - 1 elements (8 GiB); beyond that KCG_ERR_UNSUPPORTED_SHAPE is returned. */
KCG_API int kcg_gemm_f32(const float *A, const float *B, float *C, int64_t M,
                         int64_t N, int64_t K, int epilogue,
                         const kcg_gemm_sched *sched, void *stream);

/* Launch geometry the call above would use, for logging in the reference's
 * "// grid dims:(..), block dims:(..)" style (src/Backend/CUDA.cc:786-791). */
typedef struct kcg_launch_info {
  int32_t grid[3];
  int32_t block[3];
  int32_t lds_bytes;
  int32_t waves_per_block;
  char kernel[64];
  /* A matmul whose tile count leaves the last round of workgroups nearly empty is run as
   * two launches on the same stream: `main_rows` rows of C on the tile above, the
   * remaining `tail_rows` on a smaller tile.  launches == 1: the tail_* fields are 0. */
  int32_t launches;
  int32_t main_rows;
  int32_t tail_rows;
  int32_t tail_grid[3];
  int32_t tail_block[3];
  int32_t tail_lds_bytes;
  char tail_kernel[64];
} kcg_launch_info;

/* Applies the same shape checks as kcg_gemm_f32 (a shape that call refuses is refused
 * here with the same status). */
KCG_API int kcg_gemm_f32_query(int64_t M, int64_t N, int64_t K,
                               const kcg_gemm_sched *sched, kcg_launch_info *out);

/* kcg_gemm_f32 with a workspace lent by the caller.  The reference's generated kernel
 * takes A, B, C only (src/Backend/CUDA.cc:793-801) and every plan of kcg_gemm_f32 keeps to
 * that; one more plan needs device memory for partial sums: where K is a multiple of 32 and
 * N of 4 (any M; at most 6400 tiles of 64 x 64), the tile is left to the library, K is long
 * enough to pay for a second launch and the tile count is some rounds of the compute units
 * plus a rest (1536^3: 2 x 256 + 64; 1792^3: 3 x 256 + 16), or smaller than the number of
 * compute units altogether (512 x 512 x 4096), the tiles of the rest are cut along K into 2
 * to 8 pieces each and the pieces are added up by a second launch (fixed order: results do
 * not vary between runs).
 * kcg_gemm_f32_ws_bytes gives the bytes the preferred plan needs, 0 where there is none (at
 * most 32 MiB).  `workspace` must be 16-byte aligned device memory which nothing else uses
 * until the call has completed on `stream`; the call runs the best plan whose partial sums
 * fit into `workspace_bytes` (fewer pieces per tile than the preferred plan, if need be) and,
 * with NULL or where none fits, behaves exactly like kcg_gemm_f32.  Same arguments and
 * statuses otherwise. */
KCG_API int64_t kcg_gemm_f32_ws_bytes(int64_t M, int64_t N, int64_t K,
                                      const kcg_gemm_sched *sched);
KCG_API int kcg_gemm_f32_ws(const float *A, const float *B, float *C, int64_t M,
                            int64_t N, int64_t K, int epilogue,
                            const kcg_gemm_sched *sched, void *workspace,
                            int64_t workspace_bytes, void *stream);

/* Launch geometry of kcg_gemm_f32_ws for a workspace of `workspace_bytes` (the counterpart
 * of kcg_gemm_f32_query, same logging purpose, src/Backend/CUDA.cc:786-791).  Where the
 * K-split plan runs, launches == 2: grid / block / lds_bytes / kernel describe the launch
 * of whole tiles and pieces (main_rows = M, tail_rows = 0: both launches cover all rows),
 * the tail_* fields the launch that adds the pieces up.  Otherwise the answer is that of
 * kcg_gemm_f32_query.  For kcg_gemm_f32_noalloc pass 4 MiB. */
KCG_API int kcg_gemm_f32_ws_query(int64_t M, int64_t N, int64_t K,
                                  const kcg_gemm_sched *sched, int64_t workspace_bytes,
                                  kcg_launch_info *out);

/* kcg_gemm_f32_ws without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that can neither allocate device memory
 * nor lend any: code under HIP graph capture, tight serving loops, harnesses that forbid
 * allocation.  The partial sums of the K-split plan go to a 4 MiB array that is part of the
 * library's device code (one copy per GPU, held until the process ends): the call runs the
 * plan kcg_gemm_f32_ws runs when it is lent exactly 4 MiB (256 pieces at most; plans with
 * more pieces are not considered, a plan that did not fit would be refused with
 * KCG_ERR_UNSUPPORTED_SHAPE).  All calls on one GPU share that array: calls that overlap in
 * time on one GPU (two streams, two threads) race on it and must be serialised by the
 * caller.  Same arguments, statuses and results as kcg_gemm_f32_ws with 4 MiB.
 * The first call on a device looks up the array's address (hipGetSymbolAddress), and the
 * first launch of a kernel variant that needs more than 48 KiB of LDS raises that kernel's
 * limit (hipFuncSetAttribute): make one call per device and problem class outside graph
 * capture before capturing one; under capture the call then only launches kernels (no
 * memset node is recorded). */
KCG_API int kcg_gemm_f32_noalloc(const float *A, const float *B, float *C, int64_t M,
                                 int64_t N, int64_t K, int epilogue,
                                 const kcg_gemm_sched *sched, void *stream);

/* ---- fused multi-head attention ------------------------------------------ */

/* Schedule of the FMHA kernel: the reference's table (include/KernelCodeGen.h:
 * 38-41; Br = HdxBr / Hd, Bc = BrxBc / Br, src/Optimizer/Optimizer.cc:1136-1144)
 * reduced to the two tile extents.  NULL or 0 selects the gfx950 default. */
typedef struct kcg_fmha_sched {
  int32_t br; /* query rows per workgroup: 128 (4 waves) or 256 (8 waves)      */
  int32_t bc; /* key/value rows per inner step: fp32 32 or 64 (not 256 x 64 at
               * D = 128), bf16 64                                             */
} kcg_fmha_sched;

/* O = softmax(scale * Q.K^T [+ causal mask]) . V, all [B,H,S,D] contiguous fp32.
 * Replaces the kernel generated for
 * Fused_Multi_Head_Attention_<b>_<h>_SL<S>_HD<D>(Q,K,V,O)
 * (src/Optimizer/Optimizer.cc:1101-1118); semantics are those of the Frontend
 * graph BatchedMatmul(Q,K^T) -> Softmax(axis -1) -> BatchedMatmul(P,V)
 * (test/test.cc:88-90).  scale = 1 and causal = 0 give exactly that graph;
 * scale and causal are extensions.  D must be 64 or 128; any S >= 1; each tensor is
 * limited to 2^31 - 1 elements (KCG_ERR_UNSUPPORTED_SHAPE beyond; also for the bf16
 * entry point and for every operand of kcg_batched_matmul_f32). */
KCG_API int kcg_fmha_f32(const float *Q, const float *K, const float *V, float *O,
                         int32_t B, int32_t H, int32_t S, int32_t D, float scale,
                         int causal, const kcg_fmha_sched *sched, void *stream);

typedef enum kcg_dtype { KCG_F32 = 0, KCG_BF16 = 1 } kcg_dtype;

/* Same, with Q, K, V holding bf16 bit patterns (extension: the reference knows
 * only float32/float64/float16, src/Frontend/Operators.cc:5-10).  Products are
 * bf16 x bf16 accumulated in fp32; softmax in fp32; P is rounded to bf16 before
 * the second product.  O is written as o_dtype (KCG_BF16 or KCG_F32).
 *
 * Deviation from the fp32 evaluation of the same bf16 inputs: the weights of a row
 * are rounded to bf16 (unit roundoff 2^-8) and the row is normalised by the sum of
 * the rounded weights, so every element obeys
 *   |O - O_fp32| <= 2^-8 (sum_j P_ij |V_jd| + |O_id|)   (P the normalised weights)
 * up to fp32 rounding, plus 2^-8 |O_id| when O is written as bf16.  For rows that
 * average many keys this is far inside 2e-2 of the output's RMS; a causal row that
 * sees only a handful of keys with cancelling V values can reach 2.4e-2 of that RMS
 * on single elements (it stays inside the bound above and inside 2e-2 of max|O|). */
KCG_API int kcg_fmha_bf16(const uint16_t *Q, const uint16_t *K, const uint16_t *V,
                          void *O, int o_dtype, int32_t B, int32_t H, int32_t S,
                          int32_t D, float scale, int causal,
                          const kcg_fmha_sched *sched, void *stream);

KCG_API int kcg_fmha_query(int dtype, int32_t B, int32_t H, int32_t S, int32_t D,
                           int causal, const kcg_fmha_sched *sched,
                           kcg_launch_info *out);

/* ---- un-fused operators (graphs the two patterns above do not match) ------ */

/* y = maxf(0, x) elementwise; y may equal x (MemorySpace::inplace).
 * src/Frontend/Operators.cc:182-250. */
KCG_API int kcg_relu_f32(const float *x, float *y, int64_t n, void *stream);

/* C[b] = op(A[b]) . op(B[b]) for `batch` contiguous matrices.
 * transA = 0: A is [batch,M,K]; 1: [batch,K,M].  transB = 0: B is [batch,K,N];
 * 1: [batch,N,K].  src/Frontend/Operators.cc:253-420 (name suffix _NN/_NT/...,
 * :329-339).  NN and NT with 16-byte aligned rows (K % 4 == 0, and N % 4 == 0 for
 * NN) run on the tiled matmul kernel; every other case on a generic kernel. */
KCG_API int kcg_batched_matmul_f32(const float *A, int transA, const float *B,
                                   int transB, float *C, int64_t batch, int64_t M,
                                   int64_t N, int64_t K, void *stream);

/* In-place softmax over the last axis of a [rows, n] tensor:
 * x = exp(x) / sum(exp(x)), src/Frontend/Operators.cc:425-542 -- evaluated as
 * exp(x - max) / sum(exp(x - max)), which is the same number by shift invariance wherever
 * the reference's literal form is finite, and stays finite where that form overflows
 * (x > 88 gives inf / inf = NaN there).  A deliberate deviation. */
KCG_API int kcg_softmax_f32(float *x, int64_t rows, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* KCG_H */
