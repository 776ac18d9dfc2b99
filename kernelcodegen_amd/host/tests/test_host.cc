// Unit tests of the C++ host layer.  No GPU is needed: nothing here launches a
// kernel (the backend binding only asks the library for launch geometry).
//
// The structural expectations for the matmul schedule are the facts pinned by
// the stage-by-stage IR dumps in the reference's README.md (lines 9-231 there):
// loop bounds and steps after each split, loop order after reorder, grid
// (32,16) / block (16,16) and the d0*128 / d0*8 maps after parallel, the 8x8
// register buffer after bufferize, the init / k-m-n / write-back fission after
// the second reorder, and `0 to 1024 step 8` x `0 to 8` after the k split.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <functional>
#include <iostream>
#include <sstream>
#include <string>
#include <vector>

#include "IR/Interpreter.h"
#include "KernelCodeGen.h"

using namespace KernelCodeGen;
using namespace KernelCodeGen::ir;

static int g_failed = 0, g_checks = 0;
#define CHECK(cond)                                                              \
  do {                                                                           \
    ++g_checks;                                                                  \
    if (!(cond)) {                                                               \
      ++g_failed;                                                                \
      std::printf("  CHECK FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
    }                                                                            \
  } while (0)

static int count(const std::string &hay, const std::string &needle) {
  int n = 0;
  for (size_t pos = hay.find(needle); pos != std::string::npos; pos = hay.find(needle, pos + 1)) ++n;
  return n;
}

static bool contains(const std::string &hay, const std::string &needle) {
  return hay.find(needle) != std::string::npos;
}

// Runs `fn` with stderr silenced (error-path tests print the library's messages).
static void quiet(const std::function<void()> &fn) {
  std::ostringstream sink;
  auto *old = std::cerr.rdbuf(sink.rdbuf());
  fn();
  std::cerr.rdbuf(old);
}

struct MatmulFixture {
  KernelCodeGenerator gen{"ROCm"};
  ComputeDAG *graph = nullptr;
  Value A, B, C;
  FuncOp func;
  std::vector<ForOp> loops;
  MatmulFixture(int64_t m, int64_t n, int64_t k, const std::string &name = "fuse_matmul_relu") {
    gen.setLogMode(Log::Release);
    graph = &gen.createGraph(name);
    A = graph->create<PlaceHolder>(std::vector<int64_t>{m, k}, std::string{"float32"});
    B = graph->create<PlaceHolder>(std::vector<int64_t>{k, n}, std::string{"float32"});
    C = graph->create<Matmul>(A, B, MemorySpace::global);
    func = Analyzer::collectFunctions(graph->module, "Matmul")[0];
    loops = Analyzer::collectFuncLoops(func);
  }
};

static void test_frontend_matmul_nest() {
  MatmulFixture f(4096, 2048, 1024);
  CHECK(f.func.getSymName() == "Matmul_m4096n2048k1024");
  CHECK(f.func.getAttr("func.state") == "cpu");
  CHECK(f.loops.size() == 3);
  CHECK(f.loops[0].getUpperBound() == 4096 && f.loops[1].getUpperBound() == 2048 && f.loops[2].getUpperBound() == 1024);
  CHECK(f.loops[2].numIterArgs() == 1 && f.loops[0].numIterArgs() == 0);
  CHECK(verify(f.graph->module.get()).empty());
  const std::string text = f.graph->module.str();
  CHECK(contains(text, "memref<4096x1024xf32, 1>"));
  CHECK(contains(text, "memref<1024x2048xf32, 1>"));
  CHECK(contains(text, "memref<4096x2048xf32, 1>"));
  CHECK(contains(text, "affine.for %arg3 = 0 to 4096 {"));
  CHECK(contains(text, "iter_args("));
  // mulf first, then addf(product, accumulator): operand order matters for the oracle
  Op *k = f.loops[2].op;
  std::vector<Op *> body;
  for (auto &o : k->body) body.push_back(o.get());
  CHECK(body.size() == 5);
  CHECK(body[0]->kind == OpKind::Load && body[1]->kind == OpKind::Load);
  CHECK(body[2]->kind == OpKind::MulF && body[3]->kind == OpKind::AddF);
  CHECK(body[3]->operands[0] == body[2]->result() && body[3]->operands[1] == k->arg(1));
  CHECK(body[0]->memref == f.func.getArguments()[0] && body[1]->memref == f.func.getArguments()[1]);
  // A[i,k], B[k,j]
  CHECK(body[0]->indices[0].uses(f.loops[0].getInductionVar()) && body[0]->indices[1].uses(k->arg(0)));
  CHECK(body[1]->indices[0].uses(k->arg(0)) && body[1]->indices[1].uses(f.loops[1].getInductionVar()));
  // module level: three allocs, then the call A,B,C -> C
  auto calls = Analyzer::collectFuncCalls(f.graph->module);
  CHECK(calls.size() == 1 && calls[0].getArgOperands().size() == 3);
  CHECK(calls[0].getArgOperands()[0] == f.A && calls[0].getArgOperands()[1] == f.B);
  CHECK(f.C == calls[0].getResult(0));
}

static void test_schedule_stages_match_readme() {
  MatmulFixture f(4096, 2048, 1024);
  ModuleOp &module = f.graph->module;
  ForOp loopM = f.loops[0], loopN = f.loops[1], loopK = f.loops[2];

  // ---- split M, N by (8, 128) ----
  auto m_axes = Rewriter::split(loopM, 3, {8, 128});
  auto n_axes = Rewriter::split(loopN, 3, {8, 128});
  CHECK(m_axes.size() == 3 && n_axes.size() == 3);
  CHECK(m_axes[0].getUpperBound() == 4096 && m_axes[0].getStep() == 128);
  CHECK(m_axes[1].getUpperBound() == 128 && m_axes[1].getStep() == 8);
  CHECK(m_axes[2].getUpperBound() == 8 && m_axes[2].getStep() == 1);
  CHECK(n_axes[0].getUpperBound() == 2048 && n_axes[0].getStep() == 128);
  CHECK(verify(module.get()).empty());
  {
    // nesting order mo, mm, mi, no, nm, ni, k
    auto loops = Analyzer::collectFuncLoops(f.func);
    CHECK(loops.size() == 7);
    CHECK(loops[0] == m_axes[0] && loops[1] == m_axes[1] && loops[2] == m_axes[2]);
    CHECK(loops[3] == n_axes[0] && loops[4] == n_axes[1] && loops[5] == n_axes[2] && loops[6] == loopK);
    // subscripts are sums of the three induction variables
    Op *ldA = loopK->body.front().get();
    CHECK(ldA->indices[0].terms.size() == 3);
    for (auto &ax : m_axes) CHECK(ldA->indices[0].coeffOf(ax.getInductionVar()) == 1);
    CHECK(contains(module.str(), "affine.for %arg3 = 0 to 4096 step 128 {"));
    CHECK(contains(module.str(), "affine.for %arg4 = 0 to 128 step 8 {"));
    CHECK(contains(module.str(), "[%arg3 + %arg4 + %arg5, %arg9]"));
  }

  // ---- reorder ----
  ForOp m_outer = m_axes[0], m_mider = m_axes[1], m_inner = m_axes[2];
  ForOp n_outer = n_axes[0], n_mider = n_axes[1], n_inner = n_axes[2];
  Rewriter::reorder({m_outer, n_outer, m_mider, n_mider, m_inner, n_inner});
  CHECK(verify(module.get()).empty());
  {
    auto loops = Analyzer::collectFuncLoops(f.func);
    CHECK(loops.size() == 7);
    CHECK(loops[0] == m_outer && loops[1] == n_outer && loops[2] == m_mider && loops[3] == n_mider &&
          loops[4] == m_inner && loops[5] == n_inner && loops[6] == loopK);
  }

  // ---- parallel ----
  auto gridLevel = Rewriter::parallel({m_outer, n_outer});
  auto blockLevel = Rewriter::parallel({m_mider, n_mider});
  CHECK(verify(module.get()).empty());
  int64_t total = 0;
  auto grid = Analyzer::getParallelNumber(gridLevel, total);
  CHECK(grid.size() == 2 && grid[0] == 32 && grid[1] == 16 && total == 512);
  auto block = Analyzer::getParallelNumber(blockLevel, total);
  CHECK(block.size() == 2 && block[0] == 16 && block[1] == 16 && total == 256);
  {
    const std::string text = module.str();
    CHECK(contains(text, "affine.parallel (%arg3, %arg4) = (0, 0) to (32, 16) {"));
    CHECK(contains(text, "affine.parallel (%arg5, %arg6) = (0, 0) to (16, 16) {"));
    CHECK(contains(text, "affine.apply affine_map<(d0) -> (d0 * 128)>(%arg3)"));
    CHECK(contains(text, "affine.apply affine_map<(d0) -> (d0 * 128)>(%arg4)"));
    CHECK(contains(text, "affine.apply affine_map<(d0) -> (d0 * 8)>(%arg5)"));
    CHECK(contains(text, "affine.apply affine_map<(d0) -> (d0 * 8)>(%arg6)"));
    // block level is nested in the grid level, applies come first in each body
    CHECK(blockLevel->parent == gridLevel.op);
    CHECK(gridLevel->body.front()->kind == OpKind::Apply);
    CHECK(Rewriter::getParallelIdx(gridLevel).size() == 2);
  }

  // ---- bufferize the k-loop accumulator ----
  std::vector<ForOp> kmn{loopK, m_inner, n_inner};
  Value tileC = Rewriter::bufferizeLoopCarryVar(kmn);
  CHECK(bool(tileC));
  CHECK(verify(module.get()).empty());
  CHECK((tileC.getMemRefType() == MemRefType{{8, 8}, DType::f32, 3}));
  CHECK(tileC.getDefiningOp()->parent == blockLevel.op);          // allocated at the block level
  CHECK(blockLevel->body.front().get() == tileC.getDefiningOp());
  CHECK(loopK.numIterArgs() == 0 && loopK->results.empty());
  {
    Op *first = loopK->body.front().get();
    CHECK(first->kind == OpKind::Load && first->memref == tileC);
    Op *last = loopK->lastOp()->prev();
    CHECK(last->kind == OpKind::Store && last->memref == tileC);
    CHECK(loopK->prev()->kind == OpKind::Store && loopK->prev()->memref == tileC);    // init store
    CHECK(loopK->next()->kind == OpKind::Load && loopK->next()->memref == tileC);     // reload for C
    CHECK(contains(module.str(), "memref<8x8xf32, 3>"));
  }

  // ---- reorder k over (mi, ni): init nest / k,m,n nest / write-back nest ----
  Rewriter::reorder({loopK, m_inner, n_inner});
  CHECK(verify(module.get()).empty());
  {
    std::vector<Op *> nests;
    for (auto &o : blockLevel->body)
      if (o->kind == OpKind::For) nests.push_back(o.get());
    CHECK(nests.size() == 3);
    CHECK(nests[1] == loopK.op);
    // init nest: 8 x 8 with constant + store
    CHECK(nests[0]->ub == 8 && nests[0]->body.front()->kind == OpKind::For);
    Op *initInner = nests[0]->body.front().get();
    CHECK(initInner->body.front()->kind == OpKind::Constant);
    // compute nest: k { mi { ni { ... } } }
    CHECK(loopK->body.front().get() == m_inner.op && m_inner->body.front().get() == n_inner.op);
    CHECK(loopK.getUpperBound() == 1024);
    // write-back nest stores to C (function argument 2)
    Op *wbInner = nests[2]->body.front().get();
    Op *st = wbInner->lastOp()->prev();
    CHECK(st->kind == OpKind::Store && st->memref == f.func.getArguments()[2]);
  }

  // ---- split k by 8 ----
  auto k_axes = Rewriter::split(loopK, 2, {8});
  CHECK(k_axes.size() == 2);
  CHECK(k_axes[0].getUpperBound() == 1024 && k_axes[0].getStep() == 8);
  CHECK(k_axes[1].getUpperBound() == 8 && k_axes[1].getStep() == 1);
  CHECK(verify(module.get()).empty());
  CHECK(contains(module.str(), "= 0 to 1024 step 8 {"));
}

// Applies the whole recipe with small tiles and checks, with the interpreter,
// that the scheduled module computes bit-identical results to the naive one.
static void test_schedule_preserves_results() {
  const int64_t M = 32, N = 16, K = 24;
  std::vector<float> a(M * K), b(K * N);
  unsigned s = 12345u;
  auto rnd = [&]() {
    s = s * 1664525u + 1013904223u;
    return static_cast<float>(static_cast<int>(s >> 8) % 2001 - 1000) / 512.0f;
  };
  for (auto &x : a) x = rnd();
  for (auto &x : b) x = rnd();
  std::vector<float> expect(M * N);
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        volatile float mul = a[i * K + k] * b[k * N + j];
        acc = mul + acc;
      }
      expect[i * N + j] = acc;
    }
  for (int scheduled = 0; scheduled < 2; ++scheduled) {
    MatmulFixture f(M, N, K);
    if (scheduled) {
      MatmulOptimizer opt;
      MatmulOptimizer::matmulConfig = {{"BLOCK_SIZE_M", 16}, {"BLOCK_SIZE_N", 8}, {"BLOCK_SIZE_K", 4},
                                       {"THREAD_SIZE_M", 4}, {"THREAD_SIZE_N", 2}};
      CHECK(opt.applicable(f.graph->module));
      opt.applyOptimzer(f.graph->module);
      CHECK(f.func.getAttr("func.state") == "gpu");
      CHECK(f.func.getAttr("kcg.schedule") == "tiled");
      CHECK(f.func.getAttr("kcg.block_threads") == "16");   // (16/4) x (8/2)
      CHECK(f.func.getAttr("kcg.grid_blocks") == "4");      // (32/16) x (16/8)
      CHECK(verify(f.graph->module.get()).empty());
    }
    std::vector<float> c(M * N, -1.0f);
    Interpreter interp(f.graph->module);
    interp.bind(f.A, a.data());
    interp.bind(f.B, b.data());
    Value cbuf = Analyzer::collectFuncCalls(f.graph->module)[0].getArgOperands()[2];
    interp.bind(cbuf, c.data());
    const std::string err = interp.run();
    CHECK(err.empty());
    CHECK(std::memcmp(c.data(), expect.data(), c.size() * sizeof(float)) == 0);
    CHECK(interp.buffer(f.C) == c.data());   // the call result aliases the C buffer
  }
}

// The staged (SCHEDULE_DETAIL 1) and pipelined (2) schedules of the reference recipe
// (src/Optimizer/Optimizer.cc:429-546), run by the interpreter with the threads of
// a block in lock step: results must equal the naive nest bit for bit, for the
// reference's 32-wide warps and for 64-wide waves.
static void run_detailed_schedule(int detail, int warp, int64_t M, int64_t N, int64_t K, int bk, std::string *text,
                                  int bm = 128, int bn = 128, int waveM = 0, int waveN = 0) {
  std::vector<float> a(M * K), b(K * N);
  unsigned s = 777u + detail + warp;
  auto rnd = [&]() {
    s = s * 1664525u + 1013904223u;
    return static_cast<float>(static_cast<int>(s >> 8) % 2001 - 1000) / 512.0f;
  };
  for (auto &x : a) x = rnd();
  for (auto &x : b) x = rnd();
  std::vector<float> expect(M * N);
  for (int64_t i = 0; i < M; ++i)
    for (int64_t j = 0; j < N; ++j) {
      float acc = 0.0f;
      for (int64_t k = 0; k < K; ++k) {
        volatile float mul = a[i * K + k] * b[k * N + j];
        acc = mul + acc;
      }
      expect[i * N + j] = acc;
    }
  MatmulFixture f(M, N, K);
  MatmulOptimizer opt;
  MatmulOptimizer::matmulConfig = {{"BLOCK_SIZE_M", bm}, {"BLOCK_SIZE_N", bn}, {"BLOCK_SIZE_K", bk},
                                   {"THREAD_SIZE_M", 8},  {"THREAD_SIZE_N", 8},   {"VECTORIZE_WIDTH", 4},
                                   {"WARP_SIZE", warp},   {"SCHEDULE_DETAIL", detail}};
  if (waveM) MatmulOptimizer::matmulConfig["WAVE_SIZE_M"] = waveM;
  if (waveN) MatmulOptimizer::matmulConfig["WAVE_SIZE_N"] = waveN;
  CHECK(opt.applicable(f.graph->module));
  opt.applyOptimzer(f.graph->module);
  const std::string problem = verify(f.graph->module.get());
  CHECK(problem.empty());
  if (!problem.empty()) std::fprintf(stderr, "    verify: %s\n", problem.c_str());
  CHECK(f.func.getAttr("kcg.schedule") == (detail == 1 ? "staged" : detail == 2 ? "pipelined" : "direct"));
  if (text) *text = f.graph->module.str();
  std::vector<float> c(M * N, -1.0f);
  Interpreter interp(f.graph->module);
  interp.bind(f.A, a.data());
  interp.bind(f.B, b.data());
  Value cbuf = Analyzer::collectFuncCalls(f.graph->module)[0].getArgOperands()[2];
  interp.bind(cbuf, c.data());
  const std::string err = interp.run();
  CHECK(err.empty());
  if (!err.empty()) std::fprintf(stderr, "    interpreter: %s\n", err.c_str());
  CHECK(std::memcmp(c.data(), expect.data(), c.size() * sizeof(float)) == 0);
}

static void test_staged_schedule() {
  std::string text;
  run_detailed_schedule(1, 32, 128, 256, 24, 8, &text);
  // README stage "read / write / barrier / cache_read / cache_write / vectorize" facts
  CHECK(contains(text, "memref<8x128xf32, 2>"));            // smA, smB: BLOCK_SIZE_K x 128
  CHECK(contains(text, "memref<4xf32, 3>"));                // tileA / tileB: 8*128/256 registers
  CHECK(contains(text, "memref<8xf32, 3>"));                // fragA / fragB
  CHECK(count(text, "gpu.barrier") == 2);
  CHECK(count(text, "affine.vector_load %arg0[") == 1);     // one global read loop per operand
  CHECK(count(text, "affine.vector_load %arg1[") == 1);
  CHECK(contains(text, "floordiv 2"));                      // thread id -> (row, 4-wide k chunk) of the A tile
  CHECK(contains(text, "floordiv 32"));                     // thread id -> (k row, 4-wide n chunk) of the B tile
  CHECK(contains(text, ", vector<1xf32>"));                 // transposing store of A, element by element
  CHECK(contains(text, "memref<128x256xf32, 1>, vector<4xf32>"));   // C written as float4
  CHECK(!contains(text, "affine.load %arg0[") && !contains(text, "affine.load %arg1["));   // operands come from fragments
  run_detailed_schedule(1, 64, 256, 128, 16, 8, nullptr);
  run_detailed_schedule(1, 64, 128, 128, 32, 16, nullptr);
}

static void test_pipelined_schedule() {
  std::string text;
  run_detailed_schedule(2, 32, 128, 256, 32, 8, &text);
  // README final-stage facts: double-buffered shared tiles and fragments, the guard of the
  // in-loop prefetch, no always-true / never-true affine.if left
  CHECK(contains(text, "memref<2x8x128xf32, 2>"));
  CHECK(contains(text, "memref<2x8xf32, 3>"));
  CHECK(!contains(text, "memref<8x128xf32, 2>"));
  CHECK(contains(text, "affine.if affine_set<(d0) : (-d0 + 16 >= 0)>"));   // k_outer + 2*8 <= 32
  // one guard around the global loads of the next slice (top of the k_outer body), one around
  // its stores to shared memory and the barrier (after the k_inner loop); the guards along
  // k_inner were decided statically and are gone
  CHECK(count(text, "affine.if") == 2);
  CHECK(!contains(text, "(0) floordiv") && !contains(text, "(7) mod"));   // constants are folded
  CHECK(contains(text, "mod 2"));
  CHECK(contains(text, "affine.loop = \"unroll\""));
  run_detailed_schedule(2, 64, 256, 128, 48, 8, nullptr);
  run_detailed_schedule(2, 64, 128, 128, 64, 16, nullptr);
}

// SCHEDULE_DETAIL 3: global -> shared with no register tile, a ring of three copies, one
// barrier per slice -- the nest of the library's direct-load kernels.
static void test_direct_schedule() {
  std::string text;
  run_detailed_schedule(3, 64, 128, 256, 40, 8, &text);            // five slices through a ring of three
  CHECK(contains(text, "memref<3x8x128xf32, 2>"));
  CHECK(!contains(text, "memref<8x128xf32, 2>") && !contains(text, "memref<2x8x128xf32, 2>"));
  CHECK(!contains(text, "memref<4xf32, 3>"));                       // no register tile between global and shared
  CHECK(contains(text, "memref<8xf32, 3>"));                        // fragments only
  CHECK(contains(text, "mod 3"));
  CHECK(contains(text, "affine.if affine_set<(d0) : (-d0 + 16 >= 0)>"));   // k_outer + 3*8 <= 40
  CHECK(count(text, "affine.if") == 2);                             // one guard per operand's fetch
  CHECK(count(text, "gpu.barrier") == 2);                           // after the prologue, at the end of a slice
  // prologue: slices 0 and 1 of A and of B; in the loop one copy loop each
  CHECK(count(text, "affine.vector_load %arg1[") == 3);
  CHECK(contains(text, "memref<128x256xf32, 1>, vector<4xf32>"));
  run_detailed_schedule(3, 64, 256, 128, 8, 8, nullptr);             // a single slice: prologue only
  run_detailed_schedule(3, 64, 128, 128, 16, 8, nullptr);            // two slices: nothing left to fetch in the loop
  run_detailed_schedule(3, 64, 128, 128, 64, 16, nullptr);
  // the library's default tile: 256 x 128 x 16, eight waves of 64 x 64 (four by two), 8 x 8 per lane
  run_detailed_schedule(3, 64, 256, 256, 64, 16, &text, 256, 128, 64, 64);
  CHECK(contains(text, "memref<3x16x256xf32, 2>") && contains(text, "memref<3x16x128xf32, 2>"));
  CHECK(contains(text, "affine.parallel (%arg3, %arg4) = (0, 0) to (32, 16)") || contains(text, "to (32, 16)"));
  run_detailed_schedule(1, 64, 256, 128, 32, 16, nullptr, 256, 128, 64, 64);   // the same organisation, staged
  run_detailed_schedule(2, 64, 256, 128, 48, 16, nullptr, 256, 128, 64, 64);   // and pipelined
}

static void test_relu_softmax_batched_matmul_semantics() {
  KernelCodeGenerator gen;
  gen.setLogMode(Log::Release);
  auto &graph = gen.createGraph("ops");
  auto X = graph.create<PlaceHolder>(std::vector<int64_t>{2, 3, 4}, std::string{"float32"});
  auto Y = graph.create<PlaceHolder>(std::vector<int64_t>{2, 5, 4}, std::string{"float32"});
  auto S = graph.create<BatchedMatmul>(X, Layout::rowMajor, Y, Layout::colMajor);   // [2,3,5]
  auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
  auto R = graph.create<Relu>(X, MemorySpace::inplace);
  CHECK(bool(S) && bool(P) && bool(R));
  CHECK((S.getMemRefType().shape == std::vector<int64_t>{2, 3, 5}));
  CHECK(verify(graph.module.get()).empty());
  auto names = Analyzer::collectFunctions(graph.module);
  bool bmm = false, sm = false, relu = false;
  for (auto f : names) {
    bmm = bmm || f.getSymName() == "BatchMatmul_2_m3_n5_k4_NT";
    sm = sm || f.getSymName() == "Softmax_2_3_5_axis2";
    relu = relu || f.getSymName() == "Relu_Elementwise_2_3_4";
  }
  CHECK(bmm && sm && relu);

  std::vector<float> x(24), y(40);
  for (int i = 0; i < 24; ++i) x[i] = 0.25f * static_cast<float>(i % 7) - 0.6f;
  for (int i = 0; i < 40; ++i) y[i] = 0.125f * static_cast<float>(i % 5) - 0.3f;
  std::vector<float> x0 = x;
  Interpreter interp(graph.module);
  interp.bind(X, x.data());
  interp.bind(Y, y.data());
  CHECK(interp.run().empty());
  float *p = interp.buffer(P);
  CHECK(p != nullptr && p == interp.buffer(S));   // softmax is in place
  for (int b = 0; b < 2; ++b)
    for (int i = 0; i < 3; ++i) {
      float logits[5], sum = 0.0f;
      for (int j = 0; j < 5; ++j) {
        float acc = 0.0f;
        for (int k = 0; k < 4; ++k) {
          volatile float mul = x0[(b * 3 + i) * 4 + k] * y[(b * 5 + j) * 4 + k];
          acc = mul + acc;
        }
        logits[j] = acc;
      }
      for (int j = 0; j < 5; ++j) sum = std::exp(logits[j]) + sum;
      float rowsum = 0.0f;
      for (int j = 0; j < 5; ++j) {
        CHECK(p[(b * 3 + i) * 5 + j] == std::exp(logits[j]) / sum);
        rowsum += p[(b * 3 + i) * 5 + j];
      }
      CHECK(std::fabs(rowsum - 1.0f) < 1e-6f);
    }
  for (int i = 0; i < 24; ++i) CHECK(x[i] == (x0[i] > 0.0f ? x0[i] : 0.0f));   // Relu ran in place after the matmul
}

static void test_batched_matmul_layouts() {
  // the same product through all four layouts must agree bit for bit
  const int Bn = 2, M = 3, N = 4, K = 5;
  std::vector<float> a(Bn * M * K), b(Bn * K * N);
  for (size_t i = 0; i < a.size(); ++i) a[i] = 0.5f * static_cast<float>((i * 7) % 11) - 2.0f;
  for (size_t i = 0; i < b.size(); ++i) b[i] = 0.25f * static_cast<float>((i * 5) % 13) - 1.0f;
  std::vector<float> at(a.size()), bt(b.size());
  for (int q = 0; q < Bn; ++q)
    for (int i = 0; i < M; ++i)
      for (int k = 0; k < K; ++k) at[(q * K + k) * M + i] = a[(q * M + i) * K + k];
  for (int q = 0; q < Bn; ++q)
    for (int k = 0; k < K; ++k)
      for (int j = 0; j < N; ++j) bt[(q * N + j) * K + k] = b[(q * K + k) * N + j];
  std::vector<float> ref;
  for (int ta = 0; ta < 2; ++ta)
    for (int tb = 0; tb < 2; ++tb) {
      KernelCodeGenerator gen;
      gen.setLogMode(Log::Release);
      auto &graph = gen.createGraph("bmm");
      auto A = graph.create<PlaceHolder>(ta ? std::vector<int64_t>{Bn, K, M} : std::vector<int64_t>{Bn, M, K}, std::string{"float32"});
      auto B = graph.create<PlaceHolder>(tb ? std::vector<int64_t>{Bn, N, K} : std::vector<int64_t>{Bn, K, N}, std::string{"float32"});
      auto C = graph.create<BatchedMatmul>(A, ta ? Layout::colMajor : Layout::rowMajor, B,
                                           tb ? Layout::colMajor : Layout::rowMajor);
      CHECK(bool(C));
      CHECK((C.getMemRefType().shape == std::vector<int64_t>{Bn, M, N}));
      Interpreter interp(graph.module);
      interp.bind(A, ta ? at.data() : a.data());
      interp.bind(B, tb ? bt.data() : b.data());
      CHECK(interp.run().empty());
      std::vector<float> got(interp.buffer(C), interp.buffer(C) + Bn * M * N);
      if (ref.empty()) {
        ref = got;
        float acc = 0.0f;   // spot value: C[1][2][3]
        for (int k = 0; k < K; ++k) {
          volatile float mul = a[(1 * M + 2) * K + k] * b[(1 * K + k) * N + 3];
          acc = mul + acc;
        }
        CHECK(got[(1 * M + 2) * N + 3] == acc);
      } else {
        CHECK(got == ref);
      }
    }
}

static ComputeDAG &attention_graph(KernelCodeGenerator &gen, int64_t b, int64_t h, int64_t s, int64_t d,
                                   const std::string &dtype = "float32") {
  auto &graph = gen.createGraph("flash_attn_demo");
  auto Q = graph.create<PlaceHolder>(std::vector<int64_t>{b, h, s, d}, dtype);
  auto K = graph.create<PlaceHolder>(std::vector<int64_t>{b, h, s, d}, dtype);
  auto V = graph.create<PlaceHolder>(std::vector<int64_t>{b, h, s, d}, dtype);
  auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
  auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
  graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
  return graph;
}

static void test_fmha_pattern_and_fusion() {
  KernelCodeGenerator gen;
  gen.setLogMode(Log::Release);
  auto &graph = attention_graph(gen, 8, 32, 2048, 64);   // the reference's demo shape
  CHECK(verify(graph.module.get()).empty());
  {
    auto names = Analyzer::collectFunctions(graph.module);
    bool nt = false, nn = false;
    for (auto f : names) {
      nt = nt || f.getSymName() == "BatchMatmul_8_32_m2048_n2048_k64_NT";
      nn = nn || f.getSymName() == "BatchMatmul_8_32_m2048_n64_k2048_NN";
    }
    CHECK(nt && nn);
    BatchMatmulDescriptor d;
    CHECK(identifyBatchMatmul("BatchMatmul_8_32_m2048_n2048_k64_NT", d));
    CHECK(d.m == 2048 && d.n == 2048 && d.k == 64 && !d.transA && d.transB);
    CHECK((d.batch == std::vector<int>{8, 32}));
    CHECK(!identifyBatchMatmul("BatchMatmul_8_m20x8_n2_k4_NN", d));
    CHECK(!identifyBatchMatmul("Softmax_8_32_2048_2048_axis3", d));
  }
  FMHAOptimizer opt;
  FMHAOptimizer::fmhaConfig = {{"BLOCK_SIZE", 256}, {"Br", 128}, {"Bc", 32}};
  FMHAOptimizer::scale = 0.125f;
  FMHAOptimizer::causal = true;
  CHECK(opt.applicable(graph.module));
  CHECK(opt.call2callsMap.size() == 1 && opt.uniqueFuncCalls.size() == 3);
  opt.applyOptimzer(graph.module);
  FMHAOptimizer::scale = 1.0f;
  FMHAOptimizer::causal = false;
  CHECK(verify(graph.module.get()).empty());
  auto calls = Analyzer::collectFuncCalls(graph.module);
  CHECK(calls.size() == 1);
  CHECK(calls[0].getCallee() == "Fused_Multi_Head_Attention_8_32_SL2048_HD64");
  CHECK(calls[0].getArgOperands().size() == 4);
  auto funcs = Analyzer::collectFunctions(graph.module);
  CHECK(funcs.size() == 1);   // the three un-fused functions are gone
  FuncOp fused = funcs[0];
  CHECK(fused.getAttr("func.state") == "gpu");
  CHECK(fused.getAttr("kcg.Br") == "128" && fused.getAttr("kcg.Bc") == "32" && fused.getAttr("kcg.Hd") == "64");
  CHECK(fused.getAttr("kcg.causal") == "1" && fused.getAttr("kcg.scale") == "0.125");
  auto levels = Analyzer::collectFuncParallels(fused);
  CHECK(levels.size() == 2);
  int64_t total = 0;
  auto grid = Analyzer::getParallelNumber(levels[0], total);
  CHECK((grid == std::vector<int64_t>{8, 32, 16}) && total == 8 * 32 * 16);
  Analyzer::getParallelNumber(levels[1], total);
  CHECK(total == 256);
  // the S buffer (8x32x2048x2048) is no longer allocated
  CHECK(!contains(graph.module.str(), "memref<8x32x2048x2048xf32, 1>"));
  // a second pass finds nothing left to fuse
  FMHAOptimizer again;
  CHECK(!again.applicable(graph.module));
}

// The fused function as an executable nest (SCHEDULE_DETAIL 1): online softmax over K/V
// tiles, one query row per thread.  Run by the interpreter it must agree with the un-fused
// three-operator graph (same inputs, literal softmax) and, with scale and the causal mask,
// with a direct fp64 evaluation; sequence lengths that are no multiple of Br or Bc included.
static void run_fused_attention_nest(int64_t b, int64_t h, int64_t s, int64_t d, int br, int bc, int threads,
                                     float scale, bool causal, std::string *text) {
  const size_t n = static_cast<size_t>(b * h * s * d);
  std::vector<float> q(n), k(n), v(n);
  unsigned seed = 4242u + static_cast<unsigned>(s) + (causal ? 7u : 0u);
  auto rnd = [&]() {
    seed = seed * 1664525u + 1013904223u;
    return static_cast<float>(static_cast<int>(seed >> 8) % 2001 - 1000) / 1000.0f;
  };
  for (auto &x : q) x = rnd();
  for (auto &x : k) x = rnd();
  for (auto &x : v) x = rnd();
  // direct evaluation in fp64
  std::vector<double> expect(n);
  for (int64_t bh = 0; bh < b * h; ++bh)
    for (int64_t i = 0; i < s; ++i) {
      std::vector<double> w(s, 0.0);
      double sum = 0.0;
      const int64_t last = causal ? i : s - 1;
      for (int64_t j = 0; j <= last; ++j) {
        double dot = 0.0;
        for (int64_t c = 0; c < d; ++c) dot += double(q[(bh * s + i) * d + c]) * double(k[(bh * s + j) * d + c]);
        w[j] = std::exp(dot * double(scale));
        sum += w[j];
      }
      for (int64_t c = 0; c < d; ++c) {
        double o = 0.0;
        for (int64_t j = 0; j <= last; ++j) o += w[j] * double(v[(bh * s + j) * d + c]);
        expect[(bh * s + i) * d + c] = o / sum;
      }
    }
  KernelCodeGenerator gen;
  gen.setLogMode(Log::Release);
  auto &graph = gen.createGraph("fused_nest");
  std::vector<int64_t> shape{b, h, s, d};
  auto Q = graph.create<PlaceHolder>(shape, std::string{"float32"});
  auto K = graph.create<PlaceHolder>(shape, std::string{"float32"});
  auto V = graph.create<PlaceHolder>(shape, std::string{"float32"});
  auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
  auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
  auto Ou = graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
  std::vector<float> unfused;
  if (!causal && scale == 1.0f) {   // the reference graph itself has neither scale nor mask
    Interpreter plain(graph.module);
    plain.bind(Q, q.data());
    plain.bind(K, k.data());
    plain.bind(V, v.data());
    CHECK(plain.run().empty());
    const float *o = plain.buffer(Ou);
    CHECK(o != nullptr);
    if (o) unfused.assign(o, o + n);
  }
  gen.fmhaConfigs = {{{"BLOCK_SIZE", threads}, {"Br", br}, {"Bc", bc}, {"SCHEDULE_DETAIL", 1}}};
  FMHAOptimizer::scale = scale;
  FMHAOptimizer::causal = causal;
  auto module = gen.optimize(graph);
  FMHAOptimizer::scale = 1.0f;
  FMHAOptimizer::causal = false;
  const std::string problem = verify(module.get());
  CHECK(problem.empty());
  if (!problem.empty()) std::fprintf(stderr, "    verify: %s\n", problem.c_str());
  auto fused = Analyzer::collectFunctions(module, "Fused_Multi_Head_Attention");
  CHECK(fused.size() == 1 && fused[0].getAttr("kcg.schedule") == "online_softmax");
  if (text) *text = module.str();
  auto calls = Analyzer::collectFuncCalls(module);
  CHECK(calls.size() == 1);
  if (calls.size() != 1) return;
  std::vector<float> o(n, -7.0f);
  Interpreter interp(module);   // optimize() works on a copy of the graph's module: bind the copy's buffers
  auto operands = calls[0].getArgOperands();
  interp.bind(operands[0], q.data());
  interp.bind(operands[1], k.data());
  interp.bind(operands[2], v.data());
  interp.bind(operands[3], o.data());
  const std::string err = interp.run();
  CHECK(err.empty());
  if (!err.empty()) std::fprintf(stderr, "    interpreter: %s\n", err.c_str());
  double worst = 0.0, worstUnfused = 0.0;
  for (size_t i = 0; i < n; ++i) {
    worst = std::max(worst, std::fabs(double(o[i]) - expect[i]));
    if (!unfused.empty()) worstUnfused = std::max(worstUnfused, std::fabs(double(o[i]) - double(unfused[i])));
  }
  if (worst >= 2e-6) std::fprintf(stderr, "    worst %g, against the un-fused graph %g\n", worst, worstUnfused);
  CHECK(worst < 2e-6);          // |O| <= max|V| = 1
  CHECK(worstUnfused < 2e-6);
  // the fused module still binds to the kernel library from its attributes
  if (d == 64 || d == 128) {
    auto bindings = gen.bind(module);
    CHECK(bindings.size() == 1 && bindings[0].kind == KernelBinding::Fmha);
  }
}

static void test_fused_attention_nest() {
  std::string text;
  run_fused_attention_nest(1, 2, 40, 32, 16, 8, 32, 1.0f, false, &text);   // 2.5 query blocks, 5 tiles
  CHECK(contains(text, "kcg.schedule = \"online_softmax\""));
  CHECK(count(text, "math.exp") == 2);                 // rescale factor and P
  CHECK(count(text, "arith.maxf") == 1 && count(text, "arith.divf") == 1);
  CHECK(contains(text, "memref<8xf32, 3>") && contains(text, "memref<32xf32, 3>"));   // S tile, O row
  CHECK(contains(text, "affine.if affine_set<(d0, d1) : (-d0 + 15 >= 0, d1 * -16 - d0 + 39 >= 0)>"));
  CHECK(!contains(text, "func.func @Softmax") && !contains(text, "func.func @BatchMatmul"));
  run_fused_attention_nest(2, 1, 33, 16, 16, 16, 16, 0.25f, true, &text);   // ragged, causal, scaled
  CHECK(count(text, "affine.if") == 4);                // row guard + three key-validity guards
  // key < S and key <= row, with key = tile * 16 + c and row = block * 16 + thread
  CHECK(count(text, "(d0 * -16 - d1 + 32 >= 0, d2 * 16 + d3 + d0 * -16 - d1 >= 0)") == 3);
  run_fused_attention_nest(1, 1, 128, 64, 128, 32, 256, 0.125f, true, nullptr);   // the kernel's own tile, bindable
  run_fused_attention_nest(1, 1, 9, 8, 4, 4, 4, 1.0f, false, nullptr);
}

static void test_fmha_pattern_rejections() {
  {  // softmax result used twice: not fusable
    KernelCodeGenerator gen;
    gen.setLogMode(Log::Release);
    auto &graph = gen.createGraph("g");
    std::vector<int64_t> shp{1, 2, 64, 64};
    auto Q = graph.create<PlaceHolder>(shp, std::string{"float32"});
    auto K = graph.create<PlaceHolder>(shp, std::string{"float32"});
    auto V = graph.create<PlaceHolder>(shp, std::string{"float32"});
    auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
    auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
    graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
    graph.create<Relu>(P, MemorySpace::inplace);
    FMHAOptimizer opt;
    CHECK(!opt.applicable(graph.module));
  }
  {  // first product not against K^T
    KernelCodeGenerator gen;
    gen.setLogMode(Log::Release);
    auto &graph = gen.createGraph("g");
    std::vector<int64_t> shp{1, 2, 64, 64};
    auto Q = graph.create<PlaceHolder>(shp, std::string{"float32"});
    auto K = graph.create<PlaceHolder>(shp, std::string{"float32"});
    auto V = graph.create<PlaceHolder>(shp, std::string{"float32"});
    auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::rowMajor);
    auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
    graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
    FMHAOptimizer opt;
    CHECK(!opt.applicable(graph.module));
    // and the matmul recipe does not mistake BatchMatmul_* for Matmul_*
    MatmulOptimizer mm;
    CHECK(!mm.applicable(graph.module));
  }
}

// test/test.cc:8-35 of the reference: Matmul + in-place Relu, optimize, codegen, save.
static void test_facade_matmul_demo() {
  KernelCodeGenerator generator("ROCm");
  generator.setLogMode(Log::Release);
  auto &graph = generator.createGraph("matmul_demo");
  int m = 4096, n = 2048, k = 1024;
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{m, k}, std::string{"float32"});
  auto B = graph.create<PlaceHolder>(std::vector<int64_t>{k, n}, std::string{"float32"});
  auto C = graph.create<Matmul>(A, B, MemorySpace::global);
  auto D = graph.create<Relu>(C, MemorySpace::inplace);
  CHECK(bool(D));
  auto module = generator.optimize(graph);
  CHECK(verify(module.get()).empty());
  generator.dump(module);
  // the original graph is untouched (optimize works on a copy)
  CHECK(Analyzer::collectFuncCalls(graph.module).size() == 2);
  CHECK(Analyzer::collectFuncCalls(module).size() == 1);   // Relu folded into the epilogue
  auto bindings = generator.bind(module);
  CHECK(bindings.size() == 1);
  if (bindings.size() == 1) {
    auto &b = bindings[0];
    CHECK(b.kind == KernelBinding::Gemm && b.entry == "kcg_gemm_f32");
    CHECK(b.M == 4096 && b.N == 2048 && b.K == 1024 && b.epilogue == KCG_EPILOGUE_RELU);
    CHECK(b.gemmSched.block_m == 256 && b.gemmSched.block_n == 128 && b.gemmSched.block_k == 16);
    CHECK(b.launch.grid[0] == (4096 / 256) * (2048 / 128) && b.launch.block[0] == 512);
    CHECK((b.argNames == std::vector<std::string>{"A", "B", "C"}));
  }
  auto source = generator.codegen(module);
  CHECK(contains(source, "namespace matmul_demo {"));
  CHECK(contains(source, "inline int kernel0(const float* arg0 /*A*/, const float* arg1 /*B*/, float* arg2 /*C*/"));
  CHECK(contains(source, "kcg_gemm_f32(arg0, arg1, arg2, 4096, 2048, 1024, KCG_EPILOGUE_RELU, &sched, stream)"));
  CHECK(contains(source, "// grid dims:(256, 1, 1), block dims:(512, 1, 1)"));
  generator.save(source, "/tmp/kcg_test_matmulKernel.hip.cc");
  FILE *fp = std::fopen("/tmp/kcg_test_matmulKernel.hip.cc", "r");
  CHECK(fp != nullptr);
  if (fp) std::fclose(fp);
  // the scheduled function has the grid / block levels of its tile table
  FuncOp f = Analyzer::collectFunctions(module, "Matmul_m")[0];
  auto levels = Analyzer::collectFuncParallels(f);
  CHECK(levels.size() == 2);
  int64_t total = 0;
  CHECK((Analyzer::getParallelNumber(levels[0], total) == std::vector<int64_t>{16, 16}));
  CHECK((Analyzer::getParallelNumber(levels[1], total) == std::vector<int64_t>{32, 16}) && total == 512);
  // a platform without a backend yields nothing rather than undefined behaviour
  KernelCodeGenerator cuda("CUDA");
  cuda.setLogMode(Log::Release);
  std::string none = "x";
  quiet([&] { none = cuda.codegen(module); });
  CHECK(none.empty());
}

// The scheduled nest drives the binding: block_k is the extent the k split left on the
// shared tiles, the LDS buffer count is the leading dimension pipeline() gave them, the
// vector width is that of the vectorised accesses -- and a nest that contradicts the
// kcg.* attributes is refused.
static void test_schedule_drives_binding() {
  auto bindWith = [](int detail, ir::ModuleOp *keep = nullptr) {
    KernelCodeGenerator generator("ROCm");
    generator.setLogMode(Log::Release);
    generator.matmulConfigs = {{{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 8}, {"GROUP_SIZE_M", 8},
                                {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8}, {"WAVE_SIZE_M", 64}, {"WAVE_SIZE_N", 64},
                                {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}, {"SCHEDULE_DETAIL", detail}}};
    auto &graph = generator.createGraph("sched_demo");
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{512, 256}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{256, 384}, std::string{"float32"});
    graph.create<Matmul>(A, B, MemorySpace::global);
    auto module = generator.optimize(graph);
    auto bindings = generator.bind(module);
    std::string source = generator.codegen(module);
    if (keep) *keep = module;
    return std::make_pair(bindings, source);
  };
  {  // tiling stage only: the attributes speak, the library picks the buffer count
    auto [b, src] = bindWith(0);
    CHECK(b.size() == 1);
    if (b.size() == 1) {
      CHECK(b[0].scheduleSource == "attributes" && b[0].gemmSched.lds_stages == 0 && b[0].gemmSched.block_k == 8);
      CHECK(std::string(b[0].launch.kernel) == "gemm_f32_128x128x8_w2x2_dl");
      CHECK(contains(src, "from the kcg.* attributes"));
    }
  }
  {  // staged: one copy of each shared tile -> the single-buffered kernel
    auto [b, src] = bindWith(1);
    CHECK(b.size() == 1);
    if (b.size() == 1) {
      CHECK(b[0].scheduleSource == "ir" && b[0].gemmSched.block_k == 8 && b[0].gemmSched.vec_width == 4);
      CHECK(b[0].gemmSched.lds_stages == 1 && b[0].scheduleNote.empty());
      CHECK(std::string(b[0].launch.kernel) == "gemm_f32_128x128x8_w2x2_single");
      CHECK(b[0].launch.lds_bytes == (128 * (8 + 4) + 8 * (128 + 8)) * 4);
      CHECK(contains(src, "lds stages 1") && contains(src, "from the scheduled loop nest") && !contains(src, "// note: "));
      CHECK(contains(src, "sched = {128, 128, 8, 8, 64, 64, 4, 64, 1};"));
    }
  }
  ir::ModuleOp pipelined;
  {  // pipelined: memref<2x8x128xf32, 2> tiles -> two LDS stages, no note
    auto [b, src] = bindWith(2, &pipelined);
    CHECK(b.size() == 1);
    if (b.size() == 1) {
      CHECK(b[0].scheduleSource == "ir" && b[0].gemmSched.lds_stages == 2 && b[0].scheduleNote.empty());
      CHECK(std::string(b[0].launch.kernel) == "gemm_f32_128x128x8_w2x2");
      CHECK(contains(pipelined.str(), "memref<2x8x128xf32, 2>"));
    }
  }
  {  // direct: memref<3x8x128xf32, 2> rings -> the three-stage direct-load kernel, read off the nest
    ir::ModuleOp direct;
    auto [b, src] = bindWith(3, &direct);
    CHECK(b.size() == 1);
    if (b.size() == 1) {
      CHECK(b[0].scheduleSource == "ir" && b[0].gemmSched.lds_stages == 3 && b[0].scheduleNote.empty());
      CHECK(b[0].gemmSched.block_k == 8 && b[0].gemmSched.vec_width == 4);
      CHECK(std::string(b[0].launch.kernel) == "gemm_f32_128x128x8_w2x2_dl");
      CHECK(contains(direct.str(), "memref<3x8x128xf32, 2>"));
      CHECK(contains(src, "lds stages 3") && contains(src, "from the scheduled loop nest"));
      CHECK(contains(src, "sched = {128, 128, 8, 8, 64, 64, 4, 64, 3};"));
    }
  }
  {  // the library's default tile staged the same way: 256 x 128 x 16, eight waves of 64 x 64
    KernelCodeGenerator generator("ROCm");
    generator.setLogMode(Log::Release);
    generator.matmulConfigs = {{{"BLOCK_SIZE_M", 256}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8},
                                {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8}, {"WAVE_SIZE_M", 64}, {"WAVE_SIZE_N", 64},
                                {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}, {"SCHEDULE_DETAIL", 3}}};
    auto &graph = generator.createGraph("sched_demo");
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{1024, 512}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{512, 768}, std::string{"float32"});
    graph.create<Matmul>(A, B, MemorySpace::global);
    auto module = generator.optimize(graph);
    auto b = generator.bind(module);
    CHECK(b.size() == 1);
    if (b.size() == 1) {
      CHECK(b[0].scheduleSource == "ir" && b[0].gemmSched.lds_stages == 3 && b[0].gemmSched.block_k == 16);
      CHECK(contains(b[0].launch.kernel, "gemm_f32_256x128x16") && contains(b[0].launch.kernel, "_dl"));
      CHECK(b[0].launch.block[0] == 512 && b[0].launch.grid[0] == 4 * 6);
      CHECK(contains(module.str(), "memref<3x16x256xf32, 2>"));
    }
  }
  {  // the attributes must not contradict the nest
    FuncOp f = Analyzer::collectFunctions(pipelined, "Matmul_m")[0];
    f.setAttr("kcg.BLOCK_SIZE_K", "16");
    std::vector<KernelBinding> b;
    quiet([&] { b = HIPBind(pipelined); });
    CHECK(b.empty());
    f.setAttr("kcg.BLOCK_SIZE_K", "8");
    f.setAttr("kcg.VECTORIZE_WIDTH", "2");
    quiet([&] { b = HIPBind(pipelined); });
    CHECK(b.empty());
    f.setAttr("kcg.VECTORIZE_WIDTH", "4");
    quiet([&] { b = HIPBind(pipelined); });
    CHECK(b.size() == 1);
  }
  {  // the library's own refusals: a buffer count it does not build, the ring on an unaligned shape
    kcg_launch_info info;
    kcg_gemm_sched s = {128, 128, 8, 8, 64, 64, 4, 64, 4};
    CHECK(kcg_gemm_f32_query(512, 384, 256, &s, &info) == KCG_ERR_BAD_SCHEDULE);
    s.lds_stages = 1;   // one copy: built for this tile, not for 128 x 128 x 32
    CHECK(kcg_gemm_f32_query(512, 384, 256, &s, &info) == KCG_OK && contains(info.kernel, "_single"));
    s.block_k = 32;
    CHECK(kcg_gemm_f32_query(512, 384, 256, &s, &info) == KCG_ERR_BAD_SCHEDULE);
    s.block_k = 8;
    s.lds_stages = 3;
    CHECK(kcg_gemm_f32_query(512, 384, 256, &s, &info) == KCG_OK && contains(info.kernel, "_dl"));
    CHECK(kcg_gemm_f32_query(512, 384, 250, &s, &info) == KCG_ERR_BAD_SCHEDULE);  // rows not 16-byte aligned
    s.lds_stages = 2;
    CHECK(kcg_gemm_f32_query(512, 384, 250, &s, &info) == KCG_OK && !contains(info.kernel, "_dl"));
  }
}

static void test_facade_config_search_and_reference_tile() {
  KernelCodeGenerator generator;
  generator.setLogMode(Log::Release);
  auto &graph = generator.createGraph("Matmul_M512_N512_K512");
  auto A = graph.create<PlaceHolder>(std::vector<int64_t>{512, 512}, std::string{"float32"});
  auto B = graph.create<PlaceHolder>(std::vector<int64_t>{512, 512}, std::string{"float32"});
  graph.create<Matmul>(A, B, MemorySpace::global);
  // with the constant evaluator the first configuration wins, as in the reference
  auto first = generator.bind(generator.optimize(graph));
  CHECK(first.size() == 1 && first[0].gemmSched.block_m == 256 && first[0].epilogue == KCG_EPILOGUE_NONE);
  // an evaluator that prefers the 128x128x8 tile (the reference's own) selects it
  generator.setEvaluator([](ModuleOp &m) {
    FuncOp f = Analyzer::collectFunctions(m, "Matmul_m")[0];
    return f.getAttr("kcg.BLOCK_SIZE_K") == "8" ? 1.0f : 2.0f;
  });
  auto second = generator.bind(generator.optimize(graph));
  CHECK(second.size() == 1 && second[0].gemmSched.block_m == 128 && second[0].gemmSched.block_k == 8);
  CHECK(second[0].launch.grid[0] == 16 && second[0].launch.block[0] == 256);
  // the gfx950 search space: every candidate is tried once, the cheapest one is kept,
  // and a candidate the evaluator refuses (FLT_MAX) can never win
  generator.useCandidateTables();
  CHECK(generator.matmulConfigs.size() == 9 && generator.fmhaConfigs.size() == 4);
  std::vector<std::string> seen;
  generator.setEvaluator([&](ModuleOp &m) {
    FuncOp f = Analyzer::collectFunctions(m, "Matmul_m")[0];
    const std::string tile = f.getAttr("kcg.BLOCK_SIZE_M") + "x" + f.getAttr("kcg.BLOCK_SIZE_N") + "x" +
                             f.getAttr("kcg.BLOCK_SIZE_K");
    seen.push_back(tile);
    if (tile == "64x64x32") return FLT_MAX;
    return tile == "128x128x32" ? 0.5f : 1.0f + static_cast<float>(seen.size());
  });
  auto third = generator.bind(generator.optimize(graph));
  CHECK(seen.size() == 9 && seen[7] == "96x96x32" && seen.back() == "96x64x32");
  CHECK(third.size() == 1 && third[0].gemmSched.block_m == 128 && third[0].gemmSched.block_k == 32);
  CHECK(generator.bestLatency() == 0.5f);
  // nothing acceptable: the module stays un-scheduled and nothing binds
  generator.setEvaluator([](ModuleOp &) { return FLT_MAX; });
  std::vector<KernelBinding> none;
  quiet([&] { none = generator.bind(generator.optimize(graph)); });
  CHECK(none.empty());
}

// test/test.cc:64-107 of the reference: the attention graph through the facade.
static void test_facade_flash_attention_demo() {
  KernelCodeGenerator generator("ROCm");
  generator.setLogMode(Log::Release);
  auto &graph = attention_graph(generator, 1, 32, 2048, 128);
  FMHAOptimizer::scale = 0.08838834764831845f;
  auto module = generator.optimize(graph);
  FMHAOptimizer::scale = 1.0f;
  CHECK(verify(module.get()).empty());
  auto bindings = generator.bind(module);
  CHECK(bindings.size() == 1);
  if (bindings.size() == 1) {
    auto &b = bindings[0];
    CHECK(b.kind == KernelBinding::Fmha && b.entry == "kcg_fmha_f32");
    CHECK(b.B == 1 && b.H == 32 && b.S == 2048 && b.D == 128 && b.causal == 0);
    CHECK(std::fabs(b.scale - 0.0883883f) < 1e-6f);
    CHECK(b.fmhaSched.br == 128 && b.fmhaSched.bc == 32);
    CHECK(b.launch.grid[0] == 32 * 16 && b.launch.block[0] == 256);
  }
  auto source = generator.codegen(module);
  CHECK(contains(source, "namespace flash_attn_demo {"));
  CHECK(contains(source, "kcg_fmha_f32(arg0, arg1, arg2, arg3, 1, 32, 2048, 128, 0.0883883461f, 0, &sched, stream)"));
  // bf16 graph binds the bf16 entry point
  KernelCodeGenerator g2;
  g2.setLogMode(Log::Release);
  auto &graph2 = attention_graph(g2, 4, 32, 4096, 128, "bfloat16");
  g2.fmhaConfigs = {{{"BLOCK_SIZE", 256}, {"Br", 128}, {"Bc", 64}}};
  FMHAOptimizer::causal = true;
  auto module2 = g2.optimize(graph2);
  FMHAOptimizer::causal = false;
  auto b2 = g2.bind(module2);
  CHECK(b2.size() == 1 && b2[0].entry == "kcg_fmha_bf16" && b2[0].dtype == KCG_BF16 && b2[0].causal == 1);
  CHECK(contains(g2.codegen(module2), "kcg_fmha_bf16(arg0, arg1, arg2, arg3, KCG_BF16, 4, 32, 4096, 128, 1.0f, 1, &sched, stream)"));
}

// Graphs no pattern matches: every call is bound to its un-fused kernel, in module order,
// and the bindings name the module-level buffers their pointers stand for.
static void test_unfused_binding() {
  KernelCodeGenerator generator("ROCm");
  generator.setLogMode(Log::Release);
  auto &graph = generator.createGraph("unfused");
  std::vector<int64_t> shp{2, 3, 96, 64};
  auto Q = graph.create<PlaceHolder>(shp, std::string{"float32"});
  auto K = graph.create<PlaceHolder>(shp, std::string{"float32"});
  auto V = graph.create<PlaceHolder>(shp, std::string{"float32"});
  auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
  graph.create<Relu>(S, MemorySpace::global);   // second reader of the scores, own result buffer
  auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
  graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
  auto module = generator.optimize(graph);
  CHECK(verify(module.get()).empty());
  auto b = generator.bind(module);
  CHECK(b.size() == 4);
  if (b.size() == 4) {
    CHECK(b[0].kind == KernelBinding::BatchedMatmul && b[0].entry == "kcg_batched_matmul_f32");
    CHECK(b[0].batch == 6 && b[0].M == 96 && b[0].N == 96 && b[0].K == 64 && b[0].transA == 0 && b[0].transB == 1);
    CHECK(b[0].argBytes == (std::vector<size_t>{6 * 96 * 64 * 4, 6 * 96 * 64 * 4, 6 * 96 * 96 * 4}));
    CHECK(b[1].kind == KernelBinding::Relu && !b[1].inPlace && b[1].count == 6 * 96 * 96 && b[1].argNames.size() == 2);
    CHECK(b[2].kind == KernelBinding::Softmax && b[2].inPlace && b[2].rowLength == 96 && b[2].count == 6 * 96 * 96);
    CHECK(b[3].kind == KernelBinding::BatchedMatmul && b[3].transA == 0 && b[3].transB == 0 && b[3].K == 96 && b[3].N == 64);
    for (int i = 0; i < 4; ++i) CHECK(b[i].index == i && b[i].buffers.size() == b[i].argNames.size());
    // the scores: written by the first product, read by Relu, rewritten in place by Softmax,
    // and -- through Softmax's result -- the left operand of the second product
    CHECK(b[0].buffers[2] == b[1].buffers[0] && b[0].buffers[2] == b[2].buffers[0] && b[0].buffers[2] == b[3].buffers[0]);
    CHECK(b[1].buffers[1] != b[1].buffers[0]);                       // Relu's own result
    CHECK(b[0].buffers[0] != b[0].buffers[1] && b[3].buffers[1] != b[0].buffers[1]);   // Q, K, V apart
    CHECK(b[0].buffers[2].getDefiningOp() && b[0].buffers[2].getDefiningOp()->kind == OpKind::Alloc);
  }
  const std::string src = generator.codegen(module);
  CHECK(contains(src, "namespace unfused {"));
  CHECK(contains(src, "return kcg_batched_matmul_f32(arg0, 0, arg1, 1, arg2, 6, 96, 96, 64, stream);"));
  CHECK(contains(src, "inline int kernel1(const float* arg0 /*x*/, float* arg1 /*y*/, void* stream = nullptr)"));
  CHECK(contains(src, "return kcg_relu_f32(arg0, arg1, 55296, stream);"));
  CHECK(contains(src, "return kcg_softmax_f32(arg0, 576, 96, stream);"));
  CHECK(contains(src, "return kcg_batched_matmul_f32(arg0, 0, arg1, 0, arg2, 6, 96, 64, 96, stream);"));
  // a Softmax on its own, an in-place Relu on its own
  KernelCodeGenerator g2;
  g2.setLogMode(Log::Release);
  auto &lone = g2.createGraph("lone");
  auto X = lone.create<PlaceHolder>(std::vector<int64_t>{40, 1000}, std::string{"float32"});
  auto Y = lone.create<Softmax>(X, -1, MemorySpace::inplace);
  lone.create<Relu>(Y, MemorySpace::inplace);
  auto m2 = g2.optimize(lone);
  auto b2 = g2.bind(m2);
  CHECK(b2.size() == 2);
  if (b2.size() == 2) {
    CHECK(b2[0].kind == KernelBinding::Softmax && b2[0].rowLength == 1000 && b2[0].count == 40000);
    CHECK(b2[1].kind == KernelBinding::Relu && b2[1].inPlace && b2[1].argNames.size() == 1);
    CHECK(b2[0].buffers[0] == b2[1].buffers[0]);
  }
  CHECK(contains(g2.codegen(m2), "return kcg_relu_f32(arg0, arg0, 40000, stream);"));
  // a trailing in-place Relu behind a Matmul still folds into the matmul's epilogue: one binding
  KernelCodeGenerator g3;
  g3.setLogMode(Log::Release);
  auto &mm = g3.createGraph("mm");
  auto A = mm.create<PlaceHolder>(std::vector<int64_t>{256, 64}, std::string{"float32"});
  auto B = mm.create<PlaceHolder>(std::vector<int64_t>{64, 128}, std::string{"float32"});
  auto C = mm.create<Matmul>(A, B, MemorySpace::global);
  mm.create<Relu>(C, MemorySpace::inplace);
  auto b3 = g3.bind(g3.optimize(mm));
  CHECK(b3.size() == 1 && b3[0].kind == KernelBinding::Gemm && b3[0].epilogue == KCG_EPILOGUE_RELU);
  // other element types have no un-fused kernel: reported and skipped
  KernelCodeGenerator g4;
  g4.setLogMode(Log::Release);
  auto &half = g4.createGraph("half");
  auto H = half.create<PlaceHolder>(std::vector<int64_t>{8, 64}, std::string{"float16"});
  half.create<Softmax>(H, -1, MemorySpace::inplace);
  std::vector<KernelBinding> b4;
  quiet([&] { b4 = g4.bind(g4.optimize(half)); });
  CHECK(b4.empty());
}

// The reference's own attention table (include/KernelCodeGen.h:38-41 there: 128 threads,
// HdxBr = BrxBc = 8192) binds: Br 64 x Bc 128 at head dim 128, Br 128 x Bc 64 at head dim 64.
static void test_reference_attention_table_binds() {
  for (int hd : {128, 64}) {
    KernelCodeGenerator generator("ROCm");
    generator.setLogMode(Log::Release);
    generator.fmhaConfigs = {{{"BLOCK_SIZE", 128}, {"HdxBr", 8192}, {"BrxBc", 8192}, {"WARP_SIZE", 32}}};
    auto &graph = attention_graph(generator, 8, 32, 2048, hd);
    auto module = generator.optimize(graph);
    auto b = generator.bind(module);
    CHECK(b.size() == 1);
    if (b.size() != 1) continue;
    CHECK(b[0].kind == KernelBinding::Fmha && b[0].fmhaSched.br == 8192 / hd && b[0].fmhaSched.bc == hd);
    CHECK(b[0].launch.block[0] == (hd == 128 ? 128 : 256));       // two waves / four waves of 32 rows
    CHECK(b[0].launch.grid[0] == 8 * 32 * (2048 / (8192 / hd)));
    // and for bf16 operands
    KernelCodeGenerator g2;
    g2.setLogMode(Log::Release);
    g2.fmhaConfigs = generator.fmhaConfigs;
    auto &graph2 = attention_graph(g2, 2, 4, 512, hd, "bfloat16");
    auto b2 = g2.bind(g2.optimize(graph2));
    CHECK(b2.size() == 1 && b2[0].entry == "kcg_fmha_bf16" && b2[0].fmhaSched.br == 8192 / hd);
  }
}

static void test_error_paths() {
  quiet([] {
    KernelCodeGenerator gen;
    gen.setLogMode(Log::Release);
    auto &graph = gen.createGraph("errors");
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{8, 4}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{5, 8}, std::string{"float32"});
    CHECK(!graph.create<Matmul>(A, B, MemorySpace::global));                 // K mismatch
    CHECK(!graph.create<PlaceHolder>(std::vector<int64_t>{4}, std::string{"int8"}));
    CHECK(!graph.create<PlaceHolder>(std::vector<int64_t>{4, 0}, std::string{"float32"}));
    CHECK(!graph.create<Matmul>(Value(), B, MemorySpace::global));
    CHECK(!graph.create<BatchedMatmul>(A, Layout::rowMajor, B, Layout::rowMajor));
    CHECK(!graph.create<Softmax>(A, 0));                                     // only the last axis
    CHECK(!graph.create<Softmax>(A, 7));
    CHECK(!graph.create<Transpose>(A));
    CHECK(getDType("float16") == DType::f16 && getDType("nope") == DType::none);
    CHECK(verify(graph.module.get()).empty());                              // failed builds left no debris

    // split preconditions
    auto C = graph.create<PlaceHolder>(std::vector<int64_t>{4, 6}, std::string{"float32"});
    auto D = graph.create<Matmul>(A, C, MemorySpace::global);
    CHECK(bool(D));
    FuncOp f = Analyzer::collectFunctions(graph.module, "Matmul_m8")[0];
    auto loops = Analyzer::collectFuncLoops(f);
    const std::string before = graph.module.str();
    CHECK(Rewriter::split(loops[0], 3, {3, 8}).empty());    // 8 % 3
    CHECK(Rewriter::split(loops[0], 3, {2}).empty());       // wrong factor count
    CHECK(Rewriter::split(loops[2], 2, {2}).empty());       // carries a value
    CHECK(!Rewriter::parallel({loops[0], loops[2]}));       // not perfectly nested
    CHECK(graph.module.str() == before);                    // nothing was changed
    // reorder across the un-bufferized accumulator is refused and changes nothing
    Rewriter::reorder({loops[2], loops[0], loops[1]});
    CHECK(graph.module.str() == before);
    // ragged shape through the recipe: kept naive, flagged for the bounds-checked kernel
    MatmulOptimizer opt;
    MatmulOptimizer::matmulConfig = {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 8}};
    CHECK(opt.applicable(graph.module));
    opt.applyOptimzer(graph.module);
    CHECK(f.getAttr("kcg.schedule") == "edge" && f.getAttr("func.state") == "gpu");
  });
}

static void test_verify_and_clone() {
  MatmulFixture f(16, 16, 16);
  ModuleOp copy = f.graph->module.clone();
  CHECK(copy.str() == f.graph->module.str());
  // mutate the copy: the original is unaffected
  FuncOp cf = Analyzer::collectFunctions(copy, "Matmul")[0];
  auto loops = Analyzer::collectFuncLoops(cf);
  Rewriter::split(loops[0], 2, {4});
  CHECK(copy.str() != f.graph->module.str());
  CHECK(verify(copy.get()).empty() && verify(f.graph->module.get()).empty());
  // break it: a store that uses a loop's induction variable outside the loop
  Op *k = Analyzer::collectFuncLoops(cf).back().op;
  Value kiv = k->arg(0);
  Op *stray = cf->lastOp()->insertBefore(makeLoad(cf.getArguments()[0], {LinExpr(kiv), LinExpr(int64_t(0))}));
  CHECK(!verify(copy.get()).empty());
  stray->erase();
  CHECK(verify(copy.get()).empty());
  // rank mismatch
  Op *bad = cf->lastOp()->insertBefore(makeLoad(cf.getArguments()[0], {LinExpr(int64_t(0))}));
  CHECK(contains(verify(copy.get()), "rank"));
  bad->erase();
}

static void test_builders_outer_product_set_buffer() {
  KernelCodeGenerator gen;
  gen.setLogMode(Log::Release);
  auto &graph = gen.createGraph("builders");
  MemRefType t{{4}, DType::f32, 1};
  FuncOp func = buildFuction(graph.module, "Demo", {t, t}, {});
  CHECK(buildFuction(graph.module, "Demo", {t, t}, {}) == func);   // found, not duplicated
  func->pushBack(makeReturn({}));
  Value tile = Rewriter::alloc_buffer(OpHandle(func.op), MemorySpace::local, {4, 4}, DType::f32);
  Value zero = func->lastOp()->insertBefore(makeConstant(0.0, DType::f32))->result();
  Rewriter::set_buffer(OpHandle(func.op), tile, zero);
  ForOp outer = Rewriter::outer_product(OpHandle(func.op), tile, func.getArguments()[0], func.getArguments()[1], 4, 4);
  Rewriter::barrier(outer, Position::before);
  CHECK(outer->prev()->kind == OpKind::Barrier);
  CHECK(verify(graph.module.get()).empty());
  Rewriter::unrollAttribute(graph.module, 8);
  CHECK(contains(graph.module.str(), "affine.loop = \"unroll\""));
  auto a = graph.create<PlaceHolder>(std::vector<int64_t>{4}, std::string{"float32"});
  auto b = graph.create<PlaceHolder>(std::vector<int64_t>{4}, std::string{"float32"});
  graph.module->pushBack(makeCall(func.op, {a, b}));
  // a barrier outside any parallel level is harmless for the interpreter
  std::vector<float> av{1, 2, 3, 4}, bv{10, 20, 30, 40};
  Interpreter interp(graph.module);
  interp.bind(a, av.data());
  interp.bind(b, bv.data());
  CHECK(interp.run().empty());
}

int main() {
  struct Case {
    const char *name;
    void (*fn)();
  } cases[] = {
      {"frontend_matmul_nest", test_frontend_matmul_nest},
      {"schedule_stages_match_readme", test_schedule_stages_match_readme},
      {"schedule_preserves_results", test_schedule_preserves_results},
      {"staged_schedule", test_staged_schedule},
      {"pipelined_schedule", test_pipelined_schedule},
      {"direct_schedule", test_direct_schedule},
      {"relu_softmax_batched_matmul_semantics", test_relu_softmax_batched_matmul_semantics},
      {"batched_matmul_layouts", test_batched_matmul_layouts},
      {"fmha_pattern_and_fusion", test_fmha_pattern_and_fusion},
      {"fused_attention_nest", test_fused_attention_nest},
      {"fmha_pattern_rejections", test_fmha_pattern_rejections},
      {"facade_matmul_demo", test_facade_matmul_demo},
      {"schedule_drives_binding", test_schedule_drives_binding},
      {"facade_config_search_and_reference_tile", test_facade_config_search_and_reference_tile},
      {"facade_flash_attention_demo", test_facade_flash_attention_demo},
      {"unfused_binding", test_unfused_binding},
      {"reference_attention_table_binds", test_reference_attention_table_binds},
      {"error_paths", test_error_paths},
      {"verify_and_clone", test_verify_and_clone},
      {"builders_outer_product_set_buffer", test_builders_outer_product_set_buffer},
  };
  int failedCases = 0;
  for (auto &c : cases) {
    const int before = g_failed;
    c.fn();
    const bool ok = g_failed == before;
    std::printf("[%s] %s\n", ok ? "PASS" : "FAIL", c.name);
    failedCases += ok ? 0 : 1;
  }
  std::printf("%d checks, %d failed, %d/%zu cases passed\n", g_checks, g_failed,
              static_cast<int>(sizeof(cases) / sizeof(cases[0])) - failedCases, sizeof(cases) / sizeof(cases[0]));
  return g_failed == 0 ? 0 : 1;
}
