#include "Optimizer/Optimizer.h"

#include <limits>

#include <algorithm>

#include <cstdio>
#include <iostream>

void BatchMatmulDescriptor::log() const {
  std::cerr << "m = " << m << " n = " << n << " k = " << k << "\nbatch = ";
  for (auto b : batch) std::cerr << b << ",";
  std::cerr << "\ntrans A = " << transA << " transB = " << transB << "\n";
}

namespace KernelCodeGen {

using namespace ir;

std::map<std::string, int> MatmulOptimizer::matmulConfig;
std::map<std::string, int> FMHAOptimizer::fmhaConfig;
float FMHAOptimizer::scale = 1.0f;
bool FMHAOptimizer::causal = false;

#define DUMP(module)                                 \
  do {                                               \
    if (KCGLog::level == Log::Debug) (module).dump(); \
  } while (0)

bool identifyBatchMatmul(const std::string &name, BatchMatmulDescriptor &matmul) {
  std::vector<std::string> frags;
  std::string cur;
  for (char c : name) {
    if (c == '_') {
      frags.push_back(cur);
      cur.clear();
    } else {
      cur += c;
    }
  }
  frags.push_back(cur);
  // BatchMatmul, batch..., m<M>, n<N>, k<K>, <N|T><N|T>
  if (frags.size() < 5 || frags[0] != "BatchMatmul") return false;
  const std::string &lay = frags.back();
  if (lay.size() != 2 || (lay[0] != 'N' && lay[0] != 'T') || (lay[1] != 'N' && lay[1] != 'T')) return false;
  auto number = [](const std::string &s, size_t from, int &out) {
    if (s.size() <= from) return false;
    for (size_t i = from; i < s.size(); ++i)
      if (s[i] < '0' || s[i] > '9') return false;
    out = std::stoi(s.substr(from));
    return true;
  };
  const size_t n = frags.size();
  if (frags[n - 4][0] != 'm' || frags[n - 3][0] != 'n' || frags[n - 2][0] != 'k') return false;
  if (!number(frags[n - 4], 1, matmul.m) || !number(frags[n - 3], 1, matmul.n) || !number(frags[n - 2], 1, matmul.k))
    return false;
  matmul.batch.clear();
  for (size_t i = 1; i + 4 < n; ++i) {
    int b = 0;
    if (!number(frags[i], 0, b)) return false;
    matmul.batch.push_back(b);
  }
  matmul.transA = lay[0] == 'T';
  matmul.transB = lay[1] == 'T';
  return true;
}

// ----------------------------------------------------------------- Matmul
bool MatmulOptimizer::applicable(ModuleOp &module) {
  clear();
  for (auto &func : Analyzer::collectFunctions(module, "Matmul")) {
    // "BatchMatmul_..." also contains "Matmul": only the plain operator is handled here
    if (func.getSymName().rfind("Matmul_m", 0) != 0) continue;
    if (func.getAttr("func.state") != "cpu") continue;
    auto loops = Analyzer::collectFuncLoops(func);
    auto args = func.getArguments();
    if (loops.size() != 3 || args.size() != 3) continue;
    if (matmuls.count(func)) std::cerr << "Duplicated Matmul in module\n";
    matmuls.insert(func);
    matmulLoops[func] = loops;
    matmulBuffers[func] = MemoryBuffer{args[0], args[1], args[2]};
  }
  return !matmuls.empty();
}

namespace {

// thread organisation of the staged schedule: warps as 2 x (warps / 2), the lanes
// of a warp as 8 x (warp / 8), as in the reference for 8 warps of 32 lanes
struct ThreadOrg {
  int64_t bm, bn, bk, width, warp, blockDimY, blockDimX, warps, warpOrg[2], threadOrg[2];
  int64_t fragA, fragB, ldgA, ldgB;
  bool consistent;
};

ThreadOrg threadOrg(const std::map<std::string, int> &config) {
  auto cfg = [&](const char *key, int fallback) {
    auto it = config.find(key);
    return static_cast<int64_t>(it == config.end() ? fallback : it->second);
  };
  ThreadOrg o{};
  o.bm = cfg("BLOCK_SIZE_M", 128);
  o.bn = cfg("BLOCK_SIZE_N", 128);
  o.bk = cfg("BLOCK_SIZE_K", 8);
  o.width = cfg("VECTORIZE_WIDTH", 4);
  o.warp = cfg("WARP_SIZE", 64);
  const int64_t tm = cfg("THREAD_SIZE_M", 8), tn = cfg("THREAD_SIZE_N", 8);
  o.blockDimY = o.bm / tm;
  o.blockDimX = o.bn / tn;
  const int64_t threads = o.blockDimY * o.blockDimX;
  o.warps = o.warp > 0 ? threads / o.warp : 0;
  // waves as WAVE rows x columns of the block tile when WAVE_SIZE_M / WAVE_SIZE_N say so and
  // account for every wave (256 x 128 in 64 x 64 wave tiles: 4 x 2), else 2 x (warps / 2)
  o.warpOrg[0] = 2;
  o.warpOrg[1] = o.warps / 2;
  const int64_t wm = cfg("WAVE_SIZE_M", 0), wn = cfg("WAVE_SIZE_N", 0);
  if (wm > 0 && wn > 0 && o.bm % wm == 0 && o.bn % wn == 0 && (o.bm / wm) * (o.bn / wn) == o.warps) {
    o.warpOrg[0] = o.bm / wm;
    o.warpOrg[1] = o.bn / wn;
  }
  o.threadOrg[0] = 8;
  o.threadOrg[1] = o.warp / 8;
  const int64_t strideA = o.warpOrg[1] > 0 ? (o.warps / o.warpOrg[1]) * o.threadOrg[0] : 0;
  const int64_t strideB = (o.warps / o.warpOrg[0]) * o.threadOrg[1];
  o.fragA = strideA > 0 ? o.bm / strideA : 0;
  o.fragB = strideB > 0 ? o.bn / strideB : 0;
  o.ldgA = threads > 0 ? o.bk * o.bm / threads : 0;
  o.ldgB = threads > 0 ? o.bk * o.bn / threads : 0;
  o.consistent = o.warps >= 2 && o.warps % 2 == 0 && o.warp % 8 == 0 && threads % o.warp == 0 &&
                 o.warpOrg[0] > 0 && o.warpOrg[1] > 0 && o.warpOrg[0] * o.warpOrg[1] == o.warps &&
                 o.fragA == tm && o.fragB == tn && o.width > 0 && o.fragA % o.width == 0 &&
                 o.fragB % o.width == 0 && o.ldgA >= o.width && o.ldgA % o.width == 0 && o.ldgB >= o.width &&
                 o.ldgB % o.width == 0 && o.bk % o.width == 0 && o.bn % o.width == 0 &&
                 (o.bk * o.bm) % threads == 0 && (o.bk * o.bn) % threads == 0;
  return o;
}

}  // namespace

AffineMap MatmulOptimizer::getAffineMap(const std::string &id) {
  const ThreadOrg o = threadOrg(matmulConfig);
  auto d = [](int i) { return AffineExpr::dim(i); };
  const int64_t w = o.width;
  const AffineExpr tid = d(0) * o.blockDimX + d(1);
  const AffineExpr warpId = tid.floorDiv(o.warp), laneId = tid % o.warp;
  const int64_t threads = o.blockDimY * o.blockDimX;
  if (id == "loadTileA") {
    // operands: threadIdx.y, threadIdx.x, blockIdx.y, k_outer, copy step
    const AffineExpr vt = tid + d(4) * threads;
    return {5, {vt.floorDiv(o.bk / w) + d(2) * o.bm, (vt % (o.bk / w)) * w + d(3)}};
  }
  if (id == "loadTileB") {
    // operands: threadIdx.y, threadIdx.x, k_outer, blockIdx.x, copy step
    const AffineExpr vt = tid + d(4) * threads;
    return {5, {vt.floorDiv(o.bn / w) + d(2), (vt % (o.bn / w)) * w + d(3) * o.bn}};
  }
  if (id == "storeTileA") {
    // operands: threadIdx.y, threadIdx.x, copy step, element of the vector (transposing store)
    const AffineExpr vt = tid + d(2) * threads;
    return {4, {(vt % (o.bk / w)) * w + d(3), vt.floorDiv(o.bk / w)}};
  }
  if (id == "storeTileB") {
    // operands: threadIdx.y, threadIdx.x, copy step
    const AffineExpr vt = tid + d(2) * threads;
    return {3, {vt.floorDiv(o.bn / w), (vt % (o.bn / w)) * w}};
  }
  if (id == "loadFragA") {
    // operands: threadIdx.y, threadIdx.x, k_inner, copy step
    const AffineExpr m = laneId.floorDiv(o.threadOrg[1]) +
                         (warpId.floorDiv(o.warpOrg[1]) + d(3) * o.warpOrg[0]) * o.threadOrg[0];
    return {4, {d(2), m * w}};
  }
  if (id == "loadFragB") {
    const AffineExpr n = laneId % o.threadOrg[1] + (warpId % o.warpOrg[1] + d(3) * o.warpOrg[1]) * o.threadOrg[1];
    return {4, {d(2), n * w}};
  }
  if (id == "cacheReadA" || id == "cacheReadB") return {1, {d(0)}};
  if (id == "cacheWriteC") {
    // operands: threadIdx.y, threadIdx.x, blockIdx.y, blockIdx.x, mi outer, ni outer, mi inner, ni inner
    const AffineExpr m = laneId.floorDiv(o.threadOrg[1]) +
                         (warpId.floorDiv(o.warpOrg[1]) + d(4).floorDiv(w) * o.warpOrg[0]) * o.threadOrg[0];
    const AffineExpr n = laneId % o.threadOrg[1] +
                         (warpId % o.warpOrg[1] + d(5).floorDiv(w) * o.warpOrg[1]) * o.threadOrg[1];
    return {8, {d(2) * o.bm + m * w + d(6), d(3) * o.bn + n * w + d(7)}};
  }
  std::cerr << "getAffineMap: unknown map \"" << id << "\"\n";
  return {};
}

void MatmulOptimizer::applyOptimzer(ModuleOp &module) {
  auto cfg = [&](const char *key, int fallback) {
    auto it = matmulConfig.find(key);
    return it == matmulConfig.end() ? fallback : it->second;
  };
  for (auto matmul : matmuls) {
    auto loops = matmulLoops[matmul];
    ForOp loopM = loops[0], loopN = loops[1], loopK = loops[2];
    const int bm = cfg("BLOCK_SIZE_M", 128), bn = cfg("BLOCK_SIZE_N", 128), bk = cfg("BLOCK_SIZE_K", 8);
    const int tm = cfg("THREAD_SIZE_M", 8), tn = cfg("THREAD_SIZE_N", 8);
    if (loopM.getUpperBound() % bm || loopN.getUpperBound() % bn || loopK.getUpperBound() % bk || bm % tm ||
        bn % tn) {
      // ragged shapes keep the naive nest; the backend binds the bounds-checked kernel
      matmul.setAttr("func.state", "gpu");
      matmul.setAttr("kcg.schedule", "edge");
      continue;
    }
    matmul.setAttr("func.state", "gpu");

    auto m_axes = Rewriter::split(loopM, 3, {tm, bm});
    auto n_axes = Rewriter::split(loopN, 3, {tn, bn});
    DUMP(module);
    ForOp m_outer = m_axes[0], m_mider = m_axes[1], m_inner = m_axes[2];
    ForOp n_outer = n_axes[0], n_mider = n_axes[1], n_inner = n_axes[2];

    Rewriter::reorder({m_outer, n_outer, m_mider, n_mider, m_inner, n_inner});
    DUMP(module);

    auto gridLevel = Rewriter::parallel({m_outer, n_outer});
    auto blockLevel = Rewriter::parallel({m_mider, n_mider});
    DUMP(module);

    std::vector<ForOp> kmn_axes{loopK, m_inner, n_inner};
    Value tileC = Rewriter::bufferizeLoopCarryVar(kmn_axes);  // THREAD_SIZE_M x THREAD_SIZE_N registers
    DUMP(module);

    Rewriter::reorder({loopK, m_inner, n_inner});
    DUMP(module);

    auto k_axes = Rewriter::split(loopK, 2, {bk});
    DUMP(module);

    const int detail = cfg("SCHEDULE_DETAIL", 0);
    const ThreadOrg org = threadOrg(matmulConfig);
    if (detail >= 1 && !org.consistent)
      std::cerr << "MatmulOptimizer: the staged schedule needs BLOCK_SIZE = 16 x THREAD_SIZE and whole warps; "
                   "keeping the tiled nest\n";
    if (detail == 3 && org.consistent && k_axes.size() == 2) {
      // The direct-load form: global -> shared with no register tile in between, the shared
      // tiles a ring of three copies along k_outer (two slices in flight while one is
      // consumed), one barrier per slice.  This is the nest of the library's default matmul
      // kernel; the reference's recipe (staged through registers, two copies) is detail 1 / 2.
      ForOp k_outer = k_axes[0], k_inner = k_axes[1];
      const int width = static_cast<int>(org.width);
      const MemoryBuffer &buf = matmulBuffers[matmul];
      const DType elemA = buf.A.getMemRefType().elem, elemB = buf.B.getMemRefType().elem;
      Value fragB = Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {org.fragB}, elemB);
      Value fragA = Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {org.fragA}, elemA);
      Value smB = Rewriter::alloc_buffer(OpHandle(gridLevel.op), MemorySpace::shared, {org.bk, org.bn}, elemB);
      Value smA = Rewriter::alloc_buffer(OpHandle(gridLevel.op), MemorySpace::shared, {org.bk, org.bm}, elemA);
      auto blockIdx = Rewriter::getParallelIdx(gridLevel);
      auto threadIdx = Rewriter::getParallelIdx(blockLevel);
      ForOp copyA = Rewriter::copy(buf.A, getAffineMap("loadTileA"),
                                   {threadIdx[0], threadIdx[1], blockIdx[0], k_outer.getInductionVar()}, smA,
                                   getAffineMap("storeTileA"), {threadIdx[0], threadIdx[1]}, org.ldgA, width, k_outer,
                                   Position::begin);
      ForOp copyB = Rewriter::copy(buf.B, getAffineMap("loadTileB"),
                                   {threadIdx[0], threadIdx[1], k_outer.getInductionVar(), blockIdx[1]}, smB,
                                   getAffineMap("storeTileB"), {threadIdx[0], threadIdx[1]}, org.ldgB, width, copyA,
                                   Position::after);
      DUMP(module);
      ForOp loadFragA = Rewriter::read(smA, fragA, getAffineMap("loadFragA"),
                                       {threadIdx[0], threadIdx[1], k_inner.getInductionVar()}, width, k_inner,
                                       Position::begin);
      Rewriter::read(smB, fragB, getAffineMap("loadFragB"), {threadIdx[0], threadIdx[1], k_inner.getInductionVar()},
                     width, loadFragA, Position::after);
      Rewriter::cache_read(k_inner, buf.A, fragA, getAffineMap("cacheReadA"), {m_inner.getInductionVar()});
      Rewriter::cache_read(k_inner, buf.B, fragB, getAffineMap("cacheReadB"), {n_inner.getInductionVar()});
      DUMP(module);
      auto writeC = Rewriter::get_write(blockLevel, buf.C);
      if (writeC.size() == 1 && writeC[0].size() == 2) {
        auto m_inner_axes = Rewriter::split(writeC[0][0], 2, {width});
        auto n_inner_axes = Rewriter::split(writeC[0][1], 2, {width});
        ForOp m_inner_0 = m_inner_axes[0], m_inner_1 = m_inner_axes[1];
        ForOp n_inner_0 = n_inner_axes[0], n_inner_1 = n_inner_axes[1];
        Rewriter::reorder({m_inner_0, n_inner_0, m_inner_1, n_inner_1});
        Rewriter::cache_write(m_inner_0, buf.C, tileC, getAffineMap("cacheWriteC"),
                              {threadIdx[0], threadIdx[1], blockIdx[0], blockIdx[1], m_inner_0.getInductionVar(),
                               n_inner_0.getInductionVar(), m_inner_1.getInductionVar(),
                               n_inner_1.getInductionVar()});
        Rewriter::vectorize(n_inner_1, width);
        DUMP(module);
      }
      constexpr int kStages = 3;
      Rewriter::pipeline({copyB}, smB, k_outer, kStages);
      Rewriter::pipeline({copyA}, smA, k_outer, kStages);
      // the slices of the prologue are published before the first one is read, and every
      // iteration ends with the barrier that lets the next one overwrite the copy just read
      Rewriter::barrier(k_outer, Position::before);
      Rewriter::barrier(k_outer, Position::end);
      DUMP(module);
      Rewriter::take_off_true_if(module);
      Rewriter::delete_false_if(module);
      matmul.setAttr("kcg.schedule", "direct");
    } else if (detail >= 1 && org.consistent && k_axes.size() == 2) {
      ForOp k_outer = k_axes[0], k_inner = k_axes[1];
      const int width = static_cast<int>(org.width);
      const MemoryBuffer &buf = matmulBuffers[matmul];
      const DType elemA = buf.A.getMemRefType().elem, elemB = buf.B.getMemRefType().elem;

      Value fragB = Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {org.fragB}, elemB);
      Value fragA = Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {org.fragA}, elemA);
      Value tileB = Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {org.ldgB}, elemB);
      Value tileA = Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {org.ldgA}, elemA);
      Value smB = Rewriter::alloc_buffer(OpHandle(gridLevel.op), MemorySpace::shared, {org.bk, org.bn}, elemB);
      Value smA = Rewriter::alloc_buffer(OpHandle(gridLevel.op), MemorySpace::shared, {org.bk, org.bm}, elemA);
      DUMP(module);

      auto blockIdx = Rewriter::getParallelIdx(gridLevel);
      auto threadIdx = Rewriter::getParallelIdx(blockLevel);

      // global -> registers -> shared, once per k_outer step, fenced by two barriers
      ForOp loadTileA = Rewriter::read(buf.A, tileA, getAffineMap("loadTileA"),
                                       {threadIdx[0], threadIdx[1], blockIdx[0], k_outer.getInductionVar()}, width,
                                       k_outer, Position::begin);
      ForOp loadTileB = Rewriter::read(buf.B, tileB, getAffineMap("loadTileB"),
                                       {threadIdx[0], threadIdx[1], k_outer.getInductionVar(), blockIdx[1]}, width,
                                       loadTileA, Position::after);
      DUMP(module);
      ForOp storeTileA = Rewriter::write(tileA, smA, getAffineMap("storeTileA"), {threadIdx[0], threadIdx[1]}, width,
                                         loadTileB, Position::after);
      ForOp storeTileB = Rewriter::write(tileB, smB, getAffineMap("storeTileB"), {threadIdx[0], threadIdx[1]}, width,
                                         storeTileA, Position::after);
      Op *barrierPrefix = Rewriter::barrier(loadTileA, Position::before);
      Op *barrierSuffix = Rewriter::barrier(storeTileB, Position::after);
      DUMP(module);

      // shared -> register fragments, once per k_inner step
      ForOp loadFragA = Rewriter::read(smA, fragA, getAffineMap("loadFragA"),
                                       {threadIdx[0], threadIdx[1], k_inner.getInductionVar()}, width, k_inner,
                                       Position::begin);
      ForOp loadFragB = Rewriter::read(smB, fragB, getAffineMap("loadFragB"),
                                       {threadIdx[0], threadIdx[1], k_inner.getInductionVar()}, width, loadFragA,
                                       Position::after);
      DUMP(module);

      Rewriter::cache_read(k_inner, buf.A, fragA, getAffineMap("cacheReadA"), {m_inner.getInductionVar()});
      Rewriter::cache_read(k_inner, buf.B, fragB, getAffineMap("cacheReadB"), {n_inner.getInductionVar()});
      DUMP(module);

      // write-back of the register tile: width-wide vectors along n
      auto writeC = Rewriter::get_write(blockLevel, buf.C);
      if (writeC.size() == 1 && writeC[0].size() == 2) {
        auto m_inner_axes = Rewriter::split(writeC[0][0], 2, {width});
        auto n_inner_axes = Rewriter::split(writeC[0][1], 2, {width});
        ForOp m_inner_0 = m_inner_axes[0], m_inner_1 = m_inner_axes[1];
        ForOp n_inner_0 = n_inner_axes[0], n_inner_1 = n_inner_axes[1];
        Rewriter::reorder({m_inner_0, n_inner_0, m_inner_1, n_inner_1});
        DUMP(module);
        Rewriter::cache_write(m_inner_0, buf.C, tileC, getAffineMap("cacheWriteC"),
                              {threadIdx[0], threadIdx[1], blockIdx[0], blockIdx[1], m_inner_0.getInductionVar(),
                               n_inner_0.getInductionVar(), m_inner_1.getInductionVar(),
                               n_inner_1.getInductionVar()});
        DUMP(module);
        Rewriter::vectorize(n_inner_1, width);
        DUMP(module);
      } else {
        std::cerr << "MatmulOptimizer: unexpected write-back nest, leaving it scalar\n";
      }
      matmul.setAttr("kcg.schedule", "staged");

      if (detail >= 2) {
        auto doubleLoadTileB = Rewriter::pipeline({loadTileB, storeTileB}, smB, k_outer);
        auto doubleLoadTileA = Rewriter::pipeline({loadTileA, storeTileA}, smA, k_outer);
        auto doubleLoadFragB = Rewriter::pipeline({loadFragB}, fragB, k_inner);
        auto doubleLoadFragA = Rewriter::pipeline({loadFragA}, fragA, k_inner);
        DUMP(module);

        Rewriter::detach_last_loop(k_inner);
        DUMP(module);

        // prologue: A then B loads, A then B stores, one barrier
        Rewriter::schedule(doubleLoadTileA[0][0].op, doubleLoadTileB[0][0].op, Position::before);
        Rewriter::schedule(doubleLoadTileA[0][1].op, doubleLoadTileB[0][1].op, Position::before);
        Rewriter::schedule(barrierPrefix, doubleLoadTileB[0][1].op, Position::after);
        // main loop: global loads of the next slice first, its stores and the barrier after the k_inner loop
        Rewriter::schedule(doubleLoadTileB[1][0].op, doubleLoadTileA[1][0].op, Position::after);
        Rewriter::schedule(doubleLoadTileA[1][1].op, doubleLoadTileB[1][1].op, Position::before);
        Rewriter::schedule(barrierSuffix, doubleLoadTileB[1][1].op, Position::after);
        Op *ifOp = doubleLoadTileA[1][1]->parent;
        Rewriter::schedule(ifOp, k_inner.op, Position::after);
        // the first fragments of a slice are fetched before the slice's loop: once ahead of
        // k_outer, and at the end of every k_outer step for the next one
        Rewriter::extract_loop(doubleLoadFragA[0][0].op, k_outer, /*iteration*/ 0);
        Rewriter::extract_loop(doubleLoadFragB[0][0].op, k_outer, /*iteration*/ 0);
        Rewriter::schedule(doubleLoadFragB[0][0].op, k_outer.op, Position::end);
        Rewriter::schedule(doubleLoadFragA[0][0].op, k_outer.op, Position::end);
        DUMP(module);

        Rewriter::change_double_buffer(doubleLoadFragA[0][0], smA);
        Rewriter::change_double_buffer(doubleLoadFragB[0][0], smB);
        DUMP(module);

        Rewriter::take_off_true_if(module);
        Rewriter::delete_false_if(module);
        DUMP(module);

        const int64_t threshold = std::max<int64_t>(bk, std::max(tm, tn));
        Rewriter::unroll(module, [&](ForOp f) {
          return f.tripCount() < std::min<int64_t>(threshold, width);
        });
        DUMP(module);
        Rewriter::unrollAttribute(module, [&](ForOp f) { return f.tripCount() <= threshold; });
        DUMP(module);
        matmul.setAttr("kcg.schedule", "pipelined");
      }
    }

    Rewriter::unrollAttribute(module, 8);

    int64_t blockThreads = 0, gridBlocks = 0;
    Analyzer::getParallelNumber(blockLevel, blockThreads);
    Analyzer::getParallelNumber(gridLevel, gridBlocks);
    if (matmul.getAttr("kcg.schedule").empty()) matmul.setAttr("kcg.schedule", "tiled");
    matmul.setAttr("kcg.block_threads", std::to_string(blockThreads));
    matmul.setAttr("kcg.grid_blocks", std::to_string(gridBlocks));
  }

  // Fold an in-place Relu on the matmul result into the kernel epilogue.
  std::set<Op *> erased;
  for (auto call : Analyzer::collectFuncCalls(module)) {
    if (erased.count(call.op)) continue;
    FuncOp callee = Analyzer::getTargetFunction(module, call.getCallee());
    if (!callee || !matmuls.count(callee)) continue;
    auto users = Analyzer::getUsers(module, call.getResult(0));
    if (users.size() != 1 || users[0]->kind != OpKind::Call) continue;
    CallOp reluCall(users[0]);
    if (reluCall.getCallee().rfind("Relu_Elementwise", 0) != 0) continue;
    FuncOp relu = Analyzer::getTargetFunction(module, reluCall.getCallee());
    // in place: the Relu function returns its own argument
    Op *ret = relu ? relu->lastOp() : nullptr;
    if (!ret || ret->operands.empty() || ret->operands[0] != relu.getArguments()[0]) continue;
    // only if no other matmul call shares the function with a different epilogue
    callee.setAttr("kcg.epilogue", "relu");
    replaceAllUsesWith(module.get(), reluCall.getResult(0), call.getResult(0));
    erased.insert(reluCall.op);
    reluCall->erase();
    relu.setAttr("func.state", "fused");
  }

  for (auto matmul : matmuls) {
    matmul.setAttr("kcg.BLOCK_SIZE_M", std::to_string(cfg("BLOCK_SIZE_M", 128)));
    matmul.setAttr("kcg.BLOCK_SIZE_N", std::to_string(cfg("BLOCK_SIZE_N", 128)));
    matmul.setAttr("kcg.BLOCK_SIZE_K", std::to_string(cfg("BLOCK_SIZE_K", 8)));
    matmul.setAttr("kcg.GROUP_SIZE_M", std::to_string(cfg("GROUP_SIZE_M", 8)));
    matmul.setAttr("kcg.WAVE_SIZE_M", std::to_string(cfg("WAVE_SIZE_M", 64)));
    matmul.setAttr("kcg.WAVE_SIZE_N", std::to_string(cfg("WAVE_SIZE_N", 64)));
    matmul.setAttr("kcg.VECTORIZE_WIDTH", std::to_string(cfg("VECTORIZE_WIDTH", 4)));
    matmul.setAttr("kcg.WARP_SIZE", std::to_string(cfg("WARP_SIZE", 64)));
  }
}

// ------------------------------------------------------------------- FMHA
bool FMHAOptimizer::applicable(ModuleOp &module) {
  clear();
  auto isCpuFunc = [&](const std::string &callee, const char *prefix) {
    if (callee.find(prefix) == std::string::npos) return false;
    FuncOp f = Analyzer::getTargetFunction(module, callee);
    return f && f.getAttr("func.state") == "cpu";
  };
  auto onlyUserCall = [&](CallOp call) -> CallOp {
    auto users = Analyzer::getUsers(module, call.getResult(0));
    if (Analyzer::getUsersNumber(users) != 1 || users[0]->kind != OpKind::Call) return CallOp();
    return CallOp(users[0]);
  };
  for (auto call2Matmul : Analyzer::collectFuncCalls(module)) {
    if (!isCpuFunc(call2Matmul.getCallee(), "BatchMatmul")) continue;
    CallOp call2Softmax = onlyUserCall(call2Matmul);
    if (!call2Softmax || !isCpuFunc(call2Softmax.getCallee(), "Softmax")) continue;
    CallOp call2Matmul2 = onlyUserCall(call2Softmax);
    if (!call2Matmul2 || !isCpuFunc(call2Matmul2.getCallee(), "BatchMatmul")) continue;
    if (uniqueFuncCalls.count(call2Matmul) || uniqueFuncCalls.count(call2Softmax) ||
        uniqueFuncCalls.count(call2Matmul2))
      continue;
    MemoryBuffer buf;
    if (!identifyBatchMatmul(call2Matmul.getCallee(), buf.matmul1) ||
        !identifyBatchMatmul(call2Matmul2.getCallee(), buf.matmul2))
      continue;
    // S = Q.K^T ('N','T'), O = P.V ('N','N'), same batch, rows match, S columns = V rows,
    // and P (the softmax result) is the left operand of the second product
    if (buf.matmul1.transA || !buf.matmul1.transB || buf.matmul2.transA || buf.matmul2.transB) continue;
    if (buf.matmul1.batch != buf.matmul2.batch || buf.matmul1.m != buf.matmul2.m ||
        buf.matmul1.n != buf.matmul2.k)
      continue;
    if (call2Matmul2.getArgOperands()[0] != call2Softmax.getResult(0)) continue;
    buf.Q = call2Matmul.getArgOperands()[0];
    buf.K = call2Matmul.getArgOperands()[1];
    buf.S = call2Matmul.getArgOperands()[2];
    buf.V = call2Matmul2.getArgOperands()[1];
    buf.O = call2Matmul2.getArgOperands()[2];
    call2bufferMap[call2Matmul] = buf;
    call2callsMap[call2Matmul] = {call2Softmax, call2Matmul2};
    uniqueFuncCalls.insert(call2Matmul);
    uniqueFuncCalls.insert(call2Softmax);
    uniqueFuncCalls.insert(call2Matmul2);
  }
  return !call2callsMap.empty();
}

// The body of the fused function as an executable loop nest (the reference's design,
// src/Optimizer/Optimizer.cc:948-1077 and 1191-1331: Br query rows per block, K/V swept in
// Bc-row tiles, running maximum / sum / rescale), one query row per thread:
//
//   m = -inf; l = 0; acc[0..Hd) = 0
//   for each K/V tile j:
//     s[c]  = scale * sum_d Q[row, d] * K[j*Bc + c, d]          for the valid keys of the tile
//     m'    = max(m, max_c s[c]);  alpha = exp(m - m')
//     l     = l * alpha;  acc[d] = acc[d] * alpha;  m = m'
//     p     = exp(s[c] - m);  l = l + p;  acc[d] = p * V[j*Bc + c, d] + acc[d]
//   O[row, d] = acc[d] / l
//
// A key is valid when it is below the sequence length and, with the causal mask, not
// beyond the query row; every valid row sees key 0 in tile 0, so m is finite from then on.
// The nest is what the interpreter runs to check the fusion against the un-fused graph;
// the GPU kernels implement the same recurrence on MFMA tiles.
static void buildOnlineSoftmaxNest(Op *gridLevel, Op *blockLevel, Value Q, Value K, Value V, Value O,
                                   int seqLen, int Hd, int Br, int Bc, float scale, bool causal) {
  const DType f32 = DType::f32;
  Value sBuf = Rewriter::alloc_buffer(OpHandle(blockLevel), MemorySpace::local, {Bc}, f32);
  Value acc = Rewriter::alloc_buffer(OpHandle(blockLevel), MemorySpace::local, {Hd}, f32);
  Value mNew = Rewriter::alloc_buffer(OpHandle(blockLevel), MemorySpace::local, {1}, f32);
  Value ml = Rewriter::alloc_buffer(OpHandle(blockLevel), MemorySpace::local, {2}, f32);  // m, l
  const int nGrid = static_cast<int>(gridLevel->args.size());
  std::vector<LinExpr> batchIdx;
  for (int i = 0; i + 1 < nGrid; ++i) batchIdx.emplace_back(gridLevel->arg(i));
  Value qb = gridLevel->arg(nGrid - 1), t = blockLevel->arg(0);
  LinExpr row;  // qb * Br + t
  row.add(qb, Br).add(t, 1);
  auto at = [&](const LinExpr &r, const LinExpr &c) {
    auto idx = batchIdx;
    idx.push_back(r);
    idx.push_back(c);
    return idx;
  };
  // this thread owns a row: t < Br and row < seqLen
  LinExpr tInBlock(static_cast<int64_t>(Br - 1));
  tInBlock.add(t, -1);
  LinExpr rowInSeq(static_cast<int64_t>(seqLen - 1));
  rowInSeq.add(row, -1);
  Op *own = blockLevel->pushBack(makeIf({tInBlock, rowInSeq}));

  Value zero = own->pushBack(makeConstant(0.0, f32))->result();
  Value negInf = own->pushBack(makeConstant(-std::numeric_limits<double>::infinity(), f32))->result();
  Value minusOne = own->pushBack(makeConstant(-1.0, f32))->result();
  Value scaleV = own->pushBack(makeConstant(static_cast<double>(scale), f32))->result();
  own->pushBack(makeStore(negInf, ml, {LinExpr(int64_t(0))}));
  own->pushBack(makeStore(zero, ml, {LinExpr(int64_t(1))}));
  {
    Op *init = own->pushBack(makeFor(0, Hd, 1));
    init->pushBack(makeStore(zero, acc, {LinExpr(init->arg(0))}));
    init->pushBack(makeYield());
  }
  const int nTiles = (seqLen + Bc - 1) / Bc;
  Op *tiles = own->pushBack(makeFor(0, nTiles, 1));
  Value j = tiles->arg(0);
  auto keyOf = [&](Value c) {
    LinExpr key;
    key.add(j, Bc).add(c, 1);
    return key;
  };
  // `body(ifOp, c, key)` is emitted under the validity guard of key (j, c)
  auto forValidKeys = [&](auto body) {
    Op *loop = tiles->pushBack(makeFor(0, Bc, 1));
    Value c = loop->arg(0);
    LinExpr key = keyOf(c);
    LinExpr inSeq(static_cast<int64_t>(seqLen - 1));
    inSeq.add(key, -1);
    std::vector<LinExpr> cons{inSeq};
    if (causal) {
      LinExpr notAfter = row;
      notAfter.add(key, -1);
      cons.push_back(notAfter);
    }
    Op *valid = loop->pushBack(makeIf(cons));
    body(valid, c, key);
    loop->pushBack(makeYield());
  };
  // s[c] = scale * <Q[row, :], K[key, :]>
  forValidKeys([&](Op *g, Value c, const LinExpr &key) {
    Op *dot = g->pushBack(makeFor(0, Hd, 1, {zero}));
    Value q = dot->pushBack(makeLoad(Q, at(row, LinExpr(dot->arg(0)))))->result();
    Value k = dot->pushBack(makeLoad(K, at(key, LinExpr(dot->arg(0)))))->result();
    Value mul = dot->pushBack(makeBinary(OpKind::MulF, q, k))->result();
    Value sum = dot->pushBack(makeBinary(OpKind::AddF, mul, dot->arg(1)))->result();
    dot->pushBack(makeYield({sum}));
    Value sc = g->pushBack(makeBinary(OpKind::MulF, dot->result(), scaleV))->result();
    g->pushBack(makeStore(sc, sBuf, {LinExpr(c)}));
  });
  // m' = max(m, max_c s[c])
  {
    Value m = tiles->pushBack(makeLoad(ml, {LinExpr(int64_t(0))}))->result();
    tiles->pushBack(makeStore(m, mNew, {LinExpr(int64_t(0))}));
  }
  forValidKeys([&](Op *g, Value c, const LinExpr &) {
    Value cur = g->pushBack(makeLoad(mNew, {LinExpr(int64_t(0))}))->result();
    Value sc = g->pushBack(makeLoad(sBuf, {LinExpr(c)}))->result();
    Value mx = g->pushBack(makeBinary(OpKind::MaxF, cur, sc))->result();
    g->pushBack(makeStore(mx, mNew, {LinExpr(int64_t(0))}));
  });
  // alpha = exp(m - m');  l *= alpha;  acc *= alpha;  m = m'
  {
    Value m = tiles->pushBack(makeLoad(ml, {LinExpr(int64_t(0))}))->result();
    Value mn = tiles->pushBack(makeLoad(mNew, {LinExpr(int64_t(0))}))->result();
    Value neg = tiles->pushBack(makeBinary(OpKind::MulF, mn, minusOne))->result();
    Value diff = tiles->pushBack(makeBinary(OpKind::AddF, m, neg))->result();
    Value alpha = tiles->pushBack(makeExp(diff))->result();
    Value l = tiles->pushBack(makeLoad(ml, {LinExpr(int64_t(1))}))->result();
    Value l2 = tiles->pushBack(makeBinary(OpKind::MulF, l, alpha))->result();
    tiles->pushBack(makeStore(l2, ml, {LinExpr(int64_t(1))}));
    Op *resc = tiles->pushBack(makeFor(0, Hd, 1));
    Value a = resc->pushBack(makeLoad(acc, {LinExpr(resc->arg(0))}))->result();
    Value a2 = resc->pushBack(makeBinary(OpKind::MulF, a, alpha))->result();
    resc->pushBack(makeStore(a2, acc, {LinExpr(resc->arg(0))}));
    resc->pushBack(makeYield());
    tiles->pushBack(makeStore(mn, ml, {LinExpr(int64_t(0))}));
  }
  // p = exp(s[c] - m);  l += p;  acc[d] = p * V[key, d] + acc[d]
  forValidKeys([&](Op *g, Value c, const LinExpr &key) {
    Value m = g->pushBack(makeLoad(ml, {LinExpr(int64_t(0))}))->result();
    Value neg = g->pushBack(makeBinary(OpKind::MulF, m, minusOne))->result();
    Value sc = g->pushBack(makeLoad(sBuf, {LinExpr(c)}))->result();
    Value diff = g->pushBack(makeBinary(OpKind::AddF, sc, neg))->result();
    Value pv = g->pushBack(makeExp(diff))->result();
    Value l = g->pushBack(makeLoad(ml, {LinExpr(int64_t(1))}))->result();
    Value l2 = g->pushBack(makeBinary(OpKind::AddF, pv, l))->result();
    g->pushBack(makeStore(l2, ml, {LinExpr(int64_t(1))}));
    Op *upd = g->pushBack(makeFor(0, Hd, 1));
    Value v = upd->pushBack(makeLoad(V, at(key, LinExpr(upd->arg(0)))))->result();
    Value a = upd->pushBack(makeLoad(acc, {LinExpr(upd->arg(0))}))->result();
    Value mul = upd->pushBack(makeBinary(OpKind::MulF, pv, v))->result();
    Value a2 = upd->pushBack(makeBinary(OpKind::AddF, mul, a))->result();
    upd->pushBack(makeStore(a2, acc, {LinExpr(upd->arg(0))}));
    upd->pushBack(makeYield());
  });
  tiles->pushBack(makeYield());
  // O[row, d] = acc[d] / l
  {
    Value l = own->pushBack(makeLoad(ml, {LinExpr(int64_t(1))}))->result();
    Op *fin = own->pushBack(makeFor(0, Hd, 1));
    Value a = fin->pushBack(makeLoad(acc, {LinExpr(fin->arg(0))}))->result();
    Value o = fin->pushBack(makeBinary(OpKind::DivF, a, l))->result();
    fin->pushBack(makeStore(o, O, at(row, LinExpr(fin->arg(0)))));
    fin->pushBack(makeYield());
  }
}

void FMHAOptimizer::applyOptimzer(ModuleOp &module) {
  auto cfg = [&](const char *key, int fallback) {
    auto it = fmhaConfig.find(key);
    return it == fmhaConfig.end() ? fallback : it->second;
  };
  for (auto &item : call2callsMap) {
    CallOp call2Matmul = item.first;
    CallOp call2Softmax = item.second[0];
    CallOp call2Matmul2 = item.second[1];
    const MemoryBuffer &buf = call2bufferMap[call2Matmul];
    const BatchMatmulDescriptor &d1 = buf.matmul1;
    const int seq_len = d1.m, head_dim = d1.k;

    std::string fusedFuncName = "Fused_Multi_Head_Attention";
    for (auto b : d1.batch) fusedFuncName += "_" + std::to_string(b);
    fusedFuncName += "_SL" + std::to_string(seq_len) + "_HD" + std::to_string(head_dim);

    const int Hd = head_dim;
    int Br = cfg("Br", 0), Bc = cfg("Bc", 0);
    if (Br == 0) Br = cfg("HdxBr", 128 * 128) / Hd;   // the reference's derivation
    if (Bc == 0) Bc = cfg("BrxBc", 128 * 32) / Br;
    const int blockSize = cfg("BLOCK_SIZE", 256);
    fmhaConfig["Hd"] = Hd;
    fmhaConfig["Br"] = Br;
    fmhaConfig["Bc"] = Bc;

    const MemRefType tq = buf.Q.getMemRefType(), tk = buf.K.getMemRefType(), tv = buf.V.getMemRefType(),
                     to = buf.O.getMemRefType();
    FuncOp funcOp = buildFuction(module, fusedFuncName, {tq, tk, tv, to}, {to});
    Op *newCall = call2Matmul2->insertAfter(makeCall(funcOp.op, {buf.Q, buf.K, buf.V, buf.O}));
    replaceAllUsesWith(module.get(), call2Matmul2.getResult(0), newCall->result(0));
    call2Matmul2->erase();
    call2Softmax->erase();
    call2Matmul->erase();
    // the S buffer has no reader left
    if (Op *sDef = buf.S.getDefiningOp())
      if (Analyzer::getUsers(module, buf.S).empty()) sDef->erase();

    if (funcOp->body.empty()) {
      auto args = funcOp.getArguments();
      funcOp->pushBack(makeReturn({args[3]}));
      // grid (batch.., ceil(S / Br)) x block (BLOCK_SIZE): one loop per level dimension,
      // then the same for -> parallel conversion the matmul recipe uses.
      // affine.parallel carries at most three dimensions (X, Y, Z): with more than
      // two batch dimensions they are folded into one
      std::vector<int64_t> bounds;
      if (d1.batch.size() <= 2) {
        for (auto b : d1.batch) bounds.push_back(b);
      } else {
        int64_t all = 1;
        for (auto b : d1.batch) all *= b;
        bounds.push_back(all);
      }
      bounds.push_back((seq_len + Br - 1) / Br);
      std::vector<ForOp> gridLoops;
      Op *cur = funcOp.op;
      for (auto b : bounds) {
        ForOp l = Rewriter::create_constant_loop(OpHandle(cur), 0, b, 1);
        gridLoops.push_back(l);
        cur = l.op;
      }
      ForOp blockLoop = Rewriter::create_constant_loop(OpHandle(cur), 0, blockSize, 1);
      auto gridLevel = Rewriter::parallel(gridLoops);
      auto blockLevel = Rewriter::parallel({blockLoop});
      const DType elem = tq.elem;
      // LDS tiles of the gfx950 kernel: K as [Bc][Hd + pad], V as [Bc][Hd + pad]
      const int padK = elem == DType::f32 ? 4 : 8, padV = elem == DType::f32 ? 8 : 32;
      Rewriter::alloc_buffer(OpHandle(gridLevel.op), MemorySpace::shared, {Bc, Hd + padV}, elem);
      Rewriter::alloc_buffer(OpHandle(gridLevel.op), MemorySpace::shared, {Bc, Hd + padK}, elem);
      const bool detailed = cfg("SCHEDULE_DETAIL", 0) >= 1 && d1.batch.size() <= 2 && Br <= blockSize;
      if (!detailed) {
        // per-lane registers: O^T accumulators (Hd/32 MFMA blocks x 16) and the running max / sum
        Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {2}, DType::f32);
        Rewriter::alloc_buffer(OpHandle(blockLevel.op), MemorySpace::local, {Hd / 32 > 0 ? Hd / 32 : 1, 16}, DType::f32);
      } else {
        buildOnlineSoftmaxNest(gridLevel.op, blockLevel.op, args[0], args[1], args[2], args[3], seq_len, Hd, Br, Bc,
                               scale, causal);
        funcOp.setAttr("kcg.schedule", "online_softmax");
      }
      funcOp.setAttr("func.state", "gpu");
      funcOp.setAttr("kcg.Br", std::to_string(Br));
      funcOp.setAttr("kcg.Bc", std::to_string(Bc));
      funcOp.setAttr("kcg.Hd", std::to_string(Hd));
      funcOp.setAttr("kcg.BLOCK_SIZE", std::to_string(blockSize));
      char sc[64];
      snprintf(sc, sizeof sc, "%.9g", static_cast<double>(scale));
      funcOp.setAttr("kcg.scale", sc);
      funcOp.setAttr("kcg.causal", causal ? "1" : "0");
    }
    DUMP(module);
  }
  // the three un-fused functions may have no caller left
  for (auto f : Analyzer::collectFunctions(module)) {
    if (f.getAttr("func.state") != "cpu") continue;
    bool called = false;
    for (auto c : Analyzer::collectFuncCalls(module)) called = called || c.getCallee() == f.getSymName();
    if (!called) f->erase();
  }
}

}  // namespace KernelCodeGen
