// Optimizer recipes (reference: include/Optimizer/Optimizer.h).
//
// A recipe recognises its operator in a module (`applicable`) and rewrites it
// in place (`applyOptimzer`, spelling kept from the reference) into the shape
// the backend binds to a gfx950 kernel: grid and block affine.parallel levels
// and the tile sizes of its string-keyed configuration table.
#pragma once

#include <map>
#include <set>
#include <string>
#include <vector>

#include "Frontend/Operators.h"
#include "IR/IR.h"
#include "Optimizer/Analyzer.h"
#include "IR/AffineMap.h"
#include "Optimizer/Rewriter.h"

// What a BatchMatmul_<batch..>_m<M>_n<N>_k<K>_<N|T><N|T> function name encodes.
struct BatchMatmulDescriptor {
  int m = 0;
  int n = 0;
  int k = 0;
  bool transA = false;
  bool transB = false;
  std::vector<int> batch;
  void log() const;
};

namespace KernelCodeGen {

// Parses a BatchMatmul function name back into its descriptor; false if malformed.
bool identifyBatchMatmul(const std::string &name, BatchMatmulDescriptor &matmul);

struct Optimizer {
  virtual ~Optimizer() = default;
  virtual bool applicable(ir::ModuleOp &module) = 0;
  virtual void applyOptimzer(ir::ModuleOp &module) = 0;
  bool operator==(const Optimizer &other) const { return name == other.name; }
  std::string name;
};

// Tiled matmul: split M, N by (THREAD_SIZE, BLOCK_SIZE), reorder to
// (mo, no, mm, nm, mi, ni), grid = parallel(mo, no), block = parallel(mm, nm),
// the k-loop accumulator bufferized into a THREAD_SIZE_M x THREAD_SIZE_N register
// tile, k hoisted over (mi, ni) and split by BLOCK_SIZE_K.  A Relu applied in
// place to the matmul's only result is folded into the kernel's epilogue
// (extension; the reference leaves Relu un-generated).
//
// Config key SCHEDULE_DETAIL selects how far the recipe of the reference
// (src/Optimizer/Optimizer.cc:383-548) is carried on the IR:
//   0 (default)  the tiling above; the backend only needs the tile sizes
//   1            + staging: global -> registers -> shared tiles (read / write /
//                barrier), shared -> register fragments, cache_read of A and B,
//                vectorised write-back of the register tile (cache_write, vectorize)
//   2            + double buffering of the shared tiles and of the fragments
//                (pipeline), peeled last k step (detach_last_loop), the
//                reference's statement order (schedule / extract_loop /
//                change_double_buffer), affine.if clean-up and unrolling
// Levels 1 and 2 follow the reference's thread organisation (8 x 8 register tile,
// BLOCK_SIZE = 16 x THREAD_SIZE in both directions); other tile shapes stay at level 0.
struct MatmulOptimizer : Optimizer {
  MatmulOptimizer() { name = "Matmul"; }
  bool applicable(ir::ModuleOp &module) override;
  void applyOptimzer(ir::ModuleOp &module) override;
  void clear() {
    matmuls.clear();
    matmulLoops.clear();
    matmulBuffers.clear();
  }

  struct MemoryBuffer {
    ir::Value A, B, C;
  };
  std::set<ir::FuncOp, CompareFunc> matmuls;
  std::map<ir::FuncOp, std::vector<ir::ForOp>, CompareFunc> matmulLoops;  // [M, N, K]
  std::map<ir::FuncOp, MemoryBuffer, CompareFunc> matmulBuffers;

  static std::map<std::string, int> matmulConfig;
  // Index maps of the staged schedule by name: loadTileA, loadTileB, storeTileA,
  // storeTileB, loadFragA, loadFragB, cacheReadA, cacheReadB, cacheWriteC
  // (the reference's getAffineMap, Optimizer.cc:272-380, for the current config).
  static ir::AffineMap getAffineMap(const std::string &mapIdentifier);
};

// BatchedMatmul(Q, K^T) -> Softmax -> BatchedMatmul(P, V), each result used
// once, becomes one function Fused_Multi_Head_Attention_<b..>_SL<S>_HD<D>(Q,K,V,O)
// with a grid level (batch.., S / Br) and a block level (BLOCK_SIZE threads).
struct FMHAOptimizer : Optimizer {
  FMHAOptimizer() { name = "FMHA"; }
  bool applicable(ir::ModuleOp &module) override;
  void applyOptimzer(ir::ModuleOp &module) override;
  void clear() {
    uniqueFuncCalls.clear();
    call2callsMap.clear();
    call2bufferMap.clear();
  }

  struct MemoryBuffer {
    ir::Value Q, K, S, V, O;
    BatchMatmulDescriptor matmul1, matmul2;
  };
  std::set<ir::CallOp, CompareFuncCall> uniqueFuncCalls;
  std::map<ir::CallOp, std::vector<ir::CallOp>, CompareFuncCall> call2callsMap;
  std::map<ir::CallOp, MemoryBuffer, CompareFuncCall> call2bufferMap;

  static std::map<std::string, int> fmhaConfig;
  // Extensions the reference graph does not have (defaults reproduce it):
  // logits multiplier and causal mask of the generated kernel.
  static float scale;
  static bool causal;
};

}  // namespace KernelCodeGen
