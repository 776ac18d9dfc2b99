// Read-only queries over a module (reference: include/Optimizer/Analyzer.h:42-82,
// src/Optimizer/Analyzer.cc:62-107).
#pragma once

#include <string>
#include <vector>

#include "IR/IR.h"

namespace KernelCodeGen {

// Orders handles by identity, for use as map / set keys.
struct CompareLoop {
  bool operator()(const ir::ForOp &x, const ir::ForOp &y) const { return x.op < y.op; }
};
struct CompareFunc {
  bool operator()(const ir::FuncOp &x, const ir::FuncOp &y) const { return x.op < y.op; }
};
struct CompareFuncCall {
  bool operator()(const ir::CallOp &x, const ir::CallOp &y) const { return x.op < y.op; }
};

struct Analyzer {
  // Loops that sit directly in the module body.
  static std::vector<ir::ForOp> collectOutermostLoop(ir::ModuleOp &module);
  // Extent of every dimension of a parallel level (grid or block) and their product.
  static std::vector<int64_t> getParallelNumber(ir::ParallelOp parallelLevel, int64_t &totalNumber);
  // Functions whose name contains `targetFuncName` (all of them when it is empty).
  static std::vector<ir::FuncOp> collectFunctions(ir::ModuleOp &module, const std::string &targetFuncName = {""});
  // Every affine.for of the function, outermost first (pre-order).
  static std::vector<ir::ForOp> collectFuncLoops(ir::FuncOp funcOp);
  static std::vector<ir::ParallelOp> collectFuncParallels(ir::FuncOp funcOp);
  static std::vector<ir::CallOp> collectFuncCalls(ir::ModuleOp &module);
  // The function called exactly `targetFuncName`; null handle (and a message) if absent.
  static ir::FuncOp getTargetFunction(ir::ModuleOp &module, const std::string &targetFuncName);
  // Ops of the module's top level that use `v`.
  static std::vector<ir::Op *> getUsers(ir::ModuleOp &module, ir::Value v);
  static int getUsersNumber(const std::vector<ir::Op *> &users) { return static_cast<int>(users.size()); }

  // Last direct child of `father` that has the given kind (null if none).
  static ir::Op *getLastOp(ir::Op *father, ir::OpKind kind);
};

}  // namespace KernelCodeGen
