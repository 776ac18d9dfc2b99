// Reference interpreter for the affine IR: runs a module on host buffers.
// It exists so that a schedule can be checked against the nest it came from
// (run the naive module and the rewritten module on the same inputs and compare
// bit for bit).  fp32 arithmetic is performed in fp32, multiply and add as
// separate roundings, exactly as the ops are written.
//
// affine.parallel is executed as a sequential loop over its index space, which
// is exact for nests without gpu.barrier (the ones split / reorder / parallel /
// bufferize produce); a barrier inside a parallel region is rejected.
#pragma once

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "IR/IR.h"

namespace KernelCodeGen {
namespace ir {

class Interpreter {
 public:
  explicit Interpreter(const ModuleOp &module) : module_(module) {}
  // Use caller-owned storage for a module-level memref (a PlaceHolder result).
  void bind(Value memref, float *data);
  // Executes the module's top-level ops in order.  Returns "" or an error text.
  std::string run();
  // Storage behind a module-level memref or call result after run().
  float *buffer(Value memref);

 private:
  struct Frame {
    std::map<const ValueImpl *, float *> mem;
    std::map<const ValueImpl *, float> f;
    std::map<const ValueImpl *, int64_t> i;
  };
  int64_t eval(const LinExpr &e, Frame &fr);
  int64_t offset(const Op *op, Frame &fr);
  void exec(const Op *op, Frame &fr);
  void execRegion(const Op *op, Frame &fr);
  float *alloc(const MemRefType &t);

  ModuleOp module_;
  Frame top_;
  std::vector<std::unique_ptr<float[]>> owned_;
  std::string error_;
  int parallelDepth_ = 0;
};

}  // namespace ir
}  // namespace KernelCodeGen
