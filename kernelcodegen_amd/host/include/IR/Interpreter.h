// Reference interpreter for the affine IR: runs a module on host buffers.
// It exists so that a schedule can be checked against the nest it came from
// (run the naive module and the rewritten module on the same inputs and compare
// bit for bit).  fp32 arithmetic is performed in fp32, multiply and add as
// separate roundings, exactly as the ops are written.
//
// affine.parallel without a barrier inside is executed as a sequential loop over
// its index space.  A parallel level that contains gpu.barrier (a thread block
// staging tiles through shared memory) is executed in lock step: every index
// point gets its own frame (its registers and local buffers), statements that
// contain a barrier -- loops with constant bounds, affine.if with a condition all
// points agree on -- are walked once for all points together, and every other
// statement is run point by point in between.  That is exact for code whose
// barriers are reached by all threads of the block alike, which is the only kind
// the schedule primitives produce; anything else is reported as an error.
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
    Frame *parent = nullptr;
    std::map<const ValueImpl *, float *> mem;
    std::map<const ValueImpl *, float> f;
    std::map<const ValueImpl *, std::vector<float>> v;  // vector values
    std::map<const ValueImpl *, int64_t> i;
  };
  float *getMem(Frame &fr, Value v);
  float getF(Frame &fr, Value v);
  bool getI(Frame &fr, Value v, int64_t &out);
  const std::vector<float> *getV(Frame &fr, Value v);
  int64_t eval(const LinExpr &e, Frame &fr);
  int64_t offset(const Op *op, Frame &fr);
  bool holds(const Op *ifOp, Frame &fr);
  void exec(const Op *op, Frame &fr);
  void execRegion(const Op *op, Frame &fr);
  void execLockStep(const OpList &body, std::vector<Frame> &threads);
  bool containsBarrier(const Op *op);
  float *alloc(const MemRefType &t);

  ModuleOp module_;
  Frame top_;
  std::vector<std::unique_ptr<float[]>> owned_;
  std::map<const Op *, bool> barrierInside_;
  std::string error_;
};

}  // namespace ir
}  // namespace KernelCodeGen
