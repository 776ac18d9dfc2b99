// Frontend: operators described as naive affine loop nests.
//
// Mirrors the reference's interface (include/Frontend/Operators.h:9-102):
// ComputeDAG::create<Op>(args...) appends, to the graph's module, one
// func.func holding the operator's loop nest (named after the operator and its
// shapes, tagged func.state = "cpu") plus a func.call to it, and returns the
// call's result.  Differences, all deliberate:
//   * the substrate is the small IR of IR/IR.h, not MLIR;
//   * problems are reported by returning a null Value after printing a message
//     (the reference also exits the process in one place, Operators.cc:271);
//   * "bfloat16" is an accepted dtype (extension);
//   * BatchedMatmul with a col-major A indexes A[.., k, i] (the reference pushes
//     (k, j), Operators.cc:390-392, which is a latent bug);
//   * Softmax accepts axis = -1 silently (the reference prints an error for its
//     own default and continues, Operators.cc:449-451);
//   * Transpose is declared but, as in the reference (Operators.cc:422-423), not
//     implemented: it reports that and returns null.
#pragma once

#include <string>
#include <vector>

#include "IR/IR.h"
#include "enum.h"
#include "log.h"

namespace KernelCodeGen {

// Returns the function named `funcName` if the module already has it, else
// creates it at the start of the module with one block argument per input type.
ir::FuncOp buildFuction(ir::ModuleOp module, const std::string &funcName,
                        const std::vector<ir::MemRefType> &inputsTypes,
                        const std::vector<ir::MemRefType> &outputsTypes);

// "float32" | "float64" | "float16" | "bfloat16" -> element type; DType::none if unknown.
ir::DType getDType(const std::string &dtype);
std::string toStr(ir::DType t);

// Builds the graph and stores its module.
struct ComputeDAG {
  ComputeDAG() = default;

  template <typename OperatorType, typename... Args>
  ir::Value create(Args &&...args) {
    return OperatorType::build(this, std::forward<Args>(args)...);
  }

  // Prints the module (Debug log level only) and verifies it.
  void dump(const std::string &info = "");

  ir::ModuleOp module;
};

template <typename T>
struct Operator {
  template <typename... Args>
  static ir::Value build(ComputeDAG *graph, Args &&...args) {
    return T::build(graph, std::forward<Args>(args)...);
  }
};

struct PlaceHolder : Operator<PlaceHolder> {
  static ir::Value build(ComputeDAG *graph, const std::vector<int64_t> &shapes, const std::string &dtype);
};

struct Matmul : Operator<Matmul> {
  static ir::Value build(ComputeDAG *graph, ir::Value A, ir::Value B, MemorySpace ms,
                         const std::string &dtype = {""});
};

struct Relu : Operator<Relu> {
  static ir::Value build(ComputeDAG *graph, ir::Value input, MemorySpace ms, const std::string &dtype = {""});
};

struct BatchedMatmul : Operator<BatchedMatmul> {
  static ir::Value build(ComputeDAG *graph, ir::Value A, Layout layoutA, ir::Value B, Layout layoutB,
                         const std::string &dtype = {""});
};

// Softmax over the last axis: exp(x) / sum(exp(x)), no max shift.
struct Softmax : Operator<Softmax> {
  static ir::Value build(ComputeDAG *graph, ir::Value input, int axis = -1,
                         MemorySpace ms = MemorySpace::global, const std::string &dtype = {""});
};

struct Transpose : Operator<Transpose> {
  static ir::Value build(ComputeDAG *graph, ir::Value input);
};

}  // namespace KernelCodeGen
