// A small self-contained affine IR: the substrate that stands in for the MLIR
// dialects the reference loads (affine, memref, func, arith, math, gpu;
// include/KernelCodeGen.h:45-57 of the reference).  It models exactly what the
// Frontend operators, the schedule primitives and the backend binding need:
//
//   module { memref.alloc ; func.func { affine.for / affine.parallel nests with
//   affine.load / affine.store (scalar or affine.vector_load / vector_store of w
//   contiguous elements) on linear index expressions, arith.{constant, mulf,
//   addf, maxf, divf}, math.exp, affine.apply, affine.if, affine.yield,
//   gpu.barrier, func.return } ; func.call }
//
// Index expressions are linear forms  sum(coeff_i * value_i) + constant  over
// loop induction variables and affine.apply results.  floordiv / mod by a
// constant (thread-id decompositions, double-buffer selectors) are affine.apply
// ops of their own -- `(expr) floordiv c`, `(expr) mod c` -- whose results are
// ordinary index values; the printer folds them back into the subscripts that
// use them, so the text reads like MLIR's single-map form.
//
// Ownership: an Op owns its results, its block arguments (induction variables,
// iter_args, function arguments) and the ops of its single-block region.
// `Value` and the typed op handles are non-owning views.
#pragma once

#include <cstdint>
#include <functional>
#include <list>
#include <map>
#include <memory>
#include <string>
#include <utility>
#include <vector>

namespace KernelCodeGen {
namespace ir {

enum class DType { f16, bf16, f32, f64, index, none };

const char *dtypeName(DType t);  // "f32", ...

struct MemRefType {
  std::vector<int64_t> shape;
  DType elem = DType::f32;
  int space = 1;  // MemorySpace as an integer (global = 1, shared = 2, local = 3)
  int64_t numElements() const;
  bool operator==(const MemRefType &o) const {
    return shape == o.shape && elem == o.elem && space == o.space;
  }
  std::string str() const;  // memref<4096x1024xf32, 1>
};

struct Op;

struct ValueImpl {
  enum Kind { Result, InductionVar, IterArg, FuncArg };
  Kind kind = Result;
  Op *owner = nullptr;  // defining op (Result) or the op whose region declares it
  int index = 0;
  bool isMemRef = false;
  MemRefType memref;
  DType dtype = DType::none;  // scalar (or vector element) type when !isMemRef
  int lanes = 1;              // > 1: vector<lanes x dtype> (result of a vector load)
};

// Non-owning handle; null-testable like the reference's mlir::Value.
class Value {
 public:
  Value() = default;
  Value(ValueImpl *p) : impl(p) {}
  explicit operator bool() const { return impl != nullptr; }
  bool operator==(const Value &o) const { return impl == o.impl; }
  bool operator!=(const Value &o) const { return impl != o.impl; }
  bool operator<(const Value &o) const { return impl < o.impl; }
  ValueImpl *get() const { return impl; }
  bool isMemRef() const { return impl && impl->isMemRef; }
  const MemRefType &getMemRefType() const { return impl->memref; }
  DType getDType() const { return impl->isMemRef ? impl->memref.elem : impl->dtype; }
  Op *getDefiningOp() const { return impl && impl->kind == ValueImpl::Result ? impl->owner : nullptr; }
  Op *getOwner() const { return impl ? impl->owner : nullptr; }

 private:
  ValueImpl *impl = nullptr;
};

// sum(coeff * value) + constant
struct LinExpr {
  std::vector<std::pair<Value, int64_t>> terms;
  int64_t constant = 0;
  LinExpr() = default;
  LinExpr(Value v) { terms.emplace_back(v, 1); }
  LinExpr(int64_t c) : constant(c) {}
  LinExpr &add(Value v, int64_t coeff = 1);
  LinExpr &add(const LinExpr &o, int64_t scale = 1);
  int64_t coeffOf(Value v) const;
  bool uses(Value v) const { return coeffOf(v) != 0; }
  // replaces `from` by the expression `to` (scaled by from's coefficient)
  void substitute(Value from, const LinExpr &to);
};

enum class OpKind {
  Module, Func, Alloc, Call, Return, For, Parallel, Apply, Load, Store, Constant,
  MulF, AddF, MaxF, DivF, Exp, Yield, Barrier, If
};

const char *opName(OpKind k);  // "affine.for", ...

using OpList = std::list<std::unique_ptr<Op>>;

struct Op {
  OpKind kind;
  Op *parent = nullptr;
  OpList body;                    // Module / Func / For / Parallel / If
  std::vector<Value> operands;    // arith operands; call / return / yield operands; store value;
                                  // for: iter_arg initial values
  Value memref;                   // load / store
  std::vector<LinExpr> indices;   // load / store subscripts; apply: one expression;
                                  // if: constraints, each meaning expr >= 0
  std::vector<std::unique_ptr<ValueImpl>> results;
  std::vector<std::unique_ptr<ValueImpl>> args;  // for: iv [+ iter_args]; parallel: ivs; func: args
  int64_t lb = 0, ub = 0, step = 1;              // for
  std::vector<int64_t> ubs;                      // parallel (lower bound 0, step 1)
  std::string name;                              // module / func symbol, call callee
  std::map<std::string, std::string> attrs;      // e.g. func.state, affine.loop
  double fvalue = 0.0;                           // constant
  int64_t divisor = 0;                           // apply: > 0 -> floordiv / mod by it
  bool isMod = false;                            // apply: mod instead of floordiv
  int vec = 0;                                   // load / store: 0 = scalar op, w >= 1 =
                                                 // vector op on w contiguous elements
  std::vector<MemRefType> resultTypes;           // func signature results

  explicit Op(OpKind k) : kind(k) {}
  Value result(int i = 0) const { return Value(results[i].get()); }
  Value arg(int i) const { return Value(args[i].get()); }
  bool hasRegion() const {
    return kind == OpKind::Module || kind == OpKind::Func || kind == OpKind::For ||
           kind == OpKind::Parallel || kind == OpKind::If;
  }
  // position helpers (this op inside parent->body)
  OpList::iterator self();
  Op *prev();
  Op *next();
  Op *lastOp() { return body.empty() ? nullptr : body.back().get(); }
  void erase();                                   // unlink and destroy
  std::unique_ptr<Op> unlink();                   // unlink, keep alive
  Op *insertBefore(std::unique_ptr<Op> op);       // before this op
  Op *insertAfter(std::unique_ptr<Op> op);        // after this op
  Op *pushBack(std::unique_ptr<Op> op);           // at the end of this op's region
  Op *pushFront(std::unique_ptr<Op> op);
  void moveBefore(Op *other);
  void moveAfter(Op *other);
  bool isAncestorOf(const Op *other) const;       // proper ancestor
  Op *parentOfKind(OpKind k);
};

// --- construction helpers (free-standing ops, to be inserted by the caller) ---
std::unique_ptr<Op> makeModule(const std::string &name);
std::unique_ptr<Op> makeFunc(const std::string &name, const std::vector<MemRefType> &inputs,
                             const std::vector<MemRefType> &outputs);
std::unique_ptr<Op> makeAlloc(const MemRefType &t);
std::unique_ptr<Op> makeCall(Op *func, const std::vector<Value> &operands);
std::unique_ptr<Op> makeReturn(const std::vector<Value> &operands);
std::unique_ptr<Op> makeFor(int64_t lb, int64_t ub, int64_t step, const std::vector<Value> &iterInits = {});
std::unique_ptr<Op> makeParallel(const std::vector<int64_t> &ubs);
std::unique_ptr<Op> makeApply(const LinExpr &e);
std::unique_ptr<Op> makeApplyFloorDiv(const LinExpr &e, int64_t divisor);  // (e) floordiv divisor
std::unique_ptr<Op> makeApplyMod(const LinExpr &e, int64_t divisor);       // (e) mod divisor
std::unique_ptr<Op> makeLoad(Value memref, const std::vector<LinExpr> &idx);
std::unique_ptr<Op> makeStore(Value value, Value memref, const std::vector<LinExpr> &idx);
// width elements along the last dimension, starting at the subscript
std::unique_ptr<Op> makeVectorLoad(Value memref, const std::vector<LinExpr> &idx, int width);
std::unique_ptr<Op> makeVectorStore(Value value, Value memref, const std::vector<LinExpr> &idx, int width);
// affine.if: the body runs when every constraint evaluates >= 0 (no else region)
std::unique_ptr<Op> makeIf(const std::vector<LinExpr> &constraints);
std::unique_ptr<Op> makeConstant(double v, DType t);
std::unique_ptr<Op> makeBinary(OpKind k, Value a, Value b);
std::unique_ptr<Op> makeExp(Value a);
std::unique_ptr<Op> makeYield(const std::vector<Value> &operands = {});
std::unique_ptr<Op> makeBarrier();

// --- traversal / rewriting utilities ---
enum class WalkOrder { PreOrder, PostOrder };
void walk(Op *root, const std::function<void(Op *)> &fn, WalkOrder order = WalkOrder::PreOrder);
// every use of `from` in the subtree of `root` (operands, memrefs, index terms)
void replaceAllUsesWith(Op *root, Value from, Value to);
void replaceIndexUses(Op *root, Value from, const LinExpr &to);  // only inside index expressions
std::vector<Op *> getUsers(Op *root, Value v);
// deep copy of `op`; values defined outside the subtree are shared, inside are remapped.
std::unique_ptr<Op> clone(const Op *op, std::map<ValueImpl *, ValueImpl *> *mapping = nullptr);

// MLIR-flavoured text of the op (module, function or loop nest).
std::string print(const Op *op);
// Structural checks: operands visible where used, bounds sane, terminators and
// region kinds consistent.  Returns "" when valid, else the first problem.
std::string verify(const Op *op);

// --- typed, non-owning handles (the reference passes mlir::ModuleOp etc. by value) ---
struct OpHandle {
  Op *op = nullptr;
  OpHandle() = default;
  OpHandle(Op *o) : op(o) {}
  explicit operator bool() const { return op != nullptr; }
  Op *operator->() const { return op; }
  bool operator==(const OpHandle &o) const { return op == o.op; }
  bool operator!=(const OpHandle &o) const { return op != o.op; }
  bool operator<(const OpHandle &o) const { return op < o.op; }
};

struct ForOp : OpHandle {
  using OpHandle::OpHandle;
  Value getInductionVar() const { return op->arg(0); }
  int64_t getLowerBound() const { return op->lb; }
  int64_t getUpperBound() const { return op->ub; }
  int64_t getStep() const { return op->step; }
  int64_t tripCount() const { return (op->ub - op->lb + op->step - 1) / op->step; }
  size_t numIterArgs() const { return op->args.size() - 1; }
};

struct IfOp : OpHandle {
  using OpHandle::OpHandle;
  const std::vector<LinExpr> &getConstraints() const { return op->indices; }
};

struct ParallelOp : OpHandle {
  using OpHandle::OpHandle;
  size_t getNumDims() const { return op->ubs.size(); }
  std::vector<Value> getIVs() const;
};

struct FuncOp : OpHandle {
  using OpHandle::OpHandle;
  const std::string &getSymName() const { return op->name; }
  std::vector<Value> getArguments() const;
  std::string getAttr(const std::string &key) const;
  void setAttr(const std::string &key, const std::string &value) { op->attrs[key] = value; }
};

struct CallOp : OpHandle {
  using OpHandle::OpHandle;
  const std::string &getCallee() const { return op->name; }
  const std::vector<Value> &getArgOperands() const { return op->operands; }
  Value getResult(int i = 0) const { return op->result(i); }
};

// Owning module handle with value semantics (copy = deep clone), so that the
// facade's backup / reset / best-module bookkeeping reads like the reference's.
class ModuleOp {
 public:
  ModuleOp() = default;
  explicit ModuleOp(std::unique_ptr<Op> m) : root(std::move(m)) {}
  static ModuleOp create(const std::string &name) { return ModuleOp(makeModule(name)); }
  ModuleOp clone() const { return root ? ModuleOp(ir::clone(root.get())) : ModuleOp(); }
  explicit operator bool() const { return root != nullptr; }
  Op *get() const { return root.get(); }
  Op *operator->() const { return root.get(); }
  const std::string &getName() const { return root->name; }
  std::string str() const { return print(root.get()); }
  void dump() const;

 private:
  std::shared_ptr<Op> root;  // shared so handles can be passed by value cheaply
};

}  // namespace ir
}  // namespace KernelCodeGen
