// Index maps in the (map, operands) style the reference's schedule primitives
// take (mlir::AffineMap + operand list, e.g. src/Optimizer/Rewriter.cc:601-647):
// result expressions over positional dimensions d0..d(n-1), bound to values
// only when the map is applied.
//
//   auto d0 = AffineExpr::dim(0), d1 = AffineExpr::dim(1);
//   AffineMap map{2, {(d0 * 16 + d1).floorDiv(2), (d0 * 16 + d1) % 2 * 4}};
//   std::vector<LinExpr> idx = materialize(map, {ty, tx}, loadOp);
//
// materialize() lowers a map onto the IR's index expressions: linear parts
// become LinExpr terms, every floordiv / mod node becomes an affine.apply op
// inserted right before the op that will use the subscripts.
#pragma once

#include <cstdint>
#include <memory>
#include <vector>

#include "IR/IR.h"

namespace KernelCodeGen {
namespace ir {

class AffineExpr {
 public:
  enum class Kind { Dim, Const, Add, Mul, FloorDiv, Mod };
  static AffineExpr dim(int position);
  static AffineExpr constant(int64_t value);
  AffineExpr() : AffineExpr(constant(0)) {}

  AffineExpr operator+(const AffineExpr &o) const;
  AffineExpr operator+(int64_t c) const { return *this + constant(c); }
  AffineExpr operator*(int64_t factor) const;
  AffineExpr floorDiv(int64_t divisor) const;
  AffineExpr operator%(int64_t divisor) const;

  Kind kind() const { return node_->kind; }
  int64_t value() const { return node_->value; }  // dim position, constant, factor or divisor
  AffineExpr lhs() const { return AffineExpr(node_->lhs); }
  AffineExpr rhs() const { return AffineExpr(node_->rhs); }
  // dimension positions renumbered: position p becomes p + shift for p >= from
  AffineExpr shiftDims(int from, int shift) const;
  int maxDim() const;  // largest dimension position used, -1 when none

 private:
  struct Node {
    Kind kind;
    int64_t value;
    std::shared_ptr<const Node> lhs, rhs;
  };
  explicit AffineExpr(std::shared_ptr<const Node> n) : node_(std::move(n)) {}
  static AffineExpr make(Kind k, int64_t v, const AffineExpr *l = nullptr, const AffineExpr *r = nullptr) {
    auto n = std::make_shared<Node>();
    n->kind = k;
    n->value = v;
    if (l) n->lhs = l->node_;
    if (r) n->rhs = r->node_;
    return AffineExpr(std::shared_ptr<const Node>(std::move(n)));
  }
  std::shared_ptr<const Node> node_;
};

inline AffineExpr operator*(int64_t factor, const AffineExpr &e) { return e * factor; }

struct AffineMap {
  int numDims = 0;
  std::vector<AffineExpr> results;
};

// Index expressions of map(operands); apply ops for floordiv / mod nodes are
// inserted before `user`.  operands.size() must be >= map.numDims.
std::vector<LinExpr> materialize(const AffineMap &map, const std::vector<Value> &operands, Op *user);
// Same for one expression.
LinExpr materialize(const AffineExpr &e, const std::vector<Value> &operands, Op *user);

}  // namespace ir
}  // namespace KernelCodeGen
