#include "IR/AffineMap.h"

namespace KernelCodeGen {
namespace ir {

AffineExpr AffineExpr::dim(int position) {
  return make(Kind::Dim, position);
}

AffineExpr AffineExpr::constant(int64_t value) {
  return make(Kind::Const, value);
}

AffineExpr AffineExpr::operator+(const AffineExpr &o) const {
  if (kind() == Kind::Const && o.kind() == Kind::Const) return constant(value() + o.value());
  return make(Kind::Add, 0, this, &o);
}

AffineExpr AffineExpr::operator*(int64_t factor) const {
  if (kind() == Kind::Const) return constant(value() * factor);
  if (factor == 1) return *this;
  return make(Kind::Mul, factor, this);
}

AffineExpr AffineExpr::floorDiv(int64_t divisor) const {
  if (divisor == 1) return *this;
  return make(Kind::FloorDiv, divisor, this);
}

AffineExpr AffineExpr::operator%(int64_t divisor) const {
  return make(Kind::Mod, divisor, this);
}

AffineExpr AffineExpr::shiftDims(int from, int shift) const {
  switch (kind()) {
    case Kind::Dim: return value() >= from ? dim(static_cast<int>(value()) + shift) : *this;
    case Kind::Const: return *this;
    case Kind::Add: return lhs().shiftDims(from, shift) + rhs().shiftDims(from, shift);
    case Kind::Mul: return lhs().shiftDims(from, shift) * value();
    case Kind::FloorDiv: return lhs().shiftDims(from, shift).floorDiv(value());
    case Kind::Mod: return lhs().shiftDims(from, shift) % value();
  }
  return *this;
}

int AffineExpr::maxDim() const {
  switch (kind()) {
    case Kind::Dim: return static_cast<int>(value());
    case Kind::Const: return -1;
    case Kind::Add: {
      const int a = lhs().maxDim(), b = rhs().maxDim();
      return a > b ? a : b;
    }
    default: return lhs().maxDim();
  }
}

LinExpr materialize(const AffineExpr &e, const std::vector<Value> &operands, Op *user) {
  switch (e.kind()) {
    case AffineExpr::Kind::Dim: return LinExpr(operands.at(static_cast<size_t>(e.value())));
    case AffineExpr::Kind::Const: return LinExpr(e.value());
    case AffineExpr::Kind::Add: {
      LinExpr r = materialize(e.lhs(), operands, user);
      r.add(materialize(e.rhs(), operands, user));
      return r;
    }
    case AffineExpr::Kind::Mul: {
      LinExpr r;
      r.add(materialize(e.lhs(), operands, user), e.value());
      return r;
    }
    case AffineExpr::Kind::FloorDiv:
    case AffineExpr::Kind::Mod: {
      const LinExpr inner = materialize(e.lhs(), operands, user);
      const bool isMod = e.kind() == AffineExpr::Kind::Mod;
      const int64_t c = e.value();
      if (inner.terms.empty()) {  // constant folds (floor semantics)
        int64_t q = inner.constant / c, r = inner.constant % c;
        if (r < 0) {
          r += c;
          q -= 1;
        }
        return LinExpr(isMod ? r : q);
      }
      Op *apply = user->insertBefore(isMod ? makeApplyMod(inner, c) : makeApplyFloorDiv(inner, c));
      return LinExpr(apply->result());
    }
  }
  return LinExpr();
}

std::vector<LinExpr> materialize(const AffineMap &map, const std::vector<Value> &operands, Op *user) {
  std::vector<LinExpr> out;
  for (auto &e : map.results) out.push_back(materialize(e, operands, user));
  return out;
}

}  // namespace ir
}  // namespace KernelCodeGen
