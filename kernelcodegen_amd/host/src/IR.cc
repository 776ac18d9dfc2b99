#include "IR/IR.h"

#include <algorithm>
#include <cassert>
#include <cstdio>
#include <iostream>
#include <set>
#include <sstream>

namespace KernelCodeGen {
namespace ir {

const char *dtypeName(DType t) {
  switch (t) {
    case DType::f16: return "f16";
    case DType::bf16: return "bf16";
    case DType::f32: return "f32";
    case DType::f64: return "f64";
    case DType::index: return "index";
    default: return "none";
  }
}

int64_t MemRefType::numElements() const {
  int64_t n = 1;
  for (auto d : shape) n *= d;
  return n;
}

std::string MemRefType::str() const {
  std::ostringstream os;
  os << "memref<";
  for (auto d : shape) os << d << "x";
  os << dtypeName(elem) << ", " << space << ">";
  return os.str();
}

// ------------------------------------------------------------------ LinExpr
LinExpr &LinExpr::add(Value v, int64_t coeff) {
  if (coeff == 0) return *this;
  for (auto &t : terms)
    if (t.first == v) {
      t.second += coeff;
      if (t.second == 0)
        terms.erase(std::remove_if(terms.begin(), terms.end(),
                                   [](const std::pair<Value, int64_t> &p) { return p.second == 0; }),
                    terms.end());
      return *this;
    }
  terms.emplace_back(v, coeff);
  return *this;
}

LinExpr &LinExpr::add(const LinExpr &o, int64_t scale) {
  for (auto &t : o.terms) add(t.first, t.second * scale);
  constant += o.constant * scale;
  return *this;
}

int64_t LinExpr::coeffOf(Value v) const {
  for (auto &t : terms)
    if (t.first == v) return t.second;
  return 0;
}

void LinExpr::substitute(Value from, const LinExpr &to) {
  const int64_t c = coeffOf(from);
  if (c == 0) return;
  // keep the position of `from` for the first replacement term so printed
  // subscripts read in loop order (outer + middle + inner)
  std::vector<std::pair<Value, int64_t>> out;
  for (auto &t : terms) {
    if (t.first == from) {
      for (auto &n : to.terms) out.emplace_back(n.first, n.second * c);
    } else {
      out.push_back(t);
    }
  }
  terms.clear();
  const int64_t k = constant + to.constant * c;
  constant = 0;
  for (auto &t : out) add(t.first, t.second);
  constant = k;
}

// ---------------------------------------------------------------------- Op
const char *opName(OpKind k) {
  switch (k) {
    case OpKind::Module: return "module";
    case OpKind::Func: return "func.func";
    case OpKind::Alloc: return "memref.alloc";
    case OpKind::Call: return "func.call";
    case OpKind::Return: return "func.return";
    case OpKind::For: return "affine.for";
    case OpKind::Parallel: return "affine.parallel";
    case OpKind::Apply: return "affine.apply";
    case OpKind::Load: return "affine.load";
    case OpKind::Store: return "affine.store";
    case OpKind::Constant: return "arith.constant";
    case OpKind::MulF: return "arith.mulf";
    case OpKind::AddF: return "arith.addf";
    case OpKind::MaxF: return "arith.maxf";
    case OpKind::DivF: return "arith.divf";
    case OpKind::Exp: return "math.exp";
    case OpKind::Yield: return "affine.yield";
    case OpKind::Barrier: return "gpu.barrier";
    case OpKind::If: return "affine.if";
  }
  return "?";
}

OpList::iterator Op::self() {
  assert(parent && "op is not linked");
  for (auto it = parent->body.begin(); it != parent->body.end(); ++it)
    if (it->get() == this) return it;
  assert(false && "op not found in its parent");
  return parent->body.end();
}

Op *Op::prev() {
  auto it = self();
  if (it == parent->body.begin()) return nullptr;
  return std::prev(it)->get();
}

Op *Op::next() {
  auto it = std::next(self());
  return it == parent->body.end() ? nullptr : it->get();
}

void Op::erase() { parent->body.erase(self()); }

std::unique_ptr<Op> Op::unlink() {
  auto it = self();
  std::unique_ptr<Op> keep = std::move(*it);
  parent->body.erase(it);
  keep->parent = nullptr;
  return keep;
}

Op *Op::insertBefore(std::unique_ptr<Op> op) {
  op->parent = parent;
  Op *raw = op.get();
  parent->body.insert(self(), std::move(op));
  return raw;
}

Op *Op::insertAfter(std::unique_ptr<Op> op) {
  op->parent = parent;
  Op *raw = op.get();
  parent->body.insert(std::next(self()), std::move(op));
  return raw;
}

Op *Op::pushBack(std::unique_ptr<Op> op) {
  op->parent = this;
  body.push_back(std::move(op));
  return body.back().get();
}

Op *Op::pushFront(std::unique_ptr<Op> op) {
  op->parent = this;
  body.push_front(std::move(op));
  return body.front().get();
}

void Op::moveBefore(Op *other) {
  auto keep = unlink();
  other->insertBefore(std::move(keep));
}

void Op::moveAfter(Op *other) {
  auto keep = unlink();
  other->insertAfter(std::move(keep));
}

bool Op::isAncestorOf(const Op *other) const {
  for (const Op *p = other ? other->parent : nullptr; p; p = p->parent)
    if (p == this) return true;
  return false;
}

Op *Op::parentOfKind(OpKind k) {
  for (Op *p = parent; p; p = p->parent)
    if (p->kind == k) return p;
  return nullptr;
}

// ------------------------------------------------------------- construction
static ValueImpl *addResult(Op *op, DType t) {
  auto v = std::make_unique<ValueImpl>();
  v->kind = ValueImpl::Result;
  v->owner = op;
  v->index = static_cast<int>(op->results.size());
  v->dtype = t;
  op->results.push_back(std::move(v));
  return op->results.back().get();
}

static ValueImpl *addMemRefResult(Op *op, const MemRefType &t) {
  ValueImpl *v = addResult(op, t.elem);
  v->isMemRef = true;
  v->memref = t;
  return v;
}

static ValueImpl *addArg(Op *op, ValueImpl::Kind kind, DType t) {
  auto v = std::make_unique<ValueImpl>();
  v->kind = kind;
  v->owner = op;
  v->index = static_cast<int>(op->args.size());
  v->dtype = t;
  op->args.push_back(std::move(v));
  return op->args.back().get();
}

std::unique_ptr<Op> makeModule(const std::string &name) {
  auto op = std::make_unique<Op>(OpKind::Module);
  op->name = name;
  return op;
}

std::unique_ptr<Op> makeFunc(const std::string &name, const std::vector<MemRefType> &inputs,
                             const std::vector<MemRefType> &outputs) {
  auto op = std::make_unique<Op>(OpKind::Func);
  op->name = name;
  op->resultTypes = outputs;
  for (auto &t : inputs) {
    ValueImpl *a = addArg(op.get(), ValueImpl::FuncArg, t.elem);
    a->isMemRef = true;
    a->memref = t;
  }
  return op;
}

std::unique_ptr<Op> makeAlloc(const MemRefType &t) {
  auto op = std::make_unique<Op>(OpKind::Alloc);
  addMemRefResult(op.get(), t);
  return op;
}

std::unique_ptr<Op> makeCall(Op *func, const std::vector<Value> &operands) {
  auto op = std::make_unique<Op>(OpKind::Call);
  op->name = func->name;
  op->operands = operands;
  for (auto &t : func->resultTypes) addMemRefResult(op.get(), t);
  return op;
}

std::unique_ptr<Op> makeReturn(const std::vector<Value> &operands) {
  auto op = std::make_unique<Op>(OpKind::Return);
  op->operands = operands;
  return op;
}

std::unique_ptr<Op> makeFor(int64_t lb, int64_t ub, int64_t step, const std::vector<Value> &iterInits) {
  auto op = std::make_unique<Op>(OpKind::For);
  op->lb = lb;
  op->ub = ub;
  op->step = step;
  addArg(op.get(), ValueImpl::InductionVar, DType::index);
  for (auto &v : iterInits) {
    op->operands.push_back(v);
    addArg(op.get(), ValueImpl::IterArg, v.getDType());
    addResult(op.get(), v.getDType());
  }
  return op;
}

std::unique_ptr<Op> makeParallel(const std::vector<int64_t> &ubs) {
  auto op = std::make_unique<Op>(OpKind::Parallel);
  op->ubs = ubs;
  for (size_t i = 0; i < ubs.size(); ++i) addArg(op.get(), ValueImpl::InductionVar, DType::index);
  return op;
}

std::unique_ptr<Op> makeApply(const LinExpr &e) {
  auto op = std::make_unique<Op>(OpKind::Apply);
  op->indices.push_back(e);
  addResult(op.get(), DType::index);
  return op;
}

std::unique_ptr<Op> makeApplyFloorDiv(const LinExpr &e, int64_t divisor) {
  auto op = makeApply(e);
  op->divisor = divisor;
  return op;
}

std::unique_ptr<Op> makeApplyMod(const LinExpr &e, int64_t divisor) {
  auto op = makeApply(e);
  op->divisor = divisor;
  op->isMod = true;
  return op;
}

std::unique_ptr<Op> makeVectorLoad(Value memref, const std::vector<LinExpr> &idx, int width) {
  auto op = makeLoad(memref, idx);
  op->vec = width;
  op->results[0]->lanes = width;
  return op;
}

std::unique_ptr<Op> makeVectorStore(Value value, Value memref, const std::vector<LinExpr> &idx, int width) {
  auto op = makeStore(value, memref, idx);
  op->vec = width;
  return op;
}

std::unique_ptr<Op> makeIf(const std::vector<LinExpr> &constraints) {
  auto op = std::make_unique<Op>(OpKind::If);
  op->indices = constraints;
  return op;
}

std::unique_ptr<Op> makeLoad(Value memref, const std::vector<LinExpr> &idx) {
  auto op = std::make_unique<Op>(OpKind::Load);
  op->memref = memref;
  op->indices = idx;
  addResult(op.get(), memref.getMemRefType().elem);
  return op;
}

std::unique_ptr<Op> makeStore(Value value, Value memref, const std::vector<LinExpr> &idx) {
  auto op = std::make_unique<Op>(OpKind::Store);
  op->operands.push_back(value);
  op->memref = memref;
  op->indices = idx;
  return op;
}

std::unique_ptr<Op> makeConstant(double v, DType t) {
  auto op = std::make_unique<Op>(OpKind::Constant);
  op->fvalue = v;
  addResult(op.get(), t);
  return op;
}

std::unique_ptr<Op> makeBinary(OpKind k, Value a, Value b) {
  auto op = std::make_unique<Op>(k);
  op->operands = {a, b};
  addResult(op.get(), a.getDType());
  return op;
}

std::unique_ptr<Op> makeExp(Value a) {
  auto op = std::make_unique<Op>(OpKind::Exp);
  op->operands = {a};
  addResult(op.get(), a.getDType());
  return op;
}

std::unique_ptr<Op> makeYield(const std::vector<Value> &operands) {
  auto op = std::make_unique<Op>(OpKind::Yield);
  op->operands = operands;
  return op;
}

std::unique_ptr<Op> makeBarrier() { return std::make_unique<Op>(OpKind::Barrier); }

// ---------------------------------------------------------------- traversal
void walk(Op *root, const std::function<void(Op *)> &fn, WalkOrder order) {
  if (order == WalkOrder::PreOrder) fn(root);
  // copy the child pointers first: callbacks may unlink the visited op
  std::vector<Op *> kids;
  for (auto &c : root->body) kids.push_back(c.get());
  for (Op *c : kids) walk(c, fn, order);
  if (order == WalkOrder::PostOrder) fn(root);
}

void replaceAllUsesWith(Op *root, Value from, Value to) {
  walk(root, [&](Op *op) {
    for (auto &v : op->operands)
      if (v == from) v = to;
    if (op->memref == from) op->memref = to;
    for (auto &e : op->indices) e.substitute(from, LinExpr(to));
  });
}

void replaceIndexUses(Op *root, Value from, const LinExpr &to) {
  walk(root, [&](Op *op) {
    for (auto &e : op->indices) e.substitute(from, to);
  });
}

std::vector<Op *> getUsers(Op *root, Value v) {
  std::vector<Op *> users;
  walk(root, [&](Op *op) {
    bool uses = op->memref == v;
    for (auto &o : op->operands) uses = uses || (o == v);
    for (auto &e : op->indices) uses = uses || e.uses(v);
    if (uses) users.push_back(op);
  });
  return users;
}

static std::unique_ptr<Op> cloneRec(const Op *op, std::map<ValueImpl *, ValueImpl *> &m) {
  auto c = std::make_unique<Op>(op->kind);
  c->lb = op->lb;
  c->ub = op->ub;
  c->step = op->step;
  c->ubs = op->ubs;
  c->name = op->name;
  c->attrs = op->attrs;
  c->fvalue = op->fvalue;
  c->divisor = op->divisor;
  c->isMod = op->isMod;
  c->vec = op->vec;
  c->resultTypes = op->resultTypes;
  auto copyVals = [&](const std::vector<std::unique_ptr<ValueImpl>> &src,
                      std::vector<std::unique_ptr<ValueImpl>> &dst) {
    for (auto &v : src) {
      auto n = std::make_unique<ValueImpl>(*v);
      n->owner = c.get();
      m[v.get()] = n.get();
      dst.push_back(std::move(n));
    }
  };
  copyVals(op->results, c->results);
  copyVals(op->args, c->args);
  auto remap = [&](Value v) -> Value {
    auto it = m.find(v.get());
    return it == m.end() ? v : Value(it->second);
  };
  for (auto &v : op->operands) c->operands.push_back(remap(v));
  c->memref = remap(op->memref);
  for (auto &e : op->indices) {
    LinExpr n;
    n.constant = e.constant;
    for (auto &t : e.terms) n.terms.emplace_back(remap(t.first), t.second);
    c->indices.push_back(n);
  }
  for (auto &k : op->body) c->pushBack(cloneRec(k.get(), m));
  return c;
}

std::unique_ptr<Op> clone(const Op *op, std::map<ValueImpl *, ValueImpl *> *mapping) {
  std::map<ValueImpl *, ValueImpl *> local;
  return cloneRec(op, mapping ? *mapping : local);
}

// ------------------------------------------------------------------ printer
namespace {
struct Printer {
  std::ostringstream os;
  std::map<const ValueImpl *, std::string> names;
  int nextResult = 0;
  int nextArg = 0;

  std::string name(Value v) {
    if (!v) return "<<null>>";
    auto it = names.find(v.get());
    if (it != names.end()) return it->second;
    return "%?";  // defined outside the printed subtree
  }
  void defResult(const Op *op) {
    for (auto &r : op->results) names[r.get()] = "%" + std::to_string(nextResult++);
  }
  void defArgs(const Op *op) {
    for (auto &a : op->args) names[a.get()] = "%arg" + std::to_string(nextArg++);
  }
  // `(inner) floordiv c` / `(inner) mod c` for a value defined by such an apply, else its name
  std::string atom(Value v, bool &compound) {
    compound = false;
    const Op *def = v.getDefiningOp();
    if (def && def->kind == OpKind::Apply && def->divisor > 0) {
      const LinExpr &in = def->indices[0];
      const bool simple = in.terms.size() == 1 && in.terms[0].second == 1 && in.constant == 0;
      bool innerCompound = false;
      std::string inner = simple ? atom(in.terms[0].first, innerCompound) : expr(in);
      if (!simple || innerCompound) inner = "(" + inner + ")";
      compound = true;
      return inner + (def->isMod ? " mod " : " floordiv ") + std::to_string(def->divisor);
    }
    return name(v);
  }
  std::string expr(const LinExpr &e) {
    std::ostringstream s;
    bool first = true;
    for (auto &t : e.terms) {
      if (!first) s << " + ";
      first = false;
      bool compound = false;
      const std::string a = atom(t.first, compound);
      if (t.second != 1) s << (compound ? "(" + a + ")" : a) << " * " << t.second;
      else s << a;
    }
    if (e.constant != 0 || first) {
      if (!first) s << " + ";
      s << e.constant;
    }
    return s.str();
  }
  std::string subscripts(const Op *op) {
    std::string s = "[";
    for (size_t i = 0; i < op->indices.size(); ++i) s += (i ? ", " : "") + expr(op->indices[i]);
    return s + "]";
  }
  void indent(int n) { os << std::string(2 * n, ' '); }
  void region(const Op *op, int depth) {
    for (auto &k : op->body) emit(k.get(), depth);
  }
  void emit(const Op *op, int d) {
    switch (op->kind) {
      case OpKind::Module:
        indent(d);
        os << "module @" << op->name << " {\n";
        // functions first number their own values independently, like MLIR
        region(op, d + 1);
        indent(d);
        os << "}\n";
        break;
      case OpKind::Func: {
        const int savedR = nextResult, savedA = nextArg;
        nextResult = 0;
        nextArg = 0;
        defArgs(op);
        indent(d);
        os << "func.func @" << op->name << "(";
        for (size_t i = 0; i < op->args.size(); ++i)
          os << (i ? ", " : "") << names[op->args[i].get()] << ": " << op->args[i]->memref.str();
        os << ")";
        if (!op->resultTypes.empty()) {
          os << " -> ";
          for (size_t i = 0; i < op->resultTypes.size(); ++i) os << (i ? ", " : "") << op->resultTypes[i].str();
        }
        if (!op->attrs.empty()) {
          os << " attributes {";
          bool f = true;
          for (auto &a : op->attrs) {
            os << (f ? "" : ", ") << a.first << " = \"" << a.second << "\"";
            f = false;
          }
          os << "}";
        }
        os << " {\n";
        region(op, d + 1);
        indent(d);
        os << "}\n";
        nextResult = savedR;
        nextArg = savedA;
        break;
      }
      case OpKind::Alloc:
        defResult(op);
        indent(d);
        os << name(op->result()) << " = memref.alloc() : " << op->results[0]->memref.str() << "\n";
        break;
      case OpKind::Call:
        defResult(op);
        indent(d);
        if (!op->results.empty()) os << name(op->result()) << " = ";
        os << "func.call @" << op->name << "(";
        for (size_t i = 0; i < op->operands.size(); ++i) os << (i ? ", " : "") << name(op->operands[i]);
        os << ")\n";
        break;
      case OpKind::Return:
        indent(d);
        os << "func.return";
        for (size_t i = 0; i < op->operands.size(); ++i) os << (i ? ", " : " ") << name(op->operands[i]);
        os << "\n";
        break;
      case OpKind::For: {
        defResult(op);
        defArgs(op);
        indent(d);
        if (!op->results.empty()) os << name(op->result()) << " = ";
        os << "affine.for " << names[op->args[0].get()] << " = " << op->lb << " to " << op->ub;
        if (op->step != 1) os << " step " << op->step;
        if (op->args.size() > 1) {
          os << " iter_args(";
          for (size_t i = 1; i < op->args.size(); ++i)
            os << (i > 1 ? ", " : "") << names[op->args[i].get()] << " = " << name(op->operands[i - 1]);
          os << ") -> (" << dtypeName(op->args[1]->dtype) << ")";
        }
        os << " {\n";
        region(op, d + 1);
        indent(d);
        os << "}";
        if (!op->attrs.empty()) {
          os << " {";
          bool f = true;
          for (auto &a : op->attrs) {
            os << (f ? "" : ", ") << a.first << " = \"" << a.second << "\"";
            f = false;
          }
          os << "}";
        }
        os << "\n";
        break;
      }
      case OpKind::Parallel: {
        defArgs(op);
        indent(d);
        os << "affine.parallel (";
        for (size_t i = 0; i < op->args.size(); ++i) os << (i ? ", " : "") << names[op->args[i].get()];
        os << ") = (";
        for (size_t i = 0; i < op->ubs.size(); ++i) os << (i ? ", " : "") << 0;
        os << ") to (";
        for (size_t i = 0; i < op->ubs.size(); ++i) os << (i ? ", " : "") << op->ubs[i];
        os << ") {\n";
        region(op, d + 1);
        indent(d);
        os << "}\n";
        break;
      }
      case OpKind::Apply: {
        defResult(op);
        if (op->divisor > 0) break;  // folded into the expressions that use it
        indent(d);
        // affine_map<(d0) -> (d0 * 128)>(%arg0)
        const LinExpr &e = op->indices[0];
        os << name(op->result()) << " = affine.apply affine_map<(";
        for (size_t i = 0; i < e.terms.size(); ++i) os << (i ? ", " : "") << "d" << i;
        os << ") -> (";
        for (size_t i = 0; i < e.terms.size(); ++i) {
          os << (i ? " + " : "") << "d" << i;
          if (e.terms[i].second != 1) os << " * " << e.terms[i].second;
        }
        if (e.constant != 0 || e.terms.empty()) os << (e.terms.empty() ? "" : " + ") << e.constant;
        os << ")>(";
        for (size_t i = 0; i < e.terms.size(); ++i) os << (i ? ", " : "") << name(e.terms[i].first);
        os << ")\n";
        break;
      }
      case OpKind::Load:
        defResult(op);
        indent(d);
        os << name(op->result()) << (op->vec ? " = affine.vector_load " : " = affine.load ") << name(op->memref)
           << subscripts(op) << " : " << op->memref.getMemRefType().str();
        if (op->vec) os << ", vector<" << op->vec << "x" << dtypeName(op->memref.getMemRefType().elem) << ">";
        os << "\n";
        break;
      case OpKind::Store:
        indent(d);
        os << (op->vec ? "affine.vector_store " : "affine.store ") << name(op->operands[0]) << ", "
           << name(op->memref) << subscripts(op) << " : " << op->memref.getMemRefType().str();
        if (op->vec) os << ", vector<" << op->vec << "x" << dtypeName(op->memref.getMemRefType().elem) << ">";
        os << "\n";
        break;
      case OpKind::Constant: {
        defResult(op);
        indent(d);
        char buf[64];
        snprintf(buf, sizeof buf, "%.6e", op->fvalue);
        os << name(op->result()) << " = arith.constant " << buf << " : " << dtypeName(op->results[0]->dtype)
           << "\n";
        break;
      }
      case OpKind::MulF:
      case OpKind::AddF:
      case OpKind::MaxF:
      case OpKind::DivF:
        defResult(op);
        indent(d);
        os << name(op->result()) << " = " << opName(op->kind) << " " << name(op->operands[0]) << ", "
           << name(op->operands[1]) << " : " << dtypeName(op->results[0]->dtype) << "\n";
        break;
      case OpKind::Exp:
        defResult(op);
        indent(d);
        os << name(op->result()) << " = math.exp " << name(op->operands[0]) << " : "
           << dtypeName(op->results[0]->dtype) << "\n";
        break;
      case OpKind::Yield:
        if (op->operands.empty()) break;  // implicit terminator, as MLIR elides it
        indent(d);
        os << "affine.yield";
        for (size_t i = 0; i < op->operands.size(); ++i) os << (i ? ", " : " ") << name(op->operands[i]);
        os << " : " << dtypeName(op->operands[0].getDType()) << "\n";
        break;
      case OpKind::Barrier:
        indent(d);
        os << "gpu.barrier\n";
        break;
      case OpKind::If: {
        // affine.if affine_set<(d0) : (-d0 + 1008 >= 0)>(%arg4) {
        std::vector<Value> dims;
        for (auto &e : op->indices)
          for (auto &t : e.terms) {
            bool seen = false;
            for (auto &v : dims) seen = seen || v == t.first;
            if (!seen) dims.push_back(t.first);
          }
        indent(d);
        os << "affine.if affine_set<(";
        for (size_t i = 0; i < dims.size(); ++i) os << (i ? ", " : "") << "d" << i;
        os << ") : (";
        for (size_t c = 0; c < op->indices.size(); ++c) {
          const LinExpr &e = op->indices[c];
          if (c) os << ", ";
          bool first = true;
          for (auto &t : e.terms) {
            size_t di = 0;
            while (!(dims[di] == t.first)) ++di;
            if (t.second == -1) os << (first ? "-" : " - ") << "d" << di;
            else if (t.second == 1) os << (first ? "" : " + ") << "d" << di;
            else os << (first ? "" : " + ") << "d" << di << " * " << t.second;
            first = false;
          }
          if (e.constant != 0 || first) os << (first ? "" : " + ") << e.constant;
          os << " >= 0";
        }
        os << ")>(";
        for (size_t i = 0; i < dims.size(); ++i) os << (i ? ", " : "") << atomName(dims[i]);
        os << ") {\n";
        region(op, d + 1);
        indent(d);
        os << "}\n";
        break;
      }
    }
  }
  std::string atomName(Value v) {
    bool c = false;
    return atom(v, c);
  }
};
}  // namespace

std::string print(const Op *op) {
  Printer p;
  p.emit(op, 0);
  return p.os.str();
}

void ModuleOp::dump() const { std::cerr << str(); }

// ----------------------------------------------------------------- verifier
namespace {
struct Verifier {
  std::set<const ValueImpl *> visible;
  std::string error;

  void fail(const Op *op, const std::string &what) {
    if (error.empty()) error = std::string(opName(op->kind)) + ": " + what;
  }
  void use(const Op *op, Value v) {
    if (!v) return fail(op, "null operand");
    if (!visible.count(v.get())) fail(op, "operand is not defined in an enclosing scope before its use");
  }
  void check(const Op *op) {
    for (auto &v : op->operands) use(op, v);
    if (op->kind == OpKind::Load || op->kind == OpKind::Store) {
      use(op, op->memref);
      if (op->memref && !op->memref.isMemRef()) fail(op, "target is not a memref");
      if (op->memref && op->memref.isMemRef() &&
          op->indices.size() != op->memref.getMemRefType().shape.size())
        fail(op, "subscript count does not match the memref rank");
    }
    for (auto &e : op->indices)
      for (auto &t : e.terms) {
        use(op, t.first);
        if (t.first && t.first.getDType() != DType::index) fail(op, "non-index value in an index expression");
      }
    if (op->kind == OpKind::Apply && op->divisor < 0) fail(op, "negative divisor");
    if ((op->kind == OpKind::Load || op->kind == OpKind::Store) && op->vec < 0) fail(op, "negative vector width");
    if (op->kind == OpKind::Store && op->vec > 0 && op->operands[0] && op->operands[0].get()->lanes != op->vec)
      fail(op, "vector store of a value with another width");
    if (op->kind == OpKind::For) {
      if (op->step <= 0) fail(op, "non-positive step");
      if (op->ub < op->lb) fail(op, "upper bound below lower bound");
      if (op->body.empty() || op->body.back()->kind != OpKind::Yield) fail(op, "missing affine.yield");
      else if (op->body.back()->operands.size() != op->results.size()) fail(op, "yield arity");
    }
    if (op->kind == OpKind::Parallel)
      for (auto u : op->ubs)
        if (u <= 0) fail(op, "non-positive parallel extent");
    if (op->kind == OpKind::Func && (op->body.empty() || op->body.back()->kind != OpKind::Return))
      fail(op, "missing func.return");
    for (auto &k : op->body)
      if (k->parent != op) fail(k.get(), "parent link is stale");
    // scope: args are visible inside the region; results after the op
    std::vector<const ValueImpl *> added;
    for (auto &a : op->args) {
      visible.insert(a.get());
      added.push_back(a.get());
    }
    std::vector<const ValueImpl *> inner;
    for (auto &k : op->body) {
      check(k.get());
      for (auto &r : k->results) {
        visible.insert(r.get());
        inner.push_back(r.get());
      }
    }
    // values of a function or loop body do not escape; module-level ones stay visible
    if (op->kind != OpKind::Module) {
      for (auto v : inner) visible.erase(v);
      for (auto v : added) visible.erase(v);
    }
  }
};
}  // namespace

std::string verify(const Op *op) {
  Verifier v;
  // values defined outside the verified subtree (when verifying a nest) are taken as visible
  for (const Op *p = op->parent; p; p = p->parent) {
    for (auto &a : p->args) v.visible.insert(a.get());
    for (auto &k : p->body)
      for (auto &r : k->results) v.visible.insert(r.get());
  }
  v.check(op);
  return v.error;
}

std::vector<Value> ParallelOp::getIVs() const {
  std::vector<Value> r;
  for (auto &a : op->args) r.emplace_back(a.get());
  return r;
}

std::vector<Value> FuncOp::getArguments() const {
  std::vector<Value> r;
  for (auto &a : op->args) r.emplace_back(a.get());
  return r;
}

std::string FuncOp::getAttr(const std::string &key) const {
  auto it = op->attrs.find(key);
  return it == op->attrs.end() ? std::string() : it->second;
}

}  // namespace ir
}  // namespace KernelCodeGen
