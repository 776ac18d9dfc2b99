#include "Optimizer/Rewriter.h"

#include <algorithm>
#include <iostream>
#include <map>
#include <set>

namespace KernelCodeGen {

using namespace ir;

namespace {

// Appends `op` to a region owner: before the terminator of a loop, at the end otherwise.
Op *append(Op *where, std::unique_ptr<Op> op) {
  Op *last = where->lastOp();
  if (last && (last->kind == OpKind::Yield || last->kind == OpKind::Return)) return last->insertBefore(std::move(op));
  return where->pushBack(std::move(op));
}

// Closest enclosing op whose body is a buffer scope: parallel level, function or module.
Op *closestScope(Op *op) {
  for (Op *p = op->parent; p; p = p->parent)
    if (p->kind == OpKind::Parallel || p->kind == OpKind::Func || p->kind == OpKind::Module) return p;
  return nullptr;
}

// Values (results and block arguments) defined by `op` or anything nested in it.
void definedValues(Op *op, std::set<const ValueImpl *> &out) {
  walk(op, [&](Op *o) {
    for (auto &r : o->results) out.insert(r.get());
    for (auto &a : o->args) out.insert(a.get());
  });
}

bool usesAny(Op *op, const std::set<const ValueImpl *> &vals) {
  bool hit = false;
  walk(op, [&](Op *o) {
    for (auto &v : o->operands) hit = hit || vals.count(v.get());
    if (o->memref) hit = hit || vals.count(o->memref.get());
    for (auto &e : o->indices)
      for (auto &t : e.terms) hit = hit || vals.count(t.first.get());
  });
  return hit;
}

// New loop with the bounds of `like`, holding `ops` (moved), whose uses of
// like's induction variable are redirected to the new loop's.
std::unique_ptr<Op> fissionCopy(Op *like, std::vector<std::unique_ptr<Op>> ops) {
  auto copy = makeFor(like->lb, like->ub, like->step);
  copy->attrs = like->attrs;
  for (auto &o : ops) copy->pushBack(std::move(o));
  copy->pushBack(makeYield());
  replaceAllUsesWith(copy.get(), like->arg(0), copy->arg(0));
  return copy;
}

// Exchanges `outer` with its direct child loop `inner`.  Returns false (IR
// untouched) when the statements around `inner` cannot be split off.
bool swapLoops(Op *outer, Op *inner) {
  if (outer->args.size() != 1 || inner->args.size() != 1) {
    std::cerr << "reorder: a loop that carries a value cannot be exchanged; bufferize it first\n";
    return false;
  }
  std::vector<Op *> pre, post;
  bool seen = false;
  for (auto &k : outer->body) {
    if (k.get() == inner) {
      seen = true;
      continue;
    }
    if (k->kind == OpKind::Yield) continue;
    (seen ? post : pre).push_back(k.get());
  }
  // fission is only legal if no value flows from the statements before the
  // inner loop into it or past it, nor from the inner loop into those after it
  std::set<const ValueImpl *> preDefs, innerDefs;
  for (Op *p : pre) definedValues(p, preDefs);
  definedValues(inner, innerDefs);
  bool illegal = usesAny(inner, preDefs);
  for (Op *p : post) illegal = illegal || usesAny(p, preDefs) || usesAny(p, innerDefs);
  if (illegal) {
    std::cerr << "reorder: a value crosses the loop being exchanged; bufferize it first\n";
    return false;
  }
  if (!pre.empty()) {
    std::vector<std::unique_ptr<Op>> moved;
    for (Op *p : pre) moved.push_back(p->unlink());
    outer->insertBefore(fissionCopy(outer, std::move(moved)));
  }
  if (!post.empty()) {
    std::vector<std::unique_ptr<Op>> moved;
    for (Op *p : post) moved.push_back(p->unlink());
    outer->insertAfter(fissionCopy(outer, std::move(moved)));
  }
  // outer = [inner, yield]  ->  inner { outer { old inner body } }
  std::unique_ptr<Op> innerOwned = inner->unlink();
  outer->body.clear();  // drops outer's terminator
  for (auto &k : innerOwned->body) k->parent = outer;
  outer->body.splice(outer->body.end(), innerOwned->body);  // includes inner's terminator
  Op *innerRaw = outer->insertBefore(std::move(innerOwned));
  innerRaw->pushBack(outer->unlink());
  innerRaw->pushBack(makeYield());
  return true;
}

}  // namespace

std::vector<ForOp> Rewriter::split(ForOp forOp, uint64_t num_output, std::vector<int64_t> &&factors) {
  Op *loop = forOp.op;
  if (!loop || loop->kind != OpKind::For) return {};
  if (factors.size() + 1 != num_output) {
    std::cerr << "split: " << num_output << " loops need " << num_output - 1 << " tile extents\n";
    return {};
  }
  if (loop->lb != 0 || loop->step != 1 || loop->args.size() != 1) {
    std::cerr << "split: the loop must start at 0 with step 1 and carry no value\n";
    return {};
  }
  // extents outermost first: ub, factors reversed; steps: factors reversed, 1
  std::vector<int64_t> ubs{loop->ub}, steps;
  for (auto it = factors.rbegin(); it != factors.rend(); ++it) {
    ubs.push_back(*it);
    steps.push_back(*it);
  }
  steps.push_back(1);
  for (size_t i = 0; i < steps.size(); ++i)
    if (steps[i] <= 0 || ubs[i] % steps[i] != 0) {
      std::cerr << "split: extent " << ubs[i] << " is not a multiple of tile " << steps[i] << "\n";
      return {};
    }
  std::vector<ForOp> loops;
  Op *outerNew = loop->insertBefore(makeFor(0, ubs[0], steps[0]));
  loops.emplace_back(outerNew);
  Op *cur = outerNew;
  for (size_t i = 1; i < ubs.size(); ++i) {
    cur = cur->pushBack(makeFor(0, ubs[i], steps[i]));
    loops.emplace_back(cur);
  }
  // the old body (terminator included) becomes the innermost body
  for (auto &k : loop->body) k->parent = cur;
  cur->body.splice(cur->body.end(), loop->body);
  for (size_t i = 0; i + 1 < loops.size(); ++i) loops[i]->pushBack(makeYield());
  LinExpr sum;
  for (auto &l : loops) sum.add(l.getInductionVar());
  replaceIndexUses(outerNew, loop->arg(0), sum);
  loop->erase();
  return loops;
}

Value Rewriter::bufferizeLoopCarryVar(std::vector<ForOp> &loops) {
  Op *carry = nullptr;
  for (auto &l : loops)
    if (l.numIterArgs() != 0) {
      if (carry) {
        std::cerr << "Can't reorder more than one loops carrying args\n";
        return Value();
      }
      carry = l.op;
    }
  if (!carry) return Value();
  if (carry->args.size() != 2) {
    std::cerr << "bufferizeLoopCarryVar: exactly one carried value is supported\n";
    return Value();
  }
  std::vector<int64_t> shape;
  std::vector<LinExpr> address;
  for (auto &l : loops)
    if (l.op != carry && l->isAncestorOf(carry)) {
      shape.push_back(l.tripCount());
      address.emplace_back(l.getInductionVar());
    }
  Value init = carry->operands[0];
  Op *initDef = init.getDefiningOp();
  Op *scope = closestScope(loops[0].op);
  if (!initDef || !scope) {
    std::cerr << "bufferizeLoopCarryVar: the initial value must be defined by an op inside a scope\n";
    return Value();
  }
  const DType dtype = carry->args[1]->dtype;
  if (shape.empty()) shape.push_back(1), address.emplace_back(int64_t(0));
  Value buffer = scope->pushFront(makeAlloc(MemRefType{shape, dtype, static_cast<int>(MemorySpace::local)}))->result();

  // 1. initialise the buffer right after the initial value is defined
  initDef->insertAfter(makeStore(init, buffer, address));
  // 2. the carried value becomes load-at-top / store-at-bottom
  Value carried = carry->arg(1);
  Op *yield = carry->lastOp();
  Value yielded = yield->operands[0];
  Value loaded = carry->pushFront(makeLoad(buffer, address))->result();
  replaceAllUsesWith(carry, carried, loaded);
  if (yielded == carried) yielded = loaded;
  yield->insertBefore(makeStore(yielded, buffer, address));
  yield->operands.clear();
  // 3. users of the loop result read the buffer after the loop
  Value oldResult = carry->result(0);
  Value after = carry->insertAfter(makeLoad(buffer, address))->result();
  replaceAllUsesWith(scope, oldResult, after);
  carry->operands.clear();
  carry->args.pop_back();
  carry->results.clear();
  return buffer;
}

void Rewriter::reorder(const std::vector<ForOp> &loops) {
  if (loops.size() < 2) return;
  std::map<Op *, int> priority;  // larger = further out
  int p = static_cast<int>(loops.size());
  for (auto &l : loops) priority[l.op] = p--;
  bool swapped = true;
  int guard = 0;
  while (swapped && guard++ < 10000) {
    swapped = false;
    for (auto &l : loops) {
      Op *parent = l.op;
      // direct child loop of `parent` that is also listed
      Op *child = nullptr;
      for (auto &k : parent->body)
        if (k->kind == OpKind::For && priority.count(k.get())) {
          child = k.get();
          break;
        }
      if (child && priority[parent] < priority[child]) {
        if (!swapLoops(parent, child)) return;
        swapped = true;
        break;
      }
    }
  }
}

ParallelOp Rewriter::parallel(const std::vector<ForOp> &forOps) {
  if (forOps.empty() || forOps.size() > 3) {
    std::cerr << "parallel: one to three loops (X, Y, Z) can form a level\n";
    return ParallelOp();
  }
  for (size_t i = 0; i < forOps.size(); ++i) {
    Op *l = forOps[i].op;
    if (l->args.size() != 1) {
      std::cerr << "parallel: a loop that carries a value cannot become a parallel dimension\n";
      return ParallelOp();
    }
    if (i + 1 < forOps.size()) {
      // perfect nest: the next loop is the only statement
      bool perfect = l->body.size() == 2 && l->body.front().get() == forOps[i + 1].op;
      if (!perfect) {
        std::cerr << "parallel: the loops must be perfectly nested\n";
        return ParallelOp();
      }
    }
  }
  std::vector<int64_t> extents;
  for (auto &l : forOps) extents.push_back(l.tripCount());
  Op *outer = forOps.front().op;
  Op *inner = forOps.back().op;
  Op *par = outer->insertBefore(makeParallel(extents));
  // move the innermost body (without its terminator)
  inner->body.pop_back();
  for (auto &k : inner->body) k->parent = par;
  par->body.splice(par->body.end(), inner->body);
  // normalise: iv = lb + step * new_iv
  Op *firstStmt = par->body.empty() ? nullptr : par->body.front().get();
  for (size_t d = 0; d < forOps.size(); ++d) {
    Op *l = forOps[d].op;
    Value oldIv = l->arg(0), newIv = par->arg(static_cast<int>(d));
    if (l->lb == 0 && l->step == 1) {
      replaceAllUsesWith(par, oldIv, newIv);
    } else {
      LinExpr e;
      e.add(newIv, l->step);
      e.constant = l->lb;
      auto apply = makeApply(e);
      Op *a = firstStmt ? firstStmt->insertBefore(std::move(apply)) : par->pushBack(std::move(apply));
      replaceAllUsesWith(par, oldIv, a->result());
      // the apply itself must keep reading the new induction variable
      a->indices[0] = e;
    }
  }
  outer->erase();  // the emptied loop shells
  return ParallelOp(par);
}

Value Rewriter::alloc_buffer(OpHandle father, MemorySpace ms, const std::vector<int64_t> &shape, DType dtype) {
  return father->pushFront(makeAlloc(MemRefType{shape, dtype, static_cast<int>(ms)}))->result();
}

Value Rewriter::alloc_buffer(OpHandle contextOp, Position pos, MemorySpace ms, const std::vector<int64_t> &shape,
                             DType dtype) {
  auto alloc = makeAlloc(MemRefType{shape, dtype, static_cast<int>(ms)});
  if (pos == Position::before) return contextOp->insertBefore(std::move(alloc))->result();
  if (pos == Position::after) return contextOp->insertAfter(std::move(alloc))->result();
  std::cerr << "alloc_buffer: only Position::before / after are meaningful here\n";
  return Value();
}

Op *Rewriter::barrier(ForOp compute_at, Position pos) {
  switch (pos) {
    case Position::before: return compute_at->insertBefore(makeBarrier());
    case Position::after: return compute_at->insertAfter(makeBarrier());
    case Position::begin: return compute_at->pushFront(makeBarrier());
    case Position::end: return append(compute_at.op, makeBarrier());
  }
  return nullptr;
}

ForOp Rewriter::create_constant_loop(OpHandle where, int64_t lowerBound, int64_t upperBound, int64_t step) {
  Op *loop = append(where.op, makeFor(lowerBound, upperBound, step));
  loop->pushBack(makeYield());
  return ForOp(loop);
}

void Rewriter::set_buffer(OpHandle where, Value mem, Value targetValue) {
  Op *cur = where.op;
  std::vector<LinExpr> idx;
  for (auto extent : mem.getMemRefType().shape) {
    ForOp l = create_constant_loop(OpHandle(cur), 0, extent, 1);
    idx.emplace_back(l.getInductionVar());
    cur = l.op;
  }
  append(cur, makeStore(targetValue, mem, idx));
}

ForOp Rewriter::outer_product(OpHandle where, Value tileC, Value fragA, Value fragB, int64_t m, int64_t n) {
  ForOp li = create_constant_loop(where, 0, m, 1);
  ForOp lj = create_constant_loop(OpHandle(li.op), 0, n, 1);
  Value i = li.getInductionVar(), j = lj.getInductionVar();
  Value c = append(lj.op, makeLoad(tileC, {LinExpr(i), LinExpr(j)}))->result();
  Value a = append(lj.op, makeLoad(fragA, {LinExpr(i)}))->result();
  Value b = append(lj.op, makeLoad(fragB, {LinExpr(j)}))->result();
  Value mul = append(lj.op, makeBinary(OpKind::MulF, a, b))->result();
  Value add = append(lj.op, makeBinary(OpKind::AddF, mul, c))->result();
  append(lj.op, makeStore(add, tileC, {LinExpr(i), LinExpr(j)}));
  return li;
}

void Rewriter::unrollAttribute(ModuleOp module, int64_t maxTrips) {
  walk(module.get(), [&](Op *op) {
    if (op->kind == OpKind::For && ForOp(op).tripCount() <= maxTrips) op->attrs["affine.loop"] = "unroll";
  });
}

}  // namespace KernelCodeGen
