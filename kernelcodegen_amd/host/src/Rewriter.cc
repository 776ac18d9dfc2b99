#include "Optimizer/Rewriter.h"

#include <functional>
#include <map>

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

// ------------------------------------------------------------- staging
namespace {

Op *placeLoop(ForOp compute_at, Position pos, std::unique_ptr<Op> loop) {
  switch (pos) {
    case Position::before: return compute_at->insertBefore(std::move(loop));
    case Position::after: return compute_at->insertAfter(std::move(loop));
    case Position::begin: return compute_at->pushFront(std::move(loop));
    case Position::end: return append(compute_at.op, std::move(loop));
  }
  return nullptr;
}

// body of a read loop: vector load src[map(operands, iv)], vector store dst[iv * width]
void fillRead(Op *loop, Value src, Value dst, const AffineMap &map, std::vector<Value> operands, int64_t width) {
  loop->pushBack(makeYield());
  Op *yield = loop->lastOp();
  operands.push_back(loop->arg(0));
  Op *ld = yield->insertBefore(makeVectorLoad(src, {}, static_cast<int>(width)));
  ld->indices = materialize(map, operands, ld);
  LinExpr di;
  di.add(loop->arg(0), width);
  yield->insertBefore(makeVectorStore(ld->result(), dst, {di}, static_cast<int>(width)));
}

void fillWrite(Op *loop, Value src, Value dst, const AffineMap &map, std::vector<Value> operands, int64_t width) {
  loop->pushBack(makeYield());
  Op *yield = loop->lastOp();
  const bool scatter = map.numDims - static_cast<int>(operands.size()) == 2;
  operands.push_back(loop->arg(0));
  if (!scatter) {
    LinExpr si;
    si.add(loop->arg(0), width);
    Op *ld = yield->insertBefore(makeVectorLoad(src, {si}, static_cast<int>(width)));
    Op *st = yield->insertBefore(makeVectorStore(ld->result(), dst, {}, static_cast<int>(width)));
    st->indices = materialize(map, operands, st);
    return;
  }
  Op *inner = yield->insertBefore(makeFor(0, width, 1));
  inner->pushBack(makeYield());
  Op *iy = inner->lastOp();
  operands.push_back(inner->arg(0));
  LinExpr si;
  si.add(loop->arg(0), width);
  si.add(inner->arg(0), 1);
  Op *ld = iy->insertBefore(makeVectorLoad(src, {si}, 1));
  Op *st = iy->insertBefore(makeVectorStore(ld->result(), dst, {}, 1));
  st->indices = materialize(map, operands, st);
}

bool registerBuffer(Value v, const char *who) {
  if (v && v.isMemRef() && v.getMemRefType().shape.size() == 1) return true;
  std::cerr << who << ": the register-side buffer must be a one-dimensional memref\n";
  return false;
}

}  // namespace

ForOp Rewriter::read(Value src, Value dst, const AffineMap &map, std::vector<Value> operands, int64_t width,
                     ForOp compute_at, Position pos) {
  if (!registerBuffer(dst, "read") || width <= 0 || dst.getMemRefType().shape[0] % width != 0) return ForOp();
  Op *loop = placeLoop(compute_at, pos, makeFor(0, dst.getMemRefType().shape[0] / width, 1));
  fillRead(loop, src, dst, map, std::move(operands), width);
  return ForOp(loop);
}

ForOp Rewriter::read(OpHandle where, Value src, Value dst, const AffineMap &map, std::vector<Value> operands,
                     int64_t width) {
  if (!registerBuffer(dst, "read") || width <= 0 || dst.getMemRefType().shape[0] % width != 0) return ForOp();
  Op *loop = append(where.op, makeFor(0, dst.getMemRefType().shape[0] / width, 1));
  fillRead(loop, src, dst, map, std::move(operands), width);
  return ForOp(loop);
}

ForOp Rewriter::write(Value src, Value dst, const AffineMap &map, std::vector<Value> operands, int64_t width,
                      ForOp compute_at, Position pos) {
  if (!registerBuffer(src, "write") || width <= 0 || src.getMemRefType().shape[0] % width != 0) return ForOp();
  Op *loop = placeLoop(compute_at, pos, makeFor(0, src.getMemRefType().shape[0] / width, 1));
  fillWrite(loop, src, dst, map, std::move(operands), width);
  return ForOp(loop);
}

ForOp Rewriter::write(OpHandle where, Value src, Value dst, const AffineMap &map, std::vector<Value> operands,
                      int64_t width) {
  if (!registerBuffer(src, "write") || width <= 0 || src.getMemRefType().shape[0] % width != 0) return ForOp();
  Op *loop = append(where.op, makeFor(0, src.getMemRefType().shape[0] / width, 1));
  fillWrite(loop, src, dst, map, std::move(operands), width);
  return ForOp(loop);
}

ForOp Rewriter::copy(Value src, const AffineMap &srcMap, std::vector<Value> srcOperands, Value dst,
                     const AffineMap &dstMap, std::vector<Value> dstOperands, int64_t count, int64_t width,
                     ForOp compute_at, Position pos) {
  if (!src || !dst || width <= 0 || count <= 0 || count % width != 0) {
    std::cerr << "copy: needs two memrefs and a count that is a multiple of the width\n";
    return ForOp();
  }
  Op *loop = placeLoop(compute_at, pos, makeFor(0, count / width, 1));
  loop->pushBack(makeYield());
  Op *yield = loop->lastOp();
  const bool scatter = dstMap.numDims - static_cast<int>(dstOperands.size()) == 2;
  srcOperands.push_back(loop->arg(0));
  dstOperands.push_back(loop->arg(0));
  if (!scatter) {
    Op *ld = yield->insertBefore(makeVectorLoad(src, {}, static_cast<int>(width)));
    ld->indices = materialize(srcMap, srcOperands, ld);
    Op *st = yield->insertBefore(makeVectorStore(ld->result(), dst, {}, static_cast<int>(width)));
    st->indices = materialize(dstMap, dstOperands, st);
    return ForOp(loop);
  }
  // element j of the vector: the source's last subscript + j
  Op *inner = yield->insertBefore(makeFor(0, width, 1));
  inner->pushBack(makeYield());
  Op *iy = inner->lastOp();
  dstOperands.push_back(inner->arg(0));
  Op *ld = iy->insertBefore(makeVectorLoad(src, {}, 1));
  ld->indices = materialize(srcMap, srcOperands, ld);
  ld->indices.back().add(inner->arg(0), 1);
  Op *st = iy->insertBefore(makeVectorStore(ld->result(), dst, {}, 1));
  st->indices = materialize(dstMap, dstOperands, st);
  return ForOp(loop);
}

void Rewriter::cache_read(ForOp scope, Value src, Value cached, const AffineMap &map,
                          const std::vector<Value> &operands) {
  std::vector<Op *> loads;
  walk(scope.op, [&](Op *op) {
    if (op->kind == OpKind::Load && op->vec == 0 && op->memref == src) loads.push_back(op);
  });
  for (Op *ld : loads) {
    ld->memref = cached;
    ld->indices = materialize(map, operands, ld);
  }
}

void Rewriter::cache_write(ForOp scope, Value src, Value cached, const AffineMap &map,
                           const std::vector<Value> &operands) {
  (void)cached;
  std::vector<Op *> stores;
  walk(scope.op, [&](Op *op) {
    if (op->kind == OpKind::Store && op->vec == 0 && op->memref == src) stores.push_back(op);
  });
  for (Op *st : stores) st->indices = materialize(map, operands, st);
}

std::vector<std::vector<ForOp>> Rewriter::get_write(ParallelOp parallelLevel, Value dst) {
  std::vector<std::vector<ForOp>> results;
  walk(parallelLevel.op, [&](Op *op) {
    if (op->kind != OpKind::Store || op->memref != dst) return;
    std::vector<ForOp> loops;
    for (Op *p = op->parent; p && p != parallelLevel.op && p->kind == OpKind::For; p = p->parent)
      loops.insert(loops.begin(), ForOp(p));
    results.push_back(loops);
  });
  return results;
}

ForOp Rewriter::vectorize(ForOp readOrWrite, int64_t width) {
  Op *l = readOrWrite.op;
  if (!l || l->lb != 0 || l->step != 1 || width <= 0 || l->ub % width != 0) {
    std::cerr << "vectorize: the loop must run from 0 in steps of 1 over a multiple of the width\n";
    return ForOp();
  }
  l->step = width;
  walk(l, [&](Op *op) {
    if (op->kind == OpKind::Load) {
      op->vec = static_cast<int>(width);
      op->results[0]->lanes = static_cast<int>(width);
    } else if (op->kind == OpKind::Store) {
      op->vec = static_cast<int>(width);
    }
  });
  return readOrWrite;
}

// ------------------------------------------------- pipelining
namespace {

// prepends a subscript to every access of `from` under `root` and retargets it to `to`
void retarget(Op *root, Value from, Value to, const std::function<LinExpr(Op *)> &leading) {
  std::vector<Op *> hits;
  walk(root, [&](Op *op) {
    if ((op->kind == OpKind::Load || op->kind == OpKind::Store) && op->memref == from) hits.push_back(op);
  });
  for (Op *op : hits) {
    const LinExpr first = leading(op);
    op->memref = to;
    op->indices.insert(op->indices.begin(), first);
  }
}

// affine.apply ops whose expression has become a constant (after an induction variable was
// fixed) are folded into the expressions that use them
void foldConstantApplies(Op *root) {
  for (bool changed = true; changed;) {
    changed = false;
    std::vector<Op *> constant;
    walk(root, [&](Op *op) {
      if (op->kind == OpKind::Apply && op->indices[0].terms.empty()) constant.push_back(op);
    });
    for (Op *a : constant) {
      int64_t v = a->indices[0].constant;
      if (a->divisor > 0) {
        int64_t q = v / a->divisor, r = v % a->divisor;
        if (r < 0) {
          r += a->divisor;
          q -= 1;
        }
        v = a->isMod ? r : q;
      }
      Op *scope = a->parent;
      replaceIndexUses(scope, a->result(), LinExpr(v));
      a->erase();
      changed = true;
    }
  }
}

// (iv floordiv step + offset) mod copies as an index value computed right before `user`
LinExpr halfSelector(Op *user, Value iv, int64_t step, int64_t offset, int64_t copies = 2) {
  LinExpr q(iv);
  if (step != 1) q = LinExpr(user->insertBefore(makeApplyFloorDiv(LinExpr(iv), step))->result());
  q.constant += offset;
  return LinExpr(user->insertBefore(makeApplyMod(q, copies))->result());
}

}  // namespace

std::vector<std::vector<ForOp>> Rewriter::pipeline(std::vector<ForOp> readBodys, Value &buffer, ForOp compute_at,
                                                   int stages) {
  if (stages == 2) return pipeline(std::move(readBodys), buffer, compute_at);
  std::vector<std::vector<ForOp>> results;
  Op *def = buffer ? buffer.getDefiningOp() : nullptr;
  if (!def || def->kind != OpKind::Alloc || readBodys.empty() || stages < 2) {
    std::cerr << "pipeline: the buffer must come from memref.alloc, there must be a loop that fills it, and a ring "
                 "has at least two copies\n";
    return results;
  }
  for (auto r : readBodys)
    if (!compute_at->isAncestorOf(r.op)) {
      std::cerr << "pipeline: the filling loops must be inside the loop they are pipelined along\n";
      return results;
    }
  Op *loop = compute_at.op;
  Value iv = compute_at.getInductionVar();
  const int64_t step = loop->step, lb = loop->lb, ub = loop->ub;
  if (lb != 0) {
    std::cerr << "pipeline: the ring is indexed by iv floordiv step, the loop must start at 0\n";
    return results;
  }
  // 1. the ring
  MemRefType t = buffer.getMemRefType();
  t.shape.insert(t.shape.begin(), stages);
  Value ring = def->insertBefore(makeAlloc(t))->result();
  // 2. prologue: the copies of iterations 0 .. stages - 2, as far as the loop has them
  std::vector<ForOp> prologue;
  for (int s = 0; s + 1 < stages && lb + s * step < ub; ++s)
    for (auto r : readBodys) {
      Op *cp = loop->insertBefore(clone(r.op));
      replaceIndexUses(cp, iv, LinExpr(lb + s * step));
      retarget(cp, buffer, ring, [s](Op *) { return LinExpr(static_cast<int64_t>(s)); });
      foldConstantApplies(cp);
      prologue.emplace_back(cp);
    }
  results.push_back(prologue);
  results.push_back(readBodys);
  // 3. in the loop: fetch iteration i + stages - 1 while there is one
  LinExpr guard;  // ub - stages * step - iv >= 0
  guard.add(iv, -1);
  guard.constant = ub - stages * step;
  Op *ifOp = loop->pushFront(makeIf({guard}));
  for (auto r : readBodys) {
    auto owned = r->unlink();
    Op *moved = ifOp->pushBack(std::move(owned));
    LinExpr ahead(iv);
    ahead.constant = (stages - 1) * step;
    replaceIndexUses(moved, iv, ahead);
    retarget(moved, buffer, ring, [&](Op *user) { return halfSelector(user, iv, step, stages - 1, stages); });
  }
  // 4. every remaining access reads the copy of the current iteration
  Op *scope = def->parent;
  retarget(scope, buffer, ring, [&](Op *user) { return halfSelector(user, iv, step, 0, stages); });
  def->erase();
  buffer = ring;
  return results;
}

std::vector<std::vector<ForOp>> Rewriter::pipeline(std::vector<ForOp> readBodys, Value &buffer, ForOp compute_at) {
  std::vector<std::vector<ForOp>> results;
  Op *def = buffer ? buffer.getDefiningOp() : nullptr;
  if (!def || def->kind != OpKind::Alloc || readBodys.empty()) {
    std::cerr << "pipeline: the buffer must come from memref.alloc and there must be a loop that fills it\n";
    return results;
  }
  for (auto r : readBodys)
    if (!compute_at->isAncestorOf(r.op)) {
      std::cerr << "pipeline: the filling loops must be inside the loop they are pipelined along\n";
      return results;
    }
  Op *loop = compute_at.op;
  Value iv = compute_at.getInductionVar();
  const int64_t step = loop->step, lb = loop->lb, ub = loop->ub;

  // 1. the double buffer
  MemRefType t = buffer.getMemRefType();
  t.shape.insert(t.shape.begin(), 2);
  Value twice = def->insertBefore(makeAlloc(t))->result();

  // 2. prologue: copies for the first iteration, into half 0
  std::vector<ForOp> prologue;
  for (auto r : readBodys) {
    Op *copy = loop->insertBefore(clone(r.op));
    replaceIndexUses(copy, iv, LinExpr(lb));
    retarget(copy, buffer, twice, [](Op *) { return LinExpr(int64_t{0}); });
    foldConstantApplies(copy);
    prologue.emplace_back(copy);
  }
  results.push_back(prologue);
  results.push_back(readBodys);

  // 3. in the loop: fetch for the next iteration while there is one
  LinExpr guard;  // ub - 2 * step - iv >= 0
  guard.add(iv, -1);
  guard.constant = ub - 2 * step;
  Op *ifOp = loop->pushFront(makeIf({guard}));
  for (auto r : readBodys) {
    auto owned = r->unlink();
    Op *moved = ifOp->pushBack(std::move(owned));
    LinExpr next(iv);
    next.constant = step;
    replaceIndexUses(moved, iv, next);
    retarget(moved, buffer, twice, [&](Op *user) { return halfSelector(user, iv, step, 1); });
  }

  // 4. every remaining access reads the half of the current iteration
  Op *scope = def->parent;
  retarget(scope, buffer, twice, [&](Op *user) { return halfSelector(user, iv, step, 0); });

  def->erase();
  buffer = twice;
  return results;
}

void Rewriter::change_double_buffer(ForOp forOp, Value buffer) {
  // the leading subscript of an access selects the half: flip it
  walk(forOp.op, [&](Op *op) {
    if ((op->kind != OpKind::Load && op->kind != OpKind::Store) || op->memref != buffer) return;
    LinExpr &sel = op->indices[0];
    if (sel.terms.empty()) {
      sel.constant = 1 - sel.constant;
      return;
    }
    // (x) mod 2 becomes (x + 1) mod 2
    Op *def = sel.terms.size() == 1 && sel.terms[0].second == 1 && sel.constant == 0
                  ? sel.terms[0].first.getDefiningOp()
                  : nullptr;
    if (def && def->kind == OpKind::Apply && def->isMod && def->divisor == 2) {
      LinExpr inner = def->indices[0];
      inner.constant += 1;
      sel = LinExpr(op->insertBefore(makeApplyMod(inner, 2))->result());
      return;
    }
    // any other 0/1 selector s: 1 - s
    LinExpr flipped(int64_t{1});
    flipped.add(sel, -1);
    sel = flipped;
  });
}

void Rewriter::detach_last_loop(ForOp forOp) {
  Op *l = forOp.op;
  if (l->args.size() != 1 || l->ub - l->step < l->lb) {
    std::cerr << "detach_last_loop: needs a loop without iter_args and at least one iteration\n";
    return;
  }
  const int64_t last = l->ub - l->step;
  l->ub = last;
  std::map<ValueImpl *, ValueImpl *> mapping;
  auto copy = clone(l, &mapping);
  Value copyIv = copy->arg(0);
  replaceIndexUses(copy.get(), copyIv, LinExpr(last));
  foldConstantApplies(copy.get());
  copy->body.pop_back();  // the terminator
  Op *after = l;
  while (!copy->body.empty()) {
    std::unique_ptr<Op> k = std::move(copy->body.front());
    copy->body.pop_front();
    after = after->insertAfter(std::move(k));
  }
}

void Rewriter::schedule(Op *srcOp, Op *dstOp, Position pos) {
  switch (pos) {
    case Position::after: srcOp->moveAfter(dstOp); break;
    case Position::before: srcOp->moveBefore(dstOp); break;
    case Position::end:
      if (dstOp->kind == OpKind::For) srcOp->moveBefore(dstOp->lastOp());
      else std::cerr << "schedule: Position::end needs a loop as destination\n";
      break;
    default: std::cerr << "schedule: Position::begin is not supported\n"; break;
  }
}

Op *Rewriter::extract_loop(Op *srcOp, ForOp forOp, int64_t iteration) {
  Op *copy = forOp->insertBefore(clone(srcOp));
  replaceIndexUses(copy, forOp.getInductionVar(), LinExpr(forOp->lb + iteration * forOp->step));
  foldConstantApplies(copy);
  return copy;
}

// ------------------------------------------------------------ clean-up
namespace {

// value range of an index value: loop / parallel induction variables and
// floordiv / mod / linear applies of ranged values
bool rangeOf(Value v, int64_t &lo, int64_t &hi);

bool rangeOf(const LinExpr &e, int64_t &lo, int64_t &hi) {
  lo = hi = e.constant;
  for (auto &t : e.terms) {
    int64_t a, b;
    if (!rangeOf(t.first, a, b)) return false;
    if (t.second >= 0) {
      lo += a * t.second;
      hi += b * t.second;
    } else {
      lo += b * t.second;
      hi += a * t.second;
    }
  }
  return true;
}

int64_t floorDivide(int64_t a, int64_t c) {
  int64_t q = a / c;
  if (a % c != 0 && a < 0) --q;
  return q;
}

bool rangeOf(Value v, int64_t &lo, int64_t &hi) {
  ValueImpl *impl = v.get();
  if (!impl) return false;
  if (impl->kind == ValueImpl::InductionVar) {
    Op *o = impl->owner;
    if (o->kind == OpKind::For) {
      if (o->ub <= o->lb) return false;
      lo = o->lb;
      hi = o->lb + (ForOp(o).tripCount() - 1) * o->step;
      return true;
    }
    if (o->kind == OpKind::Parallel) {
      lo = 0;
      hi = o->ubs[impl->index] - 1;
      return true;
    }
    return false;
  }
  Op *def = v.getDefiningOp();
  if (!def || def->kind != OpKind::Apply) return false;
  int64_t a, b;
  if (!rangeOf(def->indices[0], a, b)) return false;
  if (def->divisor == 0) {
    lo = a;
    hi = b;
  } else if (!def->isMod) {
    lo = floorDivide(a, def->divisor);
    hi = floorDivide(b, def->divisor);
  } else if (floorDivide(a, def->divisor) == floorDivide(b, def->divisor)) {
    lo = a - floorDivide(a, def->divisor) * def->divisor;
    hi = b - floorDivide(b, def->divisor) * def->divisor;
  } else {
    lo = 0;
    hi = def->divisor - 1;
  }
  return true;
}

// +1: every constraint always holds; -1: some constraint never holds; 0: undecided
int decide(Op *ifOp) {
  bool allTrue = true;
  for (auto &c : ifOp->indices) {
    int64_t lo, hi;
    if (!rangeOf(c, lo, hi)) return 0;
    if (hi < 0) return -1;
    if (lo < 0) allTrue = false;
  }
  return allTrue ? 1 : 0;
}

std::vector<Op *> collectIfs(Op *root) {
  std::vector<Op *> ifs;
  walk(root, [&](Op *op) {
    if (op->kind == OpKind::If) ifs.push_back(op);
  }, WalkOrder::PostOrder);
  return ifs;
}

}  // namespace

void Rewriter::take_off_true_if(ModuleOp module) {
  for (Op *ifOp : collectIfs(module.get())) {
    if (decide(ifOp) != 1) continue;
    Op *after = ifOp;
    while (!ifOp->body.empty()) {
      std::unique_ptr<Op> k = std::move(ifOp->body.front());
      ifOp->body.pop_front();
      if (k->kind == OpKind::Yield) continue;
      after = after->insertAfter(std::move(k));
    }
    ifOp->erase();
  }
}

void Rewriter::delete_false_if(ModuleOp module) {
  for (Op *ifOp : collectIfs(module.get()))
    if (decide(ifOp) == -1) ifOp->erase();
}

void Rewriter::unroll(ModuleOp module, const std::function<bool(ForOp)> &unrollCheckFn) {
  std::vector<Op *> loops;
  walk(module.get(), [&](Op *op) {
    if (op->kind == OpKind::For && op->args.size() == 1 && unrollCheckFn(ForOp(op))) loops.push_back(op);
  }, WalkOrder::PostOrder);
  for (Op *l : loops) {
    Op *after = l;
    for (int64_t iv = l->lb; iv < l->ub; iv += l->step) {
      auto copy = clone(l);
      replaceIndexUses(copy.get(), copy->arg(0), LinExpr(iv));
      foldConstantApplies(copy.get());
      copy->body.pop_back();
      while (!copy->body.empty()) {
        std::unique_ptr<Op> k = std::move(copy->body.front());
        copy->body.pop_front();
        after = after->insertAfter(std::move(k));
      }
    }
    l->erase();
  }
}

void Rewriter::unrollAttribute(ModuleOp module, const std::function<bool(ForOp)> &unrollCheckFn) {
  walk(module.get(), [&](Op *op) {
    if (op->kind == OpKind::For && unrollCheckFn(ForOp(op))) op->attrs["affine.loop"] = "unroll";
  });
}

void Rewriter::unrollAttribute(ModuleOp module, int64_t maxTrips) {
  walk(module.get(), [&](Op *op) {
    if (op->kind == OpKind::For && ForOp(op).tripCount() <= maxTrips) op->attrs["affine.loop"] = "unroll";
  });
}

}  // namespace KernelCodeGen
