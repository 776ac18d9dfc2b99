#include "Frontend/Operators.h"

#include <iostream>

namespace KernelCodeGen {

using namespace ir;

Log KCGLog::level = Log::Debug;

DType getDType(const std::string &dtype) {
  if (dtype == "float32") return DType::f32;
  if (dtype == "float64") return DType::f64;
  if (dtype == "float16") return DType::f16;
  if (dtype == "bfloat16") return DType::bf16;
  return DType::none;
}

std::string toStr(DType t) {
  switch (t) {
    case DType::f16: return "float16";
    case DType::bf16: return "bfloat16";
    case DType::f32: return "float32";
    case DType::f64: return "float64";
    default: return "";
  }
}

FuncOp buildFuction(ModuleOp module, const std::string &funcName,
                    const std::vector<MemRefType> &inputsTypes,
                    const std::vector<MemRefType> &outputsTypes) {
  for (auto &k : module->body)
    if (k->kind == OpKind::Func && k->name == funcName) return FuncOp(k.get());
  return FuncOp(module->pushFront(makeFunc(funcName, inputsTypes, outputsTypes)));
}

void ComputeDAG::dump(const std::string &info) {
  const std::string problem = verify(module.get());
  if (KCGLog::level != Log::Release) {
    std::cerr << "-----------------------------------------------------------\n"
              << "           " << info << "\n"
              << "-----------------------------------------------------------\n"
              << module.str();
  }
  if (!problem.empty()) std::cerr << "graph verification error: " << problem << "\n";
}

namespace {

// Nest of `extents.size()` affine.for loops [0, extent) step 1 appended to
// `where`; returns the loops outermost first (body of the innermost is empty
// apart from its terminator).
std::vector<Op *> loopNest(Op *where, const std::vector<int64_t> &extents) {
  std::vector<Op *> loops;
  Op *cur = where;
  for (auto e : extents) {
    Op *loop = cur->pushBack(makeFor(0, e, 1));
    loops.push_back(loop);
    cur = loop;
  }
  for (Op *l : loops) l->pushBack(makeYield());
  return loops;
}

// Appends `op` to the body of `loop`, before its terminator.
Op *emit(Op *loop, std::unique_ptr<Op> op) { return loop->lastOp()->insertBefore(std::move(op)); }

std::string dims(const std::vector<int64_t> &shape, size_t from, size_t to) {
  std::string s;
  for (size_t i = from; i < to; ++i) s += "_" + std::to_string(shape[i]);
  return s;
}

bool isMemRef(Value v, const char *what) {
  if (v && v.isMemRef()) return true;
  std::cerr << what << " is not Memref.\n";
  return false;
}

}  // namespace

Value PlaceHolder::build(ComputeDAG *graph, const std::vector<int64_t> &shapes, const std::string &dtype) {
  const DType t = getDType(dtype);
  if (t == DType::none) {
    std::cerr << "PlaceHolder: unknown dtype \"" << dtype << "\".\n";
    return Value();
  }
  for (auto d : shapes)
    if (d <= 0) {
      std::cerr << "PlaceHolder: non-positive extent.\n";
      return Value();
    }
  MemRefType type{shapes, t, static_cast<int>(MemorySpace::global)};
  return graph->module->pushBack(makeAlloc(type))->result();
}

// C[i,j] = sum_k A[i,k] * B[k,j]; the k loop carries the accumulator as an
// iter_arg that starts at 0 and is updated as addf(mulf(a, b), acc).
Value Matmul::build(ComputeDAG *graph, Value A, Value B, MemorySpace ms, const std::string &dtype_) {
  if (!isMemRef(A, "Type of left operand of Matmul") || !isMemRef(B, "Type of right operand of Matmul"))
    return Value();
  const auto &ta = A.getMemRefType();
  const auto &tb = B.getMemRefType();
  if (ta.shape.size() != 2 || tb.shape.size() != 2) {
    std::cerr << "Matmul needs rank-2 operands.\n";
    return Value();
  }
  const int64_t m = ta.shape[0], k1 = ta.shape[1], k2 = tb.shape[0], n = tb.shape[1];
  if (k1 != k2) {
    std::cerr << "Can't apply Matmul Operation due to imcompatible K-dim.\n";
    return Value();
  }
  const DType elem = dtype_.empty() ? ta.elem : getDType(dtype_);
  if (elem == DType::none) {
    std::cerr << "Matmul: unknown dtype.\n";
    return Value();
  }
  const std::string funcName =
      "Matmul_m" + std::to_string(m) + "n" + std::to_string(n) + "k" + std::to_string(k1);
  MemRefType tc{{m, n}, elem, static_cast<int>(ms)};
  Value C = graph->module->pushBack(makeAlloc(tc))->result();

  FuncOp func = buildFuction(graph->module, funcName, {ta, tb, tc}, {tc});
  if (func->body.empty()) {
    auto args = func.getArguments();
    auto loops = loopNest(func.op, {m, n});
    Value i = ForOp(loops[0]).getInductionVar(), j = ForOp(loops[1]).getInductionVar();
    Op *inner = loops[1];
    Value zero = emit(inner, makeConstant(0.0, elem))->result();
    Op *kLoop = emit(inner, makeFor(0, k1, 1, {zero}));
    Value k = kLoop->arg(0), acc = kLoop->arg(1);
    Value a = kLoop->pushBack(makeLoad(args[0], {LinExpr(i), LinExpr(k)}))->result();
    Value b = kLoop->pushBack(makeLoad(args[1], {LinExpr(k), LinExpr(j)}))->result();
    Value mul = kLoop->pushBack(makeBinary(OpKind::MulF, a, b))->result();
    Value add = kLoop->pushBack(makeBinary(OpKind::AddF, mul, acc))->result();
    kLoop->pushBack(makeYield({add}));
    emit(inner, makeStore(kLoop->result(), args[2], {LinExpr(i), LinExpr(j)}));
    func->pushBack(makeReturn({args[2]}));
    func.setAttr("func.state", "cpu");
  }
  return graph->module->pushBack(makeCall(func.op, {A, B, C}))->result();
}

// y = maxf(0, x) elementwise; in place when ms == MemorySpace::inplace.
Value Relu::build(ComputeDAG *graph, Value input, MemorySpace ms, const std::string &dtype_) {
  if (!isMemRef(input, "Type of input of Relu")) return Value();
  const auto &ti = input.getMemRefType();
  const DType elem = dtype_.empty() ? ti.elem : getDType(dtype_);
  const std::string funcName = "Relu_Elementwise" + dims(ti.shape, 0, ti.shape.size());
  MemRefType to = ti;
  if (ms != MemorySpace::inplace) to.space = static_cast<int>(ms);
  to.elem = elem;

  FuncOp func = buildFuction(graph->module, funcName, {ti}, {to});
  if (func->body.empty()) {
    auto args = func.getArguments();
    Value output = args[0];
    if (ms != MemorySpace::inplace) output = func->pushBack(makeAlloc(to))->result();
    auto loops = loopNest(func.op, ti.shape);
    std::vector<LinExpr> idx;
    for (Op *l : loops) idx.emplace_back(ForOp(l).getInductionVar());
    Op *inner = loops.back();
    Value zero = emit(inner, makeConstant(0.0, elem))->result();
    Value x = emit(inner, makeLoad(args[0], idx))->result();
    Value mx = emit(inner, makeBinary(OpKind::MaxF, zero, x))->result();
    emit(inner, makeStore(mx, output, idx));
    func->pushBack(makeReturn({output}));
    func.setAttr("func.state", "cpu");
  }
  return graph->module->pushBack(makeCall(func.op, {input}))->result();
}

// Leading dimensions are the batch.  rowMajor A is [.., M, K], colMajor A is
// [.., K, M]; rowMajor B is [.., K, N], colMajor B is [.., N, K].
Value BatchedMatmul::build(ComputeDAG *graph, Value A, Layout layoutA, Value B, Layout layoutB,
                           const std::string &dtype_) {
  if (!isMemRef(A, "Type of left operand of BatchedMatmul") ||
      !isMemRef(B, "Type of right operand of BatchedMatmul"))
    return Value();
  const auto &ta = A.getMemRefType();
  const auto &tb = B.getMemRefType();
  const size_t rank = ta.shape.size();
  if (rank < 2) {
    std::cerr << "BatchedMatmul needs at least 2 dim but got " << rank << "\n";
    return Value();
  }
  if (tb.shape.size() != rank) {
    std::cerr << "BatchedMatmul: A, B dim not matched.\n";
    return Value();
  }
  for (size_t d = 0; d + 2 < rank; ++d)
    if (ta.shape[d] != tb.shape[d]) {
      std::cerr << "BatchedMatmul: A, B dim not matched.\n";
      return Value();
    }
  const bool tA = layoutA == Layout::colMajor, tB = layoutB == Layout::colMajor;
  const int64_t m = tA ? ta.shape[rank - 1] : ta.shape[rank - 2];
  const int64_t k1 = tA ? ta.shape[rank - 2] : ta.shape[rank - 1];
  const int64_t k2 = tB ? tb.shape[rank - 1] : tb.shape[rank - 2];
  const int64_t n = tB ? tb.shape[rank - 2] : tb.shape[rank - 1];
  if (k1 != k2) {
    std::cerr << "Can't apply BatchedMatmul Operation due to imcompatible K-dim.\n";
    return Value();
  }
  const DType elem = dtype_.empty() ? ta.elem : getDType(dtype_);
  std::vector<int64_t> shapeC(ta.shape.begin(), ta.shape.end() - 2);
  shapeC.push_back(m);
  shapeC.push_back(n);
  MemRefType tc{shapeC, elem, static_cast<int>(MemorySpace::global)};
  // the result buffer is a placeholder that sits right after B's definition
  Value C;
  {
    auto alloc = makeAlloc(tc);
    Op *defB = B.getDefiningOp();
    C = (defB && defB->parent == graph->module.get()) ? defB->insertAfter(std::move(alloc))->result()
                                                     : graph->module->pushBack(std::move(alloc))->result();
  }
  std::string funcName = "BatchMatmul" + dims(shapeC, 0, rank - 2) + "_m" + std::to_string(m) + "_n" +
                         std::to_string(n) + "_k" + std::to_string(k1) + "_" + (tA ? 'T' : 'N') +
                         (tB ? 'T' : 'N');

  FuncOp func = buildFuction(graph->module, funcName, {ta, tb, tc}, {tc});
  if (func->body.empty()) {
    auto args = func.getArguments();
    auto loops = loopNest(func.op, shapeC);
    std::vector<LinExpr> batch;
    for (size_t d = 0; d + 2 < rank; ++d) batch.emplace_back(ForOp(loops[d]).getInductionVar());
    Value i = ForOp(loops[rank - 2]).getInductionVar(), j = ForOp(loops[rank - 1]).getInductionVar();
    Op *inner = loops.back();
    Value zero = emit(inner, makeConstant(0.0, elem))->result();
    Op *kLoop = emit(inner, makeFor(0, k1, 1, {zero}));
    Value k = kLoop->arg(0), acc = kLoop->arg(1);
    auto idxA = batch, idxB = batch, idxC = batch;
    if (tA) { idxA.emplace_back(k); idxA.emplace_back(i); } else { idxA.emplace_back(i); idxA.emplace_back(k); }
    if (tB) { idxB.emplace_back(j); idxB.emplace_back(k); } else { idxB.emplace_back(k); idxB.emplace_back(j); }
    idxC.emplace_back(i);
    idxC.emplace_back(j);
    Value a = kLoop->pushBack(makeLoad(args[0], idxA))->result();
    Value b = kLoop->pushBack(makeLoad(args[1], idxB))->result();
    Value mul = kLoop->pushBack(makeBinary(OpKind::MulF, a, b))->result();
    Value add = kLoop->pushBack(makeBinary(OpKind::AddF, mul, acc))->result();
    kLoop->pushBack(makeYield({add}));
    emit(inner, makeStore(kLoop->result(), args[2], idxC));
    func->pushBack(makeReturn({args[2]}));
    func.setAttr("func.state", "cpu");
  }
  return graph->module->pushBack(makeCall(func.op, {A, B, C}))->result();
}

// Per row of the last axis: sum = sum_k exp(x[k]) (iter_arg from 0), then
// x[k] = exp(x[k]) / sum, stored over the input.
Value Softmax::build(ComputeDAG *graph, Value input, int axis, MemorySpace ms, const std::string &dtype_) {
  (void)ms;  // the operator is in place whatever `ms` says, as in the reference
  if (!isMemRef(input, "Type of input of Softmax")) return Value();
  const auto &ti = input.getMemRefType();
  const int rank = static_cast<int>(ti.shape.size());
  const int reduceAxis = axis == -1 ? rank - 1 : axis;
  if (reduceAxis < 0 || reduceAxis >= rank) {
    std::cerr << "Illegal reduction axis in Softmax.\n";
    return Value();
  }
  if (reduceAxis != rank - 1) {
    std::cerr << "At present, only support reduction on the last dim.\n";
    return Value();
  }
  const DType elem = dtype_.empty() ? ti.elem : getDType(dtype_);
  const std::string funcName =
      "Softmax" + dims(ti.shape, 0, ti.shape.size()) + "_axis" + std::to_string(reduceAxis);

  FuncOp func = buildFuction(graph->module, funcName, {ti}, {ti});
  if (func->body.empty()) {
    auto args = func.getArguments();
    std::vector<int64_t> outer(ti.shape.begin(), ti.shape.end() - 1);
    Op *body = func.op;
    std::vector<LinExpr> idx;
    if (!outer.empty()) {
      auto loops = loopNest(func.op, outer);
      for (Op *l : loops) idx.emplace_back(ForOp(l).getInductionVar());
      body = loops.back();
    }
    auto put = [&](std::unique_ptr<Op> op) {
      return body == func.op ? body->pushBack(std::move(op)) : emit(body, std::move(op));
    };
    const int64_t len = ti.shape.back();
    Value zero = put(makeConstant(0.0, elem))->result();
    Op *sumLoop = put(makeFor(0, len, 1, {zero}));
    {
      auto at = idx;
      at.emplace_back(sumLoop->arg(0));
      Value x = sumLoop->pushBack(makeLoad(args[0], at))->result();
      Value e = sumLoop->pushBack(makeExp(x))->result();
      Value s = sumLoop->pushBack(makeBinary(OpKind::AddF, e, sumLoop->arg(1)))->result();
      sumLoop->pushBack(makeYield({s}));
    }
    Op *divLoop = put(makeFor(0, len, 1));
    {
      auto at = idx;
      at.emplace_back(divLoop->arg(0));
      Value x = divLoop->pushBack(makeLoad(args[0], at))->result();
      Value e = divLoop->pushBack(makeExp(x))->result();
      Value q = divLoop->pushBack(makeBinary(OpKind::DivF, e, sumLoop->result()))->result();
      divLoop->pushBack(makeStore(q, args[0], at));
      divLoop->pushBack(makeYield());
    }
    func->pushBack(makeReturn({args[0]}));
    func.setAttr("func.state", "cpu");
  }
  return graph->module->pushBack(makeCall(func.op, {input}))->result();
}

Value Transpose::build(ComputeDAG *, Value) {
  std::cerr << "Transpose is not implemented (express it through BatchedMatmul's Layout argument).\n";
  return Value();
}

}  // namespace KernelCodeGen
