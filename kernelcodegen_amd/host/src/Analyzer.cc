#include "Optimizer/Analyzer.h"

#include <iostream>

namespace KernelCodeGen {

using namespace ir;

std::vector<ForOp> Analyzer::collectOutermostLoop(ModuleOp &module) {
  std::vector<ForOp> res;
  for (auto &k : module->body)
    if (k->kind == OpKind::For) res.emplace_back(k.get());
  return res;
}

std::vector<int64_t> Analyzer::getParallelNumber(ParallelOp parallelLevel, int64_t &totalNumber) {
  totalNumber = 1;
  for (auto u : parallelLevel->ubs) totalNumber *= u;
  return parallelLevel->ubs;
}

std::vector<FuncOp> Analyzer::collectFunctions(ModuleOp &module, const std::string &targetFuncName) {
  std::vector<FuncOp> result;
  walk(module.get(), [&](Op *op) {
    if (op->kind != OpKind::Func) return;
    if (targetFuncName.empty() || op->name.find(targetFuncName) != std::string::npos) result.emplace_back(op);
  });
  return result;
}

std::vector<ForOp> Analyzer::collectFuncLoops(FuncOp funcOp) {
  std::vector<ForOp> res;
  walk(funcOp.op, [&](Op *op) {
    if (op->kind == OpKind::For) res.emplace_back(op);
  });
  return res;
}

std::vector<ParallelOp> Analyzer::collectFuncParallels(FuncOp funcOp) {
  std::vector<ParallelOp> res;
  walk(funcOp.op, [&](Op *op) {
    if (op->kind == OpKind::Parallel) res.emplace_back(op);
  });
  return res;
}

std::vector<CallOp> Analyzer::collectFuncCalls(ModuleOp &module) {
  std::vector<CallOp> res;
  walk(module.get(), [&](Op *op) {
    if (op->kind == OpKind::Call) res.emplace_back(op);
  });
  return res;
}

FuncOp Analyzer::getTargetFunction(ModuleOp &module, const std::string &targetFuncName) {
  for (auto &k : module->body)
    if (k->kind == OpKind::Func && k->name == targetFuncName) return FuncOp(k.get());
  std::cerr << "Failed get the function which name is " << targetFuncName << "\n";
  return FuncOp();
}

std::vector<Op *> Analyzer::getUsers(ModuleOp &module, Value v) {
  std::vector<Op *> users;
  for (auto &k : module->body) {
    if (k->kind == OpKind::Func) continue;
    for (auto &o : k->operands)
      if (o == v) {
        users.push_back(k.get());
        break;
      }
  }
  return users;
}

Op *Analyzer::getLastOp(Op *father, OpKind kind) {
  Op *res = nullptr;
  for (auto &k : father->body)
    if (k->kind == kind) res = k.get();
  return res;
}

}  // namespace KernelCodeGen
