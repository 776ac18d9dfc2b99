#include "IR/Interpreter.h"

#include <cmath>

namespace KernelCodeGen {
namespace ir {

void Interpreter::bind(Value memref, float *data) { top_.mem[memref.get()] = data; }

float *Interpreter::buffer(Value memref) {
  auto it = top_.mem.find(memref.get());
  return it == top_.mem.end() ? nullptr : it->second;
}

float *Interpreter::alloc(const MemRefType &t) {
  owned_.emplace_back(new float[t.numElements()]());
  return owned_.back().get();
}

int64_t Interpreter::eval(const LinExpr &e, Frame &fr) {
  int64_t v = e.constant;
  for (auto &t : e.terms) {
    auto it = fr.i.find(t.first.get());
    if (it == fr.i.end()) {
      error_ = "index value used before definition";
      return 0;
    }
    v += it->second * t.second;
  }
  return v;
}

int64_t Interpreter::offset(const Op *op, Frame &fr) {
  const auto &shape = op->memref.getMemRefType().shape;
  int64_t off = 0;
  for (size_t d = 0; d < shape.size(); ++d) {
    const int64_t idx = eval(op->indices[d], fr);
    if (idx < 0 || idx >= shape[d]) {
      error_ = "subscript out of bounds";
      return 0;
    }
    off = off * shape[d] + idx;
  }
  return off;
}

void Interpreter::execRegion(const Op *op, Frame &fr) {
  for (auto &k : op->body) {
    if (!error_.empty()) return;
    exec(k.get(), fr);
  }
}

void Interpreter::exec(const Op *op, Frame &fr) {
  switch (op->kind) {
    case OpKind::Alloc:
      if (!fr.mem.count(op->results[0].get())) fr.mem[op->results[0].get()] = alloc(op->results[0]->memref);
      break;
    case OpKind::Constant:
      fr.f[op->results[0].get()] = static_cast<float>(op->fvalue);
      break;
    case OpKind::Apply:
      fr.i[op->results[0].get()] = eval(op->indices[0], fr);
      break;
    case OpKind::Load: {
      float *base = fr.mem[op->memref.get()];
      if (!base) {
        error_ = "load from an unbound memref";
        return;
      }
      const int64_t off = offset(op, fr);
      if (error_.empty()) fr.f[op->results[0].get()] = base[off];
      break;
    }
    case OpKind::Store: {
      float *base = fr.mem[op->memref.get()];
      if (!base) {
        error_ = "store to an unbound memref";
        return;
      }
      const int64_t off = offset(op, fr);
      if (error_.empty()) base[off] = fr.f[op->operands[0].get()];
      break;
    }
    case OpKind::MulF: {
      volatile float r = fr.f[op->operands[0].get()] * fr.f[op->operands[1].get()];
      fr.f[op->results[0].get()] = r;
      break;
    }
    case OpKind::AddF: {
      volatile float r = fr.f[op->operands[0].get()] + fr.f[op->operands[1].get()];
      fr.f[op->results[0].get()] = r;
      break;
    }
    case OpKind::DivF:
      fr.f[op->results[0].get()] = fr.f[op->operands[0].get()] / fr.f[op->operands[1].get()];
      break;
    case OpKind::MaxF: {
      const float a = fr.f[op->operands[0].get()], b = fr.f[op->operands[1].get()];
      fr.f[op->results[0].get()] = (a != a) ? a : (b != b) ? b : (a > b ? a : b);
      break;
    }
    case OpKind::Exp:
      fr.f[op->results[0].get()] = std::exp(fr.f[op->operands[0].get()]);
      break;
    case OpKind::For: {
      const size_t nIter = op->args.size() - 1;
      for (size_t a = 0; a < nIter; ++a) fr.f[op->args[a + 1].get()] = fr.f[op->operands[a].get()];
      for (int64_t iv = op->lb; iv < op->ub && error_.empty(); iv += op->step) {
        fr.i[op->args[0].get()] = iv;
        execRegion(op, fr);
        const Op *yield = op->body.back().get();
        for (size_t a = 0; a < nIter; ++a) fr.f[op->args[a + 1].get()] = fr.f[yield->operands[a].get()];
      }
      for (size_t a = 0; a < nIter; ++a) fr.f[op->results[a].get()] = fr.f[op->args[a + 1].get()];
      break;
    }
    case OpKind::Parallel: {
      std::vector<int64_t> idx(op->ubs.size(), 0);
      int64_t total = 1;
      for (auto u : op->ubs) total *= u;
      ++parallelDepth_;
      for (int64_t n = 0; n < total && error_.empty(); ++n) {
        int64_t r = n;
        for (int d = static_cast<int>(op->ubs.size()) - 1; d >= 0; --d) {
          fr.i[op->args[d].get()] = r % op->ubs[d];
          r /= op->ubs[d];
        }
        // a buffer allocated inside the body is private to one index point; index
        // points run one after the other here, so its storage is simply reused
        execRegion(op, fr);
      }
      --parallelDepth_;
      break;
    }
    case OpKind::Call: {
      const Op *callee = nullptr;
      for (auto &k : module_->body)
        if (k->kind == OpKind::Func && k->name == op->name) callee = k.get();
      if (!callee) {
        error_ = "call to an unknown function " + op->name;
        return;
      }
      Frame inner;
      for (size_t a = 0; a < callee->args.size(); ++a) {
        float *p = fr.mem[op->operands[a].get()];
        if (!p) {
          // an output buffer that nothing bound: allocate it on first use
          p = alloc(op->operands[a].getMemRefType());
          fr.mem[op->operands[a].get()] = p;
        }
        inner.mem[callee->args[a].get()] = p;
      }
      execRegion(callee, inner);
      const Op *ret = callee->body.back().get();
      for (size_t r = 0; r < op->results.size() && r < ret->operands.size(); ++r)
        fr.mem[op->results[r].get()] = inner.mem[ret->operands[r].get()];
      break;
    }
    case OpKind::Barrier:
      if (parallelDepth_ > 0) error_ = "gpu.barrier inside affine.parallel is not interpretable";
      break;
    case OpKind::Yield:
    case OpKind::Return:
    case OpKind::Func:
    case OpKind::Module:
      break;
  }
}

std::string Interpreter::run() {
  error_.clear();
  for (auto &k : module_->body) {
    if (k->kind == OpKind::Func) continue;
    exec(k.get(), top_);
    if (!error_.empty()) break;
  }
  return error_;
}

}  // namespace ir
}  // namespace KernelCodeGen
