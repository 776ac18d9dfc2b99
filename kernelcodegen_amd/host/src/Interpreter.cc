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

float *Interpreter::getMem(Frame &fr, Value v) {
  for (Frame *f = &fr; f; f = f->parent) {
    auto it = f->mem.find(v.get());
    if (it != f->mem.end()) return it->second;
  }
  return nullptr;
}

float Interpreter::getF(Frame &fr, Value v) {
  for (Frame *f = &fr; f; f = f->parent) {
    auto it = f->f.find(v.get());
    if (it != f->f.end()) return it->second;
  }
  error_ = "scalar value used before definition";
  return 0.0f;
}

const std::vector<float> *Interpreter::getV(Frame &fr, Value v) {
  for (Frame *f = &fr; f; f = f->parent) {
    auto it = f->v.find(v.get());
    if (it != f->v.end()) return &it->second;
  }
  return nullptr;
}

bool Interpreter::getI(Frame &fr, Value v, int64_t &out) {
  for (Frame *f = &fr; f; f = f->parent) {
    auto it = f->i.find(v.get());
    if (it != f->i.end()) {
      out = it->second;
      return true;
    }
  }
  return false;
}

int64_t Interpreter::eval(const LinExpr &e, Frame &fr) {
  int64_t v = e.constant;
  for (auto &t : e.terms) {
    int64_t x = 0;
    if (!getI(fr, t.first, x)) {
      error_ = "index value used before definition";
      return 0;
    }
    v += x * t.second;
  }
  return v;
}

int64_t Interpreter::offset(const Op *op, Frame &fr) {
  const auto &shape = op->memref.getMemRefType().shape;
  const int width = op->vec > 0 ? op->vec : 1;
  int64_t off = 0;
  for (size_t d = 0; d < shape.size(); ++d) {
    const int64_t idx = eval(op->indices[d], fr);
    const int64_t span = d + 1 == shape.size() ? width : 1;
    if (idx < 0 || idx + span > shape[d]) {
      error_ = "subscript out of bounds";
      return 0;
    }
    off = off * shape[d] + idx;
  }
  return off;
}

bool Interpreter::holds(const Op *ifOp, Frame &fr) {
  for (auto &c : ifOp->indices)
    if (eval(c, fr) < 0) return false;
  return true;
}

bool Interpreter::containsBarrier(const Op *op) {
  auto it = barrierInside_.find(op);
  if (it != barrierInside_.end()) return it->second;
  // a barrier belongs to the innermost parallel level around it
  bool any = op->kind == OpKind::Barrier;
  for (auto &k : op->body)
    if (k->kind != OpKind::Parallel) any = containsBarrier(k.get()) || any;
  barrierInside_[op] = any;
  return any;
}

void Interpreter::execRegion(const Op *op, Frame &fr) {
  for (auto &k : op->body) {
    if (!error_.empty()) return;
    exec(k.get(), fr);
  }
}

void Interpreter::execLockStep(const OpList &body, std::vector<Frame> &threads) {
  for (auto &kp : body) {
    if (!error_.empty()) return;
    const Op *k = kp.get();
    if (!containsBarrier(k)) {
      for (auto &t : threads) {
        exec(k, t);
        if (!error_.empty()) return;
      }
      continue;
    }
    switch (k->kind) {
      case OpKind::Barrier:
        break;  // every thread has finished the statements before it
      case OpKind::For: {
        const size_t nIter = k->args.size() - 1;
        for (auto &t : threads)
          for (size_t a = 0; a < nIter; ++a) t.f[k->args[a + 1].get()] = getF(t, k->operands[a]);
        for (int64_t iv = k->lb; iv < k->ub && error_.empty(); iv += k->step) {
          for (auto &t : threads) t.i[k->args[0].get()] = iv;
          execLockStep(k->body, threads);
          const Op *yield = k->body.back().get();
          for (auto &t : threads)
            for (size_t a = 0; a < nIter; ++a) t.f[k->args[a + 1].get()] = getF(t, yield->operands[a]);
        }
        for (auto &t : threads)
          for (size_t a = 0; a < nIter; ++a) t.f[k->results[a].get()] = getF(t, k->args[a + 1].get());
        break;
      }
      case OpKind::If: {
        size_t yes = 0;
        for (auto &t : threads) yes += holds(k, t) ? 1 : 0;
        if (yes == threads.size()) execLockStep(k->body, threads);
        else if (yes != 0) error_ = "gpu.barrier under a condition the threads of a block disagree on";
        break;
      }
      default:
        error_ = std::string("gpu.barrier inside ") + opName(k->kind) + " is not interpretable";
        break;
    }
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
    case OpKind::Apply: {
      int64_t v = eval(op->indices[0], fr);
      if (op->divisor > 0) {
        int64_t q = v / op->divisor, r = v % op->divisor;
        if (r < 0) {  // floor semantics
          r += op->divisor;
          q -= 1;
        }
        v = op->isMod ? r : q;
      }
      fr.i[op->results[0].get()] = v;
      break;
    }
    case OpKind::Load: {
      float *base = getMem(fr, op->memref);
      if (!base) {
        error_ = "load from an unbound memref";
        return;
      }
      const int64_t off = offset(op, fr);
      if (!error_.empty()) return;
      if (op->vec > 0) fr.v[op->results[0].get()] = std::vector<float>(base + off, base + off + op->vec);
      else fr.f[op->results[0].get()] = base[off];
      break;
    }
    case OpKind::Store: {
      float *base = getMem(fr, op->memref);
      if (!base) {
        error_ = "store to an unbound memref";
        return;
      }
      const int64_t off = offset(op, fr);
      if (!error_.empty()) return;
      if (op->vec > 0) {
        const std::vector<float> *v = getV(fr, op->operands[0]);
        if (!v || static_cast<int>(v->size()) != op->vec) {
          error_ = "vector store of a value that is not a vector of that width";
          return;
        }
        for (int l = 0; l < op->vec; ++l) base[off + l] = (*v)[l];
      } else {
        base[off] = getF(fr, op->operands[0]);
      }
      break;
    }
    case OpKind::MulF: {
      volatile float r = getF(fr, op->operands[0]) * getF(fr, op->operands[1]);
      fr.f[op->results[0].get()] = r;
      break;
    }
    case OpKind::AddF: {
      volatile float r = getF(fr, op->operands[0]) + getF(fr, op->operands[1]);
      fr.f[op->results[0].get()] = r;
      break;
    }
    case OpKind::DivF:
      fr.f[op->results[0].get()] = getF(fr, op->operands[0]) / getF(fr, op->operands[1]);
      break;
    case OpKind::MaxF: {
      const float a = getF(fr, op->operands[0]), b = getF(fr, op->operands[1]);
      fr.f[op->results[0].get()] = (a != a) ? a : (b != b) ? b : (a > b ? a : b);
      break;
    }
    case OpKind::Exp:
      fr.f[op->results[0].get()] = std::exp(getF(fr, op->operands[0]));
      break;
    case OpKind::For: {
      const size_t nIter = op->args.size() - 1;
      for (size_t a = 0; a < nIter; ++a) fr.f[op->args[a + 1].get()] = getF(fr, op->operands[a]);
      for (int64_t iv = op->lb; iv < op->ub && error_.empty(); iv += op->step) {
        fr.i[op->args[0].get()] = iv;
        execRegion(op, fr);
        const Op *yield = op->body.back().get();
        for (size_t a = 0; a < nIter; ++a) fr.f[op->args[a + 1].get()] = getF(fr, yield->operands[a]);
      }
      for (size_t a = 0; a < nIter; ++a) fr.f[op->results[a].get()] = getF(fr, op->args[a + 1].get());
      break;
    }
    case OpKind::If:
      if (holds(op, fr)) execRegion(op, fr);
      break;
    case OpKind::Parallel: {
      int64_t total = 1;
      for (auto u : op->ubs) total *= u;
      auto setIvs = [&](Frame &f, int64_t n) {
        for (int d = static_cast<int>(op->ubs.size()) - 1; d >= 0; --d) {
          f.i[op->args[d].get()] = n % op->ubs[d];
          n /= op->ubs[d];
        }
      };
      if (containsBarrier(op)) {
        // a thread block: one frame per index point, walked in lock step
        std::vector<Frame> threads(static_cast<size_t>(total));
        for (int64_t n = 0; n < total; ++n) {
          threads[n].parent = &fr;
          setIvs(threads[n], n);
        }
        execLockStep(op->body, threads);
      } else {
        for (int64_t n = 0; n < total && error_.empty(); ++n) {
          // a buffer allocated inside the body is private to one index point
          Frame point;
          point.parent = &fr;
          setIvs(point, n);
          execRegion(op, point);
        }
      }
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
        float *p = getMem(fr, op->operands[a]);
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
        fr.mem[op->results[r].get()] = getMem(inner, ret->operands[r]);
      break;
    }
    case OpKind::Barrier:  // outside any parallel level there is one thread: nothing to wait for
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
