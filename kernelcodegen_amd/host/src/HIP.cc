#include "Backend/HIP.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <iostream>
#include <set>
#include <sstream>

#include "Optimizer/Analyzer.h"
#include "Optimizer/Optimizer.h"
#include "enum.h"

namespace KernelCodeGen {

using namespace ir;

namespace {

int attrInt(FuncOp f, const std::string &key, int fallback) {
  const std::string v = f.getAttr(key);
  return v.empty() ? fallback : std::stoi(v);
}

// What the scheduled loop nest of a matmul function says about the kernel: read off the
// IR, not off the kcg.* attributes.  The reference's backend prints whatever nest the
// Rewriter calls left behind (split(k) -> BLOCK_SIZE_K, pipeline -> two copies of each
// shared tile, vectorize -> float4 accesses; src/Optimizer/Optimizer.cc:494-519,
// src/Optimizer/Rewriter.cc:786-1180); here the same facts select the prebuilt kernel.
struct NestSchedule {
  bool staged = false;      // the nest holds shared-memory tiles at all
  int64_t bk = 0;           // rows of the shared tiles = the k-split factor
  std::vector<int64_t> tileExtents;  // their columns: BLOCK_SIZE_M and BLOCK_SIZE_N
  int64_t copies = 0;       // leading dimension added by pipeline (1 without it)
  int vec = 0;              // width of the vector loads / stores (0: none)
  std::string problem;      // non-empty: the nest is not one the library can bind
};

NestSchedule readNestSchedule(FuncOp f) {
  NestSchedule n;
  std::vector<MemRefType> shared;
  std::set<int> widths;
  walk(f.op, [&](Op *o) {
    if (o->kind == OpKind::Alloc && !o->results.empty()) {
      const MemRefType &t = o->result().getMemRefType();
      if (t.space == static_cast<int>(MemorySpace::shared)) shared.push_back(t);
    }
    if ((o->kind == OpKind::Load || o->kind == OpKind::Store) && o->vec > 1) widths.insert(o->vec);
  });
  if (shared.empty()) return n;
  n.staged = true;
  if (shared.size() != 2) {
    n.problem = "expected one shared tile of A and one of B, found " + std::to_string(shared.size());
    return n;
  }
  for (const MemRefType &t : shared) {
    if (t.shape.size() != 2 && t.shape.size() != 3) {
      n.problem = "shared tile " + t.str() + " is neither [BK][B] nor [copies][BK][B]";
      return n;
    }
    const int64_t copies = t.shape.size() == 3 ? t.shape[0] : 1;
    const int64_t bk = t.shape[t.shape.size() - 2];
    if ((n.copies && n.copies != copies) || (n.bk && n.bk != bk)) {
      n.problem = "the shared tiles of A and B disagree on BLOCK_SIZE_K or on the number of copies";
      return n;
    }
    n.copies = copies;
    n.bk = bk;
    n.tileExtents.push_back(t.shape.back());
  }
  if (widths.size() > 1) {
    n.problem = "vector accesses of different widths";
    return n;
  }
  n.vec = widths.empty() ? 0 : *widths.begin();
  return n;
}

bool bindMatmul(FuncOp f, KernelBinding &b) {
  auto args = f.getArguments();
  if (args.size() != 3) return false;
  const auto &ta = args[0].getMemRefType();
  const auto &tb = args[1].getMemRefType();
  if (ta.elem != DType::f32 || tb.elem != DType::f32 || ta.shape.size() != 2 || tb.shape.size() != 2) {
    std::cerr << "HIPBind: " << f.getSymName() << ": only float32 rank-2 matmul has a gfx950 kernel\n";
    return false;
  }
  if (ta.shape[1] != tb.shape[0]) {
    std::cerr << "HIPBind: " << f.getSymName() << ": A is " << ta.shape[0] << " x " << ta.shape[1] << " but B is "
              << tb.shape[0] << " x " << tb.shape[1] << " (K extents differ)\n";
    return false;
  }
  b.kind = KernelBinding::Gemm;
  b.entry = "kcg_gemm_f32";
  b.M = ta.shape[0];
  b.K = ta.shape[1];
  b.N = tb.shape[1];
  b.epilogue = f.getAttr("kcg.epilogue") == "relu" ? KCG_EPILOGUE_RELU : KCG_EPILOGUE_NONE;
  b.gemmSched.block_m = attrInt(f, "kcg.BLOCK_SIZE_M", 0);
  b.gemmSched.block_n = attrInt(f, "kcg.BLOCK_SIZE_N", 0);
  b.gemmSched.block_k = attrInt(f, "kcg.BLOCK_SIZE_K", 0);
  b.gemmSched.group_m = attrInt(f, "kcg.GROUP_SIZE_M", 0);
  b.gemmSched.wave_m = attrInt(f, "kcg.WAVE_SIZE_M", 0);
  b.gemmSched.wave_n = attrInt(f, "kcg.WAVE_SIZE_N", 0);
  b.gemmSched.vec_width = attrInt(f, "kcg.VECTORIZE_WIDTH", 0);
  b.gemmSched.wave_size = attrInt(f, "kcg.WARP_SIZE", 0);
  b.argNames = {"A", "B", "C"};
  // A staged / pipelined nest decides block_k, the LDS buffer count and the vector width
  // itself; the attributes must not contradict it.
  const NestSchedule nest = readNestSchedule(f);
  if (!nest.problem.empty()) {
    std::cerr << "HIPBind: " << f.getSymName() << ": " << nest.problem << "\n";
    return false;
  }
  if (nest.staged) {
    std::vector<int64_t> want = {b.gemmSched.block_m, b.gemmSched.block_n}, got = nest.tileExtents;
    std::sort(want.begin(), want.end());
    std::sort(got.begin(), got.end());
    if (got != want || (b.gemmSched.block_k && b.gemmSched.block_k != nest.bk) ||
        (nest.vec && b.gemmSched.vec_width && b.gemmSched.vec_width != nest.vec)) {
      std::cerr << "HIPBind: " << f.getSymName() << ": the scheduled nest (shared tiles " << nest.bk << " x {"
                << nest.tileExtents[0] << ", " << nest.tileExtents[1] << "}, vector width " << nest.vec
                << ") contradicts the kcg.* attributes (" << b.gemmSched.block_m << " x " << b.gemmSched.block_n
                << " x " << b.gemmSched.block_k << ", width " << b.gemmSched.vec_width << ")\n";
      return false;
    }
    b.scheduleSource = "ir";
    b.gemmSched.block_k = static_cast<int>(nest.bk);
    if (nest.vec) b.gemmSched.vec_width = nest.vec;
    // one copy of each shared tile (the staged schedule), two (Rewriter::pipeline) or a ring of three
    b.gemmSched.lds_stages = static_cast<int>(nest.copies);
  }
  const int st = kcg_gemm_f32_query(b.M, b.N, b.K, &b.gemmSched, &b.launch);
  if (st != KCG_OK) {
    std::cerr << "HIPBind: " << f.getSymName() << ": " << kcg_status_str(st) << "\n";
    return false;
  }
  return true;
}

bool bindFmha(FuncOp f, KernelBinding &b) {
  auto args = f.getArguments();
  if (args.size() != 4) return false;
  const auto &tq = args[0].getMemRefType();
  if (tq.shape.size() < 3) {
    std::cerr << "HIPBind: " << f.getSymName() << ": attention needs [batch.., S, D] operands\n";
    return false;
  }
  const size_t r = tq.shape.size();
  int64_t batch = 1;
  for (size_t d = 0; d + 3 < r; ++d) batch *= tq.shape[d];
  b.kind = KernelBinding::Fmha;
  b.B = static_cast<int>(r >= 4 ? batch : 1);
  b.H = static_cast<int>(tq.shape[r - 3]);
  b.S = static_cast<int>(tq.shape[r - 2]);
  b.D = static_cast<int>(tq.shape[r - 1]);
  if (tq.elem == DType::f32) {
    b.dtype = KCG_F32;
    b.entry = "kcg_fmha_f32";
  } else if (tq.elem == DType::bf16) {
    b.dtype = KCG_BF16;
    b.entry = "kcg_fmha_bf16";
  } else {
    std::cerr << "HIPBind: " << f.getSymName() << ": only float32 and bfloat16 attention kernels exist\n";
    return false;
  }
  b.fmhaSched.br = attrInt(f, "kcg.Br", 0);
  b.fmhaSched.bc = attrInt(f, "kcg.Bc", 0);
  const std::string sc = f.getAttr("kcg.scale");
  b.scale = sc.empty() ? 1.0f : std::stof(sc);
  b.causal = attrInt(f, "kcg.causal", 0);
  b.argNames = {"Q", "K", "V", "O"};
  const int st = kcg_fmha_query(b.dtype, b.B, b.H, b.S, b.D, b.causal, &b.fmhaSched, &b.launch);
  if (st != KCG_OK) {
    std::cerr << "HIPBind: " << f.getSymName() << ": " << kcg_status_str(st) << "\n";
    return false;
  }
  return true;
}

size_t bytesOf(const MemRefType &t) {
  const size_t elem = t.elem == DType::f64 ? 8 : (t.elem == DType::f32 ? 4 : 2);
  return static_cast<size_t>(t.numElements()) * elem;
}

bool allF32(FuncOp f) {
  for (auto a : f.getArguments())
    if (!a.isMemRef() || a.getMemRefType().elem != DType::f32) return false;
  return true;
}

// Relu_Elementwise_<dims> (src/Frontend/Operators.cc:182-250): one memref in; the result is
// that memref (MemorySpace::inplace) or a buffer the function allocates itself.
bool bindRelu(FuncOp f, KernelBinding &b) {
  auto args = f.getArguments();
  if (args.size() != 1 || !allF32(f)) {
    std::cerr << "HIPBind: " << f.getSymName() << ": only the float32 Relu has a gfx950 kernel\n";
    return false;
  }
  b.kind = KernelBinding::Relu;
  b.entry = "kcg_relu_f32";
  b.count = args[0].getMemRefType().numElements();
  // in place when the function returns its own argument
  b.inPlace = true;
  walk(f.op, [&](Op *o) {
    if (o->kind == OpKind::Return && !o->operands.empty() && o->operands[0] != args[0]) b.inPlace = false;
  });
  b.argNames = b.inPlace ? std::vector<std::string>{"x"} : std::vector<std::string>{"x", "y"};
  b.argBytes.assign(b.argNames.size(), bytesOf(args[0].getMemRefType()));
  return true;
}

// BatchMatmul_<batch..>_m<M>_n<N>_k<K>_<N|T><N|T> (src/Frontend/Operators.cc:253-420; the
// name is parsed back as the reference's optimizer does, src/Optimizer/Optimizer.cc:564-584).
bool bindBatchedMatmul(FuncOp f, KernelBinding &b) {
  auto args = f.getArguments();
  BatchMatmulDescriptor d;
  if (args.size() != 3 || !identifyBatchMatmul(f.getSymName(), d)) return false;
  if (!allF32(f)) {
    std::cerr << "HIPBind: " << f.getSymName() << ": only the float32 BatchedMatmul has a gfx950 kernel\n";
    return false;
  }
  b.kind = KernelBinding::BatchedMatmul;
  b.entry = "kcg_batched_matmul_f32";
  b.batch = 1;
  for (int x : d.batch) b.batch *= x;
  b.M = d.m;
  b.N = d.n;
  b.K = d.k;
  b.transA = d.transA ? 1 : 0;
  b.transB = d.transB ? 1 : 0;
  b.argNames = {"A", "B", "C"};
  for (auto a : args) b.argBytes.push_back(bytesOf(a.getMemRefType()));
  if (b.argBytes[0] != static_cast<size_t>(b.batch * b.M * b.K) * 4 ||
      b.argBytes[1] != static_cast<size_t>(b.batch * b.K * b.N) * 4 ||
      b.argBytes[2] != static_cast<size_t>(b.batch * b.M * b.N) * 4) {
    std::cerr << "HIPBind: " << f.getSymName() << ": the operand types do not have the extents the name encodes\n";
    return false;
  }
  return true;
}

// Softmax_<dims>_axis<k> (src/Frontend/Operators.cc:425-542): last axis only, in place.
bool bindSoftmax(FuncOp f, KernelBinding &b) {
  auto args = f.getArguments();
  if (args.size() != 1 || !allF32(f)) {
    std::cerr << "HIPBind: " << f.getSymName() << ": only the float32 Softmax has a gfx950 kernel\n";
    return false;
  }
  const MemRefType &t = args[0].getMemRefType();
  const std::string &name = f.getSymName();
  const size_t at = name.rfind("_axis");
  if (t.shape.empty() || at == std::string::npos ||
      std::atoi(name.c_str() + at + 5) != static_cast<int>(t.shape.size()) - 1) {
    std::cerr << "HIPBind: " << name << ": the kernel reduces over the last axis only\n";
    return false;
  }
  b.kind = KernelBinding::Softmax;
  b.entry = "kcg_softmax_f32";
  b.rowLength = t.shape.back();
  b.count = t.numElements();
  b.inPlace = true;
  b.argNames = {"x"};
  b.argBytes = {bytesOf(t)};
  return true;
}

}  // namespace

Value HIPBufferOf(ModuleOp &module, Value v) {
  for (int hops = 0; hops < 1024 && v; ++hops) {
    Op *def = v.getDefiningOp();
    if (!def || def->kind != OpKind::Call) return v;   // an allocation of the module
    FuncOp f = Analyzer::getTargetFunction(module, def->name);
    if (!f) return v;
    // which argument the function returns: Matmul / BatchMatmul return C (their last
    // argument), Softmax and the in-place Relu their only one, the fused attention O
    auto args = f.getArguments();
    int returned = -1;
    walk(f.op, [&](Op *o) {
      if (o->kind != OpKind::Return || o->operands.empty()) return;
      for (size_t i = 0; i < args.size(); ++i)
        if (o->operands[0] == args[i]) returned = static_cast<int>(i);
    });
    if (returned < 0 || returned >= static_cast<int>(def->operands.size())) return v;  // a buffer of its own
    v = def->operands[returned];
  }
  return v;
}

std::vector<KernelBinding> HIPBind(ModuleOp &module) {
  std::vector<KernelBinding> out;
  // module order of the calls decides kernel numbering, as the emitter numbers kernels in walk order
  for (auto call : Analyzer::collectFuncCalls(module)) {
    FuncOp f = Analyzer::getTargetFunction(module, call.getCallee());
    if (!f) continue;
    const std::string state = f.getAttr("func.state");
    KernelBinding b;
    b.graph = module.getName();
    b.funcName = f.getSymName();
    bool ok = false;
    if (state == "gpu") {
      if (b.funcName.rfind("Matmul_m", 0) == 0) ok = bindMatmul(f, b);
      else if (b.funcName.rfind("Fused_Multi_Head_Attention", 0) == 0) ok = bindFmha(f, b);
      else std::cerr << "HIPBind: no gfx950 kernel is bound to " << b.funcName << "\n";
      if (ok)
        for (auto a : f.getArguments()) b.argBytes.push_back(bytesOf(a.getMemRefType()));
    } else if (state == "cpu") {
      // no pattern matched this call: the un-fused kernels
      if (b.funcName.rfind("Relu_Elementwise", 0) == 0) ok = bindRelu(f, b);
      else if (b.funcName.rfind("BatchMatmul_", 0) == 0) ok = bindBatchedMatmul(f, b);
      else if (b.funcName.rfind("Softmax_", 0) == 0) ok = bindSoftmax(f, b);
      else std::cerr << "HIPBind: no gfx950 kernel is bound to " << b.funcName << "\n";
      if (ok) snprintf(b.launch.kernel, sizeof b.launch.kernel, "%s", b.entry.c_str());
    } else {
      continue;
    }
    if (!ok) continue;
    for (auto v : call.getArgOperands()) b.buffers.push_back(HIPBufferOf(module, v));
    if (b.kind == KernelBinding::Relu && !b.inPlace) b.buffers.push_back(call.getResult(0));
    if (b.buffers.size() != b.argNames.size()) {
      std::cerr << "HIPBind: " << b.funcName << ": the call has " << b.buffers.size() << " operands, the kernel takes "
                << b.argNames.size() << "\n";
      continue;
    }
    b.index = static_cast<int>(out.size());
    out.push_back(b);
  }
  return out;
}

std::string HIPGen(ModuleOp &module) {
  std::ostringstream os;
  auto bindings = HIPBind(module);
  os << "// Launchers for graph \"" << module.getName() << "\": each kernelN forwards to a prebuilt\n"
     << "// gfx950 kernel of libkcg_hip.so (include/kcg.h).  Arguments are device pointers;\n"
     << "// the call is asynchronous on `stream` and returns a kcg_status.\n"
     << "#include \"kcg.h\"\n\n"
     << "namespace " << module.getName() << " {\n\n";
  for (auto &b : bindings) {
    if (b.kind == KernelBinding::Relu || b.kind == KernelBinding::BatchedMatmul || b.kind == KernelBinding::Softmax) {
      os << "// " << b.funcName << " -> " << b.entry << " (un-fused operator: no pattern matched this call; "
         << "the library picks the launch geometry from the extents)\n";
      if (b.kind == KernelBinding::Relu && b.inPlace)
        os << "inline int kernel" << b.index << "(float* arg0 /*x, in place*/, void* stream = nullptr) {\n"
           << "  return kcg_relu_f32(arg0, arg0, " << b.count << ", stream);\n}\n\n";
      else if (b.kind == KernelBinding::Relu)
        os << "inline int kernel" << b.index << "(const float* arg0 /*x*/, float* arg1 /*y*/, void* stream = nullptr) {\n"
           << "  return kcg_relu_f32(arg0, arg1, " << b.count << ", stream);\n}\n\n";
      else if (b.kind == KernelBinding::Softmax)
        os << "inline int kernel" << b.index << "(float* arg0 /*x, in place*/, void* stream = nullptr) {\n"
           << "  return kcg_softmax_f32(arg0, " << b.count / b.rowLength << ", " << b.rowLength << ", stream);\n}\n\n";
      else
        os << "inline int kernel" << b.index
           << "(const float* arg0 /*A*/, const float* arg1 /*B*/, float* arg2 /*C*/, void* stream = nullptr) {\n"
           << "  return kcg_batched_matmul_f32(arg0, " << b.transA << ", arg1, " << b.transB << ", arg2, " << b.batch
           << ", " << b.M << ", " << b.N << ", " << b.K << ", stream);\n}\n\n";
      continue;
    }
    os << "// " << b.funcName << " -> " << b.launch.kernel << "\n"
       << "// grid dims:(" << b.launch.grid[0] << ", " << b.launch.grid[1] << ", " << b.launch.grid[2]
       << "), block dims:(" << b.launch.block[0] << ", " << b.launch.block[1] << ", " << b.launch.block[2]
       << "), lds bytes:" << b.launch.lds_bytes << "\n";
    if (b.kind == KernelBinding::Gemm) {
      os << "// block_k " << b.gemmSched.block_k << ", lds stages " << b.gemmSched.lds_stages << " (0 = library's choice)"
         << ", vector width " << b.gemmSched.vec_width << ": from the " << (b.scheduleSource == "ir" ? "scheduled loop nest" : "kcg.* attributes")
         << "\n";
      if (!b.scheduleNote.empty()) os << "// note: " << b.scheduleNote << "\n";
    }
    if (b.launch.launches == 2)
      os << "// first launch: rows 0.." << b.launch.main_rows - 1 << "; second launch (" << b.launch.tail_kernel
         << "): the last " << b.launch.tail_rows << " rows, grid dims:(" << b.launch.tail_grid[0] << ", "
         << b.launch.tail_grid[1] << ", " << b.launch.tail_grid[2] << "), block dims:(" << b.launch.tail_block[0]
         << ", " << b.launch.tail_block[1] << ", " << b.launch.tail_block[2] << "), lds bytes:"
         << b.launch.tail_lds_bytes << "\n";
    if (b.kind == KernelBinding::Gemm) {
      os << "inline int kernel" << b.index
         << "(const float* arg0 /*A*/, const float* arg1 /*B*/, float* arg2 /*C*/, void* stream = nullptr) {\n"
         << "  static const kcg_gemm_sched sched = {" << b.gemmSched.block_m << ", " << b.gemmSched.block_n << ", "
         << b.gemmSched.block_k << ", " << b.gemmSched.group_m << ", " << b.gemmSched.wave_m << ", "
         << b.gemmSched.wave_n << ", " << b.gemmSched.vec_width << ", " << b.gemmSched.wave_size << ", "
         << b.gemmSched.lds_stages << "};\n"
         << "  return kcg_gemm_f32(arg0, arg1, arg2, " << b.M << ", " << b.N << ", " << b.K << ", "
         << (b.epilogue == KCG_EPILOGUE_RELU ? "KCG_EPILOGUE_RELU" : "KCG_EPILOGUE_NONE") << ", &sched, stream);\n"
         << "}\n\n";
    } else {
      char sc[64];
      snprintf(sc, sizeof sc, "%.9gf", static_cast<double>(b.scale));
      std::string scale = sc;
      if (scale.find('.') == std::string::npos && scale.find('e') == std::string::npos)
        scale.insert(scale.size() - 1, ".0");
      const bool bf = b.dtype == KCG_BF16;
      const char *ct = bf ? "const uint16_t*" : "const float*";
      os << "inline int kernel" << b.index << "(" << ct << " arg0 /*Q*/, " << ct << " arg1 /*K*/, " << ct
         << " arg2 /*V*/, " << (bf ? "uint16_t*" : "float*") << " arg3 /*O*/, void* stream = nullptr) {\n"
         << "  static const kcg_fmha_sched sched = {" << b.fmhaSched.br << ", " << b.fmhaSched.bc << "};\n";
      if (bf)
        os << "  return kcg_fmha_bf16(arg0, arg1, arg2, arg3, KCG_BF16, " << b.B << ", " << b.H << ", " << b.S
           << ", " << b.D << ", " << scale << ", " << b.causal << ", &sched, stream);\n";
      else
        os << "  return kcg_fmha_f32(arg0, arg1, arg2, arg3, " << b.B << ", " << b.H << ", " << b.S << ", " << b.D
           << ", " << scale << ", " << b.causal << ", &sched, stream);\n";
      os << "}\n\n";
    }
  }
  os << "}  // namespace " << module.getName() << "\n";
  return os.str();
}

int HIPLaunch(const KernelBinding &b, const std::vector<void *> &p, void *stream) {
  if (p.size() != b.argNames.size()) return KCG_ERR_BAD_ARGUMENT;
  if (b.kind == KernelBinding::Gemm)
    return kcg_gemm_f32(static_cast<const float *>(p[0]), static_cast<const float *>(p[1]),
                        static_cast<float *>(p[2]), b.M, b.N, b.K, b.epilogue, &b.gemmSched, stream);
  if (b.kind == KernelBinding::Relu)
    return kcg_relu_f32(static_cast<const float *>(p[0]), static_cast<float *>(b.inPlace ? p[0] : p[1]), b.count,
                        stream);
  if (b.kind == KernelBinding::Softmax)
    return kcg_softmax_f32(static_cast<float *>(p[0]), b.count / b.rowLength, b.rowLength, stream);
  if (b.kind == KernelBinding::BatchedMatmul)
    return kcg_batched_matmul_f32(static_cast<const float *>(p[0]), b.transA, static_cast<const float *>(p[1]),
                                  b.transB, static_cast<float *>(p[2]), b.batch, b.M, b.N, b.K, stream);
  if (b.dtype == KCG_BF16)
    return kcg_fmha_bf16(static_cast<const uint16_t *>(p[0]), static_cast<const uint16_t *>(p[1]),
                         static_cast<const uint16_t *>(p[2]), p[3], KCG_BF16, b.B, b.H, b.S, b.D, b.scale,
                         b.causal, &b.fmhaSched, stream);
  return kcg_fmha_f32(static_cast<const float *>(p[0]), static_cast<const float *>(p[1]),
                      static_cast<const float *>(p[2]), static_cast<float *>(p[3]), b.B, b.H, b.S, b.D, b.scale,
                      b.causal, &b.fmhaSched, stream);
}

}  // namespace KernelCodeGen
