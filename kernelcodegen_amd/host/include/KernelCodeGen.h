// Driver facade (reference: include/KernelCodeGen.h:25-144).
//
//   KernelCodeGenerator generator("ROCm");
//   auto& graph = generator.createGraph("matmul_demo");
//   auto A = graph.create<PlaceHolder>(std::vector<int64_t>{m, k}, std::string{"float32"});
//   ...
//   auto module = generator.optimize(graph);
//   auto source = generator.codegen(module);        // launcher text
//   generator.save(source, "matmulKernel.hip.cc");
//
// Differences from the reference: the default platform is "ROCm" (the only one
// with a backend here; "CUDA" yields an empty string and a message rather than
// falling off the end of the function); both optimizers are registered (the
// reference has MatmulOptimizer commented out); evaluate() can be given a real
// cost function instead of the constant 0.
#pragma once

#include <cfloat>
#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "Backend/HIP.h"
#include "Frontend/Operators.h"
#include "Optimizer/Optimizer.h"
#include "log.h"

namespace KernelCodeGen {

class KernelCodeGenerator {
 public:
  explicit KernelCodeGenerator(const std::string &platform_ = {"ROCm"});
  KernelCodeGenerator(const KernelCodeGenerator &) = delete;

  // Starts a new, empty module named `graphName` and returns the graph that builds it.
  ComputeDAG &createGraph(const std::string &graphName);
  ComputeDAG &getGraph() { return graph; }

  // Prints `module` with a banner (Debug log level) and verifies it.
  void dump(ir::ModuleOp &module, const std::string &info = "");

  // Writes `str` to `file` ("terminal" = stdout).
  void save(const std::string &str, const std::string &file);

  void resetModule(ir::ModuleOp &module) { module = backupModule_.clone(); }
  void backupModule(ir::ModuleOp &module) { backupModule_ = module.clone(); }
  void saveBestModule(ir::ModuleOp &module) { bestModule = module.clone(); }

  // Tries every optimizer with every configuration of its table on a copy of
  // the graph's module, keeps the one `evaluate` scores lowest, returns it.
  ir::ModuleOp &optimize(ComputeDAG &graph_);

  // Latency estimate of an optimised module; the reference's is the constant 0
  // (so its first applicable configuration wins).  setEvaluator installs a
  // measured one (e.g. timing HIPLaunch on the device).
  float evaluate(ir::ModuleOp &module) { return evaluator ? evaluator(module) : 0.0f; }
  void setEvaluator(std::function<float(ir::ModuleOp &)> fn) { evaluator = std::move(fn); }

  // Launcher source for the platform's backend.
  std::string codegen(ir::ModuleOp module);
  // Kernel bindings of the module (what codegen prints, as data).
  std::vector<KernelBinding> bind(ir::ModuleOp module) { return HIPBind(module); }

  void setLogMode(Log level) { KCGLog::level = level; }

  // Replaces the two config tables by the gfx950 search space: every tile shape
  // the kernel library builds.  Meant for use with a measured evaluator; with
  // the default evaluate() (constant 0) the first entry still wins.
  void useCandidateTables();
  // evaluate() of the module optimize() returned (FLT_MAX before any call).
  float bestLatency() const { return minLatency; }

  std::vector<std::map<std::string, int>> matmulConfigs;
  std::vector<std::map<std::string, int>> fmhaConfigs;

 private:
  ir::ModuleOp backupModule_;
  ir::ModuleOp bestModule;
  ComputeDAG graph;
  std::string platform;
  float minLatency = FLT_MAX;
  std::vector<std::unique_ptr<Optimizer>> opts;
  std::function<float(ir::ModuleOp &)> evaluator;
};

}  // namespace KernelCodeGen
