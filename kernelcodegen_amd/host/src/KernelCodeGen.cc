#include "KernelCodeGen.h"

#include <fstream>
#include <iostream>

namespace KernelCodeGen {

KernelCodeGenerator::KernelCodeGenerator(const std::string &platform_) : platform(platform_) {
  opts.push_back(std::make_unique<MatmulOptimizer>());
  opts.push_back(std::make_unique<FMHAOptimizer>());
  // gfx950 tile tables.  The first entry of each is the default the kernels are
  // tuned for; the matmul table also carries the reference's own 128x128x8 tile
  // (include/KernelCodeGen.h:34-37 there) for comparison runs.
  matmulConfigs = {
      {{"BLOCK_SIZE_M", 256}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 16}, {"GROUP_SIZE_M", 8},
       {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8}, {"WAVE_SIZE_M", 64}, {"WAVE_SIZE_N", 64},
       {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}},
      {{"BLOCK_SIZE_M", 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", 8}, {"GROUP_SIZE_M", 8},
       {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8}, {"WAVE_SIZE_M", 64}, {"WAVE_SIZE_N", 64},
       {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64}},
  };
  fmhaConfigs = {
      {{"BLOCK_SIZE", 256}, {"Br", 128}, {"Bc", 32}, {"WARP_SIZE", 64}},
      {{"BLOCK_SIZE", 256}, {"Br", 128}, {"Bc", 64}, {"WARP_SIZE", 64}},
  };
}

void KernelCodeGenerator::useCandidateTables() {
  auto mm = [](int bm, int bn, int bk, int wm, int wn) {
    return std::map<std::string, int>{{"BLOCK_SIZE_M", bm}, {"BLOCK_SIZE_N", bn}, {"BLOCK_SIZE_K", bk},
                                      {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8},
                                      {"WAVE_SIZE_M", wm}, {"WAVE_SIZE_N", wn}, {"VECTORIZE_WIDTH", 4},
                                      {"WARP_SIZE", 64}};
  };
  matmulConfigs = {mm(256, 128, 16, 64, 64), mm(256, 128, 32, 64, 64), mm(128, 128, 16, 64, 64),
                   mm(128, 128, 32, 64, 64), mm(128, 128, 8, 64, 64),  mm(128, 64, 32, 64, 32),
                   mm(64, 64, 32, 32, 32),   mm(96, 96, 32, 48, 48),
                   mm(96, 64, 32, 48, 32)};
  // fp32 attention is built for Br 128|256 x Bc 32|64 (not 256 x 64 at head dim 128), bf16 for
  // Br 128|256 x Bc 64; candidates a data type has no kernel for are refused at bind time
  // and score FLT_MAX.
  fmhaConfigs = {
      {{"BLOCK_SIZE", 256}, {"Br", 128}, {"Bc", 32}, {"WARP_SIZE", 64}},
      {{"BLOCK_SIZE", 256}, {"Br", 128}, {"Bc", 64}, {"WARP_SIZE", 64}},
      {{"BLOCK_SIZE", 512}, {"Br", 256}, {"Bc", 32}, {"WARP_SIZE", 64}},
      {{"BLOCK_SIZE", 512}, {"Br", 256}, {"Bc", 64}, {"WARP_SIZE", 64}},
  };
}

ComputeDAG &KernelCodeGenerator::createGraph(const std::string &graphName) {
  minLatency = FLT_MAX;
  graph.module = ir::ModuleOp::create(graphName);
  return graph;
}

void KernelCodeGenerator::dump(ir::ModuleOp &module, const std::string &info) {
  const std::string problem = ir::verify(module.get());
  if (KCGLog::level != Log::Release) {
    std::cerr << "----------------------------------------------------------\n"
              << "           " << info << "\n"
              << "----------------------------------------------------------\n"
              << module.str();
  }
  if (!problem.empty()) std::cerr << "module verification error: " << problem << "\n";
}

void KernelCodeGenerator::save(const std::string &str, const std::string &file) {
  if (file == "terminal") {
    std::cout << str;
    return;
  }
  std::ofstream out(file.c_str());
  if (!out.is_open()) {
    std::cerr << "Can't open file \"" << file << "\"\n";
    return;
  }
  out << str;
}

ir::ModuleOp &KernelCodeGenerator::optimize(ComputeDAG &graph_) {
  if (&graph_ != &graph) graph = graph_;
  ir::ModuleOp module = graph.module.clone();
  saveBestModule(module);
  minLatency = FLT_MAX;

  // An optimizer that applies rewrites the running module; later optimizers see
  // its result (a graph may hold a matmul and an attention block).
  for (auto &opt : opts) {
    backupModule(module);
    std::vector<std::map<std::string, int>> none{{}};
    const bool isMatmul = opt->name == "Matmul", isFmha = opt->name == "FMHA";
    auto &configs = isMatmul ? matmulConfigs : isFmha ? fmhaConfigs : none;
    float best = FLT_MAX;
    bool any = false;
    ir::ModuleOp bestHere;
    for (auto &config : configs) {
      if (isMatmul) MatmulOptimizer::matmulConfig = config;
      if (isFmha) FMHAOptimizer::fmhaConfig = config;
      resetModule(module);
      if (!opt->applicable(module)) break;
      opt->applyOptimzer(module);
      const float latency = evaluate(module);
      if (latency < best) {
        best = latency;
        bestHere = module.clone();
        any = true;
      }
    }
    if (any) {
      module = bestHere;
      minLatency = best;
      saveBestModule(module);
    } else {
      resetModule(module);
    }
  }
  return bestModule;
}

std::string KernelCodeGenerator::codegen(ir::ModuleOp module) {
  if (platform == "ROCm") return HIPGen(module);
  std::cerr << "codegen: platform \"" << platform << "\" has no backend here (use \"ROCm\")\n";
  return {};
}

}  // namespace KernelCodeGen
