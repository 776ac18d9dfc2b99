// Measured cost function for KernelCodeGenerator::setEvaluator.
//
// The reference's config trial loop (src/KernelCodeGen.cc:15-51) scores every
// candidate schedule with evaluate(), which is the constant 0 there
// (include/KernelCodeGen.h:119-121), so its first applicable configuration
// always wins.  HIPTimer makes the loop real on the device: it binds the
// optimised module, launches every bound kernel on seeded pseudo-random
// inputs and returns the measured time per pass in milliseconds.
//
//   HIPTimer timer;
//   generator.useCandidateTables();
//   generator.setEvaluator([&](ir::ModuleOp &m) { return timer(m); });
//   auto module = generator.optimize(graph);      // fastest candidate
//   for (auto &t : timer.trials()) ...            // what was tried
//
// Needs the HIP runtime (link libkcg_host_rocm.a and amdhip64); the rest of the
// host layer does not.
#pragma once

#include <cfloat>
#include <string>
#include <vector>

#include "Backend/HIP.h"

namespace KernelCodeGen {

struct TimedTrial {
  std::string func;      // optimised function
  std::string kernel;    // device kernel the library picked for it
  std::string schedule;  // "256x128x16" / "br128 bc32"
  int status = KCG_OK;   // kcg_status of the launch (non-zero: not timed)
  float ms = FLT_MAX;    // average time of one launch
};

class HIPTimer {
 public:
  explicit HIPTimer(int warmup = 2, int iters = 10);
  ~HIPTimer();
  HIPTimer(const HIPTimer &) = delete;
  HIPTimer &operator=(const HIPTimer &) = delete;

  // Sum over the module's bound kernels of the average launch time (ms).
  // FLT_MAX when nothing binds, a launch is refused or a HIP call fails.
  float operator()(ir::ModuleOp &module);

  const std::vector<TimedTrial> &trials() const { return trials_; }
  void clearTrials() { trials_.clear(); }

 private:
  // grow-only device buffer per argument slot, refilled when it grows
  void *buffer(size_t slot, size_t bytes, bool bf16);
  int warmup_, iters_;
  std::vector<void *> pool_;
  std::vector<size_t> poolBytes_;
  void *stream_ = nullptr, *start_ = nullptr, *stop_ = nullptr;
  bool ok_ = false;
  std::vector<TimedTrial> trials_;
};

}  // namespace KernelCodeGen
