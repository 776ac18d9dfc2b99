#include "Backend/HIPTimer.h"

#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <cstdio>
#include <iostream>

#include "Optimizer/Analyzer.h"

namespace KernelCodeGen {

namespace {

// xorshift stream -> uniform [-1, 1); bf16 = upper half of the float
void fill(std::vector<uint32_t> &words, bool bf16, uint64_t seed) {
  uint64_t x = seed * 0x9E3779B97F4A7C15ull + 0xD1B54A32D192ED03ull;
  auto next = [&]() {
    x ^= x << 13;
    x ^= x >> 7;
    x ^= x << 17;
    return x;
  };
  auto f32bits = [&]() {
    const float v = static_cast<float>(static_cast<double>(next() >> 40) / 8388608.0 - 1.0);
    uint32_t u;
    __builtin_memcpy(&u, &v, 4);
    return u;
  };
  for (auto &w : words) w = bf16 ? ((f32bits() >> 16) | (f32bits() & 0xffff0000u)) : f32bits();
}

std::string scheduleText(const KernelBinding &b) {
  char buf[64];
  if (b.kind == KernelBinding::Gemm)
    snprintf(buf, sizeof buf, "%dx%dx%d", b.gemmSched.block_m, b.gemmSched.block_n, b.gemmSched.block_k);
  else if (b.kind == KernelBinding::Fmha)
    snprintf(buf, sizeof buf, "br%d bc%d", b.fmhaSched.br, b.fmhaSched.bc);
  else
    snprintf(buf, sizeof buf, "unfused");
  return buf;
}

}  // namespace

HIPTimer::HIPTimer(int warmup, int iters) : warmup_(warmup), iters_(iters < 1 ? 1 : iters) {
  hipStream_t s;
  hipEvent_t a, b;
  if (hipStreamCreate(&s) != hipSuccess) return;
  if (hipEventCreate(&a) != hipSuccess || hipEventCreate(&b) != hipSuccess) return;
  stream_ = s;
  start_ = a;
  stop_ = b;
  ok_ = true;
}

HIPTimer::~HIPTimer() {
  for (void *p : pool_)
    if (p) (void)hipFree(p);
  if (start_) (void)hipEventDestroy(static_cast<hipEvent_t>(start_));
  if (stop_) (void)hipEventDestroy(static_cast<hipEvent_t>(stop_));
  if (stream_) (void)hipStreamDestroy(static_cast<hipStream_t>(stream_));
}

void *HIPTimer::buffer(size_t slot, size_t bytes, bool bf16) {
  if (pool_.size() <= slot) {
    pool_.resize(slot + 1, nullptr);
    poolBytes_.resize(slot + 1, 0);
  }
  if (poolBytes_[slot] >= bytes) return pool_[slot];
  if (pool_[slot]) (void)hipFree(pool_[slot]);
  pool_[slot] = nullptr;
  poolBytes_[slot] = 0;
  void *d = nullptr;
  if (hipMalloc(&d, bytes) != hipSuccess) return nullptr;
  std::vector<uint32_t> host((bytes + 3) / 4);
  fill(host, bf16, 0xC0DE + slot);
  if (hipMemcpy(d, host.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
    (void)hipFree(d);
    return nullptr;
  }
  pool_[slot] = d;
  poolBytes_[slot] = bytes;
  return d;
}

float HIPTimer::operator()(ir::ModuleOp &module) {
  if (!ok_) return FLT_MAX;
  auto bindings = HIPBind(module);
  if (bindings.empty()) {
    // the library refused the schedule (or there is nothing to bind): say which one
    for (auto f : Analyzer::collectFunctions(module)) {
      if (f.getAttr("func.state") != "gpu") continue;
      TimedTrial t;
      t.func = f.getSymName();
      t.status = KCG_ERR_BAD_SCHEDULE;
      if (!f.getAttr("kcg.BLOCK_SIZE_M").empty())
        t.schedule = f.getAttr("kcg.BLOCK_SIZE_M") + "x" + f.getAttr("kcg.BLOCK_SIZE_N") + "x" +
                     f.getAttr("kcg.BLOCK_SIZE_K");
      else
        t.schedule = "br" + f.getAttr("kcg.Br") + " bc" + f.getAttr("kcg.Bc");
      trials_.push_back(t);
    }
    return FLT_MAX;
  }
  float total = 0.0f;
  for (auto &b : bindings) {
    TimedTrial t;
    t.func = b.funcName;
    t.kernel = b.launch.kernel;
    t.schedule = scheduleText(b);
    const std::vector<size_t> &bytes = b.argBytes;
    const bool bf16 = b.kind == KernelBinding::Fmha && b.dtype == KCG_BF16;
    std::vector<void *> ptrs;
    for (size_t i = 0; i < bytes.size(); ++i) ptrs.push_back(buffer(i, bytes[i], bf16));
    bool allocated = true;
    for (void *p : ptrs) allocated = allocated && p != nullptr;
    if (!allocated) {
      t.status = KCG_ERR_LAUNCH;
      trials_.push_back(t);
      return FLT_MAX;
    }
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int st = KCG_OK;
    // the very first kernel of a process also pays for the clocks ramping up
    const int warm = warmup_ + (trials_.empty() ? 2 * iters_ : 0);
    for (int i = 0; i < warm && st == KCG_OK; ++i) st = HIPLaunch(b, ptrs, stream);
    if (st == KCG_OK && hipEventRecord(static_cast<hipEvent_t>(start_), stream) != hipSuccess) st = KCG_ERR_LAUNCH;
    for (int i = 0; i < iters_ && st == KCG_OK; ++i) st = HIPLaunch(b, ptrs, stream);
    if (st == KCG_OK && hipEventRecord(static_cast<hipEvent_t>(stop_), stream) != hipSuccess) st = KCG_ERR_LAUNCH;
    float ms = 0.0f;
    if (st == KCG_OK && (hipEventSynchronize(static_cast<hipEvent_t>(stop_)) != hipSuccess ||
                         hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start_),
                                             static_cast<hipEvent_t>(stop_)) != hipSuccess))
      st = KCG_ERR_LAUNCH;
    t.status = st;
    if (st != KCG_OK) {
      (void)hipStreamSynchronize(stream);
      trials_.push_back(t);
      return FLT_MAX;
    }
    t.ms = ms / static_cast<float>(iters_);
    total += t.ms;
    trials_.push_back(t);
  }
  return total;
}

}  // namespace KernelCodeGen
