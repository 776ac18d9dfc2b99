// GPU demo of the host layer: the reference's test_matmul / test_flash_attention
// flows (test/test.cc:8-107 there) carried through to a launch on the device.
//
//   demo_rocm matmul M N K relu(0|1) out.bin
//   demo_rocm sched  M N K relu(0|1) detail(0|1|2|3) out.bin   the reference's 128 x 128 x 8 tile
//                    with the staged (1), pipelined (2) or direct-load (3: no register tile,
//                    a ring of three shared copies) schedule built on the IR: the binding
//                    reads block_k, the LDS buffer count and the vector width off the
//                    scheduled nest ("schedule <source> block_k <n> lds_stages <n> vec_width
//                    <n>" is printed)
//   demo_rocm sched256 M N K relu detail out.bin   the same on the library's default tile,
//                    256 x 128 x 16 with eight waves of 64 x 64
//   demo_rocm fmha   B H S D causal(0|1) scale out.bin
//   demo_rocm fmharef B H S D causal(0|1) scale out.bin    the reference's own attention table
//                    (HdxBr = BrxBc = 8192, include/KernelCodeGen.h:38-41 there): Br 64 x Bc 128
//                    at head dim 128, Br 128 x Bc 64 at head dim 64
//   demo_rocm unfused attn B H S D out.bin     S = Q.K^T, R = Relu(S) into a buffer of its own,
//                    P = Softmax(S), O = P.V: the score tensor has two users, the attention
//                    pattern does not match, and the four calls are bound one kernel each to
//                    the un-fused entry points; out.bin holds O followed by R
//   demo_rocm unfused softmax ROWS N out.bin   a Softmax on its own, in place
//   demo_rocm tune matmul M N K relu(0|1) out.bin
//   demo_rocm tune fmha   B H S D causal(0|1) scale out.bin
//
// The tune forms run the reference's config trial loop (src/KernelCodeGen.cc:15-51)
// with a measured evaluate(): every candidate schedule is timed on the device,
// the trials are printed as "trial <schedule> <kernel> <ms|refused>", the winner
// as "best <schedule> <ms>", and the winner's output is written to out.bin.
//
// Builds the graph through KernelCodeGenerator, optimizes it, binds the result
// to the gfx950 kernel, runs it on seeded uniform[-1,1) inputs (the generator of
// kernelcodegen_amd/inputs.py: splitmix64 of seed ^ tensor<<56 ^ index, top 24
// bits), and writes the raw fp32 output to out.bin for the caller to check.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <vector>

#include "Backend/HIPTimer.h"
#include "KernelCodeGen.h"

using namespace KernelCodeGen;

static const uint64_t kSeed = 0xD3A0;

static void fill_uniform(std::vector<float> &v, uint64_t seed, uint64_t tensor) {
  for (size_t i = 0; i < v.size(); ++i) {
    uint64_t x = (seed ^ (tensor << 56) ^ static_cast<uint64_t>(i)) + 0x9E3779B97F4A7C15ull;
    uint64_t z = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    v[i] = static_cast<float>(static_cast<double>(z >> 40) / 8388608.0 - 1.0);
  }
}

#define HIP_OK(call)                                                             \
  do {                                                                           \
    hipError_t e_ = (call);                                                      \
    if (e_ != hipSuccess) {                                                      \
      std::fprintf(stderr, "%s failed: %s\n", #call, hipGetErrorString(e_));     \
      return 2;                                                                  \
    }                                                                            \
  } while (0)

static int run(const KernelBinding &b, const std::vector<std::vector<float> *> &inputs, size_t outCount,
               const char *outPath) {
  std::vector<void *> dev;
  for (auto *h : inputs) {
    void *d = nullptr;
    HIP_OK(hipMalloc(&d, h->size() * sizeof(float)));
    HIP_OK(hipMemcpy(d, h->data(), h->size() * sizeof(float), hipMemcpyHostToDevice));
    dev.push_back(d);
  }
  void *out = nullptr;
  HIP_OK(hipMalloc(&out, outCount * sizeof(float)));
  HIP_OK(hipMemset(out, 0xFF, outCount * sizeof(float)));
  dev.push_back(out);
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  const int st = HIPLaunch(b, dev, stream);
  if (st != KCG_OK) {
    std::fprintf(stderr, "launch failed: %s\n", kcg_status_str(st));
    return 3;
  }
  HIP_OK(hipStreamSynchronize(stream));
  std::vector<float> host(outCount);
  HIP_OK(hipMemcpy(host.data(), out, outCount * sizeof(float), hipMemcpyDeviceToHost));
  FILE *fp = std::fopen(outPath, "wb");
  if (!fp) return 4;
  std::fwrite(host.data(), sizeof(float), host.size(), fp);
  std::fclose(fp);
  for (void *d : dev) HIP_OK(hipFree(d));
  HIP_OK(hipStreamDestroy(stream));
  return 0;
}

// Runs every binding of a module in order.  One device buffer per distinct module-level
// buffer (KernelBinding::buffers): `inputs` are uploaded, the others start as zeros;
// `outputs` are written to outPath one after the other.
static int runGraph(const std::vector<KernelBinding> &bindings,
                    const std::vector<std::pair<ir::Value, std::vector<float> *>> &inputs,
                    const std::vector<ir::Value> &outputs, const char *outPath) {
  std::vector<std::pair<ir::Value, void *>> dev;
  std::vector<size_t> bytes;
  auto find = [&](ir::Value v) -> int {
    for (size_t i = 0; i < dev.size(); ++i)
      if (dev[i].first == v) return static_cast<int>(i);
    return -1;
  };
  for (auto &b : bindings)
    for (size_t i = 0; i < b.buffers.size(); ++i) {
      if (find(b.buffers[i]) >= 0) continue;
      void *d = nullptr;
      HIP_OK(hipMalloc(&d, b.argBytes[i]));
      HIP_OK(hipMemset(d, 0, b.argBytes[i]));
      dev.emplace_back(b.buffers[i], d);
      bytes.push_back(b.argBytes[i]);
    }
  for (auto &in : inputs) {
    const int at = find(in.first);
    if (at < 0 || bytes[at] != in.second->size() * sizeof(float)) return 6;
    HIP_OK(hipMemcpy(dev[at].second, in.second->data(), bytes[at], hipMemcpyHostToDevice));
  }
  hipStream_t stream;
  HIP_OK(hipStreamCreate(&stream));
  for (auto &b : bindings) {
    std::vector<void *> p;
    for (auto v : b.buffers) p.push_back(dev[find(v)].second);
    const int st = HIPLaunch(b, p, stream);
    if (st != KCG_OK) {
      std::fprintf(stderr, "launch of %s failed: %s\n", b.funcName.c_str(), kcg_status_str(st));
      return 3;
    }
  }
  HIP_OK(hipStreamSynchronize(stream));
  FILE *fp = std::fopen(outPath, "wb");
  if (!fp) return 4;
  for (auto v : outputs) {
    const int at = find(v);
    if (at < 0) return 6;
    std::vector<float> host(bytes[at] / sizeof(float));
    HIP_OK(hipMemcpy(host.data(), dev[at].second, bytes[at], hipMemcpyDeviceToHost));
    std::fwrite(host.data(), sizeof(float), host.size(), fp);
  }
  std::fclose(fp);
  for (auto &d : dev) HIP_OK(hipFree(d.second));
  HIP_OK(hipStreamDestroy(stream));
  return 0;
}

int main(int argc, char **argv) {
  if (argc < 2) {
    std::fprintf(stderr, "usage: demo_rocm [tune] matmul M N K relu out | demo_rocm [tune] fmha B H S D causal scale out\n");
    return 1;
  }
  KernelCodeGenerator generator("ROCm");
  generator.setLogMode(Log::Release);
  HIPTimer timer(3, 20);
  bool tune = false;
  if (std::string(argv[1]) == "tune") {
    tune = true;
    generator.useCandidateTables();
    generator.setEvaluator([&](ir::ModuleOp &m) { return timer(m); });
    --argc;
    ++argv;
  }
  auto report = [&](const std::vector<KernelBinding> &bindings) {
    if (!tune) return;
    for (auto &t : timer.trials()) {
      if (t.status == KCG_OK) std::printf("trial %s %s %.5f\n", t.schedule.c_str(), t.kernel.c_str(), t.ms);
      else std::printf("trial %s - refused\n", t.schedule.c_str());
    }
    if (!bindings.empty()) {
      const KernelBinding &b = bindings[0];
      char sched[64];
      if (b.kind == KernelBinding::Gemm)
        std::snprintf(sched, sizeof sched, "%dx%dx%d", b.gemmSched.block_m, b.gemmSched.block_n, b.gemmSched.block_k);
      else
        std::snprintf(sched, sizeof sched, "br%d bc%d", b.fmhaSched.br, b.fmhaSched.bc);
      std::printf("best %s %.5f\n", sched, generator.bestLatency());
    }
  };
  std::string mode = argv[1];
  if ((mode == "sched" || mode == "sched256") && argc == 8) {
    const int detail = std::atoi(argv[6]);
    const bool big = mode == "sched256";
    generator.matmulConfigs = {{{"BLOCK_SIZE_M", big ? 256 : 128}, {"BLOCK_SIZE_N", 128}, {"BLOCK_SIZE_K", big ? 16 : 8},
                                {"GROUP_SIZE_M", 8}, {"THREAD_SIZE_M", 8}, {"THREAD_SIZE_N", 8}, {"WAVE_SIZE_M", 64},
                                {"WAVE_SIZE_N", 64}, {"VECTORIZE_WIDTH", 4}, {"WARP_SIZE", 64},
                                {"SCHEDULE_DETAIL", detail}}};
    argv[6] = argv[7];
    --argc;
    mode = "matmul";
  }
  if (mode == "matmul" && argc == 7) {
    const int64_t m = std::atoll(argv[2]), n = std::atoll(argv[3]), k = std::atoll(argv[4]);
    const bool relu = std::atoi(argv[5]) != 0;
    auto &graph = generator.createGraph("matmul_demo");
    auto A = graph.create<PlaceHolder>(std::vector<int64_t>{m, k}, std::string{"float32"});
    auto B = graph.create<PlaceHolder>(std::vector<int64_t>{k, n}, std::string{"float32"});
    auto C = graph.create<Matmul>(A, B, MemorySpace::global);
    if (relu) graph.create<Relu>(C, MemorySpace::inplace);
    auto module = generator.optimize(graph);
    auto bindings = generator.bind(module);
    if (bindings.size() != 1) return 5;
    report(bindings);
    std::printf("schedule %s block_k %d lds_stages %d vec_width %d kernel %s\n", bindings[0].scheduleSource.c_str(),
                bindings[0].gemmSched.block_k, bindings[0].gemmSched.lds_stages, bindings[0].gemmSched.vec_width,
                bindings[0].launch.kernel);
    std::printf("%s", generator.codegen(module).c_str());
    std::vector<float> a(m * k), b(k * n);
    fill_uniform(a, kSeed, 0);
    fill_uniform(b, kSeed, 1);
    return run(bindings[0], {&a, &b}, static_cast<size_t>(m * n), argv[6]);
  }
  if (mode == "unfused" && argc == 8 && std::string(argv[2]) == "attn") {
    const int64_t bsz = std::atoll(argv[3]), h = std::atoll(argv[4]), s = std::atoll(argv[5]), d = std::atoll(argv[6]);
    auto &graph = generator.createGraph("unfused_attn_demo");
    std::vector<int64_t> shape{bsz, h, s, d};
    auto Q = graph.create<PlaceHolder>(shape, std::string{"float32"});
    auto K = graph.create<PlaceHolder>(shape, std::string{"float32"});
    auto V = graph.create<PlaceHolder>(shape, std::string{"float32"});
    auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
    auto R = graph.create<Relu>(S, MemorySpace::global);   // a second reader of the scores
    auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
    auto O = graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
    auto module = generator.optimize(graph);
    auto bindings = generator.bind(module);
    std::printf("bindings %zu:", bindings.size());
    for (auto &b : bindings) std::printf(" %s", b.entry.c_str());
    std::printf("\n%s", generator.codegen(module).c_str());
    if (bindings.size() != 4) return 5;
    // the module optimize() returned is a copy: the buffers are named through its own values
    const size_t count = static_cast<size_t>(bsz * h * s * d);
    std::vector<float> q(count), kk(count), v(count);
    fill_uniform(q, kSeed, 0);
    fill_uniform(kk, kSeed, 1);
    fill_uniform(v, kSeed, 2);
    (void)Q; (void)K; (void)V; (void)R; (void)O;
    // binding 0 = Q.K^T (A, B, C), binding 1 = Relu (x, y), binding 3 = P.V (A, B, C)
    return runGraph(bindings,
                    {{bindings[0].buffers[0], &q}, {bindings[0].buffers[1], &kk}, {bindings[3].buffers[1], &v}},
                    {bindings[3].buffers[2], bindings[1].buffers[1]}, argv[7]);
  }
  if (mode == "unfused" && argc == 6 && std::string(argv[2]) == "softmax") {
    const int64_t rows = std::atoll(argv[3]), n = std::atoll(argv[4]);
    auto &graph = generator.createGraph("softmax_demo");
    auto X = graph.create<PlaceHolder>(std::vector<int64_t>{rows, n}, std::string{"float32"});
    graph.create<Softmax>(X, -1, MemorySpace::inplace);
    auto module = generator.optimize(graph);
    auto bindings = generator.bind(module);
    std::printf("bindings %zu:", bindings.size());
    for (auto &b : bindings) std::printf(" %s", b.entry.c_str());
    std::printf("\n%s", generator.codegen(module).c_str());
    if (bindings.size() != 1) return 5;
    std::vector<float> x(static_cast<size_t>(rows * n));
    fill_uniform(x, kSeed, 0);
    for (auto &e : x) e *= 4.0f;
    return runGraph(bindings, {{bindings[0].buffers[0], &x}}, {bindings[0].buffers[0]}, argv[5]);
  }
  if (mode == "fmharef" && argc == 9) {
    // the reference's own table: 128 threads, Br = 8192 / Hd, Bc = 8192 / Br
    generator.fmhaConfigs = {{{"BLOCK_SIZE", 128}, {"HdxBr", 8192}, {"BrxBc", 8192}, {"WARP_SIZE", 32}}};
    mode = "fmha";
  }
  if (mode == "fmha" && argc == 9) {
    const int64_t bsz = std::atoll(argv[2]), h = std::atoll(argv[3]), s = std::atoll(argv[4]), d = std::atoll(argv[5]);
    FMHAOptimizer::causal = std::atoi(argv[6]) != 0;
    FMHAOptimizer::scale = static_cast<float>(std::atof(argv[7]));
    auto &graph = generator.createGraph("flash_attn_demo");
    std::vector<int64_t> shape{bsz, h, s, d};
    auto Q = graph.create<PlaceHolder>(shape, std::string{"float32"});
    auto K = graph.create<PlaceHolder>(shape, std::string{"float32"});
    auto V = graph.create<PlaceHolder>(shape, std::string{"float32"});
    auto S = graph.create<BatchedMatmul>(Q, Layout::rowMajor, K, Layout::colMajor);
    auto P = graph.create<Softmax>(S, -1, MemorySpace::inplace);
    graph.create<BatchedMatmul>(P, Layout::rowMajor, V, Layout::rowMajor);
    auto module = generator.optimize(graph);
    auto bindings = generator.bind(module);
    if (bindings.size() != 1) return 5;
    report(bindings);
    std::printf("%s", generator.codegen(module).c_str());
    const size_t count = static_cast<size_t>(bsz * h * s * d);
    std::vector<float> q(count), kk(count), v(count);
    fill_uniform(q, kSeed, 0);
    fill_uniform(kk, kSeed, 1);
    fill_uniform(v, kSeed, 2);
    return run(bindings[0], {&q, &kk, &v}, count, argv[8]);
  }
  std::fprintf(stderr, "bad arguments\n");
  return 1;
}
