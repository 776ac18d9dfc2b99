// ROCm backend: binds optimised functions to the prebuilt gfx950 kernels.
//
// Takes the place of the reference's `std::string CUDAGen(mlir::ModuleOp&)`
// (include/Backend/CUDA.h:6).  Where that prints CUDA source for every
// func.func holding an affine.parallel (src/Backend/CUDA.cc:859-890), this
// backend recognises the optimised function by name and state, reads its tile
// sizes, and produces
//   * a KernelBinding: which C-ABI entry point of include/kcg.h to call, with
//     which extents, schedule and epilogue, and the launch geometry;
//   * launcher source text (HIPGen), so KernelCodeGenerator::save() still writes
//     a translation unit that defines `<graph>::kernelN(...)`;
//   * a direct launch (HIPLaunch) for host programs linked with the library.
#pragma once

#include <string>
#include <vector>

#include "IR/IR.h"
#include "kcg.h"

namespace KernelCodeGen {

struct KernelBinding {
  enum Kind { Gemm, Fmha } kind = Gemm;
  std::string graph;      // module name = namespace of the launcher
  std::string funcName;   // Matmul_m..n..k.. / Fused_Multi_Head_Attention_..
  std::string entry;      // kcg_gemm_f32 / kcg_fmha_f32 / kcg_fmha_bf16
  int index = 0;          // kernel<index> inside the namespace
  // matmul
  int64_t M = 0, N = 0, K = 0;
  int epilogue = KCG_EPILOGUE_NONE;
  kcg_gemm_sched gemmSched{};
  // Where block_k, lds_stages and vec_width came from: "ir" when the function carries a
  // staged or pipelined schedule (they are then read off the scheduled loop nest: the
  // extents of the shared tiles, the leading dimension Rewriter::pipeline gave them, the
  // width of the vector accesses), "attributes" for a nest that stops at the tiling stage.
  std::string scheduleSource = "attributes";
  std::string scheduleNote;   // anything the binding changed, in words (empty: nothing)
  // attention
  int B = 0, H = 0, S = 0, D = 0;
  int dtype = KCG_F32;
  float scale = 1.0f;
  int causal = 0;
  kcg_fmha_sched fmhaSched{};
  // launch geometry reported by the library for this binding
  kcg_launch_info launch{};
  // device pointer order of the call: A,B,C or Q,K,V,O
  std::vector<std::string> argNames;
};

// One binding per function in state "gpu", in module order.  Functions the
// library has no kernel for are reported on stderr and skipped.
std::vector<KernelBinding> HIPBind(ir::ModuleOp &module);

// Launcher translation unit for the module (see INTEGRATION notes in kcg.h).
std::string HIPGen(ir::ModuleOp &module);

// Launches the bound kernel on `stream` with caller-owned device pointers in
// argNames order.  Returns the kcg_status of the call.
int HIPLaunch(const KernelBinding &binding, const std::vector<void *> &devicePtrs, void *stream);

}  // namespace KernelCodeGen
