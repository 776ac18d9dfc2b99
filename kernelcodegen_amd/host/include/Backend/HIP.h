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
  // Gemm and Fmha: functions the optimizers brought into state "gpu".  Relu, BatchedMatmul
  // and Softmax: calls of functions still in state "cpu" -- a graph the attention pattern
  // does not match (src/Optimizer/Optimizer.cc:597-652 of the reference falls through), or
  // an operator on its own -- bound one kernel per call to the un-fused entry points.  (The
  // reference's emitter prints nothing for them: src/Backend/CUDA.cc:859-866 only visits
  // functions that hold an affine.parallel.)
  enum Kind { Gemm, Fmha, Relu, BatchedMatmul, Softmax } kind = Gemm;
  std::string graph;      // module name = namespace of the launcher
  std::string funcName;   // Matmul_m..n..k.. / Fused_Multi_Head_Attention_.. / Relu_Elementwise_.. /
                          // BatchMatmul_.._<N|T><N|T> / Softmax_.._axis<k>
  std::string entry;      // kcg_gemm_f32 / kcg_fmha_f32 / kcg_fmha_bf16 / kcg_relu_f32 /
                          // kcg_batched_matmul_f32 / kcg_softmax_f32
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
  // un-fused operators
  int64_t batch = 1;          // BatchedMatmul: number of matrices (M, N, K above)
  int transA = 0, transB = 0; // BatchedMatmul: the name's <N|T><N|T> suffix
  int64_t count = 0;          // Relu: elements; Softmax: rows x rowLength
  int64_t rowLength = 0;      // Softmax: extent of the last axis
  bool inPlace = false;       // Relu on MemorySpace::inplace, Softmax always
  // launch geometry reported by the library for this binding (Gemm, Fmha; the un-fused
  // entry points choose theirs at launch and have no query: kernel holds the entry name)
  kcg_launch_info launch{};
  // device pointer order of the call: A,B,C / Q,K,V,O / x[,y] / x
  std::vector<std::string> argNames;
  // bytes behind each of those pointers
  std::vector<size_t> argBytes;
  // The module-level buffer each pointer stands for: a PlaceHolder / result allocation of the
  // module, looked through the calls that work in place or write into an operand (the result
  // of Softmax(S) is S's buffer, the result of a BatchedMatmul call is its C operand).  An
  // out-of-place Relu writes a buffer that only exists as its call's result: that value.
  // Two bindings that name the same buffer must be given the same device pointer.
  std::vector<ir::Value> buffers;
};

// The module-level buffer a graph value lives in (see KernelBinding::buffers).
ir::Value HIPBufferOf(ir::ModuleOp &module, ir::Value v);

// One binding per call, in module order: functions in state "gpu" through their schedule,
// the un-fused operators in state "cpu" through their shapes.  Calls the library has no
// kernel for are reported on stderr and skipped.
std::vector<KernelBinding> HIPBind(ir::ModuleOp &module);

// Launcher translation unit for the module (see INTEGRATION notes in kcg.h).
std::string HIPGen(ir::ModuleOp &module);

// Launches the bound kernel on `stream` with caller-owned device pointers in
// argNames order.  Returns the kcg_status of the call.
int HIPLaunch(const KernelBinding &binding, const std::vector<void *> &devicePtrs, void *stream);

}  // namespace KernelCodeGen
