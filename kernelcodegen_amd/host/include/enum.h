// Enumerations shared by the Frontend, the Optimizer and the backend binding.
// Values follow the reference (include/enum.h:5-29) so that memory-space
// integers printed in memref types read the same.
#pragma once

namespace KernelCodeGen {

enum class Target { CUDA = 0, ROCm = 1 };

enum class MemorySpace {
  global = 1,       // HBM
  shared = 2,       // LDS
  local = 3,        // registers
  constant = 4,
  unallocated = 5,
  inplace = 6,      // operator writes its result over its input
};

enum class Position { before = 0, after = 1, begin = 2, end = 3 };

enum class Layout { rowMajor = 0, colMajor = 1 };

}  // namespace KernelCodeGen
