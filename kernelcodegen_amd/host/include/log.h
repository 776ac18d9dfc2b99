// Two-level log switch (reference: include/log.h).  Debug prints the IR after
// every rewrite; Release is silent.
#pragma once

enum Log { Debug = 0, Release = 1 };

namespace KernelCodeGen {
struct KCGLog {
  static Log level;
};
}  // namespace KernelCodeGen
