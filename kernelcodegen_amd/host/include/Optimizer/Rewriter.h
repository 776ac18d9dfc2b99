// Schedule primitives over the affine IR (reference: include/Optimizer/Rewriter.h).
//
// The four primitives the matmul and attention recipes are built from --
// split, reorder, parallel, bufferizeLoopCarryVar -- plus buffer allocation,
// barriers and the small builders the recipes use.  Every primitive keeps the
// handles the caller already holds valid (a loop that is re-nested or loses its
// iter_arg stays the same op), and reports a violated precondition by printing
// a message and leaving the IR untouched instead of asserting.
#pragma once

#include <vector>

#include "IR/IR.h"
#include "Optimizer/Analyzer.h"
#include "enum.h"

namespace KernelCodeGen {

struct Rewriter {
  // Induction variables of a grid / block level, outermost dimension first.
  static std::vector<ir::Value> getParallelIdx(ir::ParallelOp parallelLevel) { return parallelLevel.getIVs(); }

  // Tiles `forOp` (lower bound 0, step 1, no iter_args) into `num_output` nested
  // loops.  `factors` lists the tile extents innermost first, e.g.
  //   split(i, 3, {8, 128}):  for io = 0 to N step 128 / for im = 0 to 128 step 8 / for ii = 0 to 8
  // Every subscript that used the old induction variable now uses io + im + ii.
  // Returns the new loops outermost first; empty on a violated precondition
  // (the extents must divide each other and the trip count).
  static std::vector<ir::ForOp> split(ir::ForOp forOp, uint64_t num_output, std::vector<int64_t> &&factors);

  // Turns the iter_arg of the one loop in `loops` that carries a value into a
  // register buffer (MemorySpace::local) indexed by the induction variables of
  // the other listed loops that enclose it: initial value stored where it is
  // defined, load at the top of the loop body, store in place of the yield, load
  // after the loop for the users of its result.  The buffer is allocated at the
  // start of the closest enclosing parallel / function / module body.
  // Returns the buffer (null when no listed loop carries a value).
  static ir::Value bufferizeLoopCarryVar(std::vector<ir::ForOp> &loops);

  // Re-nests the listed loops (each nested in the previous one, possibly with
  // other statements in between) into the given order, outermost first.  A loop
  // that holds statements before / after the loop it is exchanged with is
  // split into copies that keep those statements (loop fission).
  static void reorder(const std::vector<ir::ForOp> &loops);

  // Replaces a perfect nest of up to three loops by one affine.parallel with
  // lower bounds 0 and steps 1; an original step s > 1 becomes an
  // `affine.apply d0 * s` at the top of the body.
  static ir::ParallelOp parallel(const std::vector<ir::ForOp> &forOps);

  // memref.alloc at the start of `father`'s body.
  static ir::Value alloc_buffer(ir::OpHandle father, MemorySpace ms, const std::vector<int64_t> &shape,
                                ir::DType dtype);
  // memref.alloc right before / after `contextOp`.
  static ir::Value alloc_buffer(ir::OpHandle contextOp, Position pos, MemorySpace ms,
                                const std::vector<int64_t> &shape, ir::DType dtype);

  // gpu.barrier before / after `compute_at`, or at the begin / end of its body.
  static ir::Op *barrier(ir::ForOp compute_at, Position pos);

  // Empty loop [lowerBound, upperBound) by `step` appended to `where`.
  static ir::ForOp create_constant_loop(ir::OpHandle where, int64_t lowerBound, int64_t upperBound,
                                        int64_t step);

  // Fills `mem` with `targetValue` (a loop nest of stores) at the end of `where`.
  static void set_buffer(ir::OpHandle where, ir::Value mem, ir::Value targetValue);

  // tileC[i][j] += fragA[i] * fragB[j] for i < m, j < n, appended to `where`;
  // returns the outer loop.
  static ir::ForOp outer_product(ir::OpHandle where, ir::Value tileC, ir::Value fragA, ir::Value fragB,
                                 int64_t m, int64_t n);

  // Marks loops with at most `maxTrips` iterations {affine.loop = "unroll"}.
  static void unrollAttribute(ir::ModuleOp module, int64_t maxTrips);
};

}  // namespace KernelCodeGen
