// Schedule primitives over the affine IR (reference: include/Optimizer/Rewriter.h).
//
// split, reorder, parallel and bufferizeLoopCarryVar tile the nest; read, write,
// barrier, cache_read, cache_write and vectorize stage tiles through shared
// memory and registers; pipeline, change_double_buffer, detach_last_loop,
// schedule and extract_loop double-buffer and software-pipeline the staging;
// take_off_true_if, delete_false_if, unroll and unrollAttribute clean up.  Plus
// buffer allocation and the small builders the recipes use.  Every primitive keeps the
// handles the caller already holds valid (a loop that is re-nested or loses its
// iter_arg stays the same op), and reports a violated precondition by printing
// a message and leaving the IR untouched instead of asserting.
#pragma once

#include <vector>

#include <functional>

#include "IR/AffineMap.h"
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
  // Same with the reference's predicate form (src/Optimizer/Rewriter.cc:1574-1603).
  static void unrollAttribute(ir::ModuleOp module, const std::function<bool(ir::ForOp)> &unrollCheckFn);

  // ---- staging through registers and shared memory (Rewriter.cc:601-807 there) ----

  // Copy loop  for i = 0 to dst.size / width:  dst[i * width .. +width) = src[map(operands, i)] .. +width)
  // placed before / after `compute_at` or at the begin / end of its body.  `dst` is a
  // one-dimensional register buffer; the loop's induction variable is bound to the
  // map's dimension operands.size().  Returns the loop.
  static ir::ForOp read(ir::Value src, ir::Value dst, const ir::AffineMap &map, std::vector<ir::Value> operands,
                        int64_t width, ir::ForOp compute_at, Position pos);
  // The same loop appended to `where`.
  static ir::ForOp read(ir::OpHandle where, ir::Value src, ir::Value dst, const ir::AffineMap &map,
                        std::vector<ir::Value> operands, int64_t width);

  // Copy loop out of a one-dimensional register buffer `src`:
  //   for i = 0 to src.size / width:  dst[map(operands, i)] .. +width) = src[i * width .. +width)
  // When the map has two dimensions more than there are operands the vector is
  // scattered element by element (an inner loop j < width binds the last
  // dimension, src[i * width + j] goes to dst[map(operands, i, j)]): a transposing store.
  static ir::ForOp write(ir::Value src, ir::Value dst, const ir::AffineMap &map, std::vector<ir::Value> operands,
                         int64_t width, ir::ForOp compute_at, Position pos);
  static ir::ForOp write(ir::OpHandle where, ir::Value src, ir::Value dst, const ir::AffineMap &map,
                         std::vector<ir::Value> operands, int64_t width);

  // Copy loop from memory to memory, with no register buffer in between (gfx950 loads
  // global memory straight into LDS; the reference stages through registers with read +
  // write):
  //   for i = 0 to count / width:  dst[dstMap(dstOperands, i)] .. +width) = src[srcMap(srcOperands, i)] .. +width)
  // When dstMap has two dimensions more than there are dstOperands the `width` elements are
  // stored one by one (an inner loop j < width binds the last dimension), which transposes
  // on the way as write's scattering form does.
  static ir::ForOp copy(ir::Value src, const ir::AffineMap &srcMap, std::vector<ir::Value> srcOperands,
                        ir::Value dst, const ir::AffineMap &dstMap, std::vector<ir::Value> dstOperands,
                        int64_t count, int64_t width, ir::ForOp compute_at, Position pos);

  // Every scalar load of `src` inside `scope` becomes a load of cached[map(operands)].
  static void cache_read(ir::ForOp scope, ir::Value src, ir::Value cached, const ir::AffineMap &map,
                         const std::vector<ir::Value> &operands);
  // Every scalar store to `src` inside `scope` is re-subscripted: src[map(operands)].
  // (`cached` names the buffer the stored values come from; like the reference,
  // Rewriter.cc:755-762, the store keeps its target.)
  static void cache_write(ir::ForOp scope, ir::Value src, ir::Value cached, const ir::AffineMap &map,
                          const std::vector<ir::Value> &operands);

  // For every store to `dst` under `parallelLevel`: the loops that enclose it, outermost first.
  static std::vector<std::vector<ir::ForOp>> get_write(ir::ParallelOp parallelLevel, ir::Value dst);

  // Sets the step of `readOrWrite` (lower bound 0, step 1, trip count a multiple of
  // `width`) to `width` and turns the loads and stores in its body into vector
  // operations of that width.  Returns the loop (null on a violated precondition).
  static ir::ForOp vectorize(ir::ForOp readOrWrite, int64_t width);

  // ---- double buffering and software pipelining (Rewriter.cc:809-1284, 1614-1643) ----

  // Double-buffers `buffer`, which the loops `readBodys` (inside `compute_at`, in
  // program order) fill once per iteration of `compute_at`:
  //   * the buffer gets a leading dimension of extent 2 (`buffer` is updated);
  //   * copies of readBodys with iv = lower bound, filling half 0, are placed before compute_at;
  //   * inside compute_at the original readBodys are moved into
  //       affine.if (iv + 2 * step <= ub) { ... }
  //     at the top of the body, fetch for iv + step and fill half (iv / step + 1) mod 2;
  //   * every other access to the buffer reads half (iv / step) mod 2.
  // Returns {prologue loops, in-loop loops}.
  static std::vector<std::vector<ir::ForOp>> pipeline(std::vector<ir::ForOp> readBodys, ir::Value &buffer,
                                                      ir::ForOp compute_at);
  // The same with a ring of `stages` copies (the reference hard-codes 2,
  // src/Optimizer/Rewriter.cc:809-1180): the leading dimension becomes `stages`, the
  // prologue fills the copies of the first stages - 1 iterations (result[0]: those loops,
  // iteration-major), iteration i fetches iteration i + stages - 1 into copy
  // (i + stages - 1) mod stages while one exists and every other access reads copy
  // i mod stages.  One barrier per iteration (at its end) keeps such a ring coherent: the
  // copy overwritten in iteration i is the one read in iteration i - 1.
  static std::vector<std::vector<ir::ForOp>> pipeline(std::vector<ir::ForOp> readBodys, ir::Value &buffer,
                                                      ir::ForOp compute_at, int stages);
  // Accesses to the double buffer `buffer` inside `forOp` switch to the other half.
  static void change_double_buffer(ir::ForOp forOp, ir::Value buffer);
  // Peels the last iteration: the loop stops one step early and a copy of its
  // body with iv = ub - step follows it.
  static void detach_last_loop(ir::ForOp forOp);
  // Moves `srcOp` before / after `dstOp`, or to the end of the loop `dstOp`.
  static void schedule(ir::Op *srcOp, ir::Op *dstOp, Position pos);
  // Copy of `srcOp` with forOp's induction variable fixed to its value in
  // iteration `iteration`, placed before `forOp`.  Returns the copy.
  static ir::Op *extract_loop(ir::Op *srcOp, ir::ForOp forOp, int64_t iteration);

  // ---- clean-up (Rewriter.cc:1359-1603) ----

  // affine.if whose constraints hold for every value its operands can take
  // (loop and parallel index ranges): the body is spliced in its place.
  static void take_off_true_if(ir::ModuleOp module);
  // affine.if with a constraint that holds for no value of its operands: removed.
  static void delete_false_if(ir::ModuleOp module);
  // Fully unrolls every loop for which `unrollCheckFn` returns true (innermost first).
  static void unroll(ir::ModuleOp module, const std::function<bool(ir::ForOp)> &unrollCheckFn);
};

}  // namespace KernelCodeGen
