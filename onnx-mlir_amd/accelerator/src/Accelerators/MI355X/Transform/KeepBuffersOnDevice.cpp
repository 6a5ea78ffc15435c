/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===----------------------- KeepBuffersOnDevice.cpp ----------------------===//
//
// After ONNX-to-Krnl every tensor between two offloaded ops is a host
// `memref.alloc`: the first call copies its result back into it and the second
// call uploads it again.  The runtime can be told to stand GPU memory in for
// such a buffer:
//
//   %t = memref.alloc() : memref<4096x768xui8>
//   "krnl.call"(%t) {funcName = "om_mi355x_KeepOnDevice", numOfOutput = 1}
//   "krnl.call"(%t, %s, %z, %x) {funcName = "om_mi355x_DynamicQuantizeLinear"}
//   "krnl.call"(%y, %t, %w, %z, %none) {funcName = "om_mi355x_MatMulInteger"}
//   "krnl.call"(%t) {funcName = "om_mi355x_Release", numOfOutput = 1}
//
// Between the two marks the entry points use the GPU copy whenever they are
// handed %t and never read or write the host buffer, so nothing crosses PCIe
// for it and the calls in between do not wait for the device.
//
// A buffer qualifies when
//   * it is a `memref.alloc` and each of its uses is an operand of a
//     `krnl.call` to an entry point of the runtime, in the block of the alloc
//     (no loads, stores, views, returns, calls to other libraries);
//   * at least one of those calls writes it (it is among the outputs) before
//     the first call that reads it.
// The release is placed right after the last such call.  The pass runs before
// deallocations exist (they are inserted in the Krnl-to-LLVM stage,
// src/Compiler/CompilerPasses.cpp:500-508); being a use of the buffer, the
// release keeps the `memref.dealloc` behind it.  That order matters: the
// runtime finds the GPU copy by host address, and an address must be released
// before the allocator can hand it out again.
//
// Both marks name the buffer as an output.  With only read effects and no
// results (src/Dialect/Krnl/KrnlOps.cpp:168-180) the calls would count as
// trivially dead and canonicalisation would drop them.
//
//===----------------------------------------------------------------------===//

#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/Dialect/MemRef/IR/MemRef.h"
#include "mlir/IR/Builders.h"
#include "mlir/Pass/Pass.h"

#include "src/Accelerators/MI355X/Transform/MI355XPasses.hpp"
#include "src/Dialect/Krnl/KrnlOps.hpp"

using namespace mlir;

namespace onnx_mlir {
namespace {

constexpr const char *kPrefix = "om_mi355x_";

/// A call that computes on the device (not one of the bookkeeping calls).
bool isOffloadedCompute(KrnlCallOp call) {
  StringRef callee = call.getFuncName();
  return callee.starts_with(kPrefix) && callee != kMI355XMarkConstant &&
         callee != kMI355XKeepOnDevice && callee != kMI355XRelease &&
         callee != kMI355XSetQuantMode;
}

/// First and last use of `buffer` if it qualifies (see the file header).
bool qualifies(memref::AllocOp alloc, Operation *&last) {
  Value buffer = alloc.getResult();
  Operation *first = nullptr;
  last = nullptr;
  for (OpOperand &use : buffer.getUses()) {
    auto call = dyn_cast<KrnlCallOp>(use.getOwner());
    // the buffer is only that call's anchor: neither read nor written
    if (call && call.getFuncName() == kMI355XSetQuantMode)
      continue;
    if (!call || call->getBlock() != alloc->getBlock() ||
        !isOffloadedCompute(call))
      return false;
    if (!first || call->isBeforeInBlock(first))
      first = call;
    if (!last || last->isBeforeInBlock(call))
      last = call;
  }
  if (!first || first == last)
    return false; // unused, or written and never consumed
  // The first call must produce the buffer in full: it is one of its outputs
  // and not also one of its inputs.
  auto producer = cast<KrnlCallOp>(first);
  int64_t numOutputs = producer.getNumOfOutput();
  bool written = false;
  for (OpOperand &operand : producer->getOpOperands()) {
    if (operand.get() != buffer)
      continue;
    if (static_cast<int64_t>(operand.getOperandNumber()) < numOutputs)
      written = true;
    else
      return false;
  }
  return written;
}

void emitMark(OpBuilder &builder, Location loc, StringRef callee, Value buffer) {
  KrnlCallOp::create(builder, loc, callee.str(),
      /*numOfOutput=*/static_cast<int64_t>(1), ValueRange{buffer});
}

struct KeepBuffersOnMI355XPass
    : public PassWrapper<KeepBuffersOnMI355XPass,
          OperationPass<func::FuncOp>> {
  MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(KeepBuffersOnMI355XPass)

  StringRef getArgument() const override { return "keep-buffers-on-mi355x"; }
  StringRef getDescription() const override {
    return "Back host buffers that only MI355X calls touch with GPU memory";
  }

  void runOnOperation() override {
    SmallVector<std::pair<memref::AllocOp, Operation *>> work;
    getOperation().walk([&](memref::AllocOp alloc) {
      Operation *last = nullptr;
      if (qualifies(alloc, last))
        work.emplace_back(alloc, last);
    });
    OpBuilder builder(&getContext());
    for (auto &[alloc, last] : work) {
      builder.setInsertionPointAfter(alloc);
      emitMark(builder, alloc.getLoc(), kMI355XKeepOnDevice, alloc.getResult());
      builder.setInsertionPointAfter(last);
      emitMark(builder, last->getLoc(), kMI355XRelease, alloc.getResult());
    }
  }
};

} // namespace

std::unique_ptr<Pass> createKeepBuffersOnMI355XPass() {
  return std::make_unique<KeepBuffersOnMI355XPass>();
}

} // namespace onnx_mlir
