/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===---------------------- MI355XCompilerUtils.cpp -----------------------===//

#include "src/Accelerators/MI355X/Compiler/MI355XCompilerUtils.hpp"

#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/Transforms/Passes.h"

#include "src/Accelerators/MI355X/Compiler/MI355XCompilerOptions.hpp"
#include "src/Accelerators/MI355X/Transform/MI355XPasses.hpp"
#include "src/Compiler/CompilerOptions.hpp"
#include "src/Compiler/CompilerPasses.hpp"
#include "src/Pass/Passes.hpp"

using namespace mlir;

namespace onnx_mlir {

void configurePassesMI355X() {
  // The generic configuration is enough; call it so that an accelerator-only
  // driver (onnx-mlir-opt --maccel=MI355X) ends up in the same state as the
  // CPU one.
  configurePasses();
}

void addPassesMI355X(OwningOpRef<ModuleOp> &module, PassManager &pm,
    EmissionTargetType &emissionTarget, std::string outputNameNoExt) {
  configurePassesMI355X();
  InputIRLevelType inputLevel = determineInputIRLevel(module);

  if (inputLevel <= ONNXLevel) {
    // Decomposition, shape inference, constant propagation.  `targetCPU` is
    // false so that rewrites meant only for the CPU matmul are skipped.
    addONNXToMLIRPasses(pm, /*targetCPU=*/false);

    // Chains ending in a float scaling become one call each; this has to run
    // while the graph is still in the ONNX dialect and fully shaped.
    if (!mi355xDisableFusion) {
      // QDQ chains first: what they become is an op the patterns below and
      // the ONNX-to-Krnl conversion of the accelerator know.
      pm.addNestedPass<func::FuncOp>(createRecomposeQDQMatMulForMI355XPass());
      pm.addNestedPass<func::FuncOp>(createFuseQuantizedMatMulForMI355XPass());
      pm.addNestedPass<func::FuncOp>(createShapeInferencePass());
      pm.addPass(createCanonicalizerPass());
    }
  }

  if (emissionTarget >= EmitMLIR) {
    if (inputLevel <= ONNXLevel)
      addONNXToKrnlPasses(
          pm, OptimizationLevel, /*enableCSE=*/true, ONNXOpStats);
    if (inputLevel <= MLIRLevel) {
      addKrnlToAffinePasses(pm);
      // Needs the final set of users of each buffer (after write-only allocs
      // are gone) and has to come before deallocations are inserted.
      if (!mi355xDisableKeepOnDevice)
        pm.addNestedPass<func::FuncOp>(createKeepBuffersOnMI355XPass());
    }
  }

  if (emissionTarget >= EmitLLVMIR && inputLevel <= LLVMLevel)
    addKrnlToLLVMPasses(pm, outputNameNoExt, /*enableCSE=*/true);
}

} // namespace onnx_mlir
