/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===---------------------- MI355XCompilerUtils.hpp -----------------------===//

#ifndef ONNX_MLIR_MI355X_COMPILER_UTILS_H
#define ONNX_MLIR_MI355X_COMPILER_UTILS_H

#include "mlir/IR/BuiltinOps.h"
#include "mlir/IR/OwningOpRef.h"
#include "mlir/Pass/PassManager.h"
#include "src/Compiler/CompilerOptionEnums.hpp"

namespace onnx_mlir {

/// The whole compilation pipeline for --maccel=MI355X.  It is the CPU pipeline
/// of src/Compiler/CompilerPasses.cpp with one ONNX-level pass added before the
/// lowering to Krnl.
void addPassesMI355X(mlir::OwningOpRef<mlir::ModuleOp> &module,
    mlir::PassManager &pm, EmissionTargetType &emissionTarget,
    std::string outputNameNoExt);

void configurePassesMI355X();

} // namespace onnx_mlir
#endif
