/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===--------------------- MI355XCompilerOptions.hpp ----------------------===//
//
// Command-line options of the MI355X accelerator and the five macros every
// accelerator has to provide (docs/AddCustomAccelerators.md:48-72; they are
// expanded in src/Accelerators/Accelerator.hpp:49-57 and
// src/Compiler/CompilerOptions.hpp).  MI355X adds no instrumentation stage, IR
// profile or optimisation report of its own, so all five are empty.
//
//===----------------------------------------------------------------------===//

#ifndef ONNX_MLIR_MI355X_COMPILER_OPTIONS_H
#define ONNX_MLIR_MI355X_COMPILER_OPTIONS_H

#include "llvm/Support/CommandLine.h"

#define INSTRUMENTSTAGE_ENUM_MI355X
#define INSTRUMENTSTAGE_CL_ENUM_MI355X
#define PROFILEIR_CL_ENUM_MI355X
#define OPTREPORT_ENUM_MI355X
#define OPTREPORT_CL_ENUM_MI355X

namespace onnx_mlir {

extern llvm::cl::OptionCategory OnnxMlirOptions;
extern llvm::cl::OptionCategory OnnxMlirCommonOptions;

/// How QLinearMatMul narrows its 32-bit result to 8 bits.
enum class MI355XNarrowMode : int64_t {
  Wrap = 0,     // what the CPU lowering does (arith.trunci)
  Saturate = 1, // what the ONNX specification says
};

extern MI355XNarrowMode mi355xNarrowMode;
extern bool mi355xDisableFusion;
extern bool mi355xDisableMarkConstant;
extern bool mi355xDisableKeepOnDevice;
extern bool mi355xFuseGelu;
extern std::string mi355xOps;

} // namespace onnx_mlir
#endif
