/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===----------------------- ONNXToMI355XCall.hpp -------------------------===//

#ifndef ONNX_MLIR_ONNX_TO_MI355X_CALL_H
#define ONNX_MLIR_ONNX_TO_MI355X_CALL_H

#include "mlir/IR/PatternMatch.h"
#include "mlir/Transforms/DialectConversion.h"

namespace onnx_mlir {

/// Patterns for the ONNX-to-Krnl conversion that replace the quantisation ops
/// (and the `onnx.Custom` ops the MI355X fusion pass creates) by `krnl.call`s
/// to libRuntimeMI355X.a.  Their benefit is above that of the CPU patterns, and
/// they fail to match whatever the runtime does not implement, which then goes
/// to the CPU lowering.
void populateONNXToMI355XCallPatterns(mlir::RewritePatternSet &patterns,
    mlir::TypeConverter &typeConverter, mlir::MLIRContext *ctx);

} // namespace onnx_mlir
#endif
