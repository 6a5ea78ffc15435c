/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===--------------------------- MI355XPasses.hpp -------------------------===//

#ifndef ONNX_MLIR_MI355X_PASSES_H
#define ONNX_MLIR_MI355X_PASSES_H

#include <memory>

#include "mlir/Pass/Pass.h"

namespace onnx_mlir {

/// Function name an `onnx.Custom` carries after fusion (attribute
/// `function_name`); they are also the symbols the runtime exports.
constexpr const char *kMI355XMatMulIntegerDequant =
    "om_mi355x_MatMulIntegerDequant";
constexpr const char *kMI355XDynQuantMatMulDequant =
    "om_mi355x_DynQuantMatMulDequant";

/// --fuse-quantized-matmul-for-mi355x
///   MatMulInteger -> Cast(f32) -> Mul(a_scale * b_scale)
///   DynamicQuantizeLinear -> MatMulInteger -> Cast(f32) -> Mul(...)
/// become one `onnx.Custom` each.
std::unique_ptr<mlir::Pass> createFuseQuantizedMatMulForMI355XPass();

} // namespace onnx_mlir
#endif
