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

/// Bookkeeping entry points of the runtime (no computation).
constexpr const char *kMI355XMarkConstant = "om_mi355x_MarkConstant";
constexpr const char *kMI355XKeepOnDevice = "om_mi355x_KeepOnDevice";
constexpr const char *kMI355XRelease = "om_mi355x_Release";
constexpr const char *kMI355XSetQuantMode = "om_mi355x_SetQuantMode";

/// --fuse-quantized-matmul-for-mi355x
///   MatMulInteger -> Cast(f32) -> Mul(a_scale * b_scale)
///   DynamicQuantizeLinear -> MatMulInteger -> Cast(f32) -> Mul(...)
/// become one `onnx.Custom` each.
std::unique_ptr<mlir::Pass> createFuseQuantizedMatMulForMI355XPass();

/// --recompose-qdq-matmul-for-mi355x
///   DequantizeLinear(a), DequantizeLinear(W) -> MatMul -> QuantizeLinear
/// becomes onnx.QLinearMatMul, also when W has one scale per output column
/// (which the runtime's QLinearMatMul takes and the CPU lowering does not).
std::unique_ptr<mlir::Pass> createRecomposeQDQMatMulForMI355XPass();

/// --keep-buffers-on-mi355x
/// Runs on Krnl/MemRef IR.  A `memref.alloc` that only MI355X calls touch gets
/// `om_mi355x_KeepOnDevice` after the allocation and `om_mi355x_Release`
/// after its last user, so that it never travels to the host and back.
std::unique_ptr<mlir::Pass> createKeepBuffersOnMI355XPass();

} // namespace onnx_mlir
#endif
