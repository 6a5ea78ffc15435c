/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===----------------------- ONNXToMI355XCall.cpp -------------------------===//
//
// ONNX-to-Krnl patterns of the MI355X accelerator.
//
// Each pattern allocates the results of the op and emits
//
//   "krnl.call"(results..., operands...) {funcName, numOfOutput, attrs...}
//
// which KrnlCallOpLowering (src/Conversion/KrnlToLLVM/KrnlCall.cpp:34-102)
// turns into `call void @funcName(OMTensor*..., int64_t...)`: parameters in
// operand order, then the remaining attributes in the (name-sorted) order of
// the attribute dictionary.  The C prototypes are in om_mi355x.h.
//
// Two points differ from the generic op-to-call pattern of
// src/Conversion/ONNXToKrnl/ONNXToKrnlCommon.hpp:577-616:
//  * the builder used here takes the operand list as is.  The one that takes
//    the ONNX op drops `none` operands (src/Dialect/Krnl/KrnlOps.cpp:92-96),
//    which would shift an absent zero point's successors by one position; a
//    `none` that is kept arrives as a NULL pointer (KrnlCall.cpp:139-145).
//  * attributes are set by name, so that only the ones in the C prototype are
//    passed (an `onnx_node_name` would otherwise become a `const char *`).
//
//===----------------------------------------------------------------------===//

#include "src/Accelerators/MI355X/Conversion/ONNXToMI355XCall.hpp"

#include "llvm/ADT/StringSet.h"

#include "src/Accelerators/MI355X/Compiler/MI355XCompilerOptions.hpp"
#include "src/Accelerators/MI355X/Transform/MI355XPasses.hpp"
#include "src/Conversion/ONNXToKrnl/ONNXToKrnlCommon.hpp"
#include "src/Dialect/Krnl/KrnlOps.hpp"
#include "src/Dialect/ONNX/ONNXOps/ShapeHelper.hpp"

using namespace mlir;

namespace onnx_mlir {
namespace {

// Above the CPU patterns' default of 1 and above the generic op-to-call
// pattern's 10, so that --maccel=MI355X wins over --ops-for-call.
constexpr int kBenefit = 20;

//===----------------------------------------------------------------------===//
// What the runtime accepts.
//===----------------------------------------------------------------------===//

bool isQ8(Type t) {
  auto intType = dyn_cast<IntegerType>(getElementTypeOrSelf(t));
  return intType && intType.getWidth() == 8;
}
bool isF32(Type t) { return getElementTypeOrSelf(t).isF32(); }
bool isI32(Type t) {
  auto intType = dyn_cast<IntegerType>(getElementTypeOrSelf(t));
  return intType && intType.getWidth() == 32;
}
bool isAbsent(Value v) { return !v || isNoneValue(v); }

bool hasRankAtLeast(Value v, int64_t rank) {
  auto type = dyn_cast<ShapedType>(v.getType());
  return type && type.hasRank() && type.getRank() >= rank;
}

/// Selected by --mi355x-ops (all five when the option is empty).
bool isEnabled(Operation *op) {
  if (mi355xOps.empty())
    return true;
  StringRef name = op->getName().stripDialect();
  SmallVector<StringRef> parts;
  StringRef(mi355xOps).split(parts, ',', /*MaxSplit=*/-1, /*KeepEmpty=*/false);
  return llvm::any_of(parts, [&](StringRef p) { return p.trim() == name; });
}

//===----------------------------------------------------------------------===//
// Emission helpers.
//===----------------------------------------------------------------------===//

/// `krnl.call` with the operands exactly as given and integer attributes that
/// arrive as trailing int64_t parameters.  Callers list attributes whose names
/// sort in the order of the C prototype.
void emitCall(ConversionPatternRewriter &rewriter, Location loc,
    StringRef callee, ValueRange results, ValueRange inputs,
    ArrayRef<std::pair<StringRef, int64_t>> intAttrs = {}) {
  SmallVector<Value, 12> params(results.begin(), results.end());
  params.append(inputs.begin(), inputs.end());
  auto call = KrnlCallOp::create(rewriter, loc, callee.str(),
      /*numOfOutput=*/static_cast<int64_t>(results.size()), params);
  for (const auto &[name, value] : intAttrs)
    call->setAttr(name, rewriter.getI64IntegerAttr(value));
}

/// The reference's own lowerings of QuantizeLinear, DequantizeLinear and
/// DynamicQuantizeLinear change with two compiler options: --enable-fast-math
/// at -O3 (the quotient becomes x * (1 / scale),
/// src/Conversion/ONNXToKrnl/Quantization/QuantizeLinear.cpp:43-44, enabled as
/// in src/Compiler/CompilerPasses.cpp:298-301) and
/// --disable-quantization-zero-point (QuantizeLinear.cpp:231-237,
/// DynamicQuantizeLinear.cpp:142, Math/Elementwise.cpp:1453).  The runtime
/// computes either way.  Which one is a property of the compiled model, as in
/// the reference, so it travels with each op: `om_mi355x_SetQuantMode(anchor,
/// mode)` applies to the calling thread's next quantize / dequantize /
/// dynamic-quantize / fused-layer entry point only, which takes the mode and
/// leaves the default behind.  The call therefore goes directly in front of
/// every offloaded op that the options touch when one of them is on; code
/// compiled with default options emits nothing and cannot inherit a mode from
/// a model that ran on the thread before it.
/// `anchor` (the op's first result buffer) is passed as an output for the
/// reason given at markIfConstant, and because two calls that write the same
/// buffer keep their order; the runtime does not touch it.
int64_t quantModeFromOptions() {
  int64_t mode = 0;
  if (OptimizationLevel >= OptLevel::O3 && enableFastMathOption)
    mode |= 1; // OM_MI355X_QUANT_RECIPROCAL
  if (disableQuantZeroPoint)
    mode |= 2; // OM_MI355X_QUANT_NO_ZERO_POINT
  return mode;
}

void emitQuantMode(
    ConversionPatternRewriter &rewriter, Location loc, Value anchor) {
  const int64_t mode = quantModeFromOptions();
  if (mode == 0)
    return;
  auto call = KrnlCallOp::create(rewriter, loc,
      std::string(kMI355XSetQuantMode),
      /*numOfOutput=*/static_cast<int64_t>(1), ValueRange{anchor});
  call->setAttr("mode", rewriter.getI64IntegerAttr(mode));
}

/// Tell the runtime that `v` is a model constant, so that it is copied to the
/// device (and, as a matmul right-hand side, packed) once instead of on every
/// call.  After conversion an `onnx.Constant` is a `krnl.global`, whose buffer
/// keeps its address for the life of the model
/// (src/Conversion/KrnlToLLVM/KrnlGlobal.cpp:74-200).  Registering an address
/// twice is a no-op in the runtime, so the call may sit in front of every use.
/// The constant is passed as an output: a call with no results and only read
/// effects (src/Dialect/Krnl/KrnlOps.cpp:168-180) counts as trivially dead and
/// would not survive canonicalisation.
void markIfConstant(
    ConversionPatternRewriter &rewriter, Location loc, Value v) {
  if (mi355xDisableMarkConstant || isAbsent(v))
    return;
  if (!v.getDefiningOp<KrnlGlobalOp>())
    return;
  KrnlCallOp::create(rewriter, loc, std::string(kMI355XMarkConstant),
      /*numOfOutput=*/static_cast<int64_t>(1), ValueRange{v});
}

/// Allocate the results of `op` with the op's own shape helper.
template <typename OP, typename SHAPE_HELPER>
std::vector<Value> allocResults(OP op, ValueRange operands,
    ConversionPatternRewriter &rewriter, const TypeConverter *typeConverter) {
  Location loc = ONNXLoc<OP>(op.getOperation());
  MultiDialectBuilder<IndexExprBuilderForKrnl, MemRefBuilder> create(
      rewriter, loc);
  SHAPE_HELPER shapeHelper(op.getOperation(), operands, &create.krnlIE);
  shapeHelper.computeShapeAndAssertOnFailure();
  return allocForONNXOp<OP>(op, rewriter, typeConverter, shapeHelper);
}

//===----------------------------------------------------------------------===//
// QuantizeLinear: void f(y, x, y_scale, y_zero_point|NULL, axis, saturate)
//===----------------------------------------------------------------------===//

struct QuantizeLinearToMI355X
    : public OpConversionPattern<ONNXQuantizeLinearOp> {
  QuantizeLinearToMI355X(TypeConverter &tc, MLIRContext *ctx)
      : OpConversionPattern(tc, ctx, kBenefit) {}

  LogicalResult matchAndRewrite(ONNXQuantizeLinearOp op, OpAdaptor adaptor,
      ConversionPatternRewriter &rewriter) const final {
    if (!isEnabled(op) || !isF32(op.getX().getType()) ||
        !isF32(op.getYScale().getType()) || !isQ8(op.getY().getType()))
      return failure(); // f16/bf16 inputs and fp8 outputs stay on the CPU
    Location loc = ONNXLoc<ONNXQuantizeLinearOp>(op);
    std::vector<Value> y =
        allocResults<ONNXQuantizeLinearOp, ONNXQuantizeLinearOpShapeHelper>(
            op, adaptor.getOperands(), rewriter, typeConverter);
    emitQuantMode(rewriter, loc, y[0]);
    emitCall(rewriter, loc, "om_mi355x_QuantizeLinear", y,
        {adaptor.getX(), adaptor.getYScale(), adaptor.getYZeroPoint()},
        {{"axis", op.getAxis()}, {"saturate", op.getSaturate()}});
    rewriter.replaceOp(op, y);
    return success();
  }
};

//===----------------------------------------------------------------------===//
// DequantizeLinear: void f(y, x, x_scale, x_zero_point|NULL, axis)
//===----------------------------------------------------------------------===//

struct DequantizeLinearToMI355X
    : public OpConversionPattern<ONNXDequantizeLinearOp> {
  DequantizeLinearToMI355X(TypeConverter &tc, MLIRContext *ctx)
      : OpConversionPattern(tc, ctx, kBenefit) {}

  LogicalResult matchAndRewrite(ONNXDequantizeLinearOp op, OpAdaptor adaptor,
      ConversionPatternRewriter &rewriter) const final {
    Type xType = op.getX().getType();
    if (!isEnabled(op) || !(isQ8(xType) || isI32(xType)) ||
        !isF32(op.getXScale().getType()) || !isF32(op.getY().getType()))
      return failure();
    Location loc = ONNXLoc<ONNXDequantizeLinearOp>(op);
    markIfConstant(rewriter, loc, adaptor.getX());
    std::vector<Value> y =
        allocResults<ONNXDequantizeLinearOp, ONNXDequantizeLinearOpShapeHelper>(
            op, adaptor.getOperands(), rewriter, typeConverter);
    emitQuantMode(rewriter, loc, y[0]);
    emitCall(rewriter, loc, "om_mi355x_DequantizeLinear", y,
        {adaptor.getX(), adaptor.getXScale(), adaptor.getXZeroPoint()},
        {{"axis", op.getAxis()}});
    rewriter.replaceOp(op, y);
    return success();
  }
};

//===----------------------------------------------------------------------===//
// DynamicQuantizeLinear: void f(y, y_scale, y_zero_point, x)
//===----------------------------------------------------------------------===//

struct DynamicQuantizeLinearToMI355X
    : public OpConversionPattern<ONNXDynamicQuantizeLinearOp> {
  DynamicQuantizeLinearToMI355X(TypeConverter &tc, MLIRContext *ctx)
      : OpConversionPattern(tc, ctx, kBenefit) {}

  LogicalResult matchAndRewrite(ONNXDynamicQuantizeLinearOp op,
      OpAdaptor adaptor, ConversionPatternRewriter &rewriter) const final {
    if (!isEnabled(op))
      return failure();
    Location loc = ONNXLoc<ONNXDynamicQuantizeLinearOp>(op);
    std::vector<Value> results = allocResults<ONNXDynamicQuantizeLinearOp,
        ONNXDynamicQuantizeLinearOpShapeHelper>(
        op, adaptor.getOperands(), rewriter, typeConverter);
    emitQuantMode(rewriter, loc, results[0]);
    emitCall(rewriter, loc, "om_mi355x_DynamicQuantizeLinear", results,
        {adaptor.getX()});
    rewriter.replaceOp(op, results);
    return success();
  }
};

//===----------------------------------------------------------------------===//
// MatMulInteger: void f(y, a, b, a_zero_point|NULL, b_zero_point|NULL)
//===----------------------------------------------------------------------===//

struct MatMulIntegerToMI355X
    : public OpConversionPattern<ONNXMatMulIntegerOp> {
  MatMulIntegerToMI355X(TypeConverter &tc, MLIRContext *ctx)
      : OpConversionPattern(tc, ctx, kBenefit) {}

  LogicalResult matchAndRewrite(ONNXMatMulIntegerOp op, OpAdaptor adaptor,
      ConversionPatternRewriter &rewriter) const final {
    // Any ranked pair of operands: the runtime pairs batch dimensions by the
    // rules of ONNXMatMulOpShapeHelper (src/Dialect/ONNX/ONNXOps/Math/
    // MatMul.cpp:200-292), the same that sized `y` here.
    if (!isEnabled(op) || !hasRankAtLeast(op.getB(), 1) ||
        !hasRankAtLeast(op.getA(), 1))
      return failure();
    Location loc = ONNXLoc<ONNXMatMulIntegerOp>(op);
    markIfConstant(rewriter, loc, adaptor.getB());
    std::vector<Value> y =
        allocResults<ONNXMatMulIntegerOp, ONNXMatMulIntegerOpShapeHelper>(
            op, adaptor.getOperands(), rewriter, typeConverter);
    emitCall(rewriter, loc, "om_mi355x_MatMulInteger", y,
        {adaptor.getA(), adaptor.getB(), adaptor.getAZeroPoint(),
            adaptor.getBZeroPoint()});
    rewriter.replaceOp(op, y);
    return success();
  }
};

//===----------------------------------------------------------------------===//
// QLinearMatMul: void f(y, a, a_scale, a_zp, b, b_scale, b_zp, y_scale, y_zp,
//                       narrow_mode)
//===----------------------------------------------------------------------===//

struct QLinearMatMulToMI355X
    : public OpConversionPattern<ONNXQLinearMatMulOp> {
  QLinearMatMulToMI355X(TypeConverter &tc, MLIRContext *ctx)
      : OpConversionPattern(tc, ctx, kBenefit) {}

  LogicalResult matchAndRewrite(ONNXQLinearMatMulOp op, OpAdaptor adaptor,
      ConversionPatternRewriter &rewriter) const final {
    if (!isEnabled(op) || !hasRankAtLeast(op.getB(), 1) ||
        !hasRankAtLeast(op.getA(), 1))
      return failure();
    Location loc = ONNXLoc<ONNXQLinearMatMulOp>(op);
    markIfConstant(rewriter, loc, adaptor.getB());
    std::vector<Value> y =
        allocResults<ONNXQLinearMatMulOp, ONNXQLinearMatMulOpShapeHelper>(
            op, adaptor.getOperands(), rewriter, typeConverter);
    emitCall(rewriter, loc, "om_mi355x_QLinearMatMul", y,
        adaptor.getOperands(),
        {{"narrow_mode", static_cast<int64_t>(mi355xNarrowMode)}});
    rewriter.replaceOp(op, y);
    return success();
  }
};

//===----------------------------------------------------------------------===//
// onnx.Custom created by the fusion pass.
//   void om_mi355x_MatMulIntegerDequant(y, a, b, a_zp|NULL, b_zp|NULL,
//                                       a_scale, b_scale, bias|NULL,
//                                       activation)
//   void om_mi355x_DynQuantMatMulDequant(y, x, b, b_zp|NULL, b_scale,
//                                        bias|NULL, activation)
// In both, input 0 is [.., M, K] and input 1 is [K, N]; the result is
// [.., M, N].  onnx.Custom has no shape rule for that, so the dimensions are
// taken from the operands here.
//===----------------------------------------------------------------------===//

struct FusedMatMulToMI355X : public OpConversionPattern<ONNXCustomOp> {
  FusedMatMulToMI355X(TypeConverter &tc, MLIRContext *ctx)
      : OpConversionPattern(tc, ctx, kBenefit) {}

  LogicalResult matchAndRewrite(ONNXCustomOp op, OpAdaptor adaptor,
      ConversionPatternRewriter &rewriter) const final {
    StringRef callee = op.getFunctionName();
    if (callee != kMI355XMatMulIntegerDequant &&
        callee != kMI355XDynQuantMatMulDequant)
      return failure();
    if (op->getNumResults() != 1)
      return failure();
    Location loc = op.getLoc();
    ValueRange inputs = adaptor.getInputs();
    auto yType = dyn_cast_or_null<MemRefType>(
        typeConverter->convertType(op->getResult(0).getType()));
    if (!yType)
      return failure();

    // [K, N] weights only: with any other rank the last dimension of the
    // result would not be dimension 1 of input 1.
    auto bType = dyn_cast<MemRefType>(inputs[1].getType());
    if (!bType || bType.getRank() != 2)
      return failure();

    MultiDialectBuilder<IndexExprBuilderForKrnl, MemRefBuilder> create(
        rewriter, loc);
    IndexExprScope scope(create.krnlIE);
    DimsExpr dims;
    create.krnlIE.getShapeAsDims(inputs[0], dims);
    if (dims.empty() || static_cast<int64_t>(dims.size()) != yType.getRank())
      return failure();
    dims.back() = create.krnlIE.getShapeAsDim(inputs[1], 1);
    Value y = create.mem.alignedAlloc(yType, dims);

    // Weights, and whichever of zero point, scales and bias are constants:
    // uploaded once instead of with every call.
    for (size_t i = 1; i < inputs.size(); ++i)
      markIfConstant(rewriter, loc, inputs[i]);
    int64_t activation = 0;
    if (auto attr = op->getAttrOfType<IntegerAttr>("activation"))
      activation = attr.getInt();
    if (callee == kMI355XDynQuantMatMulDequant) // it quantizes; the other fused op does not
      emitQuantMode(rewriter, loc, y);
    emitCall(rewriter, loc, callee, {y}, inputs, {{"activation", activation}});
    rewriter.replaceOp(op, y);
    return success();
  }
};

} // namespace

void populateONNXToMI355XCallPatterns(RewritePatternSet &patterns,
    TypeConverter &typeConverter, MLIRContext *ctx) {
  patterns.insert<QuantizeLinearToMI355X, DequantizeLinearToMI355X,
      DynamicQuantizeLinearToMI355X, MatMulIntegerToMI355X,
      QLinearMatMulToMI355X, FusedMatMulToMI355X>(typeConverter, ctx);
}

} // namespace onnx_mlir
