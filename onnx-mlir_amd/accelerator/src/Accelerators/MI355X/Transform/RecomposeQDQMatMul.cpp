/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===----------------------- RecomposeQDQMatMul.cpp -----------------------===//
//
// Statically quantized models in the QDQ format carry a linear layer as
//
//   %af = DequantizeLinear(%a, %a_scale, %a_zp)             per tensor
//   %wf = DequantizeLinear(%W, %w_scale, %w_zp) {axis = 1}  per column of W
//   %yf = MatMul(%af, %wf)
//   %y  = QuantizeLinear(%yf, %y_scale, %y_zp)
//
// The reference recomposes the per-tensor form of this chain into
// onnx.QLinearMatMul (src/Dialect/ONNX/Transforms/Recompose.cpp:592-646) and
// then lowers that op with scalar scales only
// (src/Conversion/ONNXToKrnl/Math/QLinearMatMul.cpp:53-68): with one scale per
// output channel of W -- what weight quantizers emit -- the weights are
// dequantized to f32 and the product is a float MatMul.  The MI355X runtime's
// om_mi355x_QLinearMatMul takes b_scale and b_zero_point as one value or one
// per column, so here the chain becomes an onnx.QLinearMatMul also when the
// scale of W is 1-D along its last axis; the int8 weights are then what the
// kernel reads (a quarter of the bytes), the product is exact in int32 and
//   y = narrow(roundEven(f32(acc) * ((a_scale * w_scale[j]) / y_scale)) + y_zp).
//
// What is matched, besides the shape of the chain:
//   - %a's scale and zero point hold one element; %W is 2-D with a static
//     number of columns N; its scale is one element, or 1-D of N elements with
//     the DequantizeLinear's axis naming the last dimension; a zero point has
//     its scale's shape;
//   - a DequantizeLinear without zero point gets a zero of the quantized
//     type (QLinearMatMul's zero points are required operands);
//   - the float tensors in between have no other user.
// The same pattern on a MatMul whose B is dequantized per row (axis = 0) or in
// blocks is left alone: that is not a scale per output column.
//
//===----------------------------------------------------------------------===//

#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/IR/PatternMatch.h"
#include "mlir/Pass/Pass.h"
#include "mlir/Transforms/GreedyPatternRewriteDriver.h"

#include "src/Accelerators/MI355X/Transform/MI355XPasses.hpp"
#include "src/Dialect/ONNX/ONNXOps.hpp"
#include "src/Dialect/ONNX/ONNXOps/OpHelper.hpp"

using namespace mlir;

namespace onnx_mlir {
namespace {

bool isAbsent(Value v) { return !v || isa<NoneType>(v.getType()); }

int64_t staticElements(Value v) {
  auto type = dyn_cast<RankedTensorType>(v.getType());
  return type && type.hasStaticShape() ? type.getNumElements() : -1;
}

bool isQ8Tensor(Value v) {
  auto type = dyn_cast<RankedTensorType>(v.getType());
  return type && type.getElementType().isInteger(8);
}

/// Scale and zero point of a DequantizeLinear that quantizes its whole input
/// with one pair of values.
bool isPerTensor(ONNXDequantizeLinearOp dq) {
  if (staticElements(dq.getXScale()) != 1)
    return false;
  return isAbsent(dq.getXZeroPoint()) ||
         staticElements(dq.getXZeroPoint()) == 1;
}

/// ... or with one pair per column of a 2-D input.
bool isPerColumnOf2D(ONNXDequantizeLinearOp dq) {
  auto xType = dyn_cast<RankedTensorType>(dq.getX().getType());
  auto sType = dyn_cast<RankedTensorType>(dq.getXScale().getType());
  if (!xType || !sType || xType.getRank() != 2 || sType.getRank() != 1)
    return false;
  int64_t n = xType.getShape()[1];
  if (ShapedType::isDynamic(n) || sType.getShape()[0] != n)
    return false;
  int64_t axis = dq.getAxis();
  if (axis != 1 && axis != -1)
    return false;
  if (isAbsent(dq.getXZeroPoint()))
    return true;
  auto zType = dyn_cast<RankedTensorType>(dq.getXZeroPoint().getType());
  return zType && zType.getRank() == 1 && zType.getShape()[0] == n;
}

/// The zero point of `dq`, or zeros of its quantized type and its scale's
/// shape when it has none.
Value zeroPointOf(
    PatternRewriter &rewriter, Location loc, ONNXDequantizeLinearOp dq) {
  if (!isAbsent(dq.getXZeroPoint()))
    return dq.getXZeroPoint();
  auto xType = cast<RankedTensorType>(dq.getX().getType());
  auto sType = cast<RankedTensorType>(dq.getXScale().getType());
  auto zType = RankedTensorType::get(sType.getShape(), xType.getElementType());
  Attribute zeros = DenseElementsAttr::get(
      zType, rewriter.getIntegerAttr(xType.getElementType(), 0));
  return ONNXConstantOp::create(rewriter, loc, zType, Attribute(), zeros,
      FloatAttr(), ArrayAttr(), IntegerAttr(), ArrayAttr(), StringAttr(),
      ArrayAttr())
      .getResult();
}

struct RecomposeQDQMatMul : public OpRewritePattern<ONNXQuantizeLinearOp> {
  using OpRewritePattern<ONNXQuantizeLinearOp>::OpRewritePattern;

  LogicalResult matchAndRewrite(
      ONNXQuantizeLinearOp q, PatternRewriter &rewriter) const final {
    // y = QuantizeLinear(MatMul(..)), per tensor, 8-bit.
    if (staticElements(q.getYScale()) != 1 || isAbsent(q.getYZeroPoint()) ||
        staticElements(q.getYZeroPoint()) != 1 || !isQ8Tensor(q.getY()))
      return failure();
    auto matmul = q.getX().getDefiningOp<ONNXMatMulOp>();
    if (!matmul || !matmul.getResult().hasOneUse())
      return failure();
    auto dqA = matmul.getA().getDefiningOp<ONNXDequantizeLinearOp>();
    auto dqB = matmul.getB().getDefiningOp<ONNXDequantizeLinearOp>();
    if (!dqA || !dqB || !dqA.getResult().hasOneUse() ||
        !dqB.getResult().hasOneUse())
      return failure();
    if (!isQ8Tensor(dqA.getX()) || !isQ8Tensor(dqB.getX()))
      return failure();
    if (!isPerTensor(dqA))
      return failure();
    // One scale for all of W, or one per column.  (One element counts as per
    // tensor whatever `axis` says.)
    if (!isPerTensor(dqB) && !isPerColumnOf2D(dqB))
      return failure();
    // What the reference takes itself is left to it: this pass adds the
    // per-column form only when asked to recompose both (see the pass option).
    if (isPerTensor(dqB) && perColumnOnly)
      return failure();

    Location loc = q.getLoc();
    rewriter.setInsertionPoint(q);
    Value aZp = zeroPointOf(rewriter, loc, dqA);
    Value bZp = zeroPointOf(rewriter, loc, dqB);
    auto qmm = ONNXQLinearMatMulOp::create(rewriter, loc, q.getY().getType(),
        dqA.getX(), dqA.getXScale(), aZp, dqB.getX(), dqB.getXScale(), bZp,
        q.getYScale(), q.getYZeroPoint());
    if (Attribute nodeName = matmul->getAttr("onnx_node_name"))
      qmm->setAttr("onnx_node_name", nodeName);
    rewriter.replaceOp(q, qmm.getResult());
    // MatMul and the two DequantizeLinear are dead and pure now.
    return success();
  }

  RecomposeQDQMatMul(MLIRContext *ctx, bool perColumnOnly)
      : OpRewritePattern(ctx), perColumnOnly(perColumnOnly) {}
  bool perColumnOnly;
};

struct RecomposeQDQMatMulForMI355XPass
    : public PassWrapper<RecomposeQDQMatMulForMI355XPass,
          OperationPass<func::FuncOp>> {
  MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(RecomposeQDQMatMulForMI355XPass)

  RecomposeQDQMatMulForMI355XPass() = default;
  RecomposeQDQMatMulForMI355XPass(const RecomposeQDQMatMulForMI355XPass &pass)
      : PassWrapper(pass) {}

  StringRef getArgument() const override {
    return "recompose-qdq-matmul-for-mi355x";
  }
  StringRef getDescription() const override {
    return "DequantizeLinear x 2 -> MatMul -> QuantizeLinear becomes "
           "onnx.QLinearMatMul, also with one weight scale per output column";
  }

  Option<bool> perColumnOnly{*this, "per-column-only",
      llvm::cl::desc("Leave the per-tensor form to the ONNX dialect's own "
                     "recomposition"),
      llvm::cl::init(false)};

  void runOnOperation() final {
    RewritePatternSet patterns(&getContext());
    patterns.insert<RecomposeQDQMatMul>(&getContext(), perColumnOnly);
    if (failed(applyPatternsGreedily(getOperation(), std::move(patterns))))
      signalPassFailure();
  }
};

} // namespace

std::unique_ptr<Pass> createRecomposeQDQMatMulForMI355XPass() {
  return std::make_unique<RecomposeQDQMatMulForMI355XPass>();
}

} // namespace onnx_mlir
