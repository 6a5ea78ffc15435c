/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===---------------------- FuseQuantizedMatMul.cpp -----------------------===//
//
// Dynamic quantisation of a linear layer is exported as the chain
//
//   %aq, %as, %azp = DynamicQuantizeLinear(%x)
//   %acc           = MatMulInteger(%aq, %W, %azp, %wzp)
//   %f             = Cast(%acc) {to = f32}
//   %s             = Mul(%as, %ws)
//   %y             = Mul(%f, %s)
//   %z             = Add(%y, %bias)          (optional)
//   %r             = Relu(%z) or Gelu(%z)    (optional)
//
// On the CPU that is five or six ops and as many intermediate tensors.  The
// MI355X runtime has one entry point for everything after the quantisation
// (the int32 accumulator never reaches memory) and one for the whole chain
// (the 8-bit activation stays on the device).  A bias that is added to the
// scaled result -- one value, or one per column -- goes along: the kernel
// rounds the product to f32 and then adds, as Mul followed by Add does.  A Relu
// that is the only user of that result goes along too, as the integer
// attribute `activation` = 1 (max(0, x) is exact, so where it is applied does
// not change a bit of the result).  With --mi355x-fuse-gelu an onnx.Gelu with
// approximate = "none" in that place goes along as `activation` = 2; that is
// not the default because the runtime's erf and the polynomial the CPU code
// evaluates differ in the last bits.  This pass replaces the chain by an
// `onnx.Custom` naming that entry point; the ONNX-to-Krnl patterns of the
// accelerator lower it.
//
// Only the association `f32(acc) * (a_scale * b_scale)` is matched.  The other
// one the reference knows, `(f32(acc) * a_scale) * b_scale`
// (src/Accelerators/NNPA/Conversion/ONNXToZHigh/ONNXToZHigh.cpp:895-912),
// rounds differently and is left to the unfused ops so that results stay
// bit-identical to the CPU's.
//
//===----------------------------------------------------------------------===//

#include "mlir/Dialect/Func/IR/FuncOps.h"
#include "mlir/IR/PatternMatch.h"
#include "mlir/Pass/Pass.h"
#include "mlir/Transforms/GreedyPatternRewriteDriver.h"

#include "src/Accelerators/MI355X/Compiler/MI355XCompilerOptions.hpp"
#include "src/Accelerators/MI355X/Transform/MI355XPasses.hpp"
#include "src/Dialect/ONNX/ONNXOps.hpp"
#include "src/Dialect/ONNX/ONNXOps/OpHelper.hpp"

using namespace mlir;

namespace onnx_mlir {
namespace {

bool isF32Tensor(Value v) {
  auto type = dyn_cast<RankedTensorType>(v.getType());
  return type && type.getElementType().isF32();
}

/// A tensor that statically holds exactly one element.
bool isSingleElement(Value v) {
  auto type = dyn_cast<RankedTensorType>(v.getType());
  return type && type.hasStaticShape() && type.getNumElements() == 1;
}

/// Scale of the right-hand side: one value, or one per column of `b`.
bool isColumnScale(Value scale, Value b) {
  if (isSingleElement(scale))
    return true;
  auto scaleType = dyn_cast<RankedTensorType>(scale.getType());
  auto bType = dyn_cast<RankedTensorType>(b.getType());
  if (!scaleType || !bType || scaleType.getRank() != 1 || bType.getRank() < 2)
    return false;
  int64_t n = bType.getShape().back();
  return !ShapedType::isDynamic(n) && scaleType.getShape()[0] == n;
}

struct Chain {
  ONNXMatMulIntegerOp matmul;
  ONNXCastOp cast;
  ONNXMulOp scaleProduct;
  Value aScale, bScale;
};

/// Match `Mul(Cast(MatMulInteger), Mul(sa, sb))` in either operand order.  The
/// intermediate values must have no other user: they disappear.
bool matchChain(ONNXMulOp mul, Chain &chain) {
  for (int swap = 0; swap < 2; ++swap) {
    Value accSide = swap ? mul.getB() : mul.getA();
    Value scaleSide = swap ? mul.getA() : mul.getB();
    auto cast = accSide.getDefiningOp<ONNXCastOp>();
    auto product = scaleSide.getDefiningOp<ONNXMulOp>();
    if (!cast || !product || !cast->hasOneUse() || !product->hasOneUse())
      continue;
    if (!isF32Tensor(cast.getResult()))
      continue;
    auto matmul = cast.getInput().getDefiningOp<ONNXMatMulIntegerOp>();
    if (!matmul || !matmul->hasOneUse())
      continue;
    // The fused entry points take a 2-D right-hand side (the weights of a
    // linear layer) and a left-hand side of rank >= 1, as the unfused
    // MatMulInteger pattern of the fused epilogue does; a batched B stays
    // unfused.
    auto aType = dyn_cast<RankedTensorType>(matmul.getA().getType());
    auto bType = dyn_cast<RankedTensorType>(matmul.getB().getType());
    if (!aType || !bType || bType.getRank() != 2 || aType.getRank() < 1)
      continue;
    // The accumulator tensor must already have the shape of the result: a
    // scale that broadcasts the result to more dimensions is not this chain.
    auto accType = dyn_cast<RankedTensorType>(matmul.getResult().getType());
    auto outType = dyn_cast<RankedTensorType>(mul.getResult().getType());
    if (!accType || !outType || accType.getShape() != outType.getShape())
      continue;
    // a_scale is per tensor; b_scale per tensor or per column.
    for (int swapScale = 0; swapScale < 2; ++swapScale) {
      Value sa = swapScale ? product.getB() : product.getA();
      Value sb = swapScale ? product.getA() : product.getB();
      if (!isF32Tensor(sa) || !isF32Tensor(sb) || !isSingleElement(sa) ||
          !isColumnScale(sb, matmul.getB()))
        continue;
      chain = {matmul, cast, product, sa, sb};
      return true;
    }
  }
  return false;
}

Value noneIfAbsent(PatternRewriter &rewriter, Location loc, Value v) {
  if (v && !isNoneValue(v))
    return v;
  return ONNXNoneOp::create(rewriter, loc).getResult();
}

struct FuseScaledMatMulInteger : public OpRewritePattern<ONNXMulOp> {
  using OpRewritePattern<ONNXMulOp>::OpRewritePattern;

  LogicalResult matchAndRewrite(
      ONNXMulOp mul, PatternRewriter &rewriter) const final {
    Chain chain;
    if (!matchChain(mul, chain))
      return failure();
    Location loc = mul.getLoc();
    ONNXMatMulIntegerOp matmul = chain.matmul;

    // If the left operand comes straight from DynamicQuantizeLinear of which
    // this chain is the only consumer, take the quantisation along.
    auto dynQuant = matmul.getA().getDefiningOp<ONNXDynamicQuantizeLinearOp>();
    bool wholeLayer =
        dynQuant && matmul.getA() == dynQuant.getY() &&
        matmul.getAZeroPoint() == dynQuant.getYZeroPoint() &&
        chain.aScale == dynQuant.getYScale() && dynQuant.getY().hasOneUse() &&
        dynQuant.getYScale().hasOneUse() && dynQuant.getYZeroPoint().hasOneUse();

    // A bias added to the scaled result (its only user) is taken along.
    Operation *root = mul;
    Value bias;
    if (mul->hasOneUse()) {
      if (auto add = dyn_cast<ONNXAddOp>(*mul->user_begin())) {
        Value other = add.getA() == mul.getResult() ? add.getB() : add.getA();
        bool shaped =
            isF32Tensor(other) &&
            (isSingleElement(other) || isColumnScale(other, matmul.getB())) &&
            add.getResult().getType() == mul.getResult().getType();
        if (shaped && other != mul.getResult()) {
          root = add;
          bias = other;
        }
      }
    }
    // ... and so is a Relu that is the only user of what has been matched.
    int64_t activation = 0;
    if (root->hasOneUse()) {
      if (auto relu = dyn_cast<ONNXReluOp>(*root->user_begin())) {
        if (relu.getResult().getType() == root->getResult(0).getType()) {
          root = relu;
          activation = 1;
        }
      } else if (auto gelu = dyn_cast<ONNXGeluOp>(*root->user_begin())) {
        // Only on request: the entry point and the CPU code evaluate erf by
        // different approximations, so the last bits differ.
        if (mi355xFuseGelu && gelu.getApproximate().equals_insensitive("none") &&
            gelu.getResult().getType() == root->getResult(0).getType()) {
          root = gelu;
          activation = 2;
        }
      }
    }
    rewriter.setInsertionPoint(root);

    SmallVector<Value, 8> inputs;
    StringRef callee;
    if (wholeLayer) {
      callee = kMI355XDynQuantMatMulDequant;
      inputs = {dynQuant.getX(), matmul.getB(),
          noneIfAbsent(rewriter, loc, matmul.getBZeroPoint()), chain.bScale,
          noneIfAbsent(rewriter, loc, bias)};
    } else {
      callee = kMI355XMatMulIntegerDequant;
      inputs = {matmul.getA(), matmul.getB(),
          noneIfAbsent(rewriter, loc, matmul.getAZeroPoint()),
          noneIfAbsent(rewriter, loc, matmul.getBZeroPoint()), chain.aScale,
          chain.bScale, noneIfAbsent(rewriter, loc, bias)};
    }

    SmallVector<NamedAttribute, 3> attrs;
    attrs.emplace_back(
        rewriter.getNamedAttr("function_name", rewriter.getStringAttr(callee)));
    attrs.emplace_back(rewriter.getNamedAttr(
        "activation", rewriter.getI64IntegerAttr(activation)));
    if (Attribute nodeName = mul->getAttr("onnx_node_name"))
      attrs.emplace_back(rewriter.getNamedAttr("onnx_node_name", nodeName));
    auto fused = ONNXCustomOp::create(rewriter, loc,
        TypeRange{root->getResult(0).getType()}, ValueRange(inputs), attrs);
    rewriter.replaceOp(root, fused.getResults());
    // Mul and Add (when a later op was the root), Cast, MatMulInteger, the scale product
    // and (for the whole layer) DynamicQuantizeLinear are now dead and pure:
    // the driver erases them.
    return success();
  }
};

struct FuseQuantizedMatMulForMI355XPass
    : public PassWrapper<FuseQuantizedMatMulForMI355XPass,
          OperationPass<func::FuncOp>> {
  MLIR_DEFINE_EXPLICIT_INTERNAL_INLINE_TYPE_ID(FuseQuantizedMatMulForMI355XPass)

  StringRef getArgument() const override {
    return "fuse-quantized-matmul-for-mi355x";
  }
  StringRef getDescription() const override {
    return "Fuse (DynamicQuantizeLinear ->) MatMulInteger -> Cast -> Mul into "
           "one call of the MI355X runtime";
  }

  void runOnOperation() final {
    RewritePatternSet patterns(&getContext());
    patterns.insert<FuseScaledMatMulInteger>(&getContext());
    if (failed(applyPatternsGreedily(getOperation(), std::move(patterns))))
      signalPassFailure();
  }
};

} // namespace

std::unique_ptr<Pass> createFuseQuantizedMatMulForMI355XPass() {
  return std::make_unique<FuseQuantizedMatMulForMI355XPass>();
}

} // namespace onnx_mlir
