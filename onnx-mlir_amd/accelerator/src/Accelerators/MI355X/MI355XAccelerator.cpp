/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===------------------------ MI355XAccelerator.cpp -----------------------===//

#include "src/Accelerators/MI355X/MI355XAccelerator.hpp"

#include "mlir/Pass/Pass.h"
#include "mlir/Pass/PassRegistry.h"
#include "llvm/Support/Debug.h"

#include "src/Accelerators/MI355X/Compiler/MI355XCompilerOptions.hpp"
#include "src/Accelerators/MI355X/Compiler/MI355XCompilerUtils.hpp"
#include "src/Accelerators/MI355X/Conversion/ONNXToMI355XCall.hpp"
#include "src/Accelerators/MI355X/Transform/MI355XPasses.hpp"
#include "src/Compiler/CompilerOptions.hpp"

#define DEBUG_TYPE "MI355XAccelerator"

namespace onnx_mlir {
namespace accel {

// Must stay equal to OM_MI355X_VERSION in om_mi355x.h: the runtime refuses a
// model compiled for a newer major.minor than its own.
static constexpr uint64_t kRuntimeVersion = 0x010100;

Accelerator *createMI355X() { return MI355XAccelerator::getInstance(); }

MI355XAccelerator *MI355XAccelerator::getInstance() {
  // Never destroyed: `acceleratorTargets` keeps a raw pointer to it until the
  // process ends.
  static MI355XAccelerator *theInstance = new MI355XAccelerator();
  return theInstance;
}

MI355XAccelerator::MI355XAccelerator()
    : Accelerator(Accelerator::Kind::MI355X) {
  LLVM_DEBUG(llvm::dbgs() << "Creating the MI355X accelerator\n");
  acceleratorTargets.push_back(this);

  // Libraries a compiled model is linked against, in dependency order
  // (the option mechanism is src/Compiler/CompilerOptions.cpp:1559-1575): the
  // runtime as a static archive, libRuntimeMI355X.a, the way
  // src/Accelerators/NNPA/NNPAAccelerator.cpp:60-81 names libRuntimeNNPA.a,
  // then the HIP runtime it calls.  The archive leaves the omTensor*
  // accessors undefined; the model's libcruntime provides them.
  addCompilerConfig(CCM_SHARED_LIB_DEPS, {"RuntimeMI355X", "amdhip64"},
      /*exclusive=*/true);
  std::vector<std::string> libDirs;
#ifdef OM_MI355X_RUNTIME_DIR
  libDirs.emplace_back(OM_MI355X_RUNTIME_DIR);
#endif
  libDirs.emplace_back("/opt/rocm/lib");
  addCompilerConfig(CCM_SHARED_LIB_PATH_DEPS, libDirs, /*exclusive=*/true);
}

uint64_t MI355XAccelerator::getVersionNumber() const { return kRuntimeVersion; }

std::string MI355XAccelerator::getAccelCompileInfo() const {
  std::string version = std::to_string((kRuntimeVersion >> 16) & 0xFF) + "." +
                        std::to_string((kRuntimeVersion >> 8) & 0xFF) + "." +
                        std::to_string(kRuntimeVersion & 0xFF);
  return "{\"gfx\": \"gfx950\", \"om_mi355x_version\": \"" + version + "\"}";
}

void MI355XAccelerator::addPasses(mlir::OwningOpRef<mlir::ModuleOp> &module,
    mlir::PassManager &pm, onnx_mlir::EmissionTargetType &emissionTarget,
    std::string outputNameNoExt) const {
  addPassesMI355X(module, pm, emissionTarget, outputNameNoExt);
}

void MI355XAccelerator::registerDialects(
    mlir::DialectRegistry & /*registry*/) const {
  // The accelerated ops remain ONNX ops until they become krnl.call: there is
  // nothing to add to what the drivers register anyway.
}

void MI355XAccelerator::registerPasses(int /*optLevel*/) const {
  mlir::registerPass([]() -> std::unique_ptr<mlir::Pass> {
    return onnx_mlir::createFuseQuantizedMatMulForMI355XPass();
  });
  mlir::registerPass([]() -> std::unique_ptr<mlir::Pass> {
    return onnx_mlir::createRecomposeQDQMatMulForMI355XPass();
  });
  mlir::registerPass([]() -> std::unique_ptr<mlir::Pass> {
    return onnx_mlir::createKeepBuffersOnMI355XPass();
  });
}

void MI355XAccelerator::configurePasses() const { configurePassesMI355X(); }

mlir::MemRefType MI355XAccelerator::convertTensorTypeToMemRefType(
    const mlir::TensorType /*tensorType*/) const {
  // Plain row-major tensors only: let the generic converter decide.
  return nullptr;
}

int64_t MI355XAccelerator::getDefaultAllocAlignment(
    const mlir::TensorType tensorType) const {
  // The runtime reads and writes whole tensors with DMA copies and 16-byte
  // vector accesses.  Page alignment for 8-bit and 32-bit tensors keeps the
  // host side of those copies on page boundaries; -1 (the value the base
  // class returns) leaves every other type to the default.
  mlir::Type elementType = tensorType.getElementType();
  if (elementType.isInteger(8) || elementType.isInteger(32) ||
      elementType.isF32())
    return 4096;
  return -1;
}

void MI355XAccelerator::conversionTargetONNXToKrnl(
    mlir::ConversionTarget & /*target*/) const {
  // The ONNX-to-Krnl pass already marks every ONNX op illegal and krnl.call
  // legal; ops this accelerator declines fall through to the CPU patterns.
}

void MI355XAccelerator::rewritePatternONNXToKrnl(
    mlir::RewritePatternSet &patterns, mlir::TypeConverter &typeConverter,
    mlir::MLIRContext *ctx) const {
  onnx_mlir::populateONNXToMI355XCallPatterns(patterns, typeConverter, ctx);
}

void MI355XAccelerator::conversionTargetKrnlToLLVM(
    mlir::ConversionTarget & /*target*/) const {}

void MI355XAccelerator::rewritePatternKrnlToLLVM(
    mlir::RewritePatternSet & /*patterns*/,
    mlir::LLVMTypeConverter & /*typeConverter*/,
    mlir::MLIRContext * /*ctx*/) const {
  // krnl.call is lowered by the stock KrnlCallOpLowering
  // (src/Conversion/KrnlToLLVM/KrnlCall.cpp:34-102).
}

} // namespace accel
} // namespace onnx_mlir
