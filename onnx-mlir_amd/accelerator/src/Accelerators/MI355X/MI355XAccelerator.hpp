/*
 * SPDX-License-Identifier: Apache-2.0
 */

//===------------------------ MI355XAccelerator.hpp -----------------------===//
//
// Accelerator plug-in that sends the 8-bit quantisation ops of a model to an
// AMD Instinct MI355X through the C entry points of libRuntimeMI355X.a.
//
// It introduces no dialect: the ops stay in the ONNX dialect until the
// ONNX-to-Krnl conversion, where patterns of a higher benefit than the CPU ones
// turn each of them into one `krnl.call`.  Everything after that (KrnlCallOp
// lowering, OMTensor marshalling, accelerator initialisation in the entry
// point) is the stock onnx-mlir machinery.
//
//===----------------------------------------------------------------------===//

#ifndef ONNX_MLIR_MI355X_ACCELERATOR_H
#define ONNX_MLIR_MI355X_ACCELERATOR_H

#include "mlir/IR/BuiltinTypes.h"
#include "src/Accelerators/Accelerator.hpp"

namespace onnx_mlir {
namespace accel {

/// One instance per process, created on demand by createMI355X(), the factory
/// that src/Accelerators/Accelerator.hpp:34-38 declares for every name in
/// ONNX_MLIR_ACCELERATORS.
class MI355XAccelerator final : public Accelerator {
public:
  MI355XAccelerator(const MI355XAccelerator &) = delete;
  MI355XAccelerator &operator=(const MI355XAccelerator &) = delete;

  static MI355XAccelerator *getInstance();

  static bool classof(const Accelerator *accel) {
    return accel->getKind() == Accelerator::Kind::MI355X;
  }
  static bool classof(const MI355XAccelerator *) { return true; }

  /// 0x[major][minor][patch]; handed to OMInitCompatibleAccelMI355X() by the
  /// generated entry point.
  uint64_t getVersionNumber() const final;
  std::string getAccelCompileInfo() const final;

  // onnx-mlir driver.
  void addPasses(mlir::OwningOpRef<mlir::ModuleOp> &module,
      mlir::PassManager &pm, onnx_mlir::EmissionTargetType &emissionTarget,
      std::string outputNameNoExt) const final;

  // onnx-mlir-opt driver.
  void registerDialects(mlir::DialectRegistry &registry) const final;
  void registerPasses(int optLevel) const final;
  void configurePasses() const final;

  // ONNX-to-Krnl pass.
  mlir::MemRefType convertTensorTypeToMemRefType(
      const mlir::TensorType tensorType) const final;
  int64_t getDefaultAllocAlignment(
      const mlir::TensorType tensorType) const final;
  void conversionTargetONNXToKrnl(mlir::ConversionTarget &target) const final;
  void rewritePatternONNXToKrnl(mlir::RewritePatternSet &patterns,
      mlir::TypeConverter &typeConverter, mlir::MLIRContext *ctx) const final;

  // Krnl-to-LLVM pass.
  void conversionTargetKrnlToLLVM(mlir::ConversionTarget &target) const final;
  void rewritePatternKrnlToLLVM(mlir::RewritePatternSet &patterns,
      mlir::LLVMTypeConverter &typeConverter,
      mlir::MLIRContext *ctx) const final;

private:
  MI355XAccelerator();
};

} // namespace accel
} // namespace onnx_mlir
#endif
