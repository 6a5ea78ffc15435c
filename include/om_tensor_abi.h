/*
 * The slice of onnx-mlir's OMTensor C API that the MI355X runtime uses.
 *
 * This header restates declarations of the reference's public runtime API
 * (include/onnx-mlir/Runtime/OMTensor.h:92-347, data-type codes from
 * include/onnx-mlir/Runtime/OnnxDataTypeMetaData.inc:22-44) so that the
 * runtime can be built without the reference tree.  When the runtime is linked
 * into a compiled model these symbols come from the model's libcruntime; the
 * stand-alone harness gets them from libom_tensor_shim.so, whose struct is
 * byte-compatible with src/Runtime/OMTensor.inc:125-140.
 */
#ifndef OM_TENSOR_ABI_H
#define OM_TENSOR_ABI_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct OMTensor OMTensor;

/* ONNX element-type codes (only the ones this path touches are named). */
typedef enum {
  OM_MI355X_TYPE_UNDEFINED = 0,
  OM_MI355X_TYPE_FLOAT = 1,
  OM_MI355X_TYPE_UINT8 = 2,
  OM_MI355X_TYPE_INT8 = 3,
  OM_MI355X_TYPE_INT32 = 6,
  OM_MI355X_TYPE_INT64 = 7
} OM_MI355X_DATA_TYPE;

/* include/onnx-mlir/Runtime/OMTensor.h:92,159,168,197,228,279,319,327,335 */
OMTensor *omTensorCreate(
    void *data_ptr, const int64_t *shape, int64_t rank, int dtype);
void omTensorDestroy(OMTensor *tensor);
void *omTensorGetDataPtr(const OMTensor *tensor);
const int64_t *omTensorGetShape(const OMTensor *tensor);
const int64_t *omTensorGetStrides(const OMTensor *tensor);
int omTensorGetDataType(const OMTensor *tensor);
int64_t omTensorGetBufferSize(const OMTensor *tensor);
int64_t omTensorGetRank(const OMTensor *tensor);
int64_t omTensorGetNumElems(const OMTensor *tensor);

#ifdef __cplusplus
}
#endif
#endif
