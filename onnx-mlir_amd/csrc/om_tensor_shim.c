/*
 * Stand-alone provider of the OMTensor accessors for harnesses that do not
 * link a compiled model (tests, benchmark, smoke check).  A compiled model
 * brings its own from libcruntime; this file is not part of the runtime
 * library proper.
 *
 * Field order and types follow src/Runtime/OMTensor.inc:125-140 so that a
 * tensor made here can be read by the reference's accessors and vice versa.
 * Strides are in elements, row-major (src/Runtime/OMTensor.inc:185-192).
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#include "om_tensor_abi.h"

struct OMTensor {
  void *allocatedPtr;
  void *alignedPtr;
  int64_t offset;
  int64_t *shape;
  int64_t *strides;
  int64_t rank;
  int dataType;
  int64_t owning;
};

static int64_t dtype_size(int dtype) {
  switch (dtype) {
  case OM_MI355X_TYPE_FLOAT:
  case OM_MI355X_TYPE_INT32:
    return 4;
  case OM_MI355X_TYPE_UINT8:
  case OM_MI355X_TYPE_INT8:
    return 1;
  case OM_MI355X_TYPE_INT64:
    return 8;
  default:
    return 0;
  }
}

OMTensor *omTensorCreate(
    void *data_ptr, const int64_t *shape, int64_t rank, int dtype) {
  OMTensor *t = (OMTensor *)calloc(1, sizeof(OMTensor));
  if (!t)
    return NULL;
  size_t dims = (size_t)(rank > 0 ? rank : 1);
  t->shape = (int64_t *)malloc(dims * sizeof(int64_t));
  t->strides = (int64_t *)malloc(dims * sizeof(int64_t));
  if (!t->shape || !t->strides) {
    free(t->shape);
    free(t->strides);
    free(t);
    return NULL;
  }
  t->allocatedPtr = data_ptr;
  t->alignedPtr = data_ptr;
  t->offset = 0;
  t->rank = rank;
  t->dataType = dtype;
  t->owning = 0;
  int64_t stride = 1;
  for (int64_t i = rank - 1; i >= 0; --i) {
    t->shape[i] = shape[i];
    t->strides[i] = stride;
    stride *= shape[i];
  }
  return t;
}

void omTensorDestroy(OMTensor *t) {
  if (!t)
    return;
  if (t->owning)
    free(t->allocatedPtr);
  free(t->shape);
  free(t->strides);
  free(t);
}

void *omTensorGetDataPtr(const OMTensor *t) { return t->alignedPtr; }
const int64_t *omTensorGetShape(const OMTensor *t) { return t->shape; }
const int64_t *omTensorGetStrides(const OMTensor *t) { return t->strides; }
int omTensorGetDataType(const OMTensor *t) { return t->dataType; }
int64_t omTensorGetRank(const OMTensor *t) { return t->rank; }

int64_t omTensorGetNumElems(const OMTensor *t) {
  int64_t n = 1;
  for (int64_t i = 0; i < t->rank; ++i)
    n *= t->shape[i];
  return n;
}

int64_t omTensorGetBufferSize(const OMTensor *t) {
  return omTensorGetNumElems(t) * dtype_size(t->dataType);
}
