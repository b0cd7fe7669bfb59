/*
 * Tensor metadata objects (dtype, shape, element strides); they never own data.
 * Replaces the reference's include/infiniop/tensor_descriptor.h:6-12.
 */
#ifndef INFINICORE_AMD_INFINIOP_TENSOR_DESCRIPTOR_H
#define INFINICORE_AMD_INFINIOP_TENSOR_DESCRIPTOR_H

#include "../infinicore.h"

struct InfiniopTensorDescriptor;
typedef struct InfiniopTensorDescriptor *infiniopTensorDescriptor_t;

/* shape has ndim entries; strides are in ELEMENTS and may be NULL, which means C-contiguous.
 * Reference: src/infiniop/tensor_descriptor.cc:8-24. */
__INFINI_C __export infiniStatus_t infiniopCreateTensorDescriptor(
    infiniopTensorDescriptor_t *desc_ptr,
    size_t ndim,
    const size_t *shape,
    const ptrdiff_t *strides,
    infiniDtype_t dtype);

/* Reference: src/infiniop/tensor_descriptor.cc:26-29. */
__INFINI_C __export infiniStatus_t infiniopDestroyTensorDescriptor(infiniopTensorDescriptor_t desc);

#endif
