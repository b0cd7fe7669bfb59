/*
 * Base of every operator descriptor. The object starts with {int device_type; int device_id;}
 * (reference src/infiniop/operator.h:6-9). Replaces include/infiniop/operator_descriptor.h:7-12.
 */
#ifndef INFINICORE_AMD_INFINIOP_OPERATOR_DESCRIPTOR_H
#define INFINICORE_AMD_INFINIOP_OPERATOR_DESCRIPTOR_H

#include "handle.h"
#include "tensor_descriptor.h"

struct InfiniopDescriptor;

/* Reference: src/infiniop/operator_descriptor.cc:3-8. */
__INFINI_C __export infiniStatus_t infiniopGetDescriptorDeviceType(
    const struct InfiniopDescriptor *desc_ptr, infiniDevice_t *device_type);

/* Reference: src/infiniop/operator_descriptor.cc:10-15. */
__INFINI_C __export infiniStatus_t infiniopGetDescriptorDeviceId(
    const struct InfiniopDescriptor *desc_ptr, int *device_id);

#endif
