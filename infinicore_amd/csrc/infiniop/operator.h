// Common head of every operator descriptor (reference src/infiniop/operator.h:6-9): the entry
// points read device_type to pick the backend class the pointer really refers to.
#ifndef INFINICORE_AMD_INFINIOP_OPERATOR_IMPL_H
#define INFINICORE_AMD_INFINIOP_OPERATOR_IMPL_H

#include "infiniop/operator_descriptor.h"

struct InfiniopDescriptor {
    infiniDevice_t device_type;
    int device_id;
};

#endif
