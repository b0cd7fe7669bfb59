#include "operator.h"

__INFINI_C infiniStatus_t infiniopGetDescriptorDeviceType(const InfiniopDescriptor *desc_ptr, infiniDevice_t *device_type) {
    if (desc_ptr == nullptr || device_type == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    *device_type = desc_ptr->device_type;
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infiniopGetDescriptorDeviceId(const InfiniopDescriptor *desc_ptr, int *device_id) {
    if (desc_ptr == nullptr || device_id == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    *device_id = desc_ptr->device_id;
    return INFINI_STATUS_SUCCESS;
}
