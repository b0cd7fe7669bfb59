// Handle factory: a handle records the calling thread's current runtime device
// (reference src/infiniop/devices/handle.cc:27-130). CPU handles exist so that callers can probe
// the library without a GPU; the paged operators answer DEVICE_TYPE_NOT_SUPPORTED for them, as the
// reference does.
#include "../handle.h"
#include "infinirt.h"

__INFINI_C infiniStatus_t infiniopCreateHandle(infiniopHandle_t *handle_ptr) {
    if (handle_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    infiniStatus_t status = infinirtGetDevice(&device, &device_id);
    if (status != INFINI_STATUS_SUCCESS) {
        return status;
    }
    if (device != INFINI_DEVICE_CPU && device != INFINI_DEVICE_AMD) {
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
    *handle_ptr = new InfiniopHandle{device, device_id};
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infiniopDestroyHandle(infiniopHandle_t handle) {
    if (handle == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (handle->device != INFINI_DEVICE_CPU && handle->device != INFINI_DEVICE_AMD) {
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
    delete handle;
    return INFINI_STATUS_SUCCESS;
}
