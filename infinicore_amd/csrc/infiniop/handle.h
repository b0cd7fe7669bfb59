// What an infiniopHandle_t points to. The two leading ints are part of the ABI
// (reference src/infiniop/handle.h:6-9; language bindings read them). The AMD handle adds nothing:
// per-device facts the operators need (CU count, ...) live in a process-wide table keyed by
// device_id (devices/amd/amd_device.h), so a handle is exactly these eight bytes.
#ifndef INFINICORE_AMD_INFINIOP_HANDLE_IMPL_H
#define INFINICORE_AMD_INFINIOP_HANDLE_IMPL_H

#include "infiniop/handle.h"

struct InfiniopHandle {
    infiniDevice_t device;
    int device_id;
};

#endif
