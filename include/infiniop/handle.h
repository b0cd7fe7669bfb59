/*
 * Library context handle. Replaces the reference's include/infiniop/handle.h:6-12.
 * The object behind the pointer starts with {int device; int device_id;}
 * (reference src/infiniop/handle.h:6-9); foreign-language bindings read those two fields.
 */
#ifndef INFINICORE_AMD_INFINIOP_HANDLE_H
#define INFINICORE_AMD_INFINIOP_HANDLE_H

#include "../infinicore.h"

struct InfiniopHandle;
typedef struct InfiniopHandle *infiniopHandle_t;

/* Creates a handle for the calling thread's current InfiniRT device (infinirtSetDevice).
 * NULL handle_ptr -> NULL_POINTER; a device without a backend -> DEVICE_TYPE_NOT_SUPPORTED.
 * Reference: src/infiniop/devices/handle.cc:27-80. */
__INFINI_C __export infiniStatus_t infiniopCreateHandle(infiniopHandle_t *handle_ptr);

/* Frees a handle. Descriptors created from it stay usable (they copy what they need).
 * Reference: src/infiniop/devices/handle.cc:82-130. */
__INFINI_C __export infiniStatus_t infiniopDestroyHandle(infiniopHandle_t handle);

#endif
