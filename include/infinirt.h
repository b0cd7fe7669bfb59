/*
 * InfiniRT: the small device runtime under InfiniOP (current device per thread, streams, events,
 * memory, stream capture). This build implements it on HIP for INFINI_DEVICE_AMD and keeps a host
 * backend for INFINI_DEVICE_CPU. Function names, argument order and enum values follow the
 * reference's include/infinirt.h:49-132, so a caller linked against the reference's libinfinirt.so
 * resolves the same symbols here. Each prototype cites the reference definition it replaces.
 */
#ifndef INFINICORE_AMD_INFINIRT_H
#define INFINICORE_AMD_INFINIRT_H

#include "infinicore.h"
#include <stdint.h>

/* Opaque handles: on the AMD device these are hipStream_t, hipEvent_t, hipGraph_t,
 * hipGraphNode_t and hipGraphExec_t passed through unchanged. */
typedef void *infinirtStream_t;
typedef void *infinirtEvent_t;
typedef void *infinirtGraph_t;
typedef void *infinirtGraphNode_t;
typedef void *infinirtGraphExec_t;

/* Which members of a resource snapshot a backend filled in (include/infinirt.h:16-23). */
typedef enum {
    INFINIRT_RESOURCE_FIELD_NONE = 0,
    INFINIRT_RESOURCE_FIELD_MEMORY_CAPACITY = 1ull << 0,
    INFINIRT_RESOURCE_FIELD_COMPUTE_UTILIZATION = 1ull << 1,
    INFINIRT_RESOURCE_FIELD_MEMORY_BANDWIDTH_UTILIZATION = 1ull << 2,
    INFINIRT_RESOURCE_FIELD_KERNEL_TIME_RATIO = 1ull << 3,
    INFINIRT_RESOURCE_FIELD_COMMUNICATION = 1ull << 4
} infinirtResourceField_t;

/* Same member order and types as include/infinirt.h:29-47. The AMD backend fills the memory
 * members only and sets just INFINIRT_RESOURCE_FIELD_MEMORY_CAPACITY in valid_fields. */
typedef struct {
    infiniDevice_t device_type;
    int device_id;
    uint64_t valid_fields;
    uint64_t estimated_fields;
    size_t free_bytes;
    size_t total_bytes;
    size_t used_bytes;
    size_t reserved_bytes;
    float compute_utilization;
    float memory_bandwidth_utilization;
    float kernel_time_ratio;
    float communication_time_ratio;
    uint64_t communication_bytes;
} infinirtDeviceResourceSnapshot_t;

typedef enum {
    INFINIRT_EVENT_COMPLETE = 0,
    INFINIRT_EVENT_NOT_READY = 1
} infinirtEventStatus_t;

typedef enum {
    INFINIRT_EVENT_DEFAULT = 0x0,
    INFINIRT_EVENT_DISABLE_TIMING = 0x1,
    INFINIRT_EVENT_BLOCKING_SYNC = 0x2
} infinirtEventFlags_t;

typedef enum {
    INFINIRT_MEMCPY_H2H = 0,
    INFINIRT_MEMCPY_H2D = 1,
    INFINIRT_MEMCPY_D2H = 2,
    INFINIRT_MEMCPY_D2D = 3
} infinirtMemcpyKind_t;

typedef enum {
    INFINIRT_STREAM_CAPTURE_MODE_GLOBAL = 0,
    INFINIRT_STREAM_CAPTURE_MODE_THREAD_LOCAL = 1,
    INFINIRT_STREAM_CAPTURE_MODE_RELAXED = 2
} infinirtStreamCaptureMode_t;

/* ---- library / device (reference src/infinirt/infinirt.cc:16-138) ---- */
__INFINI_C __export infiniStatus_t infinirtInit(void);                                      /* infinirt.cc:16 */
/* count_array must have INFINI_DEVICE_TYPE_COUNT entries. */
__INFINI_C __export infiniStatus_t infinirtGetAllDeviceCount(int *count_array);             /* infinirt.cc:23 */
__INFINI_C __export infiniStatus_t infinirtGetDeviceCount(infiniDevice_t device, int *count); /* infinirt.cc:96 */
/* Makes (device, device_id) the calling thread's current device; every later call on this thread
 * that takes no device argument acts on it. */
__INFINI_C __export infiniStatus_t infinirtSetDevice(infiniDevice_t device, int device_id); /* infinirt.cc:103 */
__INFINI_C __export infiniStatus_t infinirtGetDevice(infiniDevice_t *device_ptr, int *device_id_ptr); /* infinirt.cc:36 */
__INFINI_C __export infiniStatus_t infinirtGetMemInfo(infiniDevice_t device, int device_id,
                                                      size_t *free_bytes, size_t *total_bytes); /* infinirt.cc:119 */
__INFINI_C __export infiniStatus_t infinirtGetDeviceResourceSnapshot(
    infiniDevice_t device, int device_id, infinirtDeviceResourceSnapshot_t *snapshot);      /* infinirt.cc:126 */
__INFINI_C __export infiniStatus_t infinirtDeviceSynchronize(void);                         /* infinirt.cc:136 */

/* ---- streams (infinirt.cc:140-154) ---- */
__INFINI_C __export infiniStatus_t infinirtStreamCreate(infinirtStream_t *stream_ptr);
__INFINI_C __export infiniStatus_t infinirtStreamDestroy(infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinirtStreamSynchronize(infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinirtStreamWaitEvent(infinirtStream_t stream, infinirtEvent_t event);

/* ---- events (infinirt.cc:156-182) ---- */
__INFINI_C __export infiniStatus_t infinirtEventCreate(infinirtEvent_t *event_ptr);
__INFINI_C __export infiniStatus_t infinirtEventCreateWithFlags(infinirtEvent_t *event_ptr, uint32_t flags);
__INFINI_C __export infiniStatus_t infinirtEventRecord(infinirtEvent_t event, infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinirtEventQuery(infinirtEvent_t event, infinirtEventStatus_t *status_ptr);
__INFINI_C __export infiniStatus_t infinirtEventSynchronize(infinirtEvent_t event);
__INFINI_C __export infiniStatus_t infinirtEventDestroy(infinirtEvent_t event);
/* Milliseconds between two recorded, completed events. */
__INFINI_C __export infiniStatus_t infinirtEventElapsedTime(float *ms_ptr, infinirtEvent_t start, infinirtEvent_t end);

/* ---- memory (infinirt.cc:184-222) ---- */
__INFINI_C __export infiniStatus_t infinirtMalloc(void **p_ptr, size_t size);
__INFINI_C __export infiniStatus_t infinirtMallocHost(void **p_ptr, size_t size); /* pinned */
__INFINI_C __export infiniStatus_t infinirtFree(void *ptr);
__INFINI_C __export infiniStatus_t infinirtFreeHost(void *ptr);
__INFINI_C __export infiniStatus_t infinirtMemcpy(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind);
__INFINI_C __export infiniStatus_t infinirtMemcpyAsync(void *dst, const void *src, size_t size,
                                                       infinirtMemcpyKind_t kind, infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinirtMallocAsync(void **p_ptr, size_t size, infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinirtFreeAsync(void *ptr, infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinirtMemset(void *ptr, int value, size_t count);
__INFINI_C __export infiniStatus_t infinirtMemsetAsync(void *ptr, int value, size_t count, infinirtStream_t stream);

/* ---- stream capture and graphs (infinirt.cc:224-251) ---- */
__INFINI_C __export infiniStatus_t infinirtStreamBeginCapture(infinirtStream_t stream, infinirtStreamCaptureMode_t mode);
__INFINI_C __export infiniStatus_t infinirtStreamEndCapture(infinirtStream_t stream, infinirtGraph_t *graph_ptr);
__INFINI_C __export infiniStatus_t infinirtGraphDestroy(infinirtGraph_t graph);
__INFINI_C __export infiniStatus_t infinirtGraphInstantiate(infinirtGraphExec_t *graph_exec_ptr, infinirtGraph_t graph,
                                                            infinirtGraphNode_t *node_ptr, char *log_buffer,
                                                            size_t buffer_size);
__INFINI_C __export infiniStatus_t infinirtGraphExecDestroy(infinirtGraphExec_t graph_exec);
/* The reference exports this spelling (infinirt.cc:249); it is kept so existing callers link. */
__INFINI_C __export infiniStatus_t infinirtGraphLuanch(infinirtGraphExec_t graph_exec, infinirtStream_t stream);

#endif /* INFINICORE_AMD_INFINIRT_H */
