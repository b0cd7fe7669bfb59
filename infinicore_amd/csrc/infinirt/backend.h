// Per-backend function table of the runtime. Each backend namespace declares the same set of
// functions (reference: the INFINIRT_DEVICE_API macro, src/infinirt/infinirt_impl.h:6-52); the
// dispatcher in infinirt.cc picks the namespace from the calling thread's current device type.
#ifndef INFINICORE_AMD_INFINIRT_BACKEND_H
#define INFINICORE_AMD_INFINIRT_BACKEND_H

#include "infinirt.h"

#define INFINIRT_BACKEND_DECLARATIONS                                                                            \
    infiniStatus_t getDeviceCount(int *count);                                                                   \
    infiniStatus_t setDevice(int device_id);                                                                     \
    infiniStatus_t getMemInfo(int device_id, size_t *free_bytes, size_t *total_bytes);                           \
    infiniStatus_t getDeviceResourceSnapshot(int device_id, infinirtDeviceResourceSnapshot_t *snapshot);         \
    infiniStatus_t deviceSynchronize();                                                                          \
    infiniStatus_t streamCreate(infinirtStream_t *stream_ptr);                                                   \
    infiniStatus_t streamDestroy(infinirtStream_t stream);                                                       \
    infiniStatus_t streamSynchronize(infinirtStream_t stream);                                                   \
    infiniStatus_t streamWaitEvent(infinirtStream_t stream, infinirtEvent_t event);                              \
    infiniStatus_t eventCreate(infinirtEvent_t *event_ptr);                                                      \
    infiniStatus_t eventCreateWithFlags(infinirtEvent_t *event_ptr, uint32_t flags);                             \
    infiniStatus_t eventRecord(infinirtEvent_t event, infinirtStream_t stream);                                  \
    infiniStatus_t eventQuery(infinirtEvent_t event, infinirtEventStatus_t *status_ptr);                         \
    infiniStatus_t eventSynchronize(infinirtEvent_t event);                                                      \
    infiniStatus_t eventDestroy(infinirtEvent_t event);                                                          \
    infiniStatus_t eventElapsedTime(float *ms_ptr, infinirtEvent_t start, infinirtEvent_t end);                  \
    infiniStatus_t mallocDevice(void **p_ptr, size_t size);                                                      \
    infiniStatus_t mallocHost(void **p_ptr, size_t size);                                                        \
    infiniStatus_t freeDevice(void *ptr);                                                                        \
    infiniStatus_t freeHost(void *ptr);                                                                          \
    infiniStatus_t memcpy(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind);                   \
    infiniStatus_t memcpyAsync(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind,               \
                               infinirtStream_t stream);                                                         \
    infiniStatus_t mallocAsync(void **p_ptr, size_t size, infinirtStream_t stream);                              \
    infiniStatus_t freeAsync(void *ptr, infinirtStream_t stream);                                                \
    infiniStatus_t memsetDevice(void *ptr, int value, size_t count);                                             \
    infiniStatus_t memsetDeviceAsync(void *ptr, int value, size_t count, infinirtStream_t stream);               \
    infiniStatus_t streamBeginCapture(infinirtStream_t stream, infinirtStreamCaptureMode_t mode);                \
    infiniStatus_t streamEndCapture(infinirtStream_t stream, infinirtGraph_t *graph_ptr);                        \
    infiniStatus_t graphDestroy(infinirtGraph_t graph);                                                          \
    infiniStatus_t graphInstantiate(infinirtGraphExec_t *graph_exec_ptr, infinirtGraph_t graph,                  \
                                    infinirtGraphNode_t *node_ptr, char *log_buffer, size_t buffer_size);        \
    infiniStatus_t graphExecDestroy(infinirtGraphExec_t graph_exec);                                             \
    infiniStatus_t graphLaunch(infinirtGraphExec_t graph_exec, infinirtStream_t stream);

namespace infinirt::amd {
INFINIRT_BACKEND_DECLARATIONS
}
namespace infinirt::cpu {
INFINIRT_BACKEND_DECLARATIONS
}

#endif
