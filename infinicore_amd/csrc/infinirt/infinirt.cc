// C entry points of libinfinirt.so: a thread-local "current device" plus dispatch of every call
// to the backend of that device's type. Behaviour follows the reference's
// src/infinirt/infinirt.cc:11-251; backends here are amd (HIP) and cpu (host).
#include "backend.h"
#include "../utils/check.h"

namespace {

// The device every argument-less runtime call of this thread acts on
// (reference: CURRENT_DEVICE_TYPE / CURRENT_DEVICE_ID, infinirt.cc:11-12).
thread_local infiniDevice_t tls_device_type = INFINI_DEVICE_CPU;
thread_local int tls_device_id = 0;

} // namespace

// Expands to `return <backend>::CALL;` for the backend that serves TYPE.
#define DISPATCH(TYPE, CALL)                                  \
    switch (TYPE) {                                           \
    case INFINI_DEVICE_CPU:                                   \
        return infinirt::cpu::CALL;                           \
    case INFINI_DEVICE_AMD:                                   \
        return infinirt::amd::CALL;                           \
    default:                                                  \
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;       \
    }

#define DISPATCH_CURRENT(CALL) DISPATCH(tls_device_type, CALL)

__INFINI_C infiniStatus_t infinirtInit(void) {
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infinirtGetAllDeviceCount(int *count_array) {
    if (count_array == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    for (int t = 0; t < INFINI_DEVICE_TYPE_COUNT; ++t) {
        // Device types without a backend in this build report zero devices.
        count_array[t] = 0;
        if (t == INFINI_DEVICE_CPU || t == INFINI_DEVICE_AMD) {
            CHECK_STATUS(infinirtGetDeviceCount(static_cast<infiniDevice_t>(t), &count_array[t]));
        }
    }
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infinirtGetDeviceCount(infiniDevice_t device, int *count) {
    if (count == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH(device, getDeviceCount(count));
}

__INFINI_C infiniStatus_t infinirtSetDevice(infiniDevice_t device, int device_id) {
    infiniStatus_t status;
    switch (device) {
    case INFINI_DEVICE_CPU:
        status = infinirt::cpu::setDevice(device_id);
        break;
    case INFINI_DEVICE_AMD:
        status = infinirt::amd::setDevice(device_id);
        break;
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
    if (status == INFINI_STATUS_SUCCESS) {
        tls_device_type = device;
        tls_device_id = device_id;
    }
    return status;
}

__INFINI_C infiniStatus_t infinirtGetDevice(infiniDevice_t *device_ptr, int *device_id_ptr) {
    if (device_ptr == nullptr && device_id_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (device_ptr != nullptr) {
        *device_ptr = tls_device_type;
    }
    if (device_id_ptr != nullptr) {
        *device_id_ptr = tls_device_id;
    }
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infinirtGetMemInfo(infiniDevice_t device, int device_id, size_t *free_bytes, size_t *total_bytes) {
    if (free_bytes == nullptr || total_bytes == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH(device, getMemInfo(device_id, free_bytes, total_bytes));
}

__INFINI_C infiniStatus_t infinirtGetDeviceResourceSnapshot(infiniDevice_t device, int device_id,
                                                            infinirtDeviceResourceSnapshot_t *snapshot) {
    if (snapshot == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH(device, getDeviceResourceSnapshot(device_id, snapshot));
}

__INFINI_C infiniStatus_t infinirtDeviceSynchronize(void) { DISPATCH_CURRENT(deviceSynchronize()); }

__INFINI_C infiniStatus_t infinirtStreamCreate(infinirtStream_t *stream_ptr) {
    if (stream_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(streamCreate(stream_ptr));
}
__INFINI_C infiniStatus_t infinirtStreamDestroy(infinirtStream_t stream) { DISPATCH_CURRENT(streamDestroy(stream)); }
__INFINI_C infiniStatus_t infinirtStreamSynchronize(infinirtStream_t stream) { DISPATCH_CURRENT(streamSynchronize(stream)); }
__INFINI_C infiniStatus_t infinirtStreamWaitEvent(infinirtStream_t stream, infinirtEvent_t event) {
    DISPATCH_CURRENT(streamWaitEvent(stream, event));
}

__INFINI_C infiniStatus_t infinirtEventCreate(infinirtEvent_t *event_ptr) {
    if (event_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(eventCreate(event_ptr));
}
__INFINI_C infiniStatus_t infinirtEventCreateWithFlags(infinirtEvent_t *event_ptr, uint32_t flags) {
    if (event_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(eventCreateWithFlags(event_ptr, flags));
}
__INFINI_C infiniStatus_t infinirtEventRecord(infinirtEvent_t event, infinirtStream_t stream) {
    DISPATCH_CURRENT(eventRecord(event, stream));
}
__INFINI_C infiniStatus_t infinirtEventQuery(infinirtEvent_t event, infinirtEventStatus_t *status_ptr) {
    if (status_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(eventQuery(event, status_ptr));
}
__INFINI_C infiniStatus_t infinirtEventSynchronize(infinirtEvent_t event) { DISPATCH_CURRENT(eventSynchronize(event)); }
__INFINI_C infiniStatus_t infinirtEventDestroy(infinirtEvent_t event) { DISPATCH_CURRENT(eventDestroy(event)); }
__INFINI_C infiniStatus_t infinirtEventElapsedTime(float *ms_ptr, infinirtEvent_t start, infinirtEvent_t end) {
    if (ms_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(eventElapsedTime(ms_ptr, start, end));
}

__INFINI_C infiniStatus_t infinirtMalloc(void **p_ptr, size_t size) {
    if (p_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(mallocDevice(p_ptr, size));
}
__INFINI_C infiniStatus_t infinirtMallocHost(void **p_ptr, size_t size) {
    if (p_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(mallocHost(p_ptr, size));
}
__INFINI_C infiniStatus_t infinirtFree(void *ptr) { DISPATCH_CURRENT(freeDevice(ptr)); }
__INFINI_C infiniStatus_t infinirtFreeHost(void *ptr) { DISPATCH_CURRENT(freeHost(ptr)); }
__INFINI_C infiniStatus_t infinirtMemcpy(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind) {
    DISPATCH_CURRENT(memcpy(dst, src, size, kind));
}
__INFINI_C infiniStatus_t infinirtMemcpyAsync(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind,
                                              infinirtStream_t stream) {
    DISPATCH_CURRENT(memcpyAsync(dst, src, size, kind, stream));
}
__INFINI_C infiniStatus_t infinirtMallocAsync(void **p_ptr, size_t size, infinirtStream_t stream) {
    if (p_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(mallocAsync(p_ptr, size, stream));
}
__INFINI_C infiniStatus_t infinirtFreeAsync(void *ptr, infinirtStream_t stream) { DISPATCH_CURRENT(freeAsync(ptr, stream)); }
__INFINI_C infiniStatus_t infinirtMemset(void *ptr, int value, size_t count) { DISPATCH_CURRENT(memsetDevice(ptr, value, count)); }
__INFINI_C infiniStatus_t infinirtMemsetAsync(void *ptr, int value, size_t count, infinirtStream_t stream) {
    DISPATCH_CURRENT(memsetDeviceAsync(ptr, value, count, stream));
}

__INFINI_C infiniStatus_t infinirtStreamBeginCapture(infinirtStream_t stream, infinirtStreamCaptureMode_t mode) {
    DISPATCH_CURRENT(streamBeginCapture(stream, mode));
}
__INFINI_C infiniStatus_t infinirtStreamEndCapture(infinirtStream_t stream, infinirtGraph_t *graph_ptr) {
    if (graph_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(streamEndCapture(stream, graph_ptr));
}
__INFINI_C infiniStatus_t infinirtGraphDestroy(infinirtGraph_t graph) { DISPATCH_CURRENT(graphDestroy(graph)); }
__INFINI_C infiniStatus_t infinirtGraphInstantiate(infinirtGraphExec_t *graph_exec_ptr, infinirtGraph_t graph,
                                                   infinirtGraphNode_t *node_ptr, char *log_buffer, size_t buffer_size) {
    if (graph_exec_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    DISPATCH_CURRENT(graphInstantiate(graph_exec_ptr, graph, node_ptr, log_buffer, buffer_size));
}
__INFINI_C infiniStatus_t infinirtGraphExecDestroy(infinirtGraphExec_t graph_exec) { DISPATCH_CURRENT(graphExecDestroy(graph_exec)); }
__INFINI_C infiniStatus_t infinirtGraphLuanch(infinirtGraphExec_t graph_exec, infinirtStream_t stream) {
    DISPATCH_CURRENT(graphLaunch(graph_exec, stream));
}
