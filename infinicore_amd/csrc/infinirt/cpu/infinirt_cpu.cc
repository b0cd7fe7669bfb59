// Host backend of the runtime: one "device", synchronous streams, plain heap memory.
// Same behaviour as the reference's src/infinirt/cpu/infinirt_cpu.cc (streams and events are inert,
// memory is malloc/free, copies are memcpy, graphs are unsupported).
#include "../backend.h"
#include <chrono>
#include <cstdlib>
#include <cstring>

namespace infinirt::cpu {

using Clock = std::chrono::steady_clock;

infiniStatus_t getDeviceCount(int *count) {
    *count = 1;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t setDevice(int) { return INFINI_STATUS_SUCCESS; }
infiniStatus_t getMemInfo(int, size_t *free_bytes, size_t *total_bytes) {
    *free_bytes = 0;
    *total_bytes = 0;
    return INFINI_STATUS_NOT_IMPLEMENTED;
}
infiniStatus_t getDeviceResourceSnapshot(int device_id, infinirtDeviceResourceSnapshot_t *snapshot) {
    std::memset(snapshot, 0, sizeof(*snapshot));
    snapshot->device_type = INFINI_DEVICE_CPU;
    snapshot->device_id = device_id;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t deviceSynchronize() { return INFINI_STATUS_SUCCESS; }

infiniStatus_t streamCreate(infinirtStream_t *stream_ptr) {
    *stream_ptr = nullptr;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t streamDestroy(infinirtStream_t) { return INFINI_STATUS_SUCCESS; }
infiniStatus_t streamSynchronize(infinirtStream_t) { return INFINI_STATUS_SUCCESS; }
infiniStatus_t streamWaitEvent(infinirtStream_t, infinirtEvent_t) { return INFINI_STATUS_SUCCESS; }

// A host event is a heap-allocated time point; work is synchronous, so it is complete once recorded.
infiniStatus_t eventCreate(infinirtEvent_t *event_ptr) {
    *event_ptr = new Clock::time_point(Clock::now());
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventCreateWithFlags(infinirtEvent_t *event_ptr, uint32_t) { return eventCreate(event_ptr); }
infiniStatus_t eventRecord(infinirtEvent_t event, infinirtStream_t) {
    if (event == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    *static_cast<Clock::time_point *>(event) = Clock::now();
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventQuery(infinirtEvent_t, infinirtEventStatus_t *status_ptr) {
    *status_ptr = INFINIRT_EVENT_COMPLETE;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventSynchronize(infinirtEvent_t) { return INFINI_STATUS_SUCCESS; }
infiniStatus_t eventDestroy(infinirtEvent_t event) {
    delete static_cast<Clock::time_point *>(event);
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventElapsedTime(float *ms_ptr, infinirtEvent_t start, infinirtEvent_t end) {
    if (start == nullptr || end == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    auto d = *static_cast<Clock::time_point *>(end) - *static_cast<Clock::time_point *>(start);
    *ms_ptr = std::chrono::duration<float, std::milli>(d).count();
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t mallocDevice(void **p_ptr, size_t size) {
    *p_ptr = std::malloc(size);
    return (*p_ptr == nullptr && size != 0) ? INFINI_STATUS_INTERNAL_ERROR : INFINI_STATUS_SUCCESS;
}
infiniStatus_t mallocHost(void **p_ptr, size_t size) { return mallocDevice(p_ptr, size); }
infiniStatus_t freeDevice(void *ptr) {
    std::free(ptr);
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t freeHost(void *ptr) { return freeDevice(ptr); }
infiniStatus_t memcpy(void *dst, const void *src, size_t size, infinirtMemcpyKind_t) {
    std::memcpy(dst, src, size);
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t memcpyAsync(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind, infinirtStream_t) {
    return memcpy(dst, src, size, kind);
}
infiniStatus_t mallocAsync(void **p_ptr, size_t size, infinirtStream_t) { return mallocDevice(p_ptr, size); }
infiniStatus_t freeAsync(void *ptr, infinirtStream_t) { return freeDevice(ptr); }
infiniStatus_t memsetDevice(void *ptr, int value, size_t count) {
    std::memset(ptr, value, count);
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t memsetDeviceAsync(void *ptr, int value, size_t count, infinirtStream_t) {
    return memsetDevice(ptr, value, count);
}

infiniStatus_t streamBeginCapture(infinirtStream_t, infinirtStreamCaptureMode_t) { return INFINI_STATUS_NOT_IMPLEMENTED; }
infiniStatus_t streamEndCapture(infinirtStream_t, infinirtGraph_t *) { return INFINI_STATUS_NOT_IMPLEMENTED; }
infiniStatus_t graphDestroy(infinirtGraph_t) { return INFINI_STATUS_NOT_IMPLEMENTED; }
infiniStatus_t graphInstantiate(infinirtGraphExec_t *, infinirtGraph_t, infinirtGraphNode_t *, char *, size_t) {
    return INFINI_STATUS_NOT_IMPLEMENTED;
}
infiniStatus_t graphExecDestroy(infinirtGraphExec_t) { return INFINI_STATUS_NOT_IMPLEMENTED; }
infiniStatus_t graphLaunch(infinirtGraphExec_t, infinirtStream_t) { return INFINI_STATUS_NOT_IMPLEMENTED; }

} // namespace infinirt::cpu
