// HIP backend of the runtime for AMD Instinct GPUs. Every function is a thin, status-translating
// wrapper over one HIP runtime call; stream, event and graph handles are the HIP objects themselves.
// Role of the reference's src/infinirt/cuda/infinirt_cuda.cu:282-560 for the CUDA runtime.
#include "../backend.h"
#include <cstdio>
#include <cstring>
#include <hip/hip_runtime_api.h>

// Returns INTERNAL_ERROR (and says why) when a HIP call fails. hipGetLastError clears the sticky
// per-thread error so one failure is not reported again by the next, unrelated call.
#define CHECK_HIP(CALL)                                                                                   \
    do {                                                                                                  \
        hipError_t err_ = (CALL);                                                                         \
        if (err_ != hipSuccess) {                                                                         \
            std::fprintf(stderr, "HIP error %d (%s) in `%s` at %s:%d\n", (int)err_, hipGetErrorString(err_), \
                         #CALL, __FILE__, __LINE__);                                                      \
            (void)hipGetLastError();                                                                      \
            return INFINI_STATUS_INTERNAL_ERROR;                                                          \
        }                                                                                                 \
    } while (0)

namespace infinirt::amd {

infiniStatus_t getDeviceCount(int *count) {
    // A machine without a GPU (or without the driver) has zero AMD devices; that is not an error.
    if (hipGetDeviceCount(count) != hipSuccess) {
        (void)hipGetLastError();
        *count = 0;
    }
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t setDevice(int device_id) {
    int count = 0;
    getDeviceCount(&count);
    if (device_id < 0 || device_id >= count) {
        return INFINI_STATUS_DEVICE_NOT_FOUND;
    }
    CHECK_HIP(hipSetDevice(device_id));
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t getMemInfo(int device_id, size_t *free_bytes, size_t *total_bytes) {
    int previous = 0;
    CHECK_HIP(hipGetDevice(&previous));
    if (previous != device_id) {
        CHECK_HIP(hipSetDevice(device_id));
    }
    hipError_t query = hipMemGetInfo(free_bytes, total_bytes);
    if (previous != device_id) {
        CHECK_HIP(hipSetDevice(previous));
    }
    CHECK_HIP(query);
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t getDeviceResourceSnapshot(int device_id, infinirtDeviceResourceSnapshot_t *snapshot) {
    std::memset(snapshot, 0, sizeof(*snapshot));
    snapshot->device_type = INFINI_DEVICE_AMD;
    snapshot->device_id = device_id;
    infiniStatus_t status = getMemInfo(device_id, &snapshot->free_bytes, &snapshot->total_bytes);
    if (status != INFINI_STATUS_SUCCESS) {
        return status;
    }
    snapshot->used_bytes = snapshot->total_bytes - snapshot->free_bytes;
    snapshot->valid_fields = INFINIRT_RESOURCE_FIELD_MEMORY_CAPACITY;
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t deviceSynchronize() {
    CHECK_HIP(hipDeviceSynchronize());
    return INFINI_STATUS_SUCCESS;
}

// Streams are created at the default priority on purpose: mixing priorities is not needed here.
infiniStatus_t streamCreate(infinirtStream_t *stream_ptr) {
    hipStream_t stream = nullptr;
    CHECK_HIP(hipStreamCreate(&stream));
    *stream_ptr = stream;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t streamDestroy(infinirtStream_t stream) {
    CHECK_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t streamSynchronize(infinirtStream_t stream) {
    CHECK_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t streamWaitEvent(infinirtStream_t stream, infinirtEvent_t event) {
    CHECK_HIP(hipStreamWaitEvent(static_cast<hipStream_t>(stream), static_cast<hipEvent_t>(event), 0));
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t eventCreate(infinirtEvent_t *event_ptr) {
    hipEvent_t event = nullptr;
    CHECK_HIP(hipEventCreate(&event));
    *event_ptr = event;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventCreateWithFlags(infinirtEvent_t *event_ptr, uint32_t flags) {
    unsigned hip_flags = hipEventDefault;
    if (flags & INFINIRT_EVENT_DISABLE_TIMING) {
        hip_flags |= hipEventDisableTiming;
    }
    if (flags & INFINIRT_EVENT_BLOCKING_SYNC) {
        hip_flags |= hipEventBlockingSync;
    }
    hipEvent_t event = nullptr;
    CHECK_HIP(hipEventCreateWithFlags(&event, hip_flags));
    *event_ptr = event;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventRecord(infinirtEvent_t event, infinirtStream_t stream) {
    CHECK_HIP(hipEventRecord(static_cast<hipEvent_t>(event), static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventQuery(infinirtEvent_t event, infinirtEventStatus_t *status_ptr) {
    hipError_t err = hipEventQuery(static_cast<hipEvent_t>(event));
    if (err == hipSuccess) {
        *status_ptr = INFINIRT_EVENT_COMPLETE;
    } else if (err == hipErrorNotReady) {
        (void)hipGetLastError();
        *status_ptr = INFINIRT_EVENT_NOT_READY;
    } else {
        CHECK_HIP(err);
    }
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventSynchronize(infinirtEvent_t event) {
    CHECK_HIP(hipEventSynchronize(static_cast<hipEvent_t>(event)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventDestroy(infinirtEvent_t event) {
    CHECK_HIP(hipEventDestroy(static_cast<hipEvent_t>(event)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t eventElapsedTime(float *ms_ptr, infinirtEvent_t start, infinirtEvent_t end) {
    CHECK_HIP(hipEventElapsedTime(ms_ptr, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(end)));
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t mallocDevice(void **p_ptr, size_t size) {
    CHECK_HIP(hipMalloc(p_ptr, size));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t mallocHost(void **p_ptr, size_t size) {
    CHECK_HIP(hipHostMalloc(p_ptr, size, hipHostMallocDefault));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t freeDevice(void *ptr) {
    CHECK_HIP(hipFree(ptr));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t freeHost(void *ptr) {
    CHECK_HIP(hipHostFree(ptr));
    return INFINI_STATUS_SUCCESS;
}

static hipMemcpyKind toHipKind(infinirtMemcpyKind_t kind) {
    switch (kind) {
    case INFINIRT_MEMCPY_H2H: return hipMemcpyHostToHost;
    case INFINIRT_MEMCPY_H2D: return hipMemcpyHostToDevice;
    case INFINIRT_MEMCPY_D2H: return hipMemcpyDeviceToHost;
    case INFINIRT_MEMCPY_D2D: return hipMemcpyDeviceToDevice;
    }
    return hipMemcpyDefault;
}
infiniStatus_t memcpy(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind) {
    CHECK_HIP(hipMemcpy(dst, src, size, toHipKind(kind)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t memcpyAsync(void *dst, const void *src, size_t size, infinirtMemcpyKind_t kind, infinirtStream_t stream) {
    CHECK_HIP(hipMemcpyAsync(dst, src, size, toHipKind(kind), static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t mallocAsync(void **p_ptr, size_t size, infinirtStream_t stream) {
    CHECK_HIP(hipMallocAsync(p_ptr, size, static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t freeAsync(void *ptr, infinirtStream_t stream) {
    CHECK_HIP(hipFreeAsync(ptr, static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t memsetDevice(void *ptr, int value, size_t count) {
    CHECK_HIP(hipMemset(ptr, value, count));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t memsetDeviceAsync(void *ptr, int value, size_t count, infinirtStream_t stream) {
    CHECK_HIP(hipMemsetAsync(ptr, value, count, static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t streamBeginCapture(infinirtStream_t stream, infinirtStreamCaptureMode_t mode) {
    hipStreamCaptureMode hip_mode = hipStreamCaptureModeGlobal;
    if (mode == INFINIRT_STREAM_CAPTURE_MODE_THREAD_LOCAL) {
        hip_mode = hipStreamCaptureModeThreadLocal;
    } else if (mode == INFINIRT_STREAM_CAPTURE_MODE_RELAXED) {
        hip_mode = hipStreamCaptureModeRelaxed;
    }
    CHECK_HIP(hipStreamBeginCapture(static_cast<hipStream_t>(stream), hip_mode));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t streamEndCapture(infinirtStream_t stream, infinirtGraph_t *graph_ptr) {
    hipGraph_t graph = nullptr;
    CHECK_HIP(hipStreamEndCapture(static_cast<hipStream_t>(stream), &graph));
    *graph_ptr = graph;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t graphDestroy(infinirtGraph_t graph) {
    CHECK_HIP(hipGraphDestroy(static_cast<hipGraph_t>(graph)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t graphInstantiate(infinirtGraphExec_t *graph_exec_ptr, infinirtGraph_t graph, infinirtGraphNode_t *node_ptr,
                                char *log_buffer, size_t buffer_size) {
    hipGraphExec_t exec = nullptr;
    CHECK_HIP(hipGraphInstantiate(&exec, static_cast<hipGraph_t>(graph), reinterpret_cast<hipGraphNode_t *>(node_ptr),
                                  log_buffer, buffer_size));
    *graph_exec_ptr = exec;
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t graphExecDestroy(infinirtGraphExec_t graph_exec) {
    CHECK_HIP(hipGraphExecDestroy(static_cast<hipGraphExec_t>(graph_exec)));
    return INFINI_STATUS_SUCCESS;
}
infiniStatus_t graphLaunch(infinirtGraphExec_t graph_exec, infinirtStream_t stream) {
    CHECK_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph_exec), static_cast<hipStream_t>(stream)));
    return INFINI_STATUS_SUCCESS;
}

} // namespace infinirt::amd
