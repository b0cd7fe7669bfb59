// Status-returning check helpers shared by the runtime and the operator library.
// Same names and behaviour as the reference's src/utils/check.h:9-60: a failed check writes one
// line with the expression and its location to stderr and returns the given status code.
#ifndef INFINICORE_AMD_UTILS_CHECK_H
#define INFINICORE_AMD_UTILS_CHECK_H

#include "infinicore.h"
#include <cstdio>
#include <initializer_list>

namespace utils {

inline const char *statusName(infiniStatus_t s) {
    switch (s) {
    case INFINI_STATUS_SUCCESS: return "Success";
    case INFINI_STATUS_INTERNAL_ERROR: return "Internal Error";
    case INFINI_STATUS_NOT_IMPLEMENTED: return "Not Implemented";
    case INFINI_STATUS_BAD_PARAM: return "Bad Param";
    case INFINI_STATUS_NULL_POINTER: return "Null Pointer";
    case INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED: return "Device Type Not Supported";
    case INFINI_STATUS_DEVICE_NOT_FOUND: return "Device Not Found";
    case INFINI_STATUS_DEVICE_NOT_INITIALIZED: return "Device Not Initialized";
    case INFINI_STATUS_DEVICE_ARCHITECTURE_NOT_SUPPORTED: return "Device Architecture Not Supported";
    case INFINI_STATUS_BAD_TENSOR_DTYPE: return "Bad Tensor Dtype";
    case INFINI_STATUS_BAD_TENSOR_SHAPE: return "Bad Tensor Shape";
    case INFINI_STATUS_BAD_TENSOR_STRIDES: return "Bad Tensor Strides";
    case INFINI_STATUS_INSUFFICIENT_WORKSPACE: return "Insufficient Workspace";
    }
    return "Unknown Status";
}

inline void reportFailedCheck(const char *expr, const char *func, const char *file, int line) {
    std::fprintf(stderr, "Check Failed: `(%s)` is False from %s at %s:%d\n", expr, func, file, line);
}

} // namespace utils

#define CHECK_OR_RETURN(CONDITION, ERROR)                                          \
    do {                                                                           \
        if (!(CONDITION)) {                                                        \
            utils::reportFailedCheck(#CONDITION, __func__, __FILE__, __LINE__);    \
            return ERROR;                                                          \
        }                                                                          \
    } while (0)

// Runs a call that yields infiniStatus_t and propagates anything but success.
#define CHECK_STATUS(API)                                                                       \
    do {                                                                                        \
        infiniStatus_t status_ = (API);                                                         \
        if (status_ != INFINI_STATUS_SUCCESS) {                                                 \
            std::fprintf(stderr, "Error Code %d (%s) in `%s` from %s at %s:%d\n", (int)status_, \
                         utils::statusName(status_), #API, __func__, __FILE__, __LINE__);       \
            return status_;                                                                     \
        }                                                                                       \
    } while (0)

// Accepts DT if it equals one of the listed dtypes, otherwise BAD_TENSOR_DTYPE.
#define CHECK_DTYPE(DT, ...)                                                                    \
    do {                                                                                        \
        bool dtype_ok_ = false;                                                                 \
        for (infiniDtype_t allowed_ : {__VA_ARGS__}) {                                          \
            dtype_ok_ = dtype_ok_ || (allowed_ == (DT));                                        \
        }                                                                                       \
        if (!dtype_ok_) {                                                                       \
            std::fprintf(stderr, "Unsupported dtype %d from %s at %s:%d\n", (int)(DT), __func__, \
                         __FILE__, __LINE__);                                                   \
            return INFINI_STATUS_BAD_TENSOR_DTYPE;                                              \
        }                                                                                       \
    } while (0)

// Unwraps a utils::Result<T>, returning its status when it holds an error.
#define CHECK_RESULT(RESULT)                 \
    do {                                     \
        if (!(RESULT)) {                     \
            return (RESULT).status();        \
        }                                    \
    } while (0)

#endif
