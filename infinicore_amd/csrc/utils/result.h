// Minimal "value or status" carrier used by the create-time validators
// (same role as the reference's src/utils/result.hpp: a Result<T> converts from either a T or an
// infiniStatus_t, tests true when it holds a value, and hands the value out with take()).
#ifndef INFINICORE_AMD_UTILS_RESULT_H
#define INFINICORE_AMD_UTILS_RESULT_H

#include "infinicore.h"
#include <optional>
#include <utility>

namespace utils {

template <typename T>
class Result {
    std::optional<T> _value;
    infiniStatus_t _status;

public:
    Result(T value) : _value(std::move(value)), _status(INFINI_STATUS_SUCCESS) {}
    Result(infiniStatus_t status) : _value(std::nullopt), _status(status) {}

    explicit operator bool() const { return _value.has_value(); }
    infiniStatus_t status() const { return _status; }
    T take() { return std::move(*_value); }
    const T &value() const { return *_value; }
};

} // namespace utils

#endif
