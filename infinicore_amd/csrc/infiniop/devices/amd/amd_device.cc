#include "amd_device.h"
#include <hip/hip_runtime_api.h>
#include <map>
#include <mutex>

namespace device::amd {

const DeviceInfo &deviceInfo(int device_id) {
    static std::mutex lock;
    static std::map<int, DeviceInfo> table;
    std::lock_guard<std::mutex> guard(lock);
    auto found = table.find(device_id);
    if (found != table.end()) {
        return found->second;
    }
    DeviceInfo info{256, 64, false};
    int cus = 0, wave = 0;
    if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device_id) == hipSuccess
        && hipDeviceGetAttribute(&wave, hipDeviceAttributeWarpSize, device_id) == hipSuccess && cus > 0) {
        info = DeviceInfo{cus, wave, true};
    } else {
        (void)hipGetLastError();
    }
    return table.emplace(device_id, info).first->second;
}

} // namespace device::amd
