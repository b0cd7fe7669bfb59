// Facts about an AMD GPU that launch heuristics need, looked up once per device and cached for the
// life of the process. (The reference keeps the equivalent cudaDeviceProp fields inside its nvidia
// handle, src/infiniop/devices/nvidia/nvidia_common.cu:15-63.)
#ifndef INFINICORE_AMD_DEVICE_H
#define INFINICORE_AMD_DEVICE_H

namespace device::amd {

struct DeviceInfo {
    int compute_units;   // CUs on the device (256 on MI355X)
    int wavefront_size;  // lanes per wavefront (64 on CDNA)
    bool queried;        // false when HIP could not see the device and defaults were used
};

// Never fails: if the device cannot be queried (no GPU visible to this process) it returns MI355X
// defaults with queried == false, so descriptors can still be created and validated on a host
// without a GPU.
const DeviceInfo &deviceInfo(int device_id);

} // namespace device::amd

#endif
