// Loads and stores for data that is touched once (copy and scatter kernels): the non-temporal forms keep such a stream
// from displacing anything in the caches, and on MI355X they raise the rate a half-read half-written stream reaches
// (a plain 50 MiB + 50 MiB copy kernel: 5.7 - 6.0 TB/s with both against 5.2 - 5.4 TB/s with ordinary stores and
// 5.0 TB/s for the runtime's own device-to-device copy).
#ifndef INFINICORE_AMD_STREAMING_H
#define INFINICORE_AMD_STREAMING_H

#include <cstdint>
#include <hip/hip_runtime.h>

namespace device::amd {

namespace streaming_detail {
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
template <int BYTES> struct Word;
template <> struct Word<16> { using type = u32x4; };
template <> struct Word<8> { using type = u32x2; };
template <> struct Word<4> { using type = uint32_t; };
template <> struct Word<2> { using type = uint16_t; };
template <> struct Word<1> { using type = uint8_t; };
} // namespace streaming_detail

// U: any trivially copyable type of 1, 2, 4, 8 or 16 bytes; the address aligned to its size
template <typename U>
__device__ __forceinline__ U loadStreamed(const void *address) {
    using W = typename streaming_detail::Word<sizeof(U)>::type;
    return __builtin_bit_cast(U, __builtin_nontemporal_load(static_cast<const W *>(address)));
}
template <typename U>
__device__ __forceinline__ void storeStreamed(void *address, const U &value) {
    using W = typename streaming_detail::Word<sizeof(U)>::type;
    __builtin_nontemporal_store(__builtin_bit_cast(W, value), static_cast<W *>(address));
}

} // namespace device::amd

#endif
