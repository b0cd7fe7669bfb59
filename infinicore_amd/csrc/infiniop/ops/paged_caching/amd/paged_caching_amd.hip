// paged_caching on AMD Instinct (gfx950): scatter the K and V vectors of a chunk of tokens into
// their slots of the paged pool.
//
// The operation is a pure byte copy, so the kernel is written for memory transactions, not for
// elements: a token's (head, vector) rows are moved in the widest power-of-two unit (up to 16
// bytes) that divides every row length, stride and base address involved. A workgroup is a
// (chunk lanes) x (heads) x (tokens) box of 256 threads; adjacent lanes move adjacent units of one
// row, so every wavefront load/store instruction covers whole contiguous rows.
// Semantics follow the reference kernel src/infiniop/ops/paged_caching/cuda/kernel.cuh:22-89
// (negative slot = padding, page = slot / block_size, row = slot % block_size, source heads packed).
#include "paged_caching_amd.h"
#include "../../../handle.h"
#include "../../../devices/amd/amd_streaming.h"
#include "../../../../utils/check.h"
#include <cstdint>
#include <hip/hip_runtime.h>

namespace op::paged_caching::amd {

namespace {

// Everything below is in units of the copy vector (`Unit`), not of elements.
struct ScatterArgs {
    void *k_cache;
    void *v_cache;
    const void *k;
    const void *v;
    const int64_t *slot_mapping;
    int64_t num_tokens;
    int64_t num_slots;        // num_blocks * block_size; slots at or beyond it are ignored
    int32_t num_kv_heads;
    int32_t block_size;
    int32_t block_shift;      // log2(block_size) when it is a power of two, else -1
    int32_t k_units_per_row;  // head_size * element_size / sizeof(Unit)
    int32_t v_units_per_row;
    int64_t k_src_token_stride, v_src_token_stride;
    int64_t k_block_stride, k_head_stride, k_slot_stride;
    int64_t v_block_stride, v_head_stride, v_slot_stride;
};

// The leading arguments repeat a.slot_mapping, a.num_tokens, a.k, a.v, the two source token strides,
// a.num_kv_heads and a.k_units_per_row: the file is compiled with -amdgpu-kernarg-preload-count=14, which has
// the dispatcher put the first 14 argument words into scalar registers before the wavefront starts, so the
// slot and the thread's first source units are requested at once, without waiting for the scalar load of
// the argument block. The source does not depend on the slot: it is requested before the slot is known
// (for padding tokens too, which is harmless), and only the stores wait for both. The call is a few
// microseconds of dependent round trips; these two changes remove two of them.
template <typename Unit>
__global__ void __launch_bounds__(256)
pagedCachingScatterKernel(const int64_t *early_slot_mapping, int64_t early_num_tokens, const void *early_k,
                          const void *early_v, int64_t early_k_src_token_stride, int64_t early_v_src_token_stride,
                          int32_t early_num_kv_heads, int32_t early_k_units_per_row, ScatterArgs a) {
    const int64_t token = static_cast<int64_t>(blockIdx.x) * blockDim.z + threadIdx.z;
    if (token >= early_num_tokens) {
        return;
    }
    const int64_t slot = early_slot_mapping[token];
    const Unit *k_src = static_cast<const Unit *>(early_k) + token * early_k_src_token_stride;
    const Unit *v_src = static_cast<const Unit *>(early_v) + token * early_v_src_token_stride;
    // this thread's first (with a box that covers the row and the heads: only) unit of K and of V
    const int head0 = threadIdx.y;
    const int c0 = threadIdx.x;
    const bool k_first = head0 < early_num_kv_heads && c0 < early_k_units_per_row;
    const bool v_first = head0 < early_num_kv_heads && c0 < a.v_units_per_row;
    Unit k0{}, v0{};
    if (k_first) {
        k0 = k_src[static_cast<int64_t>(head0) * early_k_units_per_row + c0];
    }
    if (v_first) {
        v0 = v_src[static_cast<int64_t>(head0) * a.v_units_per_row + c0];
    }
    // Negative = padding (kernel.cuh:61-63). Slots past the pool would be an out-of-bounds write
    // in the reference; here they are dropped.
    if (slot < 0 || slot >= a.num_slots) {
        return;
    }
    int64_t page, row;
    if (a.block_shift >= 0) {
        page = slot >> a.block_shift;
        row = slot & (a.block_size - 1);
    } else if (a.num_slots <= 0x7fffffff) {
        const uint32_t s = static_cast<uint32_t>(slot), bs = static_cast<uint32_t>(a.block_size);
        page = s / bs;
        row = s % bs;
    } else {
        page = slot / a.block_size;
        row = slot % a.block_size;
    }

    Unit *k_dst = static_cast<Unit *>(a.k_cache) + page * a.k_block_stride + row * a.k_slot_stride;
    Unit *v_dst = static_cast<Unit *>(a.v_cache) + page * a.v_block_stride + row * a.v_slot_stride;
    // streamed stores (the cache rows are not read again by this kernel; see amd_streaming.h)
    if (k_first) {
        device::amd::storeStreamed(k_dst + head0 * a.k_head_stride + c0, k0);
    }
    if (v_first) {
        device::amd::storeStreamed(v_dst + head0 * a.v_head_stride + c0, v0);
    }
    // whatever the box does not cover in one step
    for (int head = head0; head < a.num_kv_heads; head += blockDim.y) {
        const int c_begin = head == head0 ? c0 + static_cast<int>(blockDim.x) : c0;
        const Unit *ks = k_src + static_cast<int64_t>(head) * a.k_units_per_row;
        const Unit *vs = v_src + static_cast<int64_t>(head) * a.v_units_per_row;
        Unit *kd = k_dst + head * a.k_head_stride;
        Unit *vd = v_dst + head * a.v_head_stride;
        for (int c = c_begin; c < a.k_units_per_row; c += blockDim.x) {
            device::amd::storeStreamed(kd + c, ks[c]);
        }
        for (int c = c_begin; c < a.v_units_per_row; c += blockDim.x) {
            device::amd::storeStreamed(vd + c, vs[c]);
        }
    }
}

// Smallest power of two >= x, at most 2^30.
int ceilPow2(int x) {
    int p = 1;
    while (p < x && p < (1 << 30)) {
        p <<= 1;
    }
    return p;
}

// Largest power of two <= 16 that divides every byte quantity in the list.
size_t commonUnitBytes(std::initializer_list<uint64_t> byte_quantities) {
    uint64_t bits = 16;
    for (uint64_t q : byte_quantities) {
        bits |= q;
    }
    return static_cast<size_t>(bits & (~bits + 1)); // lowest set bit
}

} // namespace

struct Descriptor::Opaque {};

Descriptor::~Descriptor() { delete _opaque; }

infiniStatus_t Descriptor::create(infiniopHandle_t handle, Descriptor **desc_ptr,
                                  infiniopTensorDescriptor_t k_cache_desc, infiniopTensorDescriptor_t v_cache_desc,
                                  infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc,
                                  infiniopTensorDescriptor_t slot_mapping_desc) {
    auto info = PagedCachingInfo::create(k_cache_desc, v_cache_desc, k_desc, v_desc, slot_mapping_desc);
    CHECK_RESULT(info);
    // The scatter needs no scratch (reference: nvidia/paged_caching_nvidia.cu:47-49 reports 0 too).
    *desc_ptr = new Descriptor(new Opaque{}, info.take(), 0, handle->device, handle->device_id);
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t Descriptor::calculate(void *workspace, size_t workspace_size, void *k_cache, void *v_cache,
                                     const void *k, const void *v, const void *slot_mapping, void *stream_) const {
    (void)workspace;
    (void)workspace_size;
    const PagedCachingInfo &in = _info;
    if (in.num_tokens == 0 || in.num_kv_heads == 0 || (in.head_size == 0 && in.v_head_size == 0)) {
        return INFINI_STATUS_SUCCESS;
    }
    if (k_cache == nullptr || v_cache == nullptr || k == nullptr || v == nullptr || slot_mapping == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    // the kernel counts heads, row units and workgroups in 32 bits
    if (in.num_kv_heads > 0x7fffffff || in.head_size > 0x7fffffff || in.v_head_size > 0x7fffffff
        || in.block_size > 0x7fffffff || in.num_tokens > 0x7fffffff) {
        return INFINI_STATUS_BAD_TENSOR_SHAPE;
    }

    const uint64_t es = infiniSizeOf(in.dtype);
    auto bytes = [es](ptrdiff_t elements) { return static_cast<uint64_t>(elements) * es; };
    const size_t unit = commonUnitBytes({
        in.head_size * es, in.v_head_size * es,
        bytes(in.k_src_stride), bytes(in.v_src_stride),
        bytes(in.k_cache_block_stride), bytes(in.k_cache_head_stride), bytes(in.k_cache_slot_stride),
        bytes(in.v_cache_block_stride), bytes(in.v_cache_head_stride), bytes(in.v_cache_slot_stride),
        reinterpret_cast<uint64_t>(k_cache), reinterpret_cast<uint64_t>(v_cache),
        reinterpret_cast<uint64_t>(k), reinterpret_cast<uint64_t>(v)});
    if (unit < es) {
        return INFINI_STATUS_BAD_PARAM; // a base address that is not aligned to the element size
    }
    const int64_t per = static_cast<int64_t>(unit / es); // elements per copy unit
    auto units = [per](ptrdiff_t elements) { return static_cast<int64_t>(elements) / per; };

    ScatterArgs a{};
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.k = k;
    a.v = v;
    a.slot_mapping = static_cast<const int64_t *>(slot_mapping);
    a.num_tokens = static_cast<int64_t>(in.num_tokens);
    a.num_slots = static_cast<int64_t>(in.num_blocks) * static_cast<int64_t>(in.block_size);
    a.num_kv_heads = static_cast<int32_t>(in.num_kv_heads);
    a.block_size = static_cast<int32_t>(in.block_size);
    a.block_shift = -1;
    if (in.block_size > 0 && (in.block_size & (in.block_size - 1)) == 0) {
        a.block_shift = __builtin_ctzll(in.block_size);
    }
    a.k_units_per_row = static_cast<int32_t>(units(in.head_size));
    a.v_units_per_row = static_cast<int32_t>(units(in.v_head_size));
    a.k_src_token_stride = units(in.k_src_stride);
    a.v_src_token_stride = units(in.v_src_stride);
    a.k_block_stride = units(in.k_cache_block_stride);
    a.k_head_stride = units(in.k_cache_head_stride);
    a.k_slot_stride = units(in.k_cache_slot_stride);
    a.v_block_stride = units(in.v_cache_block_stride);
    a.v_head_stride = units(in.v_cache_head_stride);
    a.v_slot_stride = units(in.v_cache_slot_stride);

    // 256-thread box: x = units along a row, y = heads, z = tokens.
    const int row_units = a.k_units_per_row > a.v_units_per_row ? a.k_units_per_row : a.v_units_per_row;
    int bx = ceilPow2(row_units);
    bx = bx > 64 ? 64 : bx;
    int by = ceilPow2(a.num_kv_heads);
    by = by > 256 / bx ? 256 / bx : by;
    const int bz = 256 / (bx * by);
    const dim3 block(bx, by, bz);
    const dim3 grid(static_cast<unsigned>((in.num_tokens + bz - 1) / bz));
    auto stream = static_cast<hipStream_t>(stream_);

#define EARLY a.slot_mapping, a.num_tokens, a.k, a.v, a.k_src_token_stride, a.v_src_token_stride, a.num_kv_heads, a.k_units_per_row
    switch (unit) {
    case 16: pagedCachingScatterKernel<uint4><<<grid, block, 0, stream>>>(EARLY, a); break;
    case 8: pagedCachingScatterKernel<uint2><<<grid, block, 0, stream>>>(EARLY, a); break;
    case 4: pagedCachingScatterKernel<uint32_t><<<grid, block, 0, stream>>>(EARLY, a); break;
    case 2: pagedCachingScatterKernel<uint16_t><<<grid, block, 0, stream>>>(EARLY, a); break;
    default: return INFINI_STATUS_BAD_TENSOR_STRIDES;
    }
#undef EARLY
    return hipGetLastError() == hipSuccess ? INFINI_STATUS_SUCCESS : INFINI_STATUS_INTERNAL_ERROR;
}

} // namespace op::paged_caching::amd
