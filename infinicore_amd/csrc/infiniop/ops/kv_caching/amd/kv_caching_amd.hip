// kv_caching on AMD Instinct (gfx950): append the K and V vectors of the new tokens of every sequence
// to its contiguous cache, behind the positions already filled.
//
// A pure byte copy, written for memory transactions like the paged scatter next door: when every
// tensor's innermost stride is 1, a (sequence, head, token) row is moved in the widest power-of-two unit
// (up to 16 bytes) that divides the row length, every outer stride and every base address; adjacent lanes
// move adjacent units, so a wavefront instruction covers whole contiguous rows. Tensors with a strided
// innermost dimension take the same kernel with the element as unit and explicit element strides.
// Semantics follow the reference kernel src/infiniop/ops/kv_caching/cuda/kernel.cuh:32-58
// (position = past_kv_lengths[b] + s); positions outside [0, max_seq_len) are an out-of-bounds write
// there and are dropped here.
#include "kv_caching_amd.h"
#include "../../../handle.h"
#include "../../../devices/amd/amd_streaming.h"
#include "../../../../utils/check.h"
#include <cstdint>
#include <hip/hip_runtime.h>

namespace op::kv_caching::amd {

namespace {

// Strides are in units of the copy vector (`Unit`), not of elements.
struct AppendArgs {
    void *k_cache;
    void *v_cache;
    const void *k;
    const void *v;
    const void *past_kv_lengths;
    int32_t past_is_i64;
    int64_t rows;          // batch * heads * seq_len
    int32_t num_kv_heads;
    int32_t seq_len;
    int32_t max_seq_len;
    int32_t units_per_row;
    int64_t k_cache_strides[4], v_cache_strides[4], k_strides[4], v_strides[4];
};

template <typename Unit, bool PACKED_ROWS>
__global__ void __launch_bounds__(256) kvCachingAppendKernel(AppendArgs a) {
    const int64_t row = static_cast<int64_t>(blockIdx.x) * blockDim.y + threadIdx.y;
    if (row >= a.rows) {
        return;
    }
    int64_t b, h, s;
    if (a.rows <= 0x7fffffff) {
        const uint32_t r = static_cast<uint32_t>(row), n = static_cast<uint32_t>(a.seq_len);
        const uint32_t bh = r / n;
        s = r - bh * n;
        b = bh / static_cast<uint32_t>(a.num_kv_heads);
        h = bh - b * a.num_kv_heads;
    } else {
        const int64_t bh = row / a.seq_len;
        s = row - bh * a.seq_len;
        b = bh / a.num_kv_heads;
        h = bh - b * a.num_kv_heads;
    }
    const int64_t past = a.past_is_i64 ? static_cast<const int64_t *>(a.past_kv_lengths)[b]
                                       : static_cast<int64_t>(static_cast<const int32_t *>(a.past_kv_lengths)[b]);
    const int64_t pos = past + s;
    if (pos < 0 || pos >= a.max_seq_len) {
        return;
    }
    const Unit *ks = static_cast<const Unit *>(a.k) + b * a.k_strides[0] + h * a.k_strides[1] + s * a.k_strides[2];
    const Unit *vs = static_cast<const Unit *>(a.v) + b * a.v_strides[0] + h * a.v_strides[1] + s * a.v_strides[2];
    Unit *kd = static_cast<Unit *>(a.k_cache) + b * a.k_cache_strides[0] + h * a.k_cache_strides[1] + pos * a.k_cache_strides[2];
    Unit *vd = static_cast<Unit *>(a.v_cache) + b * a.v_cache_strides[0] + h * a.v_cache_strides[1] + pos * a.v_cache_strides[2];
    for (int c = threadIdx.x; c < a.units_per_row; c += blockDim.x) {
        if constexpr (PACKED_ROWS) {
            // streamed stores (the cache rows are not read again by this kernel; see amd_streaming.h)
            device::amd::storeStreamed(kd + c, ks[c]);
            device::amd::storeStreamed(vd + c, vs[c]);
        } else {
            device::amd::storeStreamed(kd + c * a.k_cache_strides[3], ks[c * a.k_strides[3]]);
            device::amd::storeStreamed(vd + c * a.v_cache_strides[3], vs[c * a.v_strides[3]]);
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

template <bool PACKED_ROWS>
infiniStatus_t launch(size_t unit, const AppendArgs &a, dim3 grid, dim3 block, hipStream_t stream) {
    switch (unit) {
    case 16: kvCachingAppendKernel<uint4, PACKED_ROWS><<<grid, block, 0, stream>>>(a); break;
    case 8: kvCachingAppendKernel<uint2, PACKED_ROWS><<<grid, block, 0, stream>>>(a); break;
    case 4: kvCachingAppendKernel<uint32_t, PACKED_ROWS><<<grid, block, 0, stream>>>(a); break;
    case 2: kvCachingAppendKernel<uint16_t, PACKED_ROWS><<<grid, block, 0, stream>>>(a); break;
    default: return INFINI_STATUS_BAD_TENSOR_STRIDES;
    }
    return hipGetLastError() == hipSuccess ? INFINI_STATUS_SUCCESS : INFINI_STATUS_INTERNAL_ERROR;
}

} // namespace

struct Descriptor::Opaque {};

Descriptor::~Descriptor() { delete _opaque; }

infiniStatus_t Descriptor::create(infiniopHandle_t handle, Descriptor **desc_ptr, infiniopTensorDescriptor_t k_cache,
                                  infiniopTensorDescriptor_t v_cache, infiniopTensorDescriptor_t k,
                                  infiniopTensorDescriptor_t v, infiniopTensorDescriptor_t past_kv_lengths) {
    auto info = KVCachingInfo::create(k_cache, v_cache, k, v, past_kv_lengths);
    CHECK_RESULT(info);
    // no scratch (the reference's nvidia backend reports 0 as well)
    *desc_ptr = new Descriptor(new Opaque{}, info.take(), 0, handle->device, handle->device_id);
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t Descriptor::calculate(void *workspace, size_t workspace_size, void *k_cache, void *v_cache,
                                     const void *k, const void *v, const void *past_kv_lengths, void *stream_) const {
    (void)workspace;
    (void)workspace_size;
    const KVCachingInfo &in = _info;
    if (in.batch_size == 0 || in.num_kv_heads == 0 || in.seq_len == 0 || in.hidden_dim == 0 || in.max_seq_len == 0) {
        return INFINI_STATUS_SUCCESS;
    }
    if (k_cache == nullptr || v_cache == nullptr || k == nullptr || v == nullptr || past_kv_lengths == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (in.num_kv_heads > 0x7fffffff || in.seq_len > 0x7fffffff || in.max_seq_len > 0x7fffffff
        || in.hidden_dim > 0x7fffffff) {
        return INFINI_STATUS_BAD_TENSOR_SHAPE;
    }

    const uint64_t es = infiniSizeOf(in.dtype);
    auto bytes = [es](ptrdiff_t elements) { return static_cast<uint64_t>(elements) * es; };
    const bool packed_rows = in.k_cache_strides[3] == 1 && in.v_cache_strides[3] == 1 && in.k_strides[3] == 1
                          && in.v_strides[3] == 1;
    size_t unit = es;
    if (packed_rows) {
        unit = commonUnitBytes({in.hidden_dim * es,
                                bytes(in.k_cache_strides[0]), bytes(in.k_cache_strides[1]), bytes(in.k_cache_strides[2]),
                                bytes(in.v_cache_strides[0]), bytes(in.v_cache_strides[1]), bytes(in.v_cache_strides[2]),
                                bytes(in.k_strides[0]), bytes(in.k_strides[1]), bytes(in.k_strides[2]),
                                bytes(in.v_strides[0]), bytes(in.v_strides[1]), bytes(in.v_strides[2]),
                                reinterpret_cast<uint64_t>(k_cache), reinterpret_cast<uint64_t>(v_cache),
                                reinterpret_cast<uint64_t>(k), reinterpret_cast<uint64_t>(v)});
    }
    const uint64_t bases = reinterpret_cast<uint64_t>(k_cache) | reinterpret_cast<uint64_t>(v_cache)
                         | reinterpret_cast<uint64_t>(k) | reinterpret_cast<uint64_t>(v);
    if (unit < es || (bases & (es - 1)) != 0) {
        return INFINI_STATUS_BAD_PARAM; // a base address that is not aligned to the element size
    }
    const int64_t per = static_cast<int64_t>(unit / es); // elements per copy unit
    auto units = [per](ptrdiff_t elements) { return static_cast<int64_t>(elements) / per; };

    AppendArgs a{};
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.k = k;
    a.v = v;
    a.past_kv_lengths = past_kv_lengths;
    a.past_is_i64 = in.past_len_dtype == INFINI_DTYPE_I64;
    a.rows = static_cast<int64_t>(in.batch_size) * static_cast<int64_t>(in.num_kv_heads) * static_cast<int64_t>(in.seq_len);
    a.num_kv_heads = static_cast<int32_t>(in.num_kv_heads);
    a.seq_len = static_cast<int32_t>(in.seq_len);
    a.max_seq_len = static_cast<int32_t>(in.max_seq_len);
    a.units_per_row = static_cast<int32_t>(units(in.hidden_dim));
    for (int i = 0; i < 3; ++i) {
        a.k_cache_strides[i] = units(in.k_cache_strides[i]);
        a.v_cache_strides[i] = units(in.v_cache_strides[i]);
        a.k_strides[i] = units(in.k_strides[i]);
        a.v_strides[i] = units(in.v_strides[i]);
    }
    a.k_cache_strides[3] = in.k_cache_strides[3];
    a.v_cache_strides[3] = in.v_cache_strides[3];
    a.k_strides[3] = in.k_strides[3];
    a.v_strides[3] = in.v_strides[3];

    // 256-thread box: x = units along a row, y = rows.
    int bx = ceilPow2(a.units_per_row);
    bx = bx > 64 ? 64 : bx;
    const int by = 256 / bx;
    const int64_t blocks = (a.rows + by - 1) / by;
    if (blocks > 0x7fffffff) {
        return INFINI_STATUS_BAD_TENSOR_SHAPE;
    }
    const dim3 block(bx, by);
    const dim3 grid(static_cast<unsigned>(blocks));
    auto stream = static_cast<hipStream_t>(stream_);
    return packed_rows ? launch<true>(unit, a, grid, block, stream) : launch<false>(unit, a, grid, block, stream);
}

} // namespace op::kv_caching::amd
