// paged_attention_prefill on AMD Instinct MI355X: descriptor, kernel choice and launches.
// Takes the place of the reference's nvidia backend host code
// (src/infiniop/ops/paged_attention_prefill/nvidia/paged_attention_prefill_nvidia.cu:1572-1886)
// for the AMD device.
#include "paged_attention_prefill_amd.h"
#include "../../../handle.h"
#include "../../../../utils/check.h"
#include "../../../devices/amd/amd_device.h"
#include "prefill_common.h"
#include "prefill_generic.h"
#include "prefill_tiled.h"
#include <cstdlib>
#include <cstring>

namespace op::paged_attention_prefill::amd {

namespace {

using op::paged_attention::amd::BFloat16;
using op::paged_attention::amd::Half;
using op::paged_attention::amd::IndexI32;
using op::paged_attention::amd::IndexI64;
using op::paged_attention::amd::IndexU32;

// Decided once, at descriptor creation, from shapes and the device alone (sequence lengths live in
// device memory and are never read on the host).
struct Plan {
    bool tiled;          // matrix-core kernel (head 64 / 128 / 192 / 256 or keys 576 with values 512 / 576, power-of-two pages >= 8, 16-byte aligned strides)
    int groups_per_wave; // tiled: R = 1 or 2 column groups per wavefront -> 64 R rows per workgroup
    int dims_per_lane;   // element-wise kernel: ceil(max(head_size, value_size) / 64)
};

bool multipleOf8(ptrdiff_t x) { return (x % 8) == 0; }

Plan makePlan(const PagedAttentionPrefillInfo &in, const device::amd::DeviceInfo &dev) {
    Plan plan{};
    const long long bs = static_cast<long long>(in.page_block_size);
    const bool pow2_page = bs >= 8 && (bs & (bs - 1)) == 0;
    const long long group = static_cast<long long>(in.num_heads / in.num_kv_heads);
    const long long rows = static_cast<long long>(in.total_q_tokens) * group; // per KV head
    const bool equal_sizes = in.value_size == in.head_size
                          && (in.head_size == 64 || in.head_size == 128 || in.head_size == 192 || in.head_size == 256);
    // keys 576 with values 512 (latent attention) or 576 (a shape of the reference's decode tests,
    // test/infiniop/paged_attention.py:106, taken here as well so that prompt and decode run the same class of kernel)
    const bool latent = in.head_size == 576 && (in.value_size == 512 || in.value_size == 576);
    plan.tiled = (equal_sizes || latent) && pow2_page
              && multipleOf8(in.q_stride) && multipleOf8(in.q_head_stride) && multipleOf8(in.o_stride)
              && multipleOf8(in.o_head_stride) && multipleOf8(in.k_batch_stride) && multipleOf8(in.k_head_stride)
              && multipleOf8(in.k_row_stride) && multipleOf8(in.v_batch_stride) && multipleOf8(in.v_head_stride)
              && multipleOf8(in.v_row_stride) && in.num_blocks > 0 && in.num_blocks <= 0x7fffffff
              && rows < (1LL << 30) && (rows / 64 + static_cast<long long>(in.num_seqs)) * static_cast<long long>(in.num_kv_heads) < (1LL << 31)
              // lane offsets inside a tile (15 rows + one row of bytes) are kept in 32 bits
              && in.k_row_stride > 0 && in.k_row_stride < (1 << 26) && in.v_row_stride > 0 && in.v_row_stride < (1 << 26)
              && static_cast<long long>(in.max_num_blocks_per_seq) * bs < (1LL << 30);
    if (const char *env = std::getenv("INFINIOP_AMD_PREFILL_KERNEL")) {
        if (std::strcmp(env, "generic") == 0) {
            plan.tiled = false;
        }
    }
    // Rows per workgroup: 128 (two column groups per wavefront: every K / V operand read from LDS then feeds two
    // matrix instructions) unless the average sequence fills no more than 64, or the batch is too small to give
    // every compute unit as many workgroups of 128 as it holds at a time: two up to head 128, one above (there the
    // accumulators of 128 rows need more than half the register file).
    const long long seqs = in.num_seqs > 0 ? static_cast<long long>(in.num_seqs) : 1;
    const long long rows_per_seq = rows / seqs;
    const long long resident = in.head_size <= 128 ? 2 : 1;
    int r = 2;
    if (rows_per_seq <= 64 || rows / 128 * static_cast<long long>(in.num_kv_heads) < resident * dev.compute_units) {
        r = 1;
    }
    if (const char *env = std::getenv("INFINIOP_AMD_PREFILL_GROUPS")) {
        const int forced = std::atoi(env);
        if (forced == 1 || forced == 2) {
            r = forced;
        }
    }
    if (latent) {
        // the accumulators of 64 rows x 512 (576) columns are half the register file: there is no kernel with two
        // groups, whatever the knob says (grid and kernel must agree on the rows per workgroup)
        r = 1;
    }
    plan.groups_per_wave = r;
    const size_t widest = in.head_size > in.value_size ? in.head_size : in.value_size;
    plan.dims_per_lane = static_cast<int>((widest + 63) / 64);
    return plan;
}

template <typename T, typename Tindex>
void launchGeneric(const PrefillArgs &a, const Plan &plan, hipStream_t stream) {
    const dim3 grid(a.total_q_tokens, a.num_heads);
    switch (plan.dims_per_lane) {
    case 1: prefillGenericKernel<T, Tindex, 1><<<grid, 64, 0, stream>>>(a); break;
    case 2: prefillGenericKernel<T, Tindex, 2><<<grid, 64, 0, stream>>>(a); break;
    case 3: prefillGenericKernel<T, Tindex, 3><<<grid, 64, 0, stream>>>(a); break;
    case 4: prefillGenericKernel<T, Tindex, 4><<<grid, 64, 0, stream>>>(a); break;
    default: prefillGenericKernel<T, Tindex, 9><<<grid, 64, 0, stream>>>(a); break;
    }
}

template <typename T, typename Tindex, int KHEAD, int VHEAD, bool PLAIN>
void launchTiledHead(const PrefillArgs &a, const Plan &plan, hipStream_t stream) {
    // sum over sequences of ceil(rows / block_rows) is at most floor(total rows / block_rows) + num_seqs
    const long long rows = static_cast<long long>(a.total_q_tokens) * a.group;
    const int groups = plan.groups_per_wave;
    const int block_rows = prefillBlockRows(groups);
    const dim3 grid(static_cast<unsigned>((rows / block_rows + a.num_seqs) * a.num_kv_heads));
    if constexpr (KHEAD == VHEAD && KHEAD <= 256) {
        if (groups == 2) {
            prefillTiledKernel<T, Tindex, KHEAD, VHEAD, 2, PLAIN><<<grid, kPrefillThreads, 0, stream>>>(a);
            return;
        }
    }
    prefillTiledKernel<T, Tindex, KHEAD, VHEAD, 1, PLAIN><<<grid, kPrefillThreads, 0, stream>>>(a);
}

template <typename T, typename Tindex, bool PLAIN>
void launchTiledPlain(const PrefillArgs &a, const Plan &plan, hipStream_t stream) {
    switch (a.head_size) {
    case 64: launchTiledHead<T, Tindex, 64, 64, PLAIN>(a, plan, stream); break;
    case 128: launchTiledHead<T, Tindex, 128, 128, PLAIN>(a, plan, stream); break;
    case 192: launchTiledHead<T, Tindex, 192, 192, PLAIN>(a, plan, stream); break;
    case 256: launchTiledHead<T, Tindex, 256, 256, PLAIN>(a, plan, stream); break;
    default:
        if (a.value_size == 576) {
            launchTiledHead<T, Tindex, 576, 576, PLAIN>(a, plan, stream);
        } else {
            launchTiledHead<T, Tindex, 576, 512, PLAIN>(a, plan, stream);
        }
        break;
    }
}

template <typename T, typename Tindex>
void launchTiled(const PrefillArgs &a, const Plan &plan, hipStream_t stream) {
    if (a.alibi_slopes == nullptr && a.scale_log2 > 0.0f) {
        launchTiledPlain<T, Tindex, true>(a, plan, stream);
    } else {
        launchTiledPlain<T, Tindex, false>(a, plan, stream);
    }
}

template <typename T>
infiniStatus_t launchByIndex(infiniDtype_t index_dtype, const PrefillArgs &a, const Plan &plan, bool tiled,
                             hipStream_t stream) {
    switch (index_dtype) {
    case INFINI_DTYPE_I64:
        tiled ? launchTiled<T, IndexI64>(a, plan, stream) : launchGeneric<typename T::Base, IndexI64>(a, plan, stream);
        break;
    case INFINI_DTYPE_I32:
        tiled ? launchTiled<T, IndexI32>(a, plan, stream) : launchGeneric<typename T::Base, IndexI32>(a, plan, stream);
        break;
    case INFINI_DTYPE_U32:
        tiled ? launchTiled<T, IndexU32>(a, plan, stream) : launchGeneric<typename T::Base, IndexU32>(a, plan, stream);
        break;
    default: return INFINI_STATUS_BAD_TENSOR_DTYPE;
    }
    return INFINI_STATUS_SUCCESS;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

} // namespace

struct Descriptor::Opaque {
    Plan plan;
};

Descriptor::~Descriptor() { delete _opaque; }

infiniStatus_t Descriptor::create(infiniopHandle_t handle, Descriptor **desc_ptr, infiniopTensorDescriptor_t out_desc,
                                  infiniopTensorDescriptor_t q_desc, infiniopTensorDescriptor_t k_cache_desc,
                                  infiniopTensorDescriptor_t v_cache_desc, infiniopTensorDescriptor_t block_tables_desc,
                                  infiniopTensorDescriptor_t seq_lens_desc, infiniopTensorDescriptor_t cum_seq_lens_q_desc,
                                  infiniopTensorDescriptor_t alibi_slopes_desc, float scale) {
    auto info = PagedAttentionPrefillInfo::create(out_desc, q_desc, k_cache_desc, v_cache_desc, block_tables_desc,
                                                  seq_lens_desc, cum_seq_lens_q_desc, alibi_slopes_desc, scale);
    CHECK_RESULT(info);
    const PagedAttentionPrefillInfo in = info.take();
    const Plan plan = makePlan(in, device::amd::deviceInfo(handle->device_id));
    // every row block keeps its softmax state in registers from the first to the last K/V token: no scratch
    *desc_ptr = new Descriptor(new Opaque{plan}, in, 0, handle->device, handle->device_id);
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t Descriptor::calculate(void *workspace, size_t workspace_size, void *out, const void *q,
                                     const void *k_cache, const void *v_cache, const void *block_tables,
                                     const void *seq_lens, const void *cum_seq_lens_q, const void *alibi_slopes,
                                     void *stream_) const {
    (void)workspace;
    const PagedAttentionPrefillInfo &in = _info;
    const Plan &plan = _opaque->plan;
    if (workspace_size < _workspace_size) {
        return INFINI_STATUS_INSUFFICIENT_WORKSPACE;
    }
    if (in.num_seqs == 0 || in.num_heads == 0 || in.total_q_tokens == 0) {
        return INFINI_STATUS_SUCCESS;
    }
    if (out == nullptr || q == nullptr || k_cache == nullptr || v_cache == nullptr || block_tables == nullptr
        || seq_lens == nullptr || cum_seq_lens_q == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (in.has_alibi && alibi_slopes == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (in.max_num_blocks_per_seq == 0 || in.num_blocks == 0 || in.page_block_size == 0) {
        return INFINI_STATUS_SUCCESS; // no sequence can hold a token
    }
    if (in.total_q_tokens > 0x7fffffff || in.num_seqs > 0x7fffffff || in.num_heads > 65535) {
        return INFINI_STATUS_BAD_TENSOR_SHAPE;
    }

    PrefillArgs a{};
    a.out = out;
    a.q = q;
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.block_tables = block_tables;
    a.kv_lens = seq_lens;
    a.cu_seqlens_q = cum_seq_lens_q;
    a.alibi_slopes = static_cast<const float *>(alibi_slopes);
    a.scale_log2 = in.scale * kLog2e;
    a.num_seqs = static_cast<int32_t>(in.num_seqs);
    a.total_q_tokens = static_cast<int32_t>(in.total_q_tokens);
    a.num_heads = static_cast<int32_t>(in.num_heads);
    a.num_kv_heads = static_cast<int32_t>(in.num_kv_heads);
    a.group = static_cast<int32_t>(in.num_heads / in.num_kv_heads);
    a.head_size = static_cast<int32_t>(in.head_size);
    a.value_size = static_cast<int32_t>(in.value_size);
    a.block_size = static_cast<int32_t>(in.page_block_size);
    a.block_shift = -1;
    if ((in.page_block_size & (in.page_block_size - 1)) == 0) {
        a.block_shift = __builtin_ctzll(in.page_block_size);
    }
    a.num_blocks = static_cast<int32_t>(in.num_blocks > 0x7fffffff ? 0x7fffffff : in.num_blocks);
    a.max_blocks_per_seq = static_cast<int32_t>(in.max_num_blocks_per_seq > 0x7fffffff ? 0x7fffffff : in.max_num_blocks_per_seq);
    a.q_stride = in.q_stride;
    a.q_head_stride = in.q_head_stride;
    a.o_stride = in.o_stride;
    a.o_head_stride = in.o_head_stride;
    a.k_batch_stride = in.k_batch_stride;
    a.k_head_stride = in.k_head_stride;
    a.k_row_stride = in.k_row_stride;
    a.v_batch_stride = in.v_batch_stride;
    a.v_head_stride = in.v_head_stride;
    a.v_row_stride = in.v_row_stride;
    a.block_table_batch_stride = in.block_table_batch_stride;

    // The tiled kernel moves 16 bytes per lane; base addresses that are not 16-byte aligned take
    // the element-wise kernel instead.
    const bool tiled = plan.tiled && aligned16(out) && aligned16(q) && aligned16(k_cache) && aligned16(v_cache);
    auto stream = static_cast<hipStream_t>(stream_);

    infiniStatus_t status;
    if (in.dtype == INFINI_DTYPE_F16) {
        status = launchByIndex<TileF16>(in.index_dtype, a, plan, tiled, stream);
    } else {
        status = launchByIndex<TileBF16>(in.index_dtype, a, plan, tiled, stream);
    }
    if (status != INFINI_STATUS_SUCCESS) {
        return status;
    }
    return hipGetLastError() == hipSuccess ? INFINI_STATUS_SUCCESS : INFINI_STATUS_INTERNAL_ERROR;
}

} // namespace op::paged_attention_prefill::amd
