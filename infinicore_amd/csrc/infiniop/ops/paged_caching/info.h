// Create-time validation of the paged_caching operands and capture of every size and stride the
// scatter needs. Checks, their order and the status each one yields follow the reference's
// src/infiniop/ops/paged_caching/info.h:35-107, so the same bad input produces the same code.
#ifndef INFINICORE_AMD_PAGED_CACHING_INFO_H
#define INFINICORE_AMD_PAGED_CACHING_INFO_H

#include "../../../utils/check.h"
#include "../../../utils/result.h"
#include "../../tensor.h"
#include <cstdio>

namespace op::paged_caching {

struct PagedCachingInfo {
    infiniDtype_t dtype;

    size_t num_tokens;   // entries of slot_mapping
    size_t num_kv_heads;
    size_t head_size;    // elements of one key vector
    size_t v_head_size;  // elements of one value vector
    size_t block_size;   // token rows per page
    size_t num_blocks;   // pages in the pool (used only to ignore slots outside the pool)

    // element strides
    ptrdiff_t k_src_stride; // between tokens of k; heads and elements inside a token are packed
    ptrdiff_t v_src_stride;
    ptrdiff_t k_cache_block_stride;
    ptrdiff_t v_cache_block_stride;
    ptrdiff_t k_cache_head_stride;
    ptrdiff_t v_cache_head_stride;
    ptrdiff_t k_cache_slot_stride;
    ptrdiff_t v_cache_slot_stride;

    static utils::Result<PagedCachingInfo> create(infiniopTensorDescriptor_t k_cache_desc,
                                                  infiniopTensorDescriptor_t v_cache_desc,
                                                  infiniopTensorDescriptor_t k_desc,
                                                  infiniopTensorDescriptor_t v_desc,
                                                  infiniopTensorDescriptor_t slot_mapping_desc) {
        if (!k_cache_desc || !v_cache_desc || !k_desc || !v_desc || !slot_mapping_desc) {
            return INFINI_STATUS_NULL_POINTER;
        }

        // dtypes (info.h:42-50)
        const infiniDtype_t dtype = k_desc->dtype();
        CHECK_DTYPE(dtype, INFINI_DTYPE_F16, INFINI_DTYPE_BF16, INFINI_DTYPE_F32);
        if (v_desc->dtype() != dtype || k_cache_desc->dtype() != dtype || v_cache_desc->dtype() != dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }
        if (slot_mapping_desc->dtype() != INFINI_DTYPE_I64) {
            std::printf("slot_mapping must be int64_t.\n");
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }

        // ranks (info.h:52-54): caches may carry extra trailing dims in the reference's check
        // (ndim >= 4); only dims 0..3 are ever used.
        if (k_desc->ndim() != 3 || v_desc->ndim() != 3 || k_cache_desc->ndim() < 4 || v_cache_desc->ndim() < 4
            || slot_mapping_desc->ndim() != 1) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }

        // sizes and cross-checks (info.h:63-80)
        PagedCachingInfo info{};
        info.dtype = dtype;
        info.num_tokens = slot_mapping_desc->dim(0);
        info.num_kv_heads = k_desc->dim(1);
        info.head_size = k_desc->dim(2);
        info.v_head_size = v_desc->dim(2);
        info.block_size = k_cache_desc->dim(2);
        info.num_blocks = k_cache_desc->dim(0);

        if (k_desc->dim(0) != info.num_tokens || v_desc->dim(0) != info.num_tokens || v_desc->dim(1) != info.num_kv_heads) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (v_cache_desc->dim(0) != k_cache_desc->dim(0) || v_cache_desc->dim(1) != info.num_kv_heads
            || v_cache_desc->dim(2) != info.block_size) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (k_cache_desc->dim(1) != info.num_kv_heads || k_cache_desc->dim(3) != info.head_size
            || v_cache_desc->dim(3) != info.v_head_size) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }

        // strides (info.h:83-90)
        info.k_src_stride = k_desc->stride(0);
        info.v_src_stride = v_desc->stride(0);
        info.k_cache_block_stride = k_cache_desc->stride(0);
        info.v_cache_block_stride = v_cache_desc->stride(0);
        info.k_cache_head_stride = k_cache_desc->stride(1);
        info.v_cache_head_stride = v_cache_desc->stride(1);
        info.k_cache_slot_stride = k_cache_desc->stride(2);
        info.v_cache_slot_stride = v_cache_desc->stride(2);
        return info;
    }
};

} // namespace op::paged_caching

#endif
