// Create-time validation of the paged-attention operands and capture of every size and stride the
// decode needs. Checks, their order and the status each one yields follow the reference's
// src/infiniop/ops/paged_attention/info.h:41-194, so the same bad input produces the same code.
// Stricter than the reference in three places where the reference would read out of bounds or
// divide by zero: num_kv_heads == 0, block_tables with fewer rows than sequences, and an
// alibi_slopes vector shorter than num_heads are rejected with BAD_TENSOR_SHAPE.
#ifndef INFINICORE_AMD_PAGED_ATTENTION_INFO_H
#define INFINICORE_AMD_PAGED_ATTENTION_INFO_H

#include "../../../utils/check.h"
#include "../../../utils/result.h"
#include "../../tensor.h"

namespace op::paged_attention {

struct PagedAttentionInfo {
    infiniDtype_t dtype;       // F16 or BF16: q, out and both caches
    infiniDtype_t index_dtype; // I64, I32 or U32: block_tables and seq_lens
    float scale;
    bool has_alibi;

    size_t num_seqs;
    size_t num_heads;
    size_t num_kv_heads;
    size_t head_size;  // elements of a query / key vector
    size_t value_size; // elements of a value / output vector
    size_t page_block_size;
    size_t max_num_blocks_per_seq; // width of block_tables
    size_t num_blocks;             // pages in the pool

    // element strides
    ptrdiff_t q_stride, q_head_stride;
    ptrdiff_t k_batch_stride, k_row_stride, k_head_stride;
    ptrdiff_t v_batch_stride, v_row_stride, v_head_stride;
    ptrdiff_t o_stride, o_head_stride;
    ptrdiff_t block_table_batch_stride;
    ptrdiff_t cache_lens_stride;

    static bool isIndexDtype(infiniDtype_t dt) {
        return dt == INFINI_DTYPE_I64 || dt == INFINI_DTYPE_I32 || dt == INFINI_DTYPE_U32;
    }

    static utils::Result<PagedAttentionInfo> create(infiniopTensorDescriptor_t out_desc,
                                                    infiniopTensorDescriptor_t q_desc,
                                                    infiniopTensorDescriptor_t k_cache_desc,
                                                    infiniopTensorDescriptor_t v_cache_desc,
                                                    infiniopTensorDescriptor_t block_tables_desc,
                                                    infiniopTensorDescriptor_t cache_lens_desc,
                                                    infiniopTensorDescriptor_t alibi_slopes_desc, // may be null
                                                    float scale) {
        if (!out_desc || !q_desc || !k_cache_desc || !v_cache_desc || !block_tables_desc || !cache_lens_desc) {
            return INFINI_STATUS_NULL_POINTER;
        }

        // data dtypes (info.h:51-55)
        const infiniDtype_t dtype = q_desc->dtype();
        CHECK_DTYPE(dtype, INFINI_DTYPE_F16, INFINI_DTYPE_BF16);
        if (out_desc->dtype() != dtype || k_cache_desc->dtype() != dtype || v_cache_desc->dtype() != dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }

        // ranks (info.h:57-65)
        if (q_desc->ndim() != 3 || out_desc->ndim() != 3) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (k_cache_desc->ndim() != 4 || v_cache_desc->ndim() != 4) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (block_tables_desc->ndim() != 2 || cache_lens_desc->ndim() != 1) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }

        // innermost dimension packed (info.h:67-70)
        CHECK_OR_RETURN(q_desc->stride(2) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(out_desc->stride(2) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(k_cache_desc->stride(3) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(v_cache_desc->stride(3) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);

        // index dtypes: one of three, and the same for both tensors (info.h:72-93)
        const infiniDtype_t index_dtype = block_tables_desc->dtype();
        if (!isIndexDtype(index_dtype) || !isIndexDtype(cache_lens_desc->dtype())) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }
        if (cache_lens_desc->dtype() != index_dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }

        CHECK_OR_RETURN(block_tables_desc->stride(1) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(cache_lens_desc->stride(0) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);

        // optional ALiBi slopes (info.h:98-106)
        if (alibi_slopes_desc != nullptr) {
            if (alibi_slopes_desc->dtype() != INFINI_DTYPE_F32) {
                return INFINI_STATUS_BAD_TENSOR_DTYPE;
            }
            if (alibi_slopes_desc->ndim() != 1) {
                return INFINI_STATUS_BAD_TENSOR_SHAPE;
            }
            CHECK_OR_RETURN(alibi_slopes_desc->stride(0) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        }

        // sizes (info.h:108-151)
        PagedAttentionInfo info{};
        info.dtype = dtype;
        info.index_dtype = index_dtype;
        info.scale = scale;
        info.has_alibi = alibi_slopes_desc != nullptr;
        info.num_seqs = q_desc->dim(0);
        info.num_heads = q_desc->dim(1);
        info.head_size = q_desc->dim(2);
        info.value_size = v_cache_desc->dim(3);
        info.num_blocks = k_cache_desc->dim(0);
        info.num_kv_heads = k_cache_desc->dim(1);
        info.page_block_size = k_cache_desc->dim(2);
        info.max_num_blocks_per_seq = block_tables_desc->dim(1);
        const bool is_mla = info.head_size == 576 && info.value_size == 512;

        const size_t hs = info.head_size;
        if (hs != 64 && hs != 128 && hs != 192 && hs != 256 && hs != 576) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (info.num_kv_heads == 0 || info.num_heads % info.num_kv_heads != 0) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (k_cache_desc->dim(3) != hs) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (v_cache_desc->dim(0) != k_cache_desc->dim(0) || v_cache_desc->dim(1) != k_cache_desc->dim(1)
            || v_cache_desc->dim(2) != k_cache_desc->dim(2)) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (!is_mla && info.value_size != hs) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (out_desc->dim(0) != info.num_seqs || out_desc->dim(1) != info.num_heads || out_desc->dim(2) != info.value_size) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (cache_lens_desc->dim(0) != info.num_seqs) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        // stricter than the reference (see the note at the top of this file)
        if (block_tables_desc->dim(0) < info.num_seqs) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (alibi_slopes_desc != nullptr && alibi_slopes_desc->dim(0) < info.num_heads) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }

        // strides (info.h:155-169); the reference assumes q/out heads are packed and does not read
        // q stride(1) - here both head strides are captured and honoured.
        info.q_stride = q_desc->stride(0);
        info.q_head_stride = q_desc->stride(1);
        info.o_stride = out_desc->stride(0);
        info.o_head_stride = out_desc->stride(1);
        info.k_batch_stride = k_cache_desc->stride(0);
        info.k_head_stride = k_cache_desc->stride(1);
        info.k_row_stride = k_cache_desc->stride(2);
        info.v_batch_stride = v_cache_desc->stride(0);
        info.v_head_stride = v_cache_desc->stride(1);
        info.v_row_stride = v_cache_desc->stride(2);
        info.block_table_batch_stride = block_tables_desc->stride(0);
        info.cache_lens_stride = cache_lens_desc->stride(0);
        return info;
    }
};

} // namespace op::paged_attention

#endif
