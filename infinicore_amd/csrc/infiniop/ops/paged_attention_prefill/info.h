// Create-time validation of the paged-attention prefill operands and capture of every size and
// stride the kernels need. Checks, their order and the status each one yields follow the
// reference's src/infiniop/ops/paged_attention_prefill/info.h:43-210. Stricter where the reference
// would read out of bounds, divide by zero or reinterpret memory: num_kv_heads == 0, block_tables
// with fewer rows than sequences, an alibi_slopes vector shorter than num_heads (BAD_TENSOR_SHAPE);
// seq_lens / cum_seq_lens_q of a different index dtype than block_tables (BAD_TENSOR_DTYPE; the
// reference reads all three through the block table's type); non-contiguous seq_lens or
// cum_seq_lens_q (BAD_TENSOR_STRIDES; the reference ignores their strides).
#ifndef INFINICORE_AMD_PAGED_ATTENTION_PREFILL_INFO_H
#define INFINICORE_AMD_PAGED_ATTENTION_PREFILL_INFO_H

#include "../../../utils/check.h"
#include "../../../utils/result.h"
#include "../../tensor.h"

namespace op::paged_attention_prefill {

struct PagedAttentionPrefillInfo {
    infiniDtype_t dtype;       // F16 or BF16: q, out and both caches
    infiniDtype_t index_dtype; // I64, I32 or U32: block_tables, seq_lens and cum_seq_lens_q
    float scale;
    bool has_alibi;

    size_t num_seqs;
    size_t total_q_tokens;
    size_t num_heads;
    size_t num_kv_heads;
    size_t head_size;
    size_t value_size;
    size_t page_block_size;
    size_t max_num_blocks_per_seq;
    size_t num_blocks;

    // element strides
    ptrdiff_t q_stride, q_head_stride;
    ptrdiff_t k_batch_stride, k_row_stride, k_head_stride;
    ptrdiff_t v_batch_stride, v_row_stride, v_head_stride;
    ptrdiff_t o_stride, o_head_stride;
    ptrdiff_t block_table_batch_stride;

    static bool isIndexDtype(infiniDtype_t dt) {
        return dt == INFINI_DTYPE_I64 || dt == INFINI_DTYPE_I32 || dt == INFINI_DTYPE_U32;
    }

    static utils::Result<PagedAttentionPrefillInfo> create(infiniopTensorDescriptor_t out_desc,
                                                           infiniopTensorDescriptor_t q_desc,
                                                           infiniopTensorDescriptor_t k_cache_desc,
                                                           infiniopTensorDescriptor_t v_cache_desc,
                                                           infiniopTensorDescriptor_t block_tables_desc,
                                                           infiniopTensorDescriptor_t total_kv_lens_desc,
                                                           infiniopTensorDescriptor_t cum_seqlens_q_desc,
                                                           infiniopTensorDescriptor_t alibi_slopes_desc, // may be null
                                                           float scale) {
        if (!out_desc || !q_desc || !k_cache_desc || !v_cache_desc || !block_tables_desc || !total_kv_lens_desc
            || !cum_seqlens_q_desc) {
            return INFINI_STATUS_NULL_POINTER;
        }

        // data dtypes (info.h:55-59)
        const infiniDtype_t dtype = q_desc->dtype();
        CHECK_DTYPE(dtype, INFINI_DTYPE_F16, INFINI_DTYPE_BF16);
        if (out_desc->dtype() != dtype || k_cache_desc->dtype() != dtype || v_cache_desc->dtype() != dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }

        // ranks (info.h:61-71)
        if (q_desc->ndim() != 3 || out_desc->ndim() != 3) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (k_cache_desc->ndim() != 4 || v_cache_desc->ndim() != 4) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (block_tables_desc->ndim() != 2 || total_kv_lens_desc->ndim() != 1 || cum_seqlens_q_desc->ndim() != 1) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }

        // innermost dimension packed (info.h:73-76)
        CHECK_OR_RETURN(q_desc->stride(2) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(out_desc->stride(2) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(k_cache_desc->stride(3) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(v_cache_desc->stride(3) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);

        // index dtypes (info.h:78-93), and all three the same
        const infiniDtype_t index_dtype = block_tables_desc->dtype();
        if (!isIndexDtype(index_dtype) || !isIndexDtype(total_kv_lens_desc->dtype())
            || !isIndexDtype(cum_seqlens_q_desc->dtype())) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }
        if (total_kv_lens_desc->dtype() != index_dtype || cum_seqlens_q_desc->dtype() != index_dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }

        CHECK_OR_RETURN(block_tables_desc->stride(1) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(total_kv_lens_desc->stride(0) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        CHECK_OR_RETURN(cum_seqlens_q_desc->stride(0) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);

        // optional ALiBi slopes (info.h:97-105)
        if (alibi_slopes_desc != nullptr) {
            if (alibi_slopes_desc->dtype() != INFINI_DTYPE_F32) {
                return INFINI_STATUS_BAD_TENSOR_DTYPE;
            }
            if (alibi_slopes_desc->ndim() != 1) {
                return INFINI_STATUS_BAD_TENSOR_SHAPE;
            }
            CHECK_OR_RETURN(alibi_slopes_desc->stride(0) == 1, INFINI_STATUS_BAD_TENSOR_STRIDES);
        }

        // sizes (info.h:107-150)
        PagedAttentionPrefillInfo info{};
        info.dtype = dtype;
        info.index_dtype = index_dtype;
        info.scale = scale;
        info.has_alibi = alibi_slopes_desc != nullptr;
        info.total_q_tokens = q_desc->dim(0);
        info.num_heads = q_desc->dim(1);
        info.head_size = q_desc->dim(2);
        info.value_size = v_cache_desc->dim(3);
        info.num_blocks = k_cache_desc->dim(0);
        info.num_kv_heads = k_cache_desc->dim(1);
        info.page_block_size = k_cache_desc->dim(2);
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
        if (v_cache_desc->dim(0) != info.num_blocks || v_cache_desc->dim(1) != info.num_kv_heads
            || v_cache_desc->dim(2) != info.page_block_size) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (!is_mla && info.value_size != hs) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (out_desc->dim(0) != q_desc->dim(0) || out_desc->dim(1) != q_desc->dim(1) || out_desc->dim(2) != info.value_size) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        info.num_seqs = total_kv_lens_desc->dim(0);
        if (cum_seqlens_q_desc->dim(0) != info.num_seqs + 1) {
            return INFINI_STATUS_BAD_PARAM;
        }
        info.max_num_blocks_per_seq = block_tables_desc->dim(1);
        // stricter than the reference (see the note at the top of this file)
        if (block_tables_desc->dim(0) < info.num_seqs) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (alibi_slopes_desc != nullptr && alibi_slopes_desc->dim(0) < info.num_heads) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }

        // strides (info.h:152-166)
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
        return info;
    }
};

} // namespace op::paged_attention_prefill

#endif
