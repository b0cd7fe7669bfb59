// Create-time validation of the fused rotary-embedding + paged_caching operands. The scatter side runs the
// checks of paged_caching (PagedCachingInfo: reference src/infiniop/ops/paged_caching/info.h:35-107), the
// rotation side those of the reference's RoPE for a [tokens, heads, head_size] tensor with one position per
// token (src/infiniop/ops/rope/rope.h:72-160), so a bad operand yields the code it would yield there.
#ifndef INFINICORE_AMD_ROPE_PAGED_CACHING_INFO_H
#define INFINICORE_AMD_ROPE_PAGED_CACHING_INFO_H

#include "../paged_caching/info.h"
#include "infiniop/ops/rope_paged_caching.h"

namespace op::rope_paged_caching {

struct RoPEPagedCachingInfo {
    op::paged_caching::PagedCachingInfo scatter;
    infiniDtype_t pos_dtype; // any integer dtype
    size_t table_len;        // rows of the sin / cos tables
    size_t table_dim;        // head_size / 2
    infiniopRoPEAlgo_t algo;
    // query rotated in the same launch (infiniopCreateRoPEQKPagedCachingDescriptor); else has_query is false
    bool has_query;
    size_t num_q_heads;
    ptrdiff_t q_token_stride, q_head_stride, q_out_token_stride, q_out_head_stride;

    static bool isInteger(infiniDtype_t dt) {
        switch (dt) {
        case INFINI_DTYPE_I8: case INFINI_DTYPE_I16: case INFINI_DTYPE_I32: case INFINI_DTYPE_I64:
        case INFINI_DTYPE_U8: case INFINI_DTYPE_U16: case INFINI_DTYPE_U32: case INFINI_DTYPE_U64:
            return true;
        default:
            return false;
        }
    }

    static utils::Result<RoPEPagedCachingInfo> create(infiniopTensorDescriptor_t k_cache_desc,
                                                      infiniopTensorDescriptor_t v_cache_desc,
                                                      infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc,
                                                      infiniopTensorDescriptor_t slot_mapping_desc,
                                                      infiniopTensorDescriptor_t pos_desc,
                                                      infiniopTensorDescriptor_t sin_desc,
                                                      infiniopTensorDescriptor_t cos_desc, infiniopRoPEAlgo_t algo,
                                                      bool with_query = false,
                                                      infiniopTensorDescriptor_t q_out_desc = nullptr,
                                                      infiniopTensorDescriptor_t q_desc = nullptr) {
        // rope.h:79-82
        if (!pos_desc || !sin_desc || !cos_desc || static_cast<int>(algo) < 0 || algo >= INFINIOP_ROPE_ALGO_COUNT) {
            return INFINI_STATUS_NULL_POINTER;
        }
        auto scatter = op::paged_caching::PagedCachingInfo::create(k_cache_desc, v_cache_desc, k_desc, v_desc, slot_mapping_desc);
        CHECK_RESULT(scatter);
        RoPEPagedCachingInfo info{};
        info.scatter = scatter.take();
        info.algo = algo;
        // dtypes (rope.h:84-89); F64, which the reference's RoPE takes, is not a paged_caching dtype
        if (sin_desc->dtype() != info.scatter.dtype || cos_desc->dtype() != info.scatter.dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }
        info.pos_dtype = pos_desc->dtype();
        if (!isInteger(info.pos_dtype)) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }
        // shapes (rope.h:99-146): one position per token, tables [table_len, head_size / 2]
        if (pos_desc->ndim() != 1 || sin_desc->ndim() != 2 || cos_desc->ndim() != 2) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        if (pos_desc->dim(0) != info.scatter.num_tokens) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        info.table_len = sin_desc->dim(0);
        info.table_dim = sin_desc->dim(1);
        if (cos_desc->dim(0) != info.table_len || cos_desc->dim(1) != info.table_dim
            || info.scatter.head_size != 2 * info.table_dim) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        // strides (rope.h:148-160): last dimension of k contiguous, tables fully contiguous; positions too
        if (k_desc->stride(2) != 1 || v_desc->stride(2) != 1 || pos_desc->stride(0) != 1) {
            return INFINI_STATUS_BAD_TENSOR_STRIDES;
        }
        if (!sin_desc->isContiguous() || !cos_desc->isContiguous()) {
            return INFINI_STATUS_BAD_TENSOR_STRIDES;
        }
        // The kernel finds head h of a token at h * head_size (as the scatter it is built on does,
        // paged_caching/cuda/kernel.cuh:70-78); the reference's RoPE would honour any head stride
        // (rope/cuda/kernel.cuh:29-31), so heads that are padded or interleaved inside a token are refused
        // here rather than read from the wrong place.
        if (info.scatter.num_kv_heads > 1
            && (k_desc->stride(1) != static_cast<ptrdiff_t>(info.scatter.head_size)
                || v_desc->stride(1) != static_cast<ptrdiff_t>(info.scatter.v_head_size))) {
            return INFINI_STATUS_BAD_TENSOR_STRIDES;
        }
        info.has_query = with_query;
        if (with_query) {
            // the checks of the reference's RoPE for its x / y pair (rope.h:79-160): both given, dtype of the
            // tables, [tokens, heads, head_size] with the tokens and head size of k, packed last dimension
            if (!q_out_desc || !q_desc) {
                return INFINI_STATUS_NULL_POINTER;
            }
            if (q_desc->dtype() != info.scatter.dtype || q_out_desc->dtype() != info.scatter.dtype) {
                return INFINI_STATUS_BAD_TENSOR_DTYPE;
            }
            if (q_desc->ndim() != 3 || q_out_desc->ndim() != 3 || q_desc->dim(0) != info.scatter.num_tokens
                || q_desc->dim(2) != info.scatter.head_size || q_out_desc->dim(0) != q_desc->dim(0)
                || q_out_desc->dim(1) != q_desc->dim(1) || q_out_desc->dim(2) != q_desc->dim(2)) {
                return INFINI_STATUS_BAD_TENSOR_SHAPE;
            }
            if (q_desc->stride(2) != 1 || q_out_desc->stride(2) != 1) {
                return INFINI_STATUS_BAD_TENSOR_STRIDES;
            }
            info.num_q_heads = q_desc->dim(1);
            info.q_token_stride = q_desc->stride(0);
            info.q_head_stride = q_desc->stride(1);
            info.q_out_token_stride = q_out_desc->stride(0);
            info.q_out_head_stride = q_out_desc->stride(1);
        }
        return info;
    }
};

} // namespace op::rope_paged_caching

#endif
