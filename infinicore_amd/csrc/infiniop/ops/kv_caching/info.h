// Create-time validation of the kv_caching operands and capture of every size and stride the copy
// needs. Follows the reference's src/infiniop/ops/kv_caching/info.h:25-104, with two checks made
// stricter (noted below) so that a descriptor that was accepted cannot index outside its operands.
#ifndef INFINICORE_AMD_KV_CACHING_INFO_H
#define INFINICORE_AMD_KV_CACHING_INFO_H

#include "../../../utils/check.h"
#include "../../../utils/result.h"
#include "../../tensor.h"

namespace op::kv_caching {

struct KVCachingInfo {
    infiniDtype_t dtype;
    infiniDtype_t past_len_dtype;
    size_t batch_size, num_kv_heads, max_seq_len, seq_len, hidden_dim;
    // element strides of dims 0..3
    ptrdiff_t k_cache_strides[4], v_cache_strides[4], k_strides[4], v_strides[4];

    static utils::Result<KVCachingInfo> create(infiniopTensorDescriptor_t k_cache, infiniopTensorDescriptor_t v_cache,
                                               infiniopTensorDescriptor_t k, infiniopTensorDescriptor_t v,
                                               infiniopTensorDescriptor_t past_kv_lengths) {
        if (!k_cache || !v_cache || !k || !v || !past_kv_lengths) {
            return INFINI_STATUS_NULL_POINTER; // info.h:32-34
        }
        KVCachingInfo info{};
        info.dtype = k_cache->dtype();
        CHECK_DTYPE(info.dtype, INFINI_DTYPE_F16, INFINI_DTYPE_BF16, INFINI_DTYPE_F32); // info.h:36-37
        info.past_len_dtype = past_kv_lengths->dtype();
        CHECK_DTYPE(info.past_len_dtype, INFINI_DTYPE_I32, INFINI_DTYPE_I64); // info.h:38-39
        // The reference reads all four tensors through k_cache's dtype without comparing them.
        if (v_cache->dtype() != info.dtype || k->dtype() != info.dtype || v->dtype() != info.dtype) {
            return INFINI_STATUS_BAD_TENSOR_DTYPE;
        }
        if (k_cache->ndim() != 4 || v_cache->ndim() != 4 || k->ndim() != 4 || v->ndim() != 4) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE; // info.h:41-45
        }
        for (size_t i = 0; i < 4; ++i) { // info.h:47-49
            if (v_cache->dim(i) != k_cache->dim(i) || v->dim(i) != k->dim(i)) {
                return INFINI_STATUS_BAD_TENSOR_SHAPE;
            }
        }
        info.batch_size = k_cache->dim(0);
        info.num_kv_heads = k_cache->dim(1);
        info.max_seq_len = k_cache->dim(2);
        info.hidden_dim = k_cache->dim(3);
        info.seq_len = k->dim(2);
        // info.h:58-61 accepts the new tensors if ANY of batch, heads, head_dim agrees with the caches
        // and then indexes them with the caches' sizes; here all three must agree.
        if (k->dim(0) != info.batch_size || k->dim(1) != info.num_kv_heads || k->dim(3) != info.hidden_dim) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        // one length per sequence, packed (the reference kernel reads past_kv_lengths[b])
        if (past_kv_lengths->ndim() != 1 || past_kv_lengths->dim(0) != info.batch_size
            || (info.batch_size > 1 && past_kv_lengths->stride(0) != 1)) {
            return INFINI_STATUS_BAD_TENSOR_SHAPE;
        }
        for (size_t i = 0; i < 4; ++i) {
            info.k_cache_strides[i] = k_cache->stride(i);
            info.v_cache_strides[i] = v_cache->stride(i);
            info.k_strides[i] = k->stride(i);
            info.v_strides[i] = v->stride(i);
        }
        return info;
    }
};

} // namespace op::kv_caching

#endif
