/*
 * KV caching (contiguous, non-paged caches): append the K/V vectors of `seq_len` new tokens per
 * sequence to per-sequence caches, behind the positions already filled.
 *
 * Same four entry points, argument order and meaning as the reference's
 * include/infiniop/ops/kv_caching.h:8-29.
 *
 * Tensors (element strides, all four dims of every tensor may be strided):
 *   k_cache, v_cache  [batch, num_kv_heads, max_seq_len, head_dim]   F16 | BF16 | F32
 *   k, v              [batch, num_kv_heads, seq_len, head_dim]       same dtype
 *   past_kv_lengths   [batch]  I32 | I64, contiguous
 *
 * cache[b, h, past_kv_lengths[b] + s, :] = new[b, h, s, :] for every b, h and s < seq_len
 * (reference kernel src/infiniop/ops/kv_caching/cuda/kernel.cuh:32-58). The copy is exact (bit for
 * bit); cache positions no new token lands on are not touched.
 */
#ifndef INFINICORE_AMD_INFINIOP_KV_CACHING_H
#define INFINICORE_AMD_INFINIOP_KV_CACHING_H

#include "../operator_descriptor.h"

typedef struct InfiniopDescriptor *infiniopKVCachingDescriptor_t;

/* Validation follows the reference's src/infiniop/ops/kv_caching/info.h:25-59.
 * Replaces src/infiniop/ops/kv_caching/operator.cc:12-58. */
__INFINI_C __export infiniStatus_t infiniopCreateKVCachingDescriptor(
    infiniopHandle_t handle,
    infiniopKVCachingDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t k_cache,
    infiniopTensorDescriptor_t v_cache,
    infiniopTensorDescriptor_t k,
    infiniopTensorDescriptor_t v,
    infiniopTensorDescriptor_t past_kv_lengths);

/* Always reports 0: the copy needs no scratch.
 * Replaces src/infiniop/ops/kv_caching/operator.cc:60-96. */
__INFINI_C __export infiniStatus_t infiniopGetKVCachingWorkspaceSize(
    infiniopKVCachingDescriptor_t desc,
    size_t *size);

/* Enqueues the copy on `stream` (NULL = default stream); workspace may be NULL.
 * Replaces src/infiniop/ops/kv_caching/operator.cc:98-140. */
__INFINI_C __export infiniStatus_t infiniopKVCaching(
    infiniopKVCachingDescriptor_t desc,
    void *workspace,
    size_t workspace_size,
    void *k_cache,
    void *v_cache,
    const void *k,
    const void *v,
    const void *past_kv_lengths,
    void *stream);

/* Replaces src/infiniop/ops/kv_caching/operator.cc:142-176. */
__INFINI_C __export infiniStatus_t infiniopDestroyKVCachingDescriptor(
    infiniopKVCachingDescriptor_t desc);

#endif
