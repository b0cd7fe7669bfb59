/*
 * Paged caching: scatter freshly computed K/V vectors of a chunk of tokens into their slots of
 * the paged KV pool.
 *
 * Same four entry points, argument order and meaning as the reference's
 * include/infiniop/ops/paged_caching.h:24-75.
 *
 * Tensors (element strides):
 *   k_cache       [num_blocks, num_kv_heads, block_size, head_size]   F16 | BF16 | F32, any strides on dims 0-2
 *   v_cache       [num_blocks, num_kv_heads, block_size, value_size]  same dtype
 *   k             [num_tokens, num_kv_heads, head_size]   same dtype; heads and elements packed, any token stride
 *   v             [num_tokens, num_kv_heads, value_size]
 *   slot_mapping  [num_tokens] I64, contiguous
 *
 * Token i goes to page slot_mapping[i] / block_size, row slot_mapping[i] % block_size, for every KV
 * head; a negative slot marks padding and is skipped. Bytes of the pool that no slot names are not
 * touched. The copy is exact (bit for bit). Two tokens naming the same slot race, as in the reference.
 */
#ifndef INFINICORE_AMD_INFINIOP_PAGED_CACHING_H
#define INFINICORE_AMD_INFINIOP_PAGED_CACHING_H

#include "../operator_descriptor.h"

typedef struct InfiniopDescriptor *infiniopPagedCachingDescriptor_t;

/* Validation follows the reference's src/infiniop/ops/paged_caching/info.h:35-107.
 * Replaces src/infiniop/ops/paged_caching/operator.cc:21-68. */
__INFINI_C __export infiniStatus_t infiniopCreatePagedCachingDescriptor(
    infiniopHandle_t handle,
    infiniopPagedCachingDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t k_cache_desc,
    infiniopTensorDescriptor_t v_cache_desc,
    infiniopTensorDescriptor_t k_desc,
    infiniopTensorDescriptor_t v_desc,
    infiniopTensorDescriptor_t slot_mapping_desc);

/* Always reports 0: the scatter needs no scratch.
 * Replaces src/infiniop/ops/paged_caching/operator.cc:70-110. */
__INFINI_C __export infiniStatus_t infiniopGetPagedCachingWorkspaceSize(
    infiniopPagedCachingDescriptor_t desc,
    size_t *size);

/* Enqueues the scatter on `stream` (NULL = default stream); workspace may be NULL.
 * Replaces src/infiniop/ops/paged_caching/operator.cc:112-156. */
__INFINI_C __export infiniStatus_t infiniopPagedCaching(
    infiniopPagedCachingDescriptor_t desc,
    void *workspace,
    size_t workspace_size,
    void *k_cache,
    void *v_cache,
    const void *k,
    const void *v,
    const void *slot_mapping,
    void *stream);

/* Replaces src/infiniop/ops/paged_caching/operator.cc:158-197. */
__INFINI_C __export infiniStatus_t infiniopDestroyPagedCachingDescriptor(
    infiniopPagedCachingDescriptor_t desc);

#endif
