/*
 * Rotary position embedding of the new K vectors fused with their scatter (and that of the new V vectors) into
 * the paged KV pool: the producer step in front of every paged-attention decode call, in one launch.
 *
 * The result is that of the reference's two operators run one after the other,
 *   infiniopRoPE(k_rotated, k, pos_ids, sin_table, cos_table, algo)        include/infiniop/ops/rope.h:15-39
 *   infiniopPagedCaching(k_cache, v_cache, k_rotated, v, slot_mapping)     include/infiniop/ops/paged_caching.h:24-75
 * without the intermediate tensor: the reference has no fused entry point, these four are new. Argument
 * meaning, layouts and status codes are those of the two operators.
 *
 * Tensors (element strides; the last dimension of every tensor has stride 1):
 *   k_cache       [num_blocks, num_kv_heads, block_size, head_size]   F16 | BF16 | F32, any strides on dims 0-2
 *   v_cache       [num_blocks, num_kv_heads, block_size, value_size]  same dtype
 *   k             [num_tokens, num_kv_heads, head_size]               same dtype, heads packed inside a token
 *   v             [num_tokens, num_kv_heads, value_size]
 *   slot_mapping  [num_tokens] I64: slot = page * block_size + row; negative = padding, the token is skipped
 *   pos_ids       [num_tokens] any integer dtype: row of the tables for token i
 *   sin_table     [table_len, head_size / 2]  same dtype as k, contiguous
 *   cos_table     [table_len, head_size / 2]
 *
 * For token i with slot s >= 0 and every KV head h, with p = pos_ids[i] and pairs (a, b) = (2j, 2j + 1) for
 * GPT_J, (j, j + head_size / 2) for GPT_NEOX, j < head_size / 2:
 *   k_cache[s / bs][h][s % bs][a] = k[i][h][a] * cos[p][j] - k[i][h][b] * sin[p][j]
 *   k_cache[s / bs][h][s % bs][b] = k[i][h][a] * sin[p][j] + k[i][h][b] * cos[p][j]
 *   v_cache[s / bs][h][s % bs][:] = v[i][h][:]
 * Products and sums are rounded to fp32 one by one (no fused multiply-add), the result once to the storage
 * dtype (round to nearest even): the arithmetic of src/infiniop/ops/rope/cpu/rope_cpu.cc:71-84. Slots outside
 * the pool are dropped; positions outside the tables use the nearest row (the reference reads out of bounds).
 */
#ifndef INFINICORE_AMD_INFINIOP_ROPE_PAGED_CACHING_H
#define INFINICORE_AMD_INFINIOP_ROPE_PAGED_CACHING_H

#include "../operator_descriptor.h"

/* Same values as the reference's include/infiniop/ops/rope.h:6-11. */
typedef enum {
    INFINIOP_ROPE_ALGO_GPT_J = 0,    /* pairs are neighbours: (2j, 2j + 1) */
    INFINIOP_ROPE_ALGO_GPT_NEOX = 1, /* pairs are half a vector apart: (j, j + head_size / 2) */
    INFINIOP_ROPE_ALGO_COUNT = 2,
} infiniopRoPEAlgo_t;

typedef struct InfiniopDescriptor *infiniopRoPEPagedCachingDescriptor_t;

/* Validates the operands (the checks of both operators: src/infiniop/ops/rope/rope.h:72-160 for k, pos_ids
 * and the tables, src/infiniop/ops/paged_caching/info.h:35-107 for the rest) and builds a descriptor that owns
 * a copy of all metadata. */
__INFINI_C __export infiniStatus_t infiniopCreateRoPEPagedCachingDescriptor(
    infiniopHandle_t handle,
    infiniopRoPEPagedCachingDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t k_cache_desc,
    infiniopTensorDescriptor_t v_cache_desc,
    infiniopTensorDescriptor_t k_desc,
    infiniopTensorDescriptor_t v_desc,
    infiniopTensorDescriptor_t slot_mapping_desc,
    infiniopTensorDescriptor_t pos_ids_desc,
    infiniopTensorDescriptor_t sin_table_desc,
    infiniopTensorDescriptor_t cos_table_desc,
    infiniopRoPEAlgo_t algo);

/* Always reports 0. */
__INFINI_C __export infiniStatus_t infiniopGetRoPEPagedCachingWorkspaceSize(
    infiniopRoPEPagedCachingDescriptor_t desc,
    size_t *size);

/* Enqueues the rotation and scatter on `stream` (NULL = default stream) and returns without waiting; one kernel
 * launch, no allocation, no synchronisation, no host read of device data. */
__INFINI_C __export infiniStatus_t infiniopRoPEPagedCaching(
    infiniopRoPEPagedCachingDescriptor_t desc,
    void *workspace,
    size_t workspace_size,
    void *k_cache,
    void *v_cache,
    const void *k,
    const void *v,
    const void *slot_mapping,
    const void *pos_ids,
    const void *sin_table,
    const void *cos_table,
    void *stream);

__INFINI_C __export infiniStatus_t infiniopDestroyRoPEPagedCachingDescriptor(
    infiniopRoPEPagedCachingDescriptor_t desc);

/*
 * The same with the rotation of the query in the launch as well: the whole producer step in front of a decode
 * call, which the reference runs as infiniopRoPE on q, infiniopRoPE on k and infiniopPagedCaching.
 *   q      [num_tokens, num_heads, head_size]  same dtype as k, any token / head strides, last dimension packed
 *   q_out  [num_tokens, num_heads, head_size]  same dtype; may be q itself (rotation in place)
 *   q_out[i][h] = rotation of q[i][h] by row pos_ids[i] of the tables, for EVERY token i - also those whose slot is
 *   negative (padding): only the cache writes are skipped for them.
 * q, k and v may be slices of one fused projection output (their token strides are taken from the descriptors).
 * The descriptor is of the same type as above: infiniopGetRoPEPagedCachingWorkspaceSize and
 * infiniopDestroyRoPEPagedCachingDescriptor serve both; each descriptor is run with the entry point that
 * matches the way it was created (the other one answers BAD_PARAM).
 */
__INFINI_C __export infiniStatus_t infiniopCreateRoPEQKPagedCachingDescriptor(
    infiniopHandle_t handle,
    infiniopRoPEPagedCachingDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t q_out_desc,
    infiniopTensorDescriptor_t q_desc,
    infiniopTensorDescriptor_t k_cache_desc,
    infiniopTensorDescriptor_t v_cache_desc,
    infiniopTensorDescriptor_t k_desc,
    infiniopTensorDescriptor_t v_desc,
    infiniopTensorDescriptor_t slot_mapping_desc,
    infiniopTensorDescriptor_t pos_ids_desc,
    infiniopTensorDescriptor_t sin_table_desc,
    infiniopTensorDescriptor_t cos_table_desc,
    infiniopRoPEAlgo_t algo);

__INFINI_C __export infiniStatus_t infiniopRoPEQKPagedCaching(
    infiniopRoPEPagedCachingDescriptor_t desc,
    void *workspace,
    size_t workspace_size,
    void *q_out,
    const void *q,
    void *k_cache,
    void *v_cache,
    const void *k,
    const void *v,
    const void *slot_mapping,
    const void *pos_ids,
    const void *sin_table,
    const void *cos_table,
    void *stream);

#endif
