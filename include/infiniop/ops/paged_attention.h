/*
 * Paged-attention decode: one query token per sequence attends over that sequence's K/V history,
 * which lives in fixed-size pages of a shared pool and is found through a per-sequence block table.
 *
 * Same four entry points, argument order and meaning as the reference's
 * include/infiniop/ops/paged_attention.h:33-91.
 *
 * Tensors (element strides; the last dimension of q, out and both caches must have stride 1):
 *   out           [num_seqs, num_heads, value_size]                 F16 | BF16
 *   q             [num_seqs, num_heads, head_size]                  same dtype
 *   k_cache       [num_blocks, num_kv_heads, block_size, head_size] same dtype, any strides on dims 0-2
 *   v_cache       [num_blocks, num_kv_heads, block_size, value_size]
 *   block_tables  [num_seqs, max_blocks_per_seq]  I64 | I32 | U32, row-contiguous
 *   seq_lens      [num_seqs]                      same index dtype, contiguous
 *   alibi_slopes  [num_heads] F32 contiguous, or NULL
 *
 * Token t of sequence s is row t % block_size of page block_tables[s][t / block_size]; query head h
 * reads KV head h / (num_heads / num_kv_heads). Only tokens t < seq_lens[s] take part; table entries
 * past the last needed page are never read. A sequence with seq_lens[s] <= 0 leaves out[s] untouched.
 * The result is sum_t(p_t * v_t) / (sum_t(p_t) + 1e-6) with p_t = exp(scale * q.k_t + alibi_h * (t - (len-1)) - max),
 * accumulated in fp32 and rounded to the storage dtype with round-to-nearest-even.
 */
#ifndef INFINICORE_AMD_INFINIOP_PAGED_ATTENTION_H
#define INFINICORE_AMD_INFINIOP_PAGED_ATTENTION_H

#include "../operator_descriptor.h"

typedef struct InfiniopDescriptor *infiniopPagedAttentionDescriptor_t;

/* Validates the tensor descriptors and builds an operator descriptor that owns a copy of all
 * metadata (the tensor descriptors may be destroyed right after this call).
 * Errors: BAD_TENSOR_DTYPE / BAD_TENSOR_SHAPE / BAD_TENSOR_STRIDES as listed in the reference's
 * src/infiniop/ops/paged_attention/info.h:41-194; DEVICE_TYPE_NOT_SUPPORTED for a handle of a
 * device other than AMD. Replaces src/infiniop/ops/paged_attention/operator.cc:21-70. */
__INFINI_C __export infiniStatus_t infiniopCreatePagedAttentionDescriptor(
    infiniopHandle_t handle,
    infiniopPagedAttentionDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t out_desc,
    infiniopTensorDescriptor_t q_desc,
    infiniopTensorDescriptor_t k_cache_desc,
    infiniopTensorDescriptor_t v_cache_desc,
    infiniopTensorDescriptor_t block_tables_desc,
    infiniopTensorDescriptor_t seq_lens_desc,
    infiniopTensorDescriptor_t alibi_slopes_desc,
    float scale);

/* Bytes of device scratch the run call needs; fixed at creation from the descriptors alone
 * (it holds the per-partition partial results of long sequences).
 * Replaces src/infiniop/ops/paged_attention/operator.cc:72-109. */
__INFINI_C __export infiniStatus_t infiniopGetPagedAttentionWorkspaceSize(
    infiniopPagedAttentionDescriptor_t desc,
    size_t *size);

/* Enqueues the decode on `stream` (NULL = the device's default stream) and returns without waiting.
 * All data pointers are device pointers. It allocates nothing, never synchronises and never reads
 * device data on the host, so it may be recorded into a stream capture.
 * workspace_size below the size reported above -> INSUFFICIENT_WORKSPACE.
 * Replaces src/infiniop/ops/paged_attention/operator.cc:111-152. */
__INFINI_C __export infiniStatus_t infiniopPagedAttention(
    infiniopPagedAttentionDescriptor_t desc,
    void *workspace,
    size_t workspace_size,
    void *out,
    const void *q,
    const void *k_cache,
    const void *v_cache,
    const void *block_tables,
    const void *seq_lens,
    const void *alibi_slopes,
    void *stream);

/* infiniopPagedAttention without the workspace argument, for callers that cannot allocate device memory
 * (code under stream capture that owns no buffer, serving loops and harnesses that forbid allocation).
 * It has no counterpart in the reference. The partial results go to an array of 32 MiB that the library
 * itself holds on every GPU it runs on; a descriptor whose workspace size (see above) exceeds that is
 * answered with INSUFFICIENT_WORKSPACE and a message on stderr. It calls no allocator. All calls on one GPU
 * share the array: calls that overlap there (two streams, two threads) race; calls on one stream are
 * ordered and safe. The calling thread's current device must be the descriptor's. Results are those of
 * infiniopPagedAttention, bit for bit. */
__INFINI_C __export infiniStatus_t infiniopPagedAttentionNoAlloc(
    infiniopPagedAttentionDescriptor_t desc,
    void *out,
    const void *q,
    const void *k_cache,
    const void *v_cache,
    const void *block_tables,
    const void *seq_lens,
    const void *alibi_slopes,
    void *stream);

/* Replaces src/infiniop/ops/paged_attention/operator.cc:154-190. */
__INFINI_C __export infiniStatus_t infiniopDestroyPagedAttentionDescriptor(
    infiniopPagedAttentionDescriptor_t desc);

#endif
