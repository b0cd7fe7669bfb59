/*
 * Paged-attention prefill: a batch of sequences each brings a run of new query tokens (packed one
 * after another in q) that attend causally over the sequence's paged K/V, which already holds the
 * history and the new tokens' own keys and values.
 *
 * Same four entry points, argument order and meaning as the reference's
 * include/infiniop/ops/paged_attention_prefill.h:32-91.
 *
 * Tensors (element strides; the last dimension of q, out and both caches must have stride 1):
 *   out             [total_q_tokens, num_heads, value_size]           F16 | BF16
 *   q               [total_q_tokens, num_heads, head_size]            same dtype
 *   k_cache         [num_blocks, num_kv_heads, block_size, head_size] same dtype, any strides on dims 0-2
 *   v_cache         [num_blocks, num_kv_heads, block_size, value_size]
 *   block_tables    [num_seqs, max_blocks_per_seq]  I64 | I32 | U32, row-contiguous
 *   seq_lens        [num_seqs]       total K/V tokens of each sequence (history + new), same index dtype
 *   cum_seq_lens_q  [num_seqs + 1]   prefix sums of the new-token counts, same index dtype
 *   alibi_slopes    [num_heads] F32 contiguous, or NULL
 *
 * Sequence s owns query rows cum_seq_lens_q[s] .. cum_seq_lens_q[s+1]-1. With
 * q_len = cum_seq_lens_q[s+1] - cum_seq_lens_q[s] and history = seq_lens[s] - q_len, its j-th new token
 * sees K/V tokens 0 .. history + j (itself included); a token for which that range is empty, and any
 * row past cum_seq_lens_q[num_seqs], is left untouched in out. Paging, head mapping, ALiBi (distance
 * to the token's own position), the 1e-6 in the normaliser and the rounding are those of the decode
 * operator (paged_attention.h).
 */
#ifndef INFINICORE_AMD_INFINIOP_PAGED_ATTENTION_PREFILL_H
#define INFINICORE_AMD_INFINIOP_PAGED_ATTENTION_PREFILL_H

#include "../operator_descriptor.h"

typedef struct InfiniopDescriptor *infiniopPagedAttentionPrefillDescriptor_t;

/* Validates the tensor descriptors and builds an operator descriptor that owns a copy of all
 * metadata. Errors as in the reference's src/infiniop/ops/paged_attention_prefill/info.h:43-210
 * (BAD_TENSOR_DTYPE / BAD_TENSOR_SHAPE / BAD_TENSOR_STRIDES, BAD_PARAM for a cum_seq_lens_q whose
 * length is not num_seqs + 1). Replaces src/infiniop/ops/paged_attention_prefill/operator.cc:21-72. */
__INFINI_C __export infiniStatus_t infiniopCreatePagedAttentionPrefillDescriptor(
    infiniopHandle_t handle,
    infiniopPagedAttentionPrefillDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t out_desc,
    infiniopTensorDescriptor_t q_desc,
    infiniopTensorDescriptor_t k_cache_desc,
    infiniopTensorDescriptor_t v_cache_desc,
    infiniopTensorDescriptor_t block_tables_desc,
    infiniopTensorDescriptor_t seq_lens_desc,
    infiniopTensorDescriptor_t cum_seq_lens_q_desc,
    infiniopTensorDescriptor_t alibi_slopes_desc,
    float scale);

/* Bytes of device scratch the run call needs (0 on this backend).
 * Replaces src/infiniop/ops/paged_attention_prefill/operator.cc:74-111. */
__INFINI_C __export infiniStatus_t infiniopGetPagedAttentionPrefillWorkspaceSize(
    infiniopPagedAttentionPrefillDescriptor_t desc,
    size_t *size);

/* Enqueues the prefill on `stream` (NULL = the device's default stream) and returns without waiting.
 * All data pointers are device pointers; nothing is allocated, synchronised or read back.
 * Replaces src/infiniop/ops/paged_attention_prefill/operator.cc:113-157. */
__INFINI_C __export infiniStatus_t infiniopPagedAttentionPrefill(
    infiniopPagedAttentionPrefillDescriptor_t desc,
    void *workspace,
    size_t workspace_size,
    void *out,
    const void *q,
    const void *k_cache,
    const void *v_cache,
    const void *block_tables,
    const void *seq_lens,
    const void *cum_seq_lens_q,
    const void *alibi_slopes,
    void *stream);

/* Replaces src/infiniop/ops/paged_attention_prefill/operator.cc:159-195. */
__INFINI_C __export infiniStatus_t infiniopDestroyPagedAttentionPrefillDescriptor(
    infiniopPagedAttentionPrefillDescriptor_t desc);

#endif
