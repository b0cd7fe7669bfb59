// Shared vocabulary of the paged-attention prefill kernels: the argument block and the per-sequence
// bookkeeping (which query rows a sequence owns, how many K/V tokens each of them may see).
#ifndef INFINICORE_AMD_PA_PREFILL_COMMON_H
#define INFINICORE_AMD_PA_PREFILL_COMMON_H

#include "../../paged_attention/amd/decode_common.h"

namespace op::paged_attention_prefill::amd {

using op::paged_attention::amd::clampPage;
using op::paged_attention::amd::fastExp2;
using op::paged_attention::amd::kLog2e;
using op::paged_attention::amd::loadIndex;

struct PrefillArgs {
    void *out;
    const void *q;
    const void *k_cache;
    const void *v_cache;
    const void *block_tables;
    const void *kv_lens;      // [num_seqs] total K/V tokens per sequence (history + new)
    const void *cu_seqlens_q; // [num_seqs + 1] prefix sums of the new-token counts
    const float *alibi_slopes; // nullptr = no ALiBi

    float scale_log2; // scale * log2(e)
    int32_t num_seqs;
    int32_t total_q_tokens;
    int32_t num_heads;
    int32_t num_kv_heads;
    int32_t group; // query heads per KV head
    int32_t head_size;
    int32_t value_size;
    int32_t block_size;
    int32_t block_shift; // log2(block_size) if a power of two, else -1
    int32_t num_blocks;  // pool size; table entries are clamped into [0, num_blocks)
    int32_t max_blocks_per_seq;

    // element strides
    int64_t q_stride, q_head_stride;
    int64_t o_stride, o_head_stride;
    int64_t k_batch_stride, k_head_stride, k_row_stride;
    int64_t v_batch_stride, v_head_stride, v_row_stride;
    int64_t block_table_batch_stride;
};

// What one sequence contributes. Query token j (0 <= j < q_len) is row q_start + j of q / out and
// sees K/V tokens [0, history + j + 1), as in the reference kernels
// (src/infiniop/ops/paged_attention_prefill/cuda/kernel_v2.cuh:290-306). The row range is clipped
// to the q tensor and the visible range to what the block table can address, so that inconsistent
// index tensors cannot cause an access outside the operands.
struct SeqSpan {
    int32_t q_start;
    int32_t q_len;   // <= 0: nothing to do
    int32_t history; // may be negative: the first -history query tokens then see nothing
    int32_t capacity; // max_blocks_per_seq * block_size, the most tokens a row may see
    int32_t kv_len;   // K/V tokens the sequence holds, forced into [0, capacity]
};

template <typename Tindex>
__device__ __forceinline__ SeqSpan loadSeqSpan(const PrefillArgs &a, int seq) {
    int64_t q0 = loadIndex<Tindex>(a.cu_seqlens_q, seq);
    int64_t q1 = loadIndex<Tindex>(a.cu_seqlens_q, seq + 1);
    const int64_t kv = loadIndex<Tindex>(a.kv_lens, seq);
    const int64_t raw_len = q1 - q0;
    q0 = q0 < 0 ? 0 : (q0 > a.total_q_tokens ? a.total_q_tokens : q0);
    q1 = q1 < q0 ? q0 : (q1 > a.total_q_tokens ? a.total_q_tokens : q1);
    int64_t history = kv - raw_len;
    const int64_t lim = int64_t(1) << 30;
    history = history < -lim ? -lim : (history > lim ? lim : history);
    SeqSpan s;
    s.q_start = static_cast<int32_t>(q0);
    s.q_len = static_cast<int32_t>(q1 - q0);
    s.history = static_cast<int32_t>(history);
    const int64_t cap = static_cast<int64_t>(a.max_blocks_per_seq) * a.block_size;
    s.capacity = static_cast<int32_t>(cap > lim ? lim : cap);
    s.kv_len = static_cast<int32_t>(kv < 0 ? 0 : (kv > s.capacity ? s.capacity : kv));
    return s;
}

// K/V tokens query token j of the span may see (0 = none: its output row stays untouched).
__device__ __forceinline__ int32_t visibleTokens(const SeqSpan &s, int32_t j) {
    const int32_t n = s.history + j + 1;
    return n < 0 ? 0 : (n > s.capacity ? s.capacity : n);
}

} // namespace op::paged_attention_prefill::amd

#endif
