// Fallback prefill kernel: any head size up to 64 * DIMS_PER_LANE, any page size, any strides and
// alignment, ALiBi, all index dtypes. One wavefront per (query token, query head); lane i owns
// dimensions i, i+64, ... It streams the visible K/V tokens one at a time with an online softmax,
// which is the arithmetic of the reference's per-warp kernel
// (src/infiniop/ops/paged_attention_prefill/cuda/kernel_v2.cuh:254-472) on a 64-lane wavefront.
// Only used for shapes the tiled kernel does not cover.
#ifndef INFINICORE_AMD_PA_PREFILL_GENERIC_H
#define INFINICORE_AMD_PA_PREFILL_GENERIC_H

#include "prefill_common.h"

namespace op::paged_attention_prefill::amd {

// Sequence that owns query row `row`: the last s with cu_seqlens_q[s] <= row, provided the row is
// below cu_seqlens_q[s + 1]; -1 for a row no sequence owns.
template <typename Tindex>
__device__ __forceinline__ int findSequence(const PrefillArgs &a, int64_t row) {
    if (a.num_seqs <= 0) {
        return -1;
    }
    int lo = 0, hi = a.num_seqs;
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (loadIndex<Tindex>(a.cu_seqlens_q, mid) <= row) {
            lo = mid;
        } else {
            hi = mid;
        }
    }
    const int64_t q0 = loadIndex<Tindex>(a.cu_seqlens_q, lo);
    const int64_t q1 = loadIndex<Tindex>(a.cu_seqlens_q, lo + 1);
    return (row >= q0 && row < q1) ? lo : -1;
}

template <typename T, typename Tindex, int DIMS_PER_LANE>
__global__ void __launch_bounds__(64) prefillGenericKernel(PrefillArgs a) {
    using S = typename T::storage;
    using op::paged_attention::amd::waveSum;
    const int row = blockIdx.x; // query token, global
    const int head = blockIdx.y;
    const int lane = threadIdx.x;

    const int seq = findSequence<Tindex>(a, row);
    if (seq < 0) {
        return;
    }
    const SeqSpan span = loadSeqSpan<Tindex>(a, seq);
    const int visible = visibleTokens(span, row - span.q_start);
    if (visible <= 0) {
        return; // the output row stays untouched (kernel_v2.cuh:302-306)
    }
    const int kv_head = head / a.group;
    const float slope = a.alibi_slopes ? a.alibi_slopes[head] : 0.0f;

    const S *q_ptr = static_cast<const S *>(a.q) + row * a.q_stride + head * a.q_head_stride;
    float q_reg[DIMS_PER_LANE], acc[DIMS_PER_LANE];
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
        const int d = lane + 64 * i;
        q_reg[i] = d < a.head_size ? T::toFloat(q_ptr[d]) : 0.0f;
        acc[i] = 0.0f;
    }

    float m = -INFINITY, l = 0.0f;
    const S *k_page = nullptr, *v_page = nullptr;
    int cached_entry = -1;
    for (int t = 0; t < visible; ++t) {
        const int entry = a.block_shift >= 0 ? (t >> a.block_shift) : (t / a.block_size);
        const int page_row = t - entry * a.block_size;
        if (entry != cached_entry) {
            cached_entry = entry;
            const int page = clampPage(loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + entry),
                                       a.num_blocks);
            k_page = static_cast<const S *>(a.k_cache) + page * a.k_batch_stride + kv_head * a.k_head_stride;
            v_page = static_cast<const S *>(a.v_cache) + page * a.v_batch_stride + kv_head * a.v_head_stride;
        }
        const S *k_row = k_page + page_row * a.k_row_stride;
        const S *v_row = v_page + page_row * a.v_row_stride;

        float dot = 0.0f;
#pragma unroll
        for (int i = 0; i < DIMS_PER_LANE; ++i) {
            const int d = lane + 64 * i;
            if (d < a.head_size) {
                dot += q_reg[i] * T::toFloat(k_row[d]);
            }
        }
        dot = waveSum(dot);

        float score = dot * a.scale_log2;
        if (slope != 0.0f) {
            score += slope * static_cast<float>(t - (visible - 1)) * kLog2e;
        }
        const float m_new = fmaxf(m, score);
        const float alpha = fastExp2(m - m_new);
        const float beta = fastExp2(score - m_new);
        l = l * alpha + beta;
        m = m_new;
#pragma unroll
        for (int i = 0; i < DIMS_PER_LANE; ++i) {
            const int d = lane + 64 * i;
            if (d < a.value_size) {
                acc[i] = acc[i] * alpha + beta * T::toFloat(v_row[d]);
            }
        }
    }

    const float inv_l = 1.0f / (l + 1e-6f);
    S *o_ptr = static_cast<S *>(a.out) + row * a.o_stride + head * a.o_head_stride;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
        const int d = lane + 64 * i;
        if (d < a.value_size) {
            o_ptr[d] = T::fromFloat(acc[i] * inv_l);
        }
    }
}

} // namespace op::paged_attention_prefill::amd

#endif
