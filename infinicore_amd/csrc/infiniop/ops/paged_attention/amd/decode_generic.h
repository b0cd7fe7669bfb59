// Fallback decode kernel: any head size up to 64 * DIMS_PER_LANE, any page size, any strides and
// alignment, ALiBi, all index dtypes. One wavefront per (partition, query head, sequence); lane i
// owns dimensions i, i+64, ... of the query, the accumulator and the output. It streams tokens one
// at a time with an online softmax, which is the arithmetic of the reference's per-warp kernel
// (src/infiniop/ops/paged_attention/cuda/kernel_v2.cuh:134-336) on a 64-lane wavefront. It does
// not share K/V between the query heads of a group and is only used for shapes the tiled kernel
// does not cover.
#ifndef INFINICORE_AMD_PA_DECODE_GENERIC_H
#define INFINICORE_AMD_PA_DECODE_GENERIC_H

#include "decode_common.h"

namespace op::paged_attention::amd {

template <typename T, typename Tindex, int DIMS_PER_LANE>
__global__ void __launch_bounds__(64) decodeGenericKernel(DecodeArgs a) {
    using S = typename T::storage;
    const int part = blockIdx.x;
    const int head = blockIdx.y;
    const int seq = blockIdx.z;
    const int lane = threadIdx.x;

    const int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
    if (len64 <= 0) {
        return; // out[seq] stays untouched (kernel_v2.cuh:164-167)
    }
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) * a.block_size;
    const int len = static_cast<int>(len64 < max_len ? len64 : max_len);
    const int start = part * a.partition_tokens;
    if (start >= len) {
        return;
    }
    const int end = min(len, start + a.partition_tokens);
    const int kv_head = head / a.group;
    const float slope = a.alibi_slopes ? a.alibi_slopes[head] : 0.0f;

    const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + head * a.q_head_stride;
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
    for (int t = start; t < end; ++t) {
        const int entry = a.block_shift >= 0 ? (t >> a.block_shift) : (t / a.block_size);
        const int row = t - entry * a.block_size;
        if (entry != cached_entry) {
            cached_entry = entry;
            const int page = clampPage(loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + entry),
                                       a.num_blocks);
            k_page = static_cast<const S *>(a.k_cache) + page * a.k_batch_stride + kv_head * a.k_head_stride;
            v_page = static_cast<const S *>(a.v_cache) + page * a.v_batch_stride + kv_head * a.v_head_stride;
        }
        const S *k_row = k_page + row * a.k_row_stride;
        const S *v_row = v_page + row * a.v_row_stride;

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
            score += slope * static_cast<float>(t - (len - 1)) * kLog2e;
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

    if (len <= a.partition_tokens) {
        // whole sequence in this partition: normalise and store (kernel_v2.cuh:318-335)
        const float inv_l = 1.0f / (l + 1e-6f);
        S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride;
#pragma unroll
        for (int i = 0; i < DIMS_PER_LANE; ++i) {
            const int d = lane + 64 * i;
            if (d < a.value_size) {
                o_ptr[d] = T::fromFloat(acc[i] * inv_l);
            }
        }
    } else {
        const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + head) * a.max_partitions + part;
        float *pa = a.part_acc + slot * a.value_size;
#pragma unroll
        for (int i = 0; i < DIMS_PER_LANE; ++i) {
            const int d = lane + 64 * i;
            if (d < a.value_size) {
                pa[d] = acc[i];
            }
        }
        if (lane == 0) {
            a.part_m[slot] = m;
            a.part_l[slot] = l;
        }
    }
}

} // namespace op::paged_attention::amd

#endif
