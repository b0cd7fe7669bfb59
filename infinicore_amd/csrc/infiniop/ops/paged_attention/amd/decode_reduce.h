// Merge of the per-partition partial results of sequences longer than one partition:
//   M = max_p m_p,  out = sum_p acc_p * 2^(m_p - M) / (sum_p l_p * 2^(m_p - M) + 1e-6)
// rounded to the storage dtype. Same arithmetic as the reference's combine kernel
// (src/infiniop/ops/paged_attention/cuda/kernel_v2.cuh:556-616), with the number of partitions
// derived from the sequence length instead of being fixed. One wavefront per (query head, sequence).
#ifndef INFINICORE_AMD_PA_DECODE_REDUCE_H
#define INFINICORE_AMD_PA_DECODE_REDUCE_H

#include "decode_common.h"

namespace op::paged_attention::amd {

template <typename T, typename Tindex, int DIMS_PER_LANE>
__global__ void __launch_bounds__(64) decodeReduceKernel(DecodeArgs a) {
    using S = typename T::storage;
    const int head = blockIdx.x;
    const int seq = blockIdx.y;
    const int lane = threadIdx.x;

    const int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) * a.block_size;
    const int len = static_cast<int>(len64 < max_len ? len64 : max_len);
    if (len <= a.partition_tokens) {
        return; // empty sequence, or already finished by the decode kernel
    }
    const int parts = (len + a.partition_tokens - 1) / a.partition_tokens;
    const int64_t slot0 = (static_cast<int64_t>(seq) * a.num_heads + head) * a.max_partitions;

    // every lane looks at a strided subset of the partitions, then the wavefront agrees
    float m = -INFINITY;
    for (int p = lane; p < parts; p += 64) {
        m = fmaxf(m, a.part_m[slot0 + p]);
    }
    m = waveMax(m);
    float l = 0.0f;
    for (int p = lane; p < parts; p += 64) {
        l += a.part_l[slot0 + p] * fastExp2(a.part_m[slot0 + p] - m);
    }
    l = waveSum(l);
    const float inv_l = 1.0f / (l + 1e-6f);

    float acc[DIMS_PER_LANE];
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
        acc[i] = 0.0f;
    }
    for (int p = 0; p < parts; ++p) {
        const float w = fastExp2(a.part_m[slot0 + p] - m);
        const float *pa = a.part_acc + (slot0 + p) * a.value_size;
#pragma unroll
        for (int i = 0; i < DIMS_PER_LANE; ++i) {
            const int d = lane + 64 * i;
            if (d < a.value_size) {
                acc[i] += pa[d] * w;
            }
        }
    }
    S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride;
#pragma unroll
    for (int i = 0; i < DIMS_PER_LANE; ++i) {
        const int d = lane + 64 * i;
        if (d < a.value_size) {
            o_ptr[d] = T::fromFloat(acc[i] * inv_l);
        }
    }
}

} // namespace op::paged_attention::amd

#endif
