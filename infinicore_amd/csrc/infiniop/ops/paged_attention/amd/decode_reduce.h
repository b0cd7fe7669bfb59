// Merge of the per-partition partial results of sequences longer than one partition:
//   M = max_p m_p,  out = sum_p acc_p * 2^(m_p - M) / (sum_p l_p * 2^(m_p - M) + 1e-6)
// rounded to the storage dtype. Same arithmetic as the reference's combine kernel
// (src/infiniop/ops/paged_attention/cuda/kernel_v2.cuh:556-616), with the number of partitions
// derived from the sequence length instead of being fixed.
//
// One 256-thread workgroup per (query head, sequence). Thread = (row group rg = tid / 16, strip
// c = tid % 16): it merges partitions rg, rg+16, ... for the value_size/16 output columns of strip
// c, so all partial rows of up to 16 partitions are fetched by one round of independent loads.
// Row groups are then merged with the same associative rule: inside a wavefront with lane swaps,
// across the four wavefronts through LDS.
#ifndef INFINICORE_AMD_PA_DECODE_REDUCE_H
#define INFINICORE_AMD_PA_DECODE_REDUCE_H

#include "decode_common.h"

namespace op::paged_attention::amd {

constexpr int kReduceThreads = 256;
constexpr int kReduceRowGroups = kReduceThreads / 16;

__device__ __forceinline__ float swapMax(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float swapSum(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// weight 2^(m - m_ref) of a partial result, 0 for an empty one (m = -inf), also when m_ref = -inf
__device__ __forceinline__ float mergeWeight(float m, float m_ref) {
    return m == -INFINITY ? 0.0f : fastExp2(m - m_ref);
}

// COLS = value_size / 16 output columns per thread (a multiple of 4).
template <typename T, typename Tindex, int COLS>
__global__ void __launch_bounds__(kReduceThreads) decodeReduceKernel(DecodeArgs a) {
    using S = typename T::storage;
    __shared__ float wave_acc[4][16][COLS];
    __shared__ float wave_m[4][16];
    __shared__ float wave_l[4][16];

    const int head = blockIdx.x;
    const int seq = blockIdx.y;
    const int tid = threadIdx.x;
    const int c = tid & 15;
    const int rg = tid >> 4;
    const int wave = tid >> 6;

    const int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) * a.block_size;
    const int len = static_cast<int>(len64 < max_len ? len64 : max_len);
    if (len <= a.partition_tokens) {
        return; // empty sequence, or already finished by the decode kernel (uniform for the workgroup)
    }
    const int parts = (len + a.partition_tokens - 1) / a.partition_tokens;
    const int64_t slot0 = (static_cast<int64_t>(seq) * a.num_heads + head) * a.max_partitions;

    // this thread's partitions: running (m, l, acc) merge
    float m_loc = -INFINITY, l_loc = 0.0f;
    float acc[COLS];
#pragma unroll
    for (int i = 0; i < COLS; ++i) {
        acc[i] = 0.0f;
    }
    for (int p = rg; p < parts; p += kReduceRowGroups) {
        const float m_p = a.part_m[slot0 + p];
        const float l_p = a.part_l[slot0 + p];
        const float4 *row = reinterpret_cast<const float4 *>(a.part_acc + (slot0 + p) * a.value_size + c * COLS);
        float4 v[COLS / 4];
#pragma unroll
        for (int i = 0; i < COLS / 4; ++i) {
            v[i] = row[i];
        }
        const float m_new = fmaxf(m_loc, m_p);
        const float w_old = mergeWeight(m_loc, m_new), w_p = mergeWeight(m_p, m_new);
        l_loc = l_loc * w_old + l_p * w_p;
#pragma unroll
        for (int i = 0; i < COLS / 4; ++i) {
            acc[4 * i + 0] = acc[4 * i + 0] * w_old + v[i].x * w_p;
            acc[4 * i + 1] = acc[4 * i + 1] * w_old + v[i].y * w_p;
            acc[4 * i + 2] = acc[4 * i + 2] * w_old + v[i].z * w_p;
            acc[4 * i + 3] = acc[4 * i + 3] * w_old + v[i].w * w_p;
        }
        m_loc = m_new;
    }

    // merge the four row groups of this wavefront (lanes c, c+16, c+32, c+48)
    const float m_w = swapMax(m_loc);
    const float f = mergeWeight(m_loc, m_w);
    const float l_w = swapSum(l_loc * f);
#pragma unroll
    for (int i = 0; i < COLS; ++i) {
        acc[i] = swapSum(acc[i] * f);
    }
    if ((tid & 63) < 16) {
        wave_m[wave][c] = m_w;
        wave_l[wave][c] = l_w;
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
            wave_acc[wave][c][i] = acc[i];
        }
    }
    __syncthreads();

    // the first 16 threads merge the four wavefronts, normalise and store COLS columns each
    if (tid < 16) {
        float m = wave_m[0][c];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            m = fmaxf(m, wave_m[w][c]);
        }
        float l = 0.0f, out_acc[COLS];
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
            out_acc[i] = 0.0f;
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float fw = mergeWeight(wave_m[w][c], m);
            l += wave_l[w][c] * fw;
#pragma unroll
            for (int i = 0; i < COLS; ++i) {
                out_acc[i] += wave_acc[w][c][i] * fw;
            }
        }
        const float inv_l = 1.0f / (l + 1e-6f);
        S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride + c * COLS;
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
            o_ptr[i] = T::fromFloat(out_acc[i] * inv_l);
        }
    }
}

} // namespace op::paged_attention::amd

#endif
