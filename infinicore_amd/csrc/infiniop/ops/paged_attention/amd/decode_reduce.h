// Merge of the per-partition partial results of sequences longer than one partition:
//   M = max_p m_p,  out = sum_p acc_p * 2^(m_p - M) / (sum_p l_p * 2^(m_p - M) + 1e-6)
// rounded to the storage dtype. Same arithmetic as the reference's combine kernel
// (src/infiniop/ops/paged_attention/cuda/kernel_v2.cuh:556-616), with the number of partitions
// derived from the sequence length instead of being fixed.
//
// One 256-thread workgroup per (query head, sequence). Thread = (row group rg = tid / 16, strip
// c = tid % 16): it merges partitions rg, rg+16, ... for the value_size/16 output columns of strip
// c (groups of four columns, 64 apart), so all partial rows of up to 16 partitions are fetched by
// one round of independent, coalesced loads.
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

// COLS = value_size / 16 output columns per thread (a multiple of 4): strip c owns the COLS/4 groups of
// four columns 64 i + 4 c .. + 3, so the 16 threads of a row group read 256 contiguous bytes of a partial
// row with every load instruction and write 128 contiguous bytes of the output row per group.
template <typename T, typename Tindex, int COLS>
__global__ void __launch_bounds__(kReduceThreads) decodeReduceKernel(DecodeArgs a) {
    using S = typename T::storage;
    constexpr int kGroups = COLS / 4;
    __shared__ float4 wave_acc[4][kGroups][16];
    __shared__ float wave_m[4];
    __shared__ float wave_l[4];

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
    float4 acc[kGroups];
#pragma unroll
    for (int i = 0; i < kGroups; ++i) {
        acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    for (int p = rg; p < parts; p += kReduceRowGroups) {
        const float m_p = a.part_m[slot0 + p];
        const float l_p = a.part_l[slot0 + p];
        const float4 *row = reinterpret_cast<const float4 *>(a.part_acc + (slot0 + p) * a.value_size) + c;
        float4 v[kGroups];
#pragma unroll
        for (int i = 0; i < kGroups; ++i) {
            v[i] = row[16 * i];
        }
        const float m_new = fmaxf(m_loc, m_p);
        const float w_old = mergeWeight(m_loc, m_new), w_p = mergeWeight(m_p, m_new);
        l_loc = l_loc * w_old + l_p * w_p;
#pragma unroll
        for (int i = 0; i < kGroups; ++i) {
            acc[i].x = acc[i].x * w_old + v[i].x * w_p;
            acc[i].y = acc[i].y * w_old + v[i].y * w_p;
            acc[i].z = acc[i].z * w_old + v[i].z * w_p;
            acc[i].w = acc[i].w * w_old + v[i].w * w_p;
        }
        m_loc = m_new;
    }

    // merge the four row groups of this wavefront (lanes c, c+16, c+32, c+48)
    const float m_w = swapMax(m_loc);
    const float f = mergeWeight(m_loc, m_w);
    const float l_w = swapSum(l_loc * f);
#pragma unroll
    for (int i = 0; i < kGroups; ++i) {
        acc[i].x = swapSum(acc[i].x * f);
        acc[i].y = swapSum(acc[i].y * f);
        acc[i].z = swapSum(acc[i].z * f);
        acc[i].w = swapSum(acc[i].w * f);
    }
    if ((tid & 63) < 16) {
        if (c == 0) {
            wave_m[wave] = m_w; // the 16 strips of a row group went through the same partitions
            wave_l[wave] = l_w;
        }
#pragma unroll
        for (int i = 0; i < kGroups; ++i) {
            wave_acc[wave][i][c] = acc[i];
        }
    }
    __syncthreads();

    // one thread per group of four columns merges the four wavefronts, normalises and stores
    for (int e = tid; e < 16 * kGroups; e += kReduceThreads) {
        const int i = e >> 4, cc = e & 15;
        const float m = fmaxf(fmaxf(wave_m[0], wave_m[1]), fmaxf(wave_m[2], wave_m[3]));
        float l = 0.0f;
        float4 sum = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float fw = mergeWeight(wave_m[w], m);
            const float4 x = wave_acc[w][i][cc];
            l += wave_l[w] * fw;
            sum.x += x.x * fw, sum.y += x.y * fw, sum.z += x.z * fw, sum.w += x.w * fw;
        }
        const float inv_l = 1.0f / (l + 1e-6f);
        S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride + 64 * i + 4 * cc;
        o_ptr[0] = T::fromFloat(sum.x * inv_l);
        o_ptr[1] = T::fromFloat(sum.y * inv_l);
        o_ptr[2] = T::fromFloat(sum.z * inv_l);
        o_ptr[3] = T::fromFloat(sum.w * inv_l);
    }
}

} // namespace op::paged_attention::amd

#endif
