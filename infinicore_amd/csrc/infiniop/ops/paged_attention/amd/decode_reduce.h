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
    const int partition_tokens = a.chosen_partition != nullptr ? a.chosen_partition[0] : a.partition_tokens;
    if (len <= partition_tokens) {
        return; // empty sequence, or already finished by the decode kernel (uniform for the workgroup)
    }
    const int parts = (len + partition_tokens - 1) / partition_tokens;
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

// The same merge for calls with few partitions per sequence (the host uses it up to 8): one WAVEFRONT
// per (query head, sequence), four per workgroup. Lane p fetches (m, l) of partition p; the partial rows
// are then added one after the other with every lane on its own columns (column lane * kVec + 64 kVec j:
// every load instruction of the wavefront reads one contiguous piece of a row), all loads independent of
// each other. No LDS, no barrier, and a sequence with three partitions keeps all 64 lanes busy, where the
// kernel above would leave thirteen of its sixteen row groups idle.
template <typename T, typename Tindex, int VALUE>
__global__ void __launch_bounds__(kReduceThreads) decodeReduceWaveKernel(DecodeArgs a) {
    using S = typename T::storage;
    constexpr int kVec = VALUE % 256 == 0 ? 4 : (VALUE % 128 == 0 ? 2 : 1); // floats per load
    constexpr int kLoads = VALUE / (64 * kVec);
    static_assert(kLoads * 64 * kVec == VALUE, "value sizes are multiples of 64");

    const int lane = threadIdx.x & 63;
    const int64_t pair = static_cast<int64_t>(blockIdx.x) * (kReduceThreads / 64) + (threadIdx.x >> 6); // seq * num_heads + head
    if (pair >= static_cast<int64_t>(a.num_seqs) * a.num_heads) {
        return;
    }
    const int seq = static_cast<int>(pair / a.num_heads);
    const int head = static_cast<int>(pair - static_cast<int64_t>(seq) * a.num_heads);
    const int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) * a.block_size;
    const int len = static_cast<int>(len64 < max_len ? len64 : max_len);
    const int partition_tokens = a.chosen_partition != nullptr ? a.chosen_partition[0] : a.partition_tokens;
    if (len <= partition_tokens) {
        return; // empty sequence, or already finished by the decode kernel (uniform for the wavefront)
    }
    const int parts = (len + partition_tokens - 1) / partition_tokens; // <= max_partitions <= 64
    const int64_t slot0 = pair * a.max_partitions;

    const float m_p = lane < parts ? a.part_m[slot0 + lane] : -INFINITY;
    const float l_p = lane < parts ? a.part_l[slot0 + lane] : 0.0f;
    float m = m_p;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        m = fmaxf(m, __shfl_xor(m, off, 64));
    }
    const float w_p = mergeWeight(m_p, m);
    float l = l_p * w_p;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        l += __shfl_xor(l, off, 64);
    }

    float acc[kLoads][kVec];
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
            acc[j][e] = 0.0f;
        }
    }
    // four partial rows per trip, so that their loads are in flight together; a trip past the last
    // partition reads the last row again with weight 0
    for (int p0 = 0; p0 < parts; p0 += 4) {
        float w[4];
        const float *row[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int p = min(p0 + u, parts - 1);
            w[u] = p0 + u < parts ? __shfl(w_p, p, 64) : 0.0f;
            row[u] = a.part_acc + (slot0 + p) * VALUE + lane * kVec;
        }
        float v[4][kLoads][kVec];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                if constexpr (kVec == 4) {
                    const float4 x = *reinterpret_cast<const float4 *>(row[u] + 64 * kVec * j);
                    v[u][j][0] = x.x, v[u][j][1] = x.y, v[u][j][2] = x.z, v[u][j][3] = x.w;
                } else if constexpr (kVec == 2) {
                    const float2 x = *reinterpret_cast<const float2 *>(row[u] + 64 * kVec * j);
                    v[u][j][0] = x.x, v[u][j][1] = x.y;
                } else {
                    v[u][j][0] = row[u][64 * j];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
#pragma unroll
                for (int e = 0; e < kVec; ++e) {
                    acc[j][e] += v[u][j][e] * w[u];
                }
            }
        }
    }
    const float inv_l = 1.0f / (l + 1e-6f);
    S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride + lane * kVec;
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
#pragma unroll
        for (int e = 0; e < kVec; ++e) {
            o_ptr[64 * kVec * j + e] = T::fromFloat(acc[j][e] * inv_l);
        }
    }
}

} // namespace op::paged_attention::amd

#endif
