// Shared vocabulary of the paged-attention decode kernels: the argument block, index loads for the
// three index dtypes, and storage-dtype <-> fp32 conversions.
#ifndef INFINICORE_AMD_PA_DECODE_COMMON_H
#define INFINICORE_AMD_PA_DECODE_COMMON_H

#include "decode_plan.h"
#include <cstdint>
#include <hip/hip_runtime.h>

namespace op::paged_attention::amd {

constexpr float kLog2e = 1.4426950408889634f;

// Scores are kept in the log2 domain (score * log2(e)), so the softmax uses exp2 directly, as the
// reference kernels do (src/infiniop/ops/paged_attention/cuda/kernel_v2.cuh:174-175,272-278).
//
// Long sequences are cut into partitions of `partition_tokens` tokens. A partition is one unit of
// work of the decode kernel and yields, per query head, an un-normalised accumulator
// acc = sum 2^(s_t - m) * v_t, the running maximum m and the sum l = sum 2^(s_t - m). A sequence
// that fits in one partition is normalised and written to `out` by the decode kernel itself; longer
// ones leave (acc, m, l) per partition in the workspace and the reduce kernel merges them.
struct DecodeArgs {
    void *out;
    const void *q;
    const void *k_cache;
    const void *v_cache;
    const void *block_tables;
    const void *seq_lens;
    const float *alibi_slopes; // nullptr = no ALiBi

    // workspace, all fp32; index of (seq, head, partition) = (seq * num_heads + head) * max_partitions + partition
    float *part_acc; // [.., value_size]
    float *part_m;
    float *part_l;
    int2 *seq_pieces; // work-equalising schedule only: per sequence {first piece, number of pieces}
    // 64-head latent-attention kernel only: the partition size the decode kernel settled on for this
    // call (>= partition_tokens), written by its first workgroup for the merge kernel; else nullptr
    int32_t *chosen_partition;

    float scale_log2; // scale * log2(e)
    int32_t num_seqs;
    int32_t num_heads;
    int32_t num_kv_heads;
    int32_t group;        // query heads per KV head
    int32_t head_size;
    int32_t value_size;
    int32_t block_size;
    int32_t block_shift;  // log2(block_size) if a power of two, else -1
    int32_t num_blocks;   // pool size; table entries are clamped into [0, num_blocks)
    int32_t max_blocks_per_seq;
    int32_t partition_tokens;
    int32_t max_partitions;
    int32_t compute_units; // of the device the call runs on

    // element strides
    int64_t q_stride, q_head_stride;
    int64_t o_stride, o_head_stride;
    int64_t k_batch_stride, k_head_stride, k_row_stride;
    int64_t v_batch_stride, v_head_stride, v_row_stride;
    int64_t block_table_batch_stride;
};

// ---- index tensors: I64, I32 or U32 ----
struct IndexI64 { using type = int64_t; };
struct IndexI32 { using type = int32_t; };
struct IndexU32 { using type = uint32_t; };

template <typename Tindex>
__device__ __forceinline__ int64_t loadIndex(const void *base, int64_t i) {
    return static_cast<int64_t>(static_cast<const typename Tindex::type *>(base)[i]);
}

// A page id read from the block table, forced into the pool so that a corrupt table can produce a
// wrong answer but never an out-of-bounds access.
__device__ __forceinline__ int32_t clampPage(int64_t page, int32_t num_blocks) {
    page = page < 0 ? 0 : page;
    return static_cast<int32_t>(page >= num_blocks ? num_blocks - 1 : page);
}

// ---- storage dtypes ----
struct Half {
    using storage = _Float16;
    static __device__ __forceinline__ float toFloat(storage x) { return static_cast<float>(x); }
    static __device__ __forceinline__ storage fromFloat(float x) { return static_cast<storage>(x); } // RNE
};
struct BFloat16 {
    using storage = __bf16;
    static __device__ __forceinline__ float toFloat(storage x) { return static_cast<float>(x); }
    static __device__ __forceinline__ storage fromFloat(float x) { return static_cast<storage>(x); } // RNE
};

__device__ __forceinline__ float fastExp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Sum / max over the 64 lanes of a wavefront; every lane receives the result.
__device__ __forceinline__ float waveSum(float x) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        x += __shfl_xor(x, offset, 64);
    }
    return x;
}
__device__ __forceinline__ float waveMax(float x) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        x = fmaxf(x, __shfl_xor(x, offset, 64));
    }
    return x;
}

} // namespace op::paged_attention::amd

#endif
