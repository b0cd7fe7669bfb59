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
    int2 *seq_pieces; // work-equalising schedule, merge by a second kernel: per sequence {first piece, number of pieces}
    // work-equalising schedule, merge inside the decode kernel: one word per partial row group
    // [(piece + sequence) x streams]; it holds `token` once the rows of that segment are complete in memory
    unsigned long long *seg_flags;
    unsigned long long token; // differs from call to call (a replayed graph repeats it: flags are cleared by their reader)
    // work-equalising schedule: per wavefront [piece x stream] kFirstTileInts words, the (page, first row) pairs of
    // the tiles its pipeline started with in the last call; any content is legal (a guess, checked before use)
    int32_t *first_tiles;
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
    int32_t odd_piece_relief; // work-equalising schedule: odd pieces hand this many 256ths of a piece to their even neighbour

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

// ---- hand-over of data between wavefronts of one kernel ----
// Each of the eight accelerator dies (XCDs) has its own L2, and the L2s are not kept coherent with one another
// for ordinary accesses inside a kernel: an ordinary store stays in the writer's L2 until the kernel ends, and an
// ordinary load may be served from the reader's own L1 / L2 copy of the line. Accesses with the sc1 bit
// ("agent scope") are the ones that work across dies: such a store is written through to memory and such a
// load is served from memory, past both caches. Measured with a ping-pong of 1 KiB rows between wavefronts
// on different dies (and on the same die), the reader's caches holding the previous round's lines: sc1 stores +
// `s_waitcnt vmcnt(0)` + an sc1 flag store, against an sc1 poll of the flag followed by sc1 loads of the rows:
// 0 wrong words in 3.4e7 hand-overs, ~1 us per hand-over on an idle device; with ordinary stores or ordinary
// loads on either side every hand-over between dies reads stale data.
// Rows travel 16 bytes per lane through raw buffer accesses that carry the sc1 bit (the compiler knows these
// instructions, so its wait-count bookkeeping covers them); the buffer descriptor holds a wave-uniform base
// and a size, lanes whose offset lies beyond the size store nothing and load zeros. Flags are relaxed atomics
// of agent scope, which compile to global_load / global_store ... sc1.
constexpr int kAgentScope = 16; // cache-policy operand of the raw buffer builtins: sc1
typedef unsigned agent_u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned agent_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t agentBuffer(const void *uniform_base, int bytes) {
    const uint64_t b = reinterpret_cast<uint64_t>(uniform_base);
    // (the lane read returns a signed int: widen both halves as unsigned, or a low half with its top bit set
    // would smear ones over the high half)
    const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b >> 32)));
    const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b)));
    const uint64_t u = (static_cast<uint64_t>(hi) << 32) | lo;
    return __builtin_amdgcn_make_buffer_rsrc(reinterpret_cast<void *>(u), 0, bytes, 0x00020000);
}
__device__ __forceinline__ void storeAgent16(__amdgpu_buffer_rsrc_t buffer, int byte_offset, float a, float b, float c, float d) {
    const agent_u32x4 w = {__float_as_uint(a), __float_as_uint(b), __float_as_uint(c), __float_as_uint(d)};
    __builtin_amdgcn_raw_buffer_store_b128(w, buffer, byte_offset, 0, kAgentScope);
}
__device__ __forceinline__ void storeAgent8(__amdgpu_buffer_rsrc_t buffer, int byte_offset, float a, float b) {
    const agent_u32x2 w = {__float_as_uint(a), __float_as_uint(b)};
    __builtin_amdgcn_raw_buffer_store_b64(w, buffer, byte_offset, 0, kAgentScope);
}
__device__ __forceinline__ float4 loadAgent16(__amdgpu_buffer_rsrc_t buffer, int byte_offset) {
    const agent_u32x4 w = __builtin_amdgcn_raw_buffer_load_b128(buffer, byte_offset, 0, kAgentScope);
    return make_float4(__uint_as_float(w[0]), __uint_as_float(w[1]), __uint_as_float(w[2]), __uint_as_float(w[3]));
}
__device__ __forceinline__ float2 loadAgent8(__amdgpu_buffer_rsrc_t buffer, int byte_offset) {
    const agent_u32x2 w = __builtin_amdgcn_raw_buffer_load_b64(buffer, byte_offset, 0, kAgentScope);
    return make_float2(__uint_as_float(w[0]), __uint_as_float(w[1]));
}
__device__ __forceinline__ void storeAgent(unsigned long long *p, unsigned long long v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long loadAgent(const unsigned long long *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// Every vector memory operation this wavefront has issued is complete: loads have delivered, stores have been
// written (agent-scope stores: to memory). Also a barrier for the compiler's own reordering of memory accesses.
__device__ __forceinline__ void waitVectorMemory() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void compilerMemoryBarrier() { asm volatile("" ::: "memory"); }

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
