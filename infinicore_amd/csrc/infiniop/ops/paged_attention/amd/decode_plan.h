// Launch plan of the paged-attention decode on AMD Instinct MI355X: which kernel family runs, how the
// sequences are cut into units of work and how large the workspace is. Decided once, at descriptor
// creation, from shapes and the device alone (sequence lengths live in device memory and are never read
// on the host). Host-only code without any HIP dependency, so that the arithmetic can be exercised on a
// machine without a GPU. Takes the place of the launch heuristics in the reference's
// src/infiniop/ops/paged_attention/nvidia/paged_attention_hd128.cu:424-667.
#ifndef INFINICORE_AMD_PA_DECODE_PLAN_H
#define INFINICORE_AMD_PA_DECODE_PLAN_H

#include "../../../devices/amd/amd_device.h"
#include "../info.h"
#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace op::paged_attention::amd {

constexpr int kTileTokens = 16;        // tokens per tile = rows of one matrix instruction
constexpr int kHeadsPerWave = 16;      // query heads of one KV head packed into one wavefront
constexpr int kPageIdsPerWave = 64;    // block-table entries a wavefront holds at a time, one per lane
constexpr int kBalancedMaxSeqs = 1024; // work-equalising schedule: prefix sums of the batch live in LDS
constexpr int kBalancedMaxStartCost = 6; // largest per-sequence start cost (in tiles) that schedule adds to its flat axis
constexpr int kFirstTileInts = 8;      // that schedule: words per wavefront that remember where its first tiles were (32 bytes)
constexpr int kMlaKeySize = 576;       // latent attention: key / query vector
constexpr int kMlaValueSize = 512;     // latent attention: value / output vector
constexpr size_t kGridLimitYZ = 65535; // largest y / z extent of a launch

struct Plan {
    bool tiled;            // tiled matrix-core kernel (head 64 / 128 / 192 / 256 or 576 with values of 512, power-of-two pages >= 16, 16-byte aligned strides)
    bool balanced;         // tiled kernel under the work-equalising schedule (decode_balanced.h)
    bool fused_merge;      // balanced: segments merged inside the decode kernel (no second launch)
    bool latent_wide;      // latent attention on 32-token tiles shared through LDS, units planned per call (decode_mla.h)
    int latent_chunks;     // that kernel: 16-head chunks that share a workgroup: 1 (eight wavefronts for the one chunk), 4 or 8 (a wavefront each)
    bool latent_roles;     // four chunks: a wavefront for the scores and a wavefront for the values of each (decodeMlaRolesKernel)
    bool partition_forced; // INFINIOP_AMD_PA_PARTITION set: the 64-head kernel keeps exactly that size
    int partition_tokens;  // grid schedule: tokens per unit of work
    int max_partitions;    // grid schedule: partitions the longest representable sequence needs
    // A descriptor planned for the work-equalising schedule runs the element-wise kernel when the operands of
    // a call turn out not to be 16-byte aligned. That kernel works on fixed partitions; these are cut so that
    // its partial results fit the workspace the work-equalising schedule asks for.
    int fallback_partition_tokens;
    int fallback_max_partitions;
    int dims_per_lane;     // element-wise kernel: ceil(max(head_size, value_size) / 64)
    int waves_per_stream;  // balanced: wavefronts that share the tiles of one (KV head, 16-head chunk)
    int odd_piece_relief;  // balanced: 256ths of a piece that every odd piece hands to its even neighbour
    // Workspace regions, each 256-byte aligned: [acc][m][l][pieces][flags][first tiles].
    size_t acc_bytes, ml_bytes, pieces_bytes, flags_bytes, first_tiles_bytes;
    size_t workspaceBytes() const {
        return acc_bytes > 0 ? acc_bytes + 2 * ml_bytes + pieces_bytes + flags_bytes + first_tiles_bytes + 256 : 0;
    }
};

inline size_t alignUp(size_t x, size_t a) { return (x + a - 1) / a * a; }

inline int floorPow2(long long x) {
    int p = 1;
    while (2LL * p <= x) {
        p *= 2;
    }
    return p;
}

inline bool multipleOf8(ptrdiff_t x) { return (x % 8) == 0; }

// Shapes no kernel of this backend can be launched for: the grid schedule and the element-wise kernel put
// sequences and heads on the y / z axes of the launch.
inline bool launchable(const PagedAttentionInfo &in) {
    return in.num_seqs <= kGridLimitYZ && in.num_heads <= kGridLimitYZ;
}

// Environment knobs (all optional, read at descriptor creation only): INFINIOP_AMD_PA_KERNEL=generic,
// INFINIOP_AMD_PA_SCHEDULE=grid|balanced, INFINIOP_AMD_PA_LATENT_KERNEL=wide|rows|narrow, INFINIOP_AMD_PA_LATENT_HEADS=64|128,
// INFINIOP_AMD_PA_PARTITION=<tokens>, INFINIOP_AMD_PA_WAVES_PER_CU=<n>, INFINIOP_AMD_PA_MERGE=kernel|fused,
// INFINIOP_AMD_PA_ODD_RELIEF=<256ths>.
inline Plan makePlan(const PagedAttentionInfo &in, const device::amd::DeviceInfo &dev) {
    Plan plan{};
    const long long bs = static_cast<long long>(in.page_block_size);
    const long long max_tokens = static_cast<long long>(in.max_num_blocks_per_seq) * bs;
    const bool pow2_page = bs >= 16 && (bs & (bs - 1)) == 0;

    const bool tiled_head = in.head_size == 64 || in.head_size == 128 || in.head_size == 192 || in.head_size == 256;
    // heads of 576: latent attention (values of 512), or values as wide as the keys (a shape of the reference's tests,
    // test/infiniop/paged_attention.py:106), which only the kernel on 16-head units of two wavefronts takes
    const bool latent_head = in.head_size == kMlaKeySize && (in.value_size == kMlaValueSize || in.value_size == kMlaKeySize);
    const bool latent_tiles_in_lds = latent_head && in.value_size == kMlaValueSize;
    plan.tiled = ((tiled_head && in.value_size == in.head_size) || latent_head) && pow2_page
              && multipleOf8(in.q_stride) && multipleOf8(in.q_head_stride) && multipleOf8(in.o_stride)
              && multipleOf8(in.o_head_stride) && multipleOf8(in.k_batch_stride) && multipleOf8(in.k_head_stride)
              && multipleOf8(in.k_row_stride) && multipleOf8(in.v_batch_stride) && multipleOf8(in.v_head_stride)
              && multipleOf8(in.v_row_stride) && in.num_blocks > 0 && in.num_blocks <= 0x7fffffff
              && max_tokens < (1LL << 30)
              // lane offsets inside a tile (15 rows + one row of bytes) are kept in 32 bits
              && in.k_row_stride > 0 && in.k_row_stride < (1 << 26) && in.v_row_stride > 0 && in.v_row_stride < (1 << 26);
    if (const char *env = std::getenv("INFINIOP_AMD_PA_KERNEL")) {
        if (std::strcmp(env, "generic") == 0) {
            plan.tiled = false;
        }
    }

    // ---- grid schedule: units of work = sequences x KV heads (x query heads for the element-wise
    // kernel) x partitions. Aim at ~16 units per compute unit for the longest sequences; keep a
    // partition between 64 and 512 tokens.
    const long long group = static_cast<long long>(in.num_heads / in.num_kv_heads);
    const long long stream_count = static_cast<long long>(in.num_kv_heads) * ((group + kHeadsPerWave - 1) / kHeadsPerWave);
    const long long units = static_cast<long long>(in.num_seqs) * (plan.tiled ? stream_count : static_cast<long long>(in.num_heads));
    // A job whose block table cannot hold more than 16 tiles per wavefront of the work-equalising schedule
    // (134 MB of K and V at head 128) is over in 10 - 30 us, and there the fixed partitions win: their
    // wavefronts start with two round trips less and share a SIMD two at a time (one sequence of 2 100
    // tokens: 10.4 vs 15.9 us; 4 ragged sequences: 14.2 vs 18.6; 8: 22.2 vs 22.0; 16: 34.6 vs 33.4).
    const long long max_tiles = (max_tokens + kTileTokens - 1) / kTileTokens;
    const bool small_job = plan.tiled && !latent_head
                        && static_cast<long long>(in.num_seqs) * stream_count * max_tiles <= 64LL * dev.compute_units;
    // A unit of the latent-attention kernel leaves 32 KiB of partial results and advances one tile per
    // ~2 us however many units there are: fewer, longer units measured best there (more units end the
    // decode kernel sooner, but writing and merging their partial results costs more than that gains).
    // Latent attention with more than one 16-head chunk per KV head shares every K / V tile between the chunks of a
    // workgroup, a wavefront per chunk (decodeMlaRowsKernel; measured against the 16-head units, 32 sequences, with
    // the first kernel of the kind: 32 heads 58.1 vs 62.0 us, 48 heads 60 vs 82, 64 heads 64 vs 104, 128 heads 83 vs
    // 165). One workgroup per compute unit there, up to 256 KiB of partial results each: about one round of
    // workgroups measured best. Four chunks (64 heads) per workgroup, or eight where there are more than four and the
    // batch fills the device without cutting the sequences finely: with eight a tile is fetched once for twice the
    // heads, but a unit leaves twice the partial results and there are half as many units to fill the device with
    // (128 heads, 4 vs 8 chunks: 32 sequences 70.2 vs 72.2 us, 64 sequences 136.7 vs 112.0, 128 sequences 276 vs 212,
    // 256 sequences 523 vs 425).
    const long long head_chunks = (group + kHeadsPerWave - 1) / kHeadsPerWave;
    // A single chunk gets all eight wavefronts of a workgroup (decodeMlaChunkKernel) up to 64 sequences x KV
    // heads (16 heads, 1 / 4 / 16 / 32 sequences: 16.0 / 18.9 / 26.2 / 37.8 vs 28.8 / 29.8 / 31.5 / 39.1 us on the
    // 16-head units; 128 sequences: 135.8 vs 134.1).
    plan.latent_wide = plan.tiled && latent_tiles_in_lds
                    && (head_chunks > 1 || static_cast<long long>(in.num_seqs) * in.num_kv_heads <= 64);
    bool latent_rows_forced = false;
    if (const char *env = std::getenv("INFINIOP_AMD_PA_LATENT_KERNEL")) {
        latent_rows_forced = std::strcmp(env, "rows") == 0;
        if (std::strcmp(env, "wide") == 0 || latent_rows_forced) {
            plan.latent_wide = plan.tiled && latent_tiles_in_lds;
        } else if (std::strcmp(env, "narrow") == 0) {
            plan.latent_wide = false;
        }
    }
    plan.latent_chunks = head_chunks <= 1 ? 1 : ((head_chunks > 4 && static_cast<long long>(in.num_seqs) * in.num_kv_heads >= 48) ? 8 : 4);
    if (const char *env = std::getenv("INFINIOP_AMD_PA_LATENT_HEADS")) {
        if (head_chunks > 1 && (std::atoi(env) == 64 || std::atoi(env) == 128)) {
            plan.latent_chunks = std::atoi(env) / kHeadsPerWave;
        }
    }
    // Four chunks per workgroup: K . Q^T with the softmax, and P . V, in different wavefronts of a SIMD, unless the knob
    // asks for one wavefront per chunk (128 heads, 32 sequences: 60.1 vs 66.5 us; 32 / 48 / 64 heads: 46.8 / 51.9 / 53.5
    // vs 48.0 / 51.0 / 55.4; 64 heads, 8 / 64 / 128 sequences: 25.5 / 86.2 / 169 vs 26.2 / 88.2 / 175).
    plan.latent_roles = plan.latent_wide && plan.latent_chunks == 4 && !latent_rows_forced;
    const long long chunks_per_group = plan.latent_chunks;
    const long long wide_units = static_cast<long long>(in.num_seqs) * in.num_kv_heads
                               * ((head_chunks + chunks_per_group - 1) / chunks_per_group);
    long long want = plan.latent_wide ? wide_units * max_tokens / dev.compute_units
                   : latent_head      ? units * max_tokens * 3 / (16LL * dev.compute_units)
                   : small_job        ? units * max_tokens / (8LL * dev.compute_units)
                                      : units * max_tokens / (16LL * dev.compute_units);
    long long p = floorPow2(want < 1 ? 1 : want);
    const long long p_min = plan.latent_wide ? 128 : (latent_head ? 256 : 64);
    p = p < p_min ? p_min : (p > 512 ? 512 : p);
    if (const char *env = std::getenv("INFINIOP_AMD_PA_PARTITION")) {
        const int forced = std::atoi(env);
        if (forced >= 16) {
            p = (forced + 15LL) / 16 * 16;
            plan.partition_forced = true;
        }
    }
    // Bound the workspace: at most 128 partitions.
    if (max_tokens > 128LL * p) {
        p = (max_tokens + 127) / 128;
        p = (p + 15) / 16 * 16;
    }
    // A wavefront of the tiled kernels fetches the page ids of its partition with one load, an entry per
    // lane. A partition whose size is a multiple of the page size starts on a page boundary and spans
    // p / bs entries; any other size can start inside a page and span one entry more. So: at most 64 pages,
    // and sizes above one page are rounded up to whole pages (a size of up to one page spans two entries at
    // most; the element-wise kernel has no such limit).
    if (plan.tiled) {
        if (p > bs) {
            p = (p + bs - 1) / bs * bs;
        }
        const long long cap = kPageIdsPerWave * bs;
        p = p > cap ? cap : p;
    }
    plan.partition_tokens = static_cast<int>(p);
    plan.max_partitions = static_cast<int>(max_tokens > 0 ? (max_tokens + p - 1) / p : 1);
    const size_t widest = in.head_size > in.value_size ? in.head_size : in.value_size;
    plan.dims_per_lane = static_cast<int>((widest + 63) / 64);
    size_t rows = plan.max_partitions > 1 ? in.num_seqs * static_cast<size_t>(plan.max_partitions) : 0;

    // ---- balanced schedule: ragged batches of up to kBalancedMaxSeqs sequences run the tiled kernel
    // with as many wavefronts as fill the device once at one wavefront per SIMD (4 per compute unit,
    // the setting that measured best: every compute unit gets the same number, each wavefront streams
    // as long as possible), each with an equal share of the tiles. The flat tile axis of a stream (all
    // tiles of the batch plus a start cost per sequence) is indexed with 32-bit integers.
    const bool flat_axis_fits = static_cast<long long>(in.num_seqs) * (max_tiles + kBalancedMaxStartCost) < (1LL << 30);
    // (an empty batch or a tensor without heads is a legal call that launches nothing: no plan to make, and the
    // arithmetic below divides by both counts)
    const bool can_balance = plan.tiled && !latent_head && flat_axis_fits && in.num_seqs <= static_cast<size_t>(kBalancedMaxSeqs)
                          && in.num_seqs > 0 && stream_count > 0;
    plan.balanced = can_balance && !small_job;
    if (const char *env = std::getenv("INFINIOP_AMD_PA_SCHEDULE")) {
        if (std::strcmp(env, "grid") == 0) {
            plan.balanced = false;
        } else if (std::strcmp(env, "balanced") == 0) {
            plan.balanced = can_balance;
        }
    }
    plan.fallback_partition_tokens = plan.partition_tokens;
    plan.fallback_max_partitions = plan.max_partitions;
    if (plan.balanced) {
        // one wavefront per SIMD at every head size (head 64, half the bytes per tile, ran two per SIMD until
        // its matrix results stayed in vector registers: now 33.3 us with four per compute unit, 34.0 - 34.7 with eight)
        int waves_per_cu = 4;
        if (const char *env = std::getenv("INFINIOP_AMD_PA_WAVES_PER_CU")) {
            const int forced = std::atoi(env);
            waves_per_cu = forced >= 1 && forced <= 64 ? forced : waves_per_cu;
        }
        const long long wps = static_cast<long long>(dev.compute_units) * waves_per_cu / stream_count;
        plan.waves_per_stream = static_cast<int>(wps < 1 ? 1 : wps);
        rows = static_cast<size_t>(plan.waves_per_stream) + in.num_seqs;
        plan.pieces_bytes = alignUp(in.num_seqs * 2 * sizeof(int), 256);
        // Workgroups go to the eight accelerator dies round-robin by linear id, so with an even number of pieces
        // per stream the odd pieces run on the odd dies, and on every MI355X measured (four of them) the odd die
        // of each pair streams the head-128 and head-192 kernels 5 - 9 % slower than the even one (per-die median
        // time in the tile loop at the Llama-3-8B batch-32 shape: 41.5 vs 44.5 us at head 128, 63 vs 66 us at
        // head 192; none at heads 64 and 256). Every odd piece therefore hands a fixed share of its slots, in
        // 256ths, to its even neighbour (head 128: 55.45 -> 54.9 us at that shape, 122.0 -> 120.2 us at the
        // long-context shape, 370 -> 362 us at the 70B share; head 192: 78.4 -> 77.4 us; heads 64 and 256 lose with
        // any share). INFINIOP_AMD_PA_ODD_RELIEF=<0..64> overrides it, 0 switches it off.
        plan.odd_piece_relief = in.head_size == 128 ? 16 : (in.head_size == 192 ? 12 : 0);
        if (const char *env = std::getenv("INFINIOP_AMD_PA_ODD_RELIEF")) {
            const int forced = std::atoi(env);
            plan.odd_piece_relief = forced >= 0 && forced <= 64 ? forced : plan.odd_piece_relief;
        }
        if (plan.waves_per_stream % 2 != 0) {
            plan.odd_piece_relief = 0; // pieces do not come in (even die, odd die) pairs
        }
        // Merging inside the decode kernel saves the second launch and pays for it with the readers' dependent
        // round trips at the end of the kernel, one batch of four segments after the other: it wins where a
        // sequence is cut into few segments and the call is short. Measured, second kernel vs merged inside
        // (us per call): 128 sequences of 1 024 - 8 192 tokens on 128 pieces per stream 362.3 vs 360.7 at head
        // 128, 193.1 vs 190.9 at head 64; 32 sequences of 512 - 4 096 tokens 33.1 vs 31.6 at head 64 but 55.4 vs
        // 55.6 at head 128 and 77.4 vs 79.6 at head 192; 8 sequences of 16 384 - 32 768 tokens 67.8 vs 70.4 at
        // head 64; head 256 always loses (102 vs 133).
        const long long pieces = plan.waves_per_stream;
        // With up to four heads per KV head the reader has eight segments in flight instead of four, and sequences cut
        // into twice as many segments still gain: head 64, 16 sequences 20.2 vs 21.3 us (8: 15.7 vs 15.8); head 128, 64
        // sequences 102.5 vs 103.4 (32: 56.4 vs 56.8 in that run, 55.6 vs 55.4 in the benchmark: left to the second
        // kernel; 16: 31.9 vs 31.6).
        const long long reach = group <= 4 ? 2 : 1;
        plan.fused_merge = (in.head_size == 64 && pieces <= 4LL * reach * static_cast<long long>(in.num_seqs))
                        || (in.head_size == 128 && pieces <= reach * static_cast<long long>(in.num_seqs));
        if (const char *env = std::getenv("INFINIOP_AMD_PA_MERGE")) {
            if (std::strcmp(env, "fused") == 0) {
                plan.fused_merge = true;
            } else if (std::strcmp(env, "kernel") == 0) {
                plan.fused_merge = false;
            }
        }
        // one flag per (row, stream), whichever way the merge runs (the knob must not change the size)
        plan.flags_bytes = alignUp(rows * static_cast<size_t>(stream_count) * sizeof(unsigned long long), 256);
        plan.first_tiles_bytes = alignUp(static_cast<size_t>(plan.waves_per_stream) * static_cast<size_t>(stream_count)
                                             * kFirstTileInts * sizeof(int), 256);
        // the element-wise kernel's rows are (sequence, partition): as many partitions as those rows hold
        long long fallback = static_cast<long long>(rows / in.num_seqs);
        fallback = fallback > plan.max_partitions ? plan.max_partitions : fallback;
        long long fp = max_tokens > 0 ? (max_tokens + fallback - 1) / fallback : 1;
        fp = fp < plan.partition_tokens ? plan.partition_tokens : fp;
        plan.fallback_partition_tokens = static_cast<int>(fp);
        plan.fallback_max_partitions = static_cast<int>(max_tokens > 0 ? (max_tokens + fp - 1) / fp : 1);
    }
    if (plan.latent_wide) {
        plan.pieces_bytes = 256; // the partition size the decode kernel chose, for the merge kernel
    }
    if (rows > 0) {
        plan.acc_bytes = alignUp(rows * in.num_heads * in.value_size * sizeof(float), 256);
        plan.ml_bytes = alignUp(rows * in.num_heads * sizeof(float), 256);
    }
    return plan;
}

} // namespace op::paged_attention::amd

#endif
