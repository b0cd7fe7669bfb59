// paged_attention (decode) on AMD Instinct MI355X: descriptor, launch plan and launches.
// Takes the place of the reference's nvidia backend host code
// (src/infiniop/ops/paged_attention/nvidia/paged_attention_nvidia.cu:182-443 and
// nvidia/paged_attention_hd128.cu:424-923) for the AMD device.
#include "paged_attention_amd.h"
#include "../../../handle.h"
#include "../../../../utils/check.h"
#include "../../../devices/amd/amd_device.h"
#include "decode_common.h"
#include "decode_generic.h"
#include "decode_reduce.h"
#include "decode_balanced.h"
#include "decode_tiled.h"
#include "decode_mla.h" // after decode_balanced.h: shares its diagnostic timestamp buffer
#include <cstdlib>
#include <cstring>

namespace op::paged_attention::amd {

namespace {

// Decided once, at descriptor creation, from shapes and the device alone (sequence lengths live in
// device memory and are never read on the host).
struct Plan {
    bool tiled;            // tiled matrix-core kernel (head 64 / 128 / 192 / 256 or 576 with values of 512, power-of-two pages >= 16, 16-byte aligned strides)
    bool balanced;         // tiled kernel under the work-equalising schedule (decode_balanced.h)
    bool latent_wide;      // latent attention with more than 16 query heads per KV head: up to 64 heads per workgroup
    bool partition_forced; // INFINIOP_AMD_PA_PARTITION set: the 64-head kernel keeps exactly that size
    int partition_tokens;  // grid schedule: tokens per unit of work
    int max_partitions;    // grid schedule: partitions the longest representable sequence needs
    int dims_per_lane;     // element-wise kernel: ceil(max(head_size, value_size) / 64)
    int waves_per_stream;  // balanced: wavefronts that share the tiles of one (KV head, 16-head chunk)
    // Workspace regions, each 256-byte aligned: [acc][m][l][pieces]. A descriptor planned for the
    // balanced schedule can still be run with the element-wise kernel (operands that turn out not
    // to be 16-byte aligned), so the regions are sized for whichever schedule needs more.
    size_t acc_bytes, ml_bytes, pieces_bytes;
    size_t workspaceBytes() const { return acc_bytes > 0 ? acc_bytes + 2 * ml_bytes + pieces_bytes + 256 : 0; }
};

size_t alignUp(size_t x, size_t a) { return (x + a - 1) / a * a; }

int floorPow2(long long x) {
    int p = 1;
    while (2LL * p <= x) {
        p *= 2;
    }
    return p;
}

bool multipleOf8(ptrdiff_t x) { return (x % 8) == 0; }

Plan makePlan(const PagedAttentionInfo &in, const device::amd::DeviceInfo &dev) {
    Plan plan{};
    const long long bs = static_cast<long long>(in.page_block_size);
    const long long max_tokens = static_cast<long long>(in.max_num_blocks_per_seq) * bs;
    const bool pow2_page = bs >= 16 && (bs & (bs - 1)) == 0;

    const bool tiled_head = in.head_size == 64 || in.head_size == 128 || in.head_size == 192 || in.head_size == 256;
    const bool latent_head = in.head_size == kMlaKeySize && in.value_size == kMlaValueSize;
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
    // Latent attention with more than one 16-head chunk per KV head runs up to 64 heads per workgroup
    // (measured against the 16-head units, 32 sequences: 16 heads 54.4 vs 40.7 us, 32 heads 58.1 vs 62.0,
    // 48 heads 60 vs 82, 64 heads 64 vs 104, 128 heads 83 vs 165; 128 sequences of 32 heads 163 vs 245, of
    // 128 heads 314 vs 708). One workgroup per compute unit there, up to 128 KiB of partial results each:
    // about one round of workgroups measured best.
    const long long head_chunks = (group + kHeadsPerWave - 1) / kHeadsPerWave;
    // A single chunk gets all eight wavefronts of such a workgroup (decodeMlaWideKernel<.., 1>) up to 64
    // sequences x KV heads (16 heads, 1 / 4 / 16 / 32 sequences: 16.0 / 18.9 / 26.2 / 37.8 vs 28.8 / 29.8 /
    // 31.5 / 39.1 us on the 16-head units; 128 sequences: 135.8 vs 134.1).
    plan.latent_wide = plan.tiled && latent_head
                    && (head_chunks > 1 || static_cast<long long>(in.num_seqs) * in.num_kv_heads <= 64);
    if (const char *env = std::getenv("INFINIOP_AMD_PA_LATENT_KERNEL")) {
        if (std::strcmp(env, "wide") == 0) {
            plan.latent_wide = plan.tiled && latent_head;
        } else if (std::strcmp(env, "narrow") == 0) {
            plan.latent_wide = false;
        }
    }
    const long long wide_units = static_cast<long long>(in.num_seqs) * in.num_kv_heads
                               * ((head_chunks + kMlaWideChunks - 1) / kMlaWideChunks);
    long long want = plan.latent_wide ? wide_units * max_tokens / dev.compute_units
                   : latent_head      ? units * max_tokens * 3 / (16LL * dev.compute_units)
                   : small_job        ? units * max_tokens / (8LL * dev.compute_units)
                                      : units * max_tokens / (16LL * dev.compute_units);
    int p = floorPow2(want < 1 ? 1 : want);
    const int p_min = plan.latent_wide ? 128 : (latent_head ? 256 : 64);
    p = p < p_min ? p_min : (p > 512 ? 512 : p);
    if (const char *env = std::getenv("INFINIOP_AMD_PA_PARTITION")) {
        const int forced = std::atoi(env);
        if (forced >= 16) {
            p = (forced + 15) / 16 * 16;
            plan.partition_forced = true;
        }
    }
    // Bound the workspace: at most 128 partitions, unless that would exceed what one wavefront of
    // the tiled kernel can address through its single page-id load (64 table entries).
    const long long cap = plan.tiled ? 64 * bs : (1LL << 30);
    if (max_tokens > 128LL * p) {
        long long grown = (max_tokens + 127) / 128;
        grown = (grown + 15) / 16 * 16;
        p = static_cast<int>(grown);
    }
    if (p > cap) {
        p = static_cast<int>(cap);
    }
    plan.partition_tokens = p;
    plan.max_partitions = static_cast<int>(max_tokens > 0 ? (max_tokens + p - 1) / p : 1);
    const size_t widest = in.head_size > in.value_size ? in.head_size : in.value_size;
    plan.dims_per_lane = static_cast<int>((widest + 63) / 64);
    size_t rows = plan.max_partitions > 1 ? in.num_seqs * static_cast<size_t>(plan.max_partitions) : 0;

    // ---- balanced schedule: ragged batches of up to kBalancedMaxSeqs sequences run the tiled kernel
    // with as many wavefronts as fill the device once at one wavefront per SIMD (4 per compute unit,
    // the setting that measured best: every compute unit gets the same number, each wavefront streams
    // as long as possible), each with an equal share of the tiles.
    plan.balanced = plan.tiled && !latent_head && !small_job && in.num_seqs <= static_cast<size_t>(kBalancedMaxSeqs);
    if (const char *env = std::getenv("INFINIOP_AMD_PA_SCHEDULE")) {
        if (std::strcmp(env, "grid") == 0) {
            plan.balanced = false;
        } else if (std::strcmp(env, "balanced") == 0) {
            plan.balanced = plan.tiled && !latent_head && in.num_seqs <= static_cast<size_t>(kBalancedMaxSeqs);
        }
    }
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
        const size_t balanced_rows = static_cast<size_t>(plan.waves_per_stream) + in.num_seqs;
        rows = rows > balanced_rows ? rows : balanced_rows;
        plan.pieces_bytes = alignUp(in.num_seqs * 2 * sizeof(int), 256);
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

template <typename T, typename Tindex>
void launchGeneric(const DecodeArgs &a, const Plan &plan, hipStream_t stream) {
    const dim3 grid(plan.max_partitions, a.num_heads, a.num_seqs);
    switch (plan.dims_per_lane) {
    case 1: decodeGenericKernel<T, Tindex, 1><<<grid, 64, 0, stream>>>(a); break;
    case 2: decodeGenericKernel<T, Tindex, 2><<<grid, 64, 0, stream>>>(a); break;
    case 3: decodeGenericKernel<T, Tindex, 3><<<grid, 64, 0, stream>>>(a); break;
    case 4: decodeGenericKernel<T, Tindex, 4><<<grid, 64, 0, stream>>>(a); break;
    default: decodeGenericKernel<T, Tindex, 9><<<grid, 64, 0, stream>>>(a); break;
    }
}

template <typename T, typename Tindex>
void launchReduce(const DecodeArgs &a, hipStream_t stream) {
    if (a.max_partitions <= 8) {
        // few partitions per sequence: one wavefront per (head, sequence) (up to 8: m2 14.6 -> 8.2 us; with
        // 16, of which m1 uses up to 16, the workgroup-per-row kernel is the faster one: 4.7 vs 5.4 us)
        const long long pairs = static_cast<long long>(a.num_heads) * a.num_seqs;
        const dim3 few(static_cast<unsigned>((pairs + 3) / 4));
        switch (a.value_size / 64) {
        case 1: decodeReduceWaveKernel<T, Tindex, 64><<<few, kReduceThreads, 0, stream>>>(a); break;
        case 2: decodeReduceWaveKernel<T, Tindex, 128><<<few, kReduceThreads, 0, stream>>>(a); break;
        case 3: decodeReduceWaveKernel<T, Tindex, 192><<<few, kReduceThreads, 0, stream>>>(a); break;
        case 4: decodeReduceWaveKernel<T, Tindex, 256><<<few, kReduceThreads, 0, stream>>>(a); break;
        case 8: decodeReduceWaveKernel<T, Tindex, 512><<<few, kReduceThreads, 0, stream>>>(a); break;
        default: decodeReduceWaveKernel<T, Tindex, 576><<<few, kReduceThreads, 0, stream>>>(a); break;
        }
        return;
    }
    const dim3 grid(a.num_heads, a.num_seqs);
    switch (a.value_size / 16) { // value sizes the validator lets through: 64, 128, 192, 256, 512, 576
    case 4: decodeReduceKernel<T, Tindex, 4><<<grid, kReduceThreads, 0, stream>>>(a); break;
    case 8: decodeReduceKernel<T, Tindex, 8><<<grid, kReduceThreads, 0, stream>>>(a); break;
    case 12: decodeReduceKernel<T, Tindex, 12><<<grid, kReduceThreads, 0, stream>>>(a); break;
    case 16: decodeReduceKernel<T, Tindex, 16><<<grid, kReduceThreads, 0, stream>>>(a); break;
    case 32: decodeReduceKernel<T, Tindex, 32><<<grid, kReduceThreads, 0, stream>>>(a); break;
    default: decodeReduceKernel<T, Tindex, 36><<<grid, kReduceThreads, 0, stream>>>(a); break;
    }
}

// The tiled kernels of one head size: work-equalising schedule + merge, or fixed partitions.
template <typename T, typename Tindex, int HEAD>
void launchTiled(const DecodeArgs &a, const Plan &plan, hipStream_t stream) {
    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    if (plan.balanced) {
        const dim3 grid(plan.waves_per_stream, a.num_kv_heads * head_chunks);
        decodeBalancedKernel<T, Tindex, HEAD><<<grid, 64, 0, stream>>>(a.seq_lens, a.num_seqs, a.max_blocks_per_seq,
                                                                       a.block_shift, a, plan.waves_per_stream);
        decodeBalancedMergeKernel<T, Tindex, HEAD><<<dim3((a.num_heads + 3) / 4, a.num_seqs), 256, 0, stream>>>(
            a.seq_lens, a.seq_pieces, a.num_heads, a);
    } else {
        const dim3 grid(plan.max_partitions, a.num_kv_heads * head_chunks, a.num_seqs);
        decodeTiledKernel<T, Tindex, HEAD><<<grid, 64, 0, stream>>>(a);
    }
}

template <typename T, typename Tindex>
void launchAll(const DecodeArgs &a, const Plan &plan, bool tiled, hipStream_t stream) {
    if (tiled) {
        switch (a.head_size) {
        case 64: launchTiled<T, Tindex, 64>(a, plan, stream); break;
        case 128: launchTiled<T, Tindex, 128>(a, plan, stream); break;
        case 192: launchTiled<T, Tindex, 192>(a, plan, stream); break;
        case 256: launchTiled<T, Tindex, 256>(a, plan, stream); break;
        default: {
            const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
            const dim3 grid(plan.max_partitions, a.num_kv_heads * head_chunks, a.num_seqs);
            if (plan.latent_wide) {
                // a single chunk of 16 heads gets the whole workgroup; otherwise four chunks share one
                const bool one_chunk = head_chunks == 1;
                const int groups_of_chunks = one_chunk ? 1 : (head_chunks + kMlaWideChunks - 1) / kMlaWideChunks;
                const int streams = a.num_kv_heads * groups_of_chunks;
                dim3 wide(plan.max_partitions, streams, a.num_seqs);
                if (a.chosen_partition != nullptr) {
                    // units planned by the kernel from the actual lengths: at most one per (sequence, planned partition)
                    const long long units = static_cast<long long>(a.num_seqs) * plan.max_partitions;
                    wide = dim3(static_cast<unsigned>((units + 7) / 8 * 8 * streams));
                }
                if (one_chunk) {
                    decodeMlaWideKernel<T, Tindex, 1><<<wide, kMlaWideThreads, 0, stream>>>(a);
                } else {
                    decodeMlaWideKernel<T, Tindex, kMlaWideChunks><<<wide, kMlaWideThreads, 0, stream>>>(a);
                }
                break;
            }
            decodeMlaKernel<T, Tindex><<<grid, kMlaThreads, 0, stream>>>(a);
            break;
        }
        }
        if (plan.balanced) {
            return; // merged by its own kernel
        }
    } else {
        launchGeneric<typename T::Base, Tindex>(a, plan, stream);
    }
    if (plan.max_partitions > 1) {
        launchReduce<typename T::Base, Tindex>(a, stream);
    }
}

template <typename T>
infiniStatus_t launchByIndex(infiniDtype_t index_dtype, const DecodeArgs &a, const Plan &plan, bool tiled,
                             hipStream_t stream) {
    switch (index_dtype) {
    case INFINI_DTYPE_I64: launchAll<T, IndexI64>(a, plan, tiled, stream); break;
    case INFINI_DTYPE_I32: launchAll<T, IndexI32>(a, plan, tiled, stream); break;
    case INFINI_DTYPE_U32: launchAll<T, IndexU32>(a, plan, tiled, stream); break;
    default: return INFINI_STATUS_BAD_TENSOR_DTYPE;
    }
    return INFINI_STATUS_SUCCESS;
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

} // namespace

#ifdef INFINIOP_AMD_PA_TRACE
// Diagnostic build only: point the decode kernel's timestamp buffer at device memory.
extern "C" __attribute__((visibility("default"))) int infiniopAmdPaTraceSet(void *device_buffer) {
    return static_cast<int>(hipMemcpyToSymbol(HIP_SYMBOL(g_pa_trace), &device_buffer, sizeof(void *)));
}
// Diagnostic build only: workgroups of the balanced decode kernel the runtime expects to fit on one compute unit.
extern "C" __attribute__((visibility("default"))) int infiniopAmdPaOccupancy() {
    int blocks = -1;
    hipFuncAttributes attr{};
    (void)hipFuncGetAttributes(&attr, reinterpret_cast<const void *>(&decodeBalancedKernel<TileBF16, IndexI64, 128>));
    std::fprintf(stderr, "decodeBalancedKernel: numRegs=%d sharedSizeBytes=%zu localSizeBytes=%zu maxThreadsPerBlock=%d\n",
                 attr.numRegs, attr.sharedSizeBytes, attr.localSizeBytes, attr.maxThreadsPerBlock);
    (void)hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, decodeBalancedKernel<TileBF16, IndexI64, 128>, 64, 0);
    return blocks;
}
#endif

struct Descriptor::Opaque {
    Plan plan;
};

Descriptor::~Descriptor() { delete _opaque; }

infiniStatus_t Descriptor::create(infiniopHandle_t handle, Descriptor **desc_ptr, infiniopTensorDescriptor_t out_desc,
                                  infiniopTensorDescriptor_t q_desc, infiniopTensorDescriptor_t k_cache_desc,
                                  infiniopTensorDescriptor_t v_cache_desc, infiniopTensorDescriptor_t block_tables_desc,
                                  infiniopTensorDescriptor_t seq_lens_desc, infiniopTensorDescriptor_t alibi_slopes_desc,
                                  float scale) {
    auto info = PagedAttentionInfo::create(out_desc, q_desc, k_cache_desc, v_cache_desc, block_tables_desc,
                                           seq_lens_desc, alibi_slopes_desc, scale);
    CHECK_RESULT(info);
    const PagedAttentionInfo in = info.take();
    const Plan plan = makePlan(in, device::amd::deviceInfo(handle->device_id));
    // includes 256 spare bytes that let calculate() align the carve-up itself, whatever pointer the caller passes
    const size_t workspace_bytes = plan.workspaceBytes();
    *desc_ptr = new Descriptor(new Opaque{plan}, in, workspace_bytes, handle->device, handle->device_id);
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t Descriptor::calculate(void *workspace, size_t workspace_size, void *out, const void *q,
                                     const void *k_cache, const void *v_cache, const void *block_tables,
                                     const void *seq_lens, const void *alibi_slopes, void *stream_) const {
    const PagedAttentionInfo &in = _info;
    const Plan &plan = _opaque->plan;
    if (workspace_size < _workspace_size || (_workspace_size > 0 && workspace == nullptr)) {
        return INFINI_STATUS_INSUFFICIENT_WORKSPACE;
    }
    if (in.num_seqs == 0 || in.num_heads == 0) {
        return INFINI_STATUS_SUCCESS;
    }
    if (out == nullptr || q == nullptr || k_cache == nullptr || v_cache == nullptr || block_tables == nullptr
        || seq_lens == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (in.has_alibi && alibi_slopes == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (in.max_num_blocks_per_seq == 0 || in.num_blocks == 0) {
        return INFINI_STATUS_SUCCESS; // no sequence can hold a token
    }

    DecodeArgs a{};
    a.out = out;
    a.q = q;
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.block_tables = block_tables;
    a.seq_lens = seq_lens;
    a.alibi_slopes = static_cast<const float *>(alibi_slopes);
    if (plan.acc_bytes > 0) {
        char *ws = reinterpret_cast<char *>((reinterpret_cast<uintptr_t>(workspace) + 255) & ~static_cast<uintptr_t>(255));
        a.part_acc = reinterpret_cast<float *>(ws);
        a.part_m = reinterpret_cast<float *>(ws + plan.acc_bytes);
        a.part_l = reinterpret_cast<float *>(ws + plan.acc_bytes + plan.ml_bytes);
        a.seq_pieces = reinterpret_cast<int2 *>(ws + plan.acc_bytes + 2 * plan.ml_bytes);
        if (plan.latent_wide && !plan.partition_forced && in.num_seqs <= 256 && plan.tiled && aligned16(out) && aligned16(q) && aligned16(k_cache) && aligned16(v_cache)) {
            a.chosen_partition = reinterpret_cast<int32_t *>(ws + plan.acc_bytes + 2 * plan.ml_bytes);
        }
    }
    a.scale_log2 = in.scale * kLog2e;
    a.num_seqs = static_cast<int32_t>(in.num_seqs);
    a.num_heads = static_cast<int32_t>(in.num_heads);
    a.num_kv_heads = static_cast<int32_t>(in.num_kv_heads);
    a.group = static_cast<int32_t>(in.num_heads / in.num_kv_heads);
    a.head_size = static_cast<int32_t>(in.head_size);
    a.value_size = static_cast<int32_t>(in.value_size);
    a.block_size = static_cast<int32_t>(in.page_block_size);
    a.block_shift = -1;
    if (in.page_block_size > 0 && (in.page_block_size & (in.page_block_size - 1)) == 0) {
        a.block_shift = __builtin_ctzll(in.page_block_size);
    }
    a.num_blocks = static_cast<int32_t>(in.num_blocks > 0x7fffffff ? 0x7fffffff : in.num_blocks);
    a.max_blocks_per_seq = static_cast<int32_t>(in.max_num_blocks_per_seq);
    a.partition_tokens = plan.partition_tokens;
    a.max_partitions = plan.max_partitions;
    a.compute_units = device::amd::deviceInfo(device_id).compute_units;
    a.q_stride = in.q_stride;
    a.q_head_stride = in.q_head_stride;
    a.o_stride = in.o_stride;
    a.o_head_stride = in.o_head_stride;
    a.k_batch_stride = in.k_batch_stride;
    a.k_head_stride = in.k_head_stride;
    a.k_row_stride = in.k_row_stride;
    a.v_batch_stride = in.v_batch_stride;
    a.v_head_stride = in.v_head_stride;
    a.v_row_stride = in.v_row_stride;
    a.block_table_batch_stride = in.block_table_batch_stride;

    // The tiled kernel moves 16 bytes per lane; base addresses that are not 16-byte aligned take
    // the element-wise kernel instead.
    const bool tiled = plan.tiled && aligned16(out) && aligned16(q) && aligned16(k_cache) && aligned16(v_cache);
    auto stream = static_cast<hipStream_t>(stream_);

    infiniStatus_t status;
    if (in.dtype == INFINI_DTYPE_F16) {
        status = launchByIndex<TileF16>(in.index_dtype, a, plan, tiled, stream);
    } else {
        status = launchByIndex<TileBF16>(in.index_dtype, a, plan, tiled, stream);
    }
    if (status != INFINI_STATUS_SUCCESS) {
        return status;
    }
    return hipGetLastError() == hipSuccess ? INFINI_STATUS_SUCCESS : INFINI_STATUS_INTERNAL_ERROR;
}

} // namespace op::paged_attention::amd
