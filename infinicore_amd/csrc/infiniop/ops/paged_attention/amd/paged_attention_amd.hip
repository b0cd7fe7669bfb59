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
#include "decode_mla.h"
#include "decode_plan.h"
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <mutex>

namespace op::paged_attention::amd {

namespace {

template <typename T, typename Tindex>
void launchGeneric(const DecodeArgs &a, const Plan &plan, hipStream_t stream) {
    const dim3 grid(a.max_partitions, a.num_heads, a.num_seqs);
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
        if (plan.fused_merge) {
            decodeBalancedKernel<T, Tindex, HEAD, true><<<grid, 64, 0, stream>>>(
                a.seq_lens, a.num_seqs, a.max_blocks_per_seq, a.block_shift, a, plan.waves_per_stream);
            return;
        }
        decodeBalancedKernel<T, Tindex, HEAD, false><<<grid, 64, 0, stream>>>(
            a.seq_lens, a.num_seqs, a.max_blocks_per_seq, a.block_shift, a, plan.waves_per_stream);
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
                // a single chunk of 16 heads gets the whole workgroup; otherwise a wavefront per chunk, four or eight
                const int groups_of_chunks = (head_chunks + plan.latent_chunks - 1) / plan.latent_chunks;
                const int streams = a.num_kv_heads * groups_of_chunks;
                dim3 wide(plan.max_partitions, streams, a.num_seqs);
                if (a.chosen_partition != nullptr) {
                    // units planned by the kernel from the actual lengths: at most one per (sequence, planned partition)
                    const long long units = static_cast<long long>(a.num_seqs) * plan.max_partitions;
                    wide = dim3(static_cast<unsigned>((units + 7) / 8 * 8 * streams));
                }
                // one workgroup per (partition, sequence, KV head): its tiles are fetched once
                const bool once = groups_of_chunks == 1;
                if (plan.latent_chunks == 1) {
                    decodeMlaChunkKernel<T, Tindex><<<wide, kMlaWideThreads, 0, stream>>>(a);
                } else if (plan.latent_chunks == 8) {
                    if (once) {
                        decodeMlaRowsKernel<T, Tindex, 8, true><<<wide, 512, 0, stream>>>(a);
                    } else {
                        decodeMlaRowsKernel<T, Tindex, 8, false><<<wide, 512, 0, stream>>>(a);
                    }
                } else if (plan.latent_roles) {
                    if (once) {
                        decodeMlaRolesKernel<T, Tindex, true><<<wide, 512, 0, stream>>>(a);
                    } else {
                        decodeMlaRolesKernel<T, Tindex, false><<<wide, 512, 0, stream>>>(a);
                    }
                } else {
                    decodeMlaRowsKernel<T, Tindex, 4, false><<<wide, 256, 0, stream>>>(a);
                }
                break;
            }
            if (a.value_size == kMlaKeySize) {
                decodeMlaKernel<T, Tindex, kMlaKeySize><<<grid, kMlaThreads, 0, stream>>>(a);
            } else {
                decodeMlaKernel<T, Tindex, kMlaValueSize><<<grid, kMlaThreads, 0, stream>>>(a);
            }
            break;
        }
        }
        if (plan.balanced) {
            return; // merged by its own kernel
        }
    } else {
        launchGeneric<typename T::Base, Tindex>(a, plan, stream);
    }
    if (a.max_partitions > 1) {
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

// A 64-bit value no earlier call of this process has used and that is never 0 (the value of a cleared flag):
// a counter that starts at a point of the clock, spread over the word by an odd multiplier. What a workspace
// holds before its first use can only be mistaken for it by a 2^-64 accident.
unsigned long long nextToken() {
    static std::atomic<unsigned long long> counter{
        static_cast<unsigned long long>(std::chrono::steady_clock::now().time_since_epoch().count()) | 1ull};
    unsigned long long t = counter.fetch_add(1, std::memory_order_relaxed) * 0x9e3779b97f4a7c15ull;
    return t != 0 ? t : 0x9e3779b97f4a7c15ull;
}

} // namespace

// ---- scratch of the entry point that takes no workspace (infiniopPagedAttentionNoAlloc) ----
// One array per GPU, held from the moment the library's code is loaded on that GPU until the process
// ends. In host code the array's name is only a handle for the runtime: the address a kernel can use is
// looked up once per device (with that device current) and kept; every use below goes through that address.
constexpr size_t kScratchBytes = size_t{32} << 20;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {

constexpr int kMaxScratchDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxScratchDevices] = {};

// Device address of this GPU's scratch array; nullptr (and a status) when it cannot be had. The caller's
// current device must be `device_id`: the lookup answers for the current device.
infiniStatus_t scratchAddress(int device_id, void **ptr) {
    *ptr = nullptr;
    if (device_id < 0 || device_id >= kMaxScratchDevices) {
        return INFINI_STATUS_DEVICE_NOT_FOUND;
    }
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[device_id] == nullptr) {
        int current = -1;
        if (hipGetDevice(&current) != hipSuccess || current != device_id) {
            return INFINI_STATUS_BAD_PARAM;
        }
        void *address = nullptr;
        if (hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)) != hipSuccess || address == nullptr) {
            (void)hipGetLastError();
            return INFINI_STATUS_INTERNAL_ERROR;
        }
        g_scratch_ptr[device_id] = address;
    }
    *ptr = g_scratch_ptr[device_id];
    return INFINI_STATUS_SUCCESS;
}

} // namespace

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
    if (!launchable(in)) {
        return INFINI_STATUS_BAD_TENSOR_SHAPE; // more sequences or heads than one launch can index
    }
    const Plan plan = makePlan(in, device::amd::deviceInfo(handle->device_id));
    // includes 256 spare bytes that let calculate() align the carve-up itself, whatever pointer the caller passes
    const size_t workspace_bytes = plan.workspaceBytes();
    *desc_ptr = new Descriptor(new Opaque{plan}, in, workspace_bytes, handle->device, handle->device_id);
    // Set-up for calculateNoAlloc(): look the scratch array up now if this thread is on the descriptor's
    // GPU, so that the first call (which may sit inside a stream capture) finds the address ready. Not an
    // error when it cannot be done here (no GPU visible, another device current): the call does it then.
    if (device::amd::deviceInfo(handle->device_id).queried && workspace_bytes > 0 && workspace_bytes <= kScratchBytes) {
        void *unused = nullptr;
        (void)scratchAddress(handle->device_id, &unused);
    }
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t Descriptor::calculate(void *workspace, size_t workspace_size, void *out, const void *q,
                                     const void *k_cache, const void *v_cache, const void *block_tables,
                                     const void *seq_lens, const void *alibi_slopes, void *stream_) const {
    if (workspace_size < _workspace_size || (_workspace_size > 0 && workspace == nullptr)) {
        return INFINI_STATUS_INSUFFICIENT_WORKSPACE;
    }
    return launch(workspace, out, q, k_cache, v_cache, block_tables, seq_lens, alibi_slopes, stream_);
}

// The call without a workspace argument: partial results go to this GPU's scratch array (32 MiB). Calls
// whose descriptor needs more are refused. Nothing in the array has to start at zero (every row that is
// read was written by the same call), so nothing is cleared; two calls that overlap on one GPU (different
// streams, or threads) share the array and race.
infiniStatus_t Descriptor::calculateNoAlloc(void *out, const void *q, const void *k_cache, const void *v_cache,
                                            const void *block_tables, const void *seq_lens, const void *alibi_slopes,
                                            void *stream_) const {
    if (_workspace_size > kScratchBytes) {
        std::fprintf(stderr,
                     "infiniopPagedAttentionNoAlloc: this descriptor needs %zu bytes of scratch, the built-in array holds "
                     "%zu; use infiniopPagedAttention with a caller-provided workspace\n",
                     _workspace_size, kScratchBytes);
        return INFINI_STATUS_INSUFFICIENT_WORKSPACE;
    }
    void *ptr = nullptr;
    if (_workspace_size > 0) {
        const infiniStatus_t status = scratchAddress(device_id, &ptr);
        if (status != INFINI_STATUS_SUCCESS) {
            return status;
        }
    }
    return launch(ptr, out, q, k_cache, v_cache, block_tables, seq_lens, alibi_slopes, stream_);
}

infiniStatus_t Descriptor::launch(void *workspace, void *out, const void *q, const void *k_cache, const void *v_cache,
                                  const void *block_tables, const void *seq_lens, const void *alibi_slopes,
                                  void *stream_) const {
    const PagedAttentionInfo &in = _info;
    const Plan &plan = _opaque->plan;
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
    // The launches go to the calling thread's current device, and the plan (compute units, wavefronts per
    // stream) was made for the descriptor's: they must be the same.
    int current_device = -1;
    if (hipGetDevice(&current_device) != hipSuccess || current_device != device_id) {
        return INFINI_STATUS_BAD_PARAM;
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
        a.seg_flags = reinterpret_cast<unsigned long long *>(ws + plan.acc_bytes + 2 * plan.ml_bytes + plan.pieces_bytes);
        a.first_tiles = reinterpret_cast<int32_t *>(ws + plan.acc_bytes + 2 * plan.ml_bytes + plan.pieces_bytes + plan.flags_bytes);
        a.token = nextToken();
        // the 64-head latent-attention kernel plans its units per call from the actual lengths and leaves the
        // partition size it chose in the first word of the pieces region, for the merge kernel
        if (plan.latent_wide && !plan.partition_forced && in.num_seqs <= 256 && plan.tiled && aligned16(out) && aligned16(q)
            && aligned16(k_cache) && aligned16(v_cache)) {
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
    // The tiled kernel moves 16 bytes per lane; base addresses that are not 16-byte aligned take
    // the element-wise kernel instead, on partitions cut to fit the workspace of the planned schedule.
    const bool tiled = plan.tiled && aligned16(out) && aligned16(q) && aligned16(k_cache) && aligned16(v_cache);
    a.partition_tokens = tiled ? plan.partition_tokens : plan.fallback_partition_tokens;
    a.max_partitions = tiled ? plan.max_partitions : plan.fallback_max_partitions;
    a.compute_units = device::amd::deviceInfo(device_id).compute_units;
    a.odd_piece_relief = plan.odd_piece_relief;
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
