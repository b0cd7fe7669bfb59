// Tiled prefill kernel on gfx950 (CDNA4, 64-lane wavefronts) for head_size = value_size = 64, 128, 192 or 256 and
// for latent attention (keys of 576, values of 512 elements). Figures below are for head 128; the geometry per
// size is PrefillGeometry below.
//
// Work unit: one 256-thread workgroup = 64*R "rows" of one (sequence, KV head). A row is a (new
// token, query head of the KV head's group) pair, token-major: row = token * group + head_in_group.
// Packing the heads of a group into the row dimension means a K/V tile fetched once serves all of
// them, and short prompts still fill the matrix instructions. Each of the four wavefronts owns 16*R
// consecutive rows (R = 1 or 2 column groups of 16).
//
// The K/V tokens the rows may see are consumed in steps of 64 (32 where LDS or registers ask for it: see
// prefillStepTokens). Per step the workgroup brings that many K rows and V rows (16 KiB each) from the paged pool
// straight into LDS (16 bytes per lane, no register in between), a wavefront 16 tokens at a time, double-buffered:
// the loads of step j+2 are issued after the barrier that ends step j and awaited before the barrier that ends
// step j+1; one barrier per step separates writers and readers. Which global chunk a lane asks for decides the
// layout in LDS:
//   * K row-major, 16-byte chunks XOR-swizzled by the row so that the later row-wise reads are conflict-free: the
//     matrix instruction wants lane i to hold token i.
//   * V row-major in blocks of 16 columns (see v_lds): the operand of P.V wants 8 tokens of one column per lane,
//     which the transposing LDS read of gfx950 (ds_read_b64_tr_b16) delivers from row-major data, four tokens per
//     read.
//
// Arithmetic per step and column group, lane = 16*g + c:
//   S[token][row] = K . Q^T   16 x v_mfma_f32_16x16x32 (A = K tile from LDS, B = Q held in registers
//                             for the whole kernel; lane holds S[16T + 4g + 0..3][row c], T = 0..3)
//   causal mask (only in steps that touch the diagonal), online softmax in fp32 / log2 domain
//   O[row][dim] += P . V      16 x v_mfma_f32_16x16x32 (A = P rounded to the storage dtype, straight
//                             from the registers S came out in; B = V from LDS; lane holds
//                             O[row 4g + 0..3][16 e + c], e = 0..7)
//   l[row]      += P . 1       2 x v_mfma_f32_16x16x32: the denominator sums the rounded probabilities
// K/V fragments read from LDS are shared by the R column groups of a wavefront. A step whose tokens
// lie beyond everything a wavefront's rows may see is skipped by that wavefront (it still takes part
// in the copy).
//
// The math follows the reference's prefill kernels (src/infiniop/ops/paged_attention_prefill/cuda/
// kernel_v2.cuh:254-472: visible range, ALiBi distance, 1e-6 in the normaliser, rounding).
#ifndef INFINICORE_AMD_PA_PREFILL_TILED_H
#define INFINICORE_AMD_PA_PREFILL_TILED_H

#include "../../paged_attention/amd/decode_tiled.h"
#include "prefill_common.h"

namespace op::paged_attention_prefill::amd {

using op::paged_attention::amd::f32x4;
using op::paged_attention::amd::maxAcrossTokenGroups;
using op::paged_attention::amd::maxOf;
using op::paged_attention::amd::sumAcrossTokenGroups;
using op::paged_attention::amd::TileBF16;
using op::paged_attention::amd::TileF16;

using op::paged_attention::amd::kTileTokens;
using op::paged_attention::amd::loadLane16ToLds;
using op::paged_attention::amd::loadLane16ToLdsMasked;

constexpr int kPrefillThreads = 256;
// K / V operands are requested from LDS this many uses before the matrix instructions that take them (an LDS read
// takes longer than the R instructions one operand feeds; left alone the compiler requests one or two ahead and
// the matrix unit waits). At the Llama-3-8B chunked-prefill shape, head 128, three to six ahead are within 1.5 % of
// each other, the run-to-run spread (571 - 578 us; with V staged through registers 600 - 620 us against 639 us left
// to the compiler); above head 128, where the registers allow more, 8 is no better than 4.
constexpr int kOperandsAhead = 4;
constexpr float kLazyLog2 = 8.0f; // how far (in powers of two) a row maximum may outgrow its reference point

// 16-byte load from (wave-uniform base) + (32-bit per-lane byte offset), through the caches: K/V tiles
// are read again by the other row blocks of the sequence. The empty asm keeps the offset a value
// defined where it is used, so that the scalar-base form of the load is selected.
__device__ __forceinline__ uint4 loadLane16Cached(const char *uniform_base, uint32_t lane_offset) {
    asm volatile("" : "+v"(lane_offset));
    return *reinterpret_cast<const uint4 *>(uniform_base + lane_offset);
}

// Rows of one workgroup for R column groups per wavefront.
__host__ __device__ constexpr int prefillBlockRows(int r) { return 64 * r; }

// Which (sequence, row block) workgroup `x` of a KV head works on. Blocks are numbered from the last
// block of the last sequence backwards, so that within a sequence the blocks that see the most
// tokens start first. Every wavefront runs this on its own (no LDS, no barrier); all values are
// wave-uniform. Returns false for a workgroup beyond the last block.
// `span` receives the sequence's span as the lane that looked at it read it (lane reads: loading it again
// would be one more memory round trip at the head of every workgroup).
template <typename Tindex>
__device__ __forceinline__ bool findRowBlock(const PrefillArgs &a, int lane, int block_rows, int x, int &seq, int &block,
                                             SeqSpan &span_out) {
    int running = 0;
    for (int base = 0; base < a.num_seqs; base += 64) {
        const int idx = base + lane;
        const int s = a.num_seqs - 1 - idx;
        int nb = 0;
        SeqSpan span{0, 0, 0, 0, 0};
        if (idx < a.num_seqs) {
            span = loadSeqSpan<Tindex>(a, s);
            const int64_t rows = static_cast<int64_t>(span.q_len) * a.group;
            nb = rows > 0 ? static_cast<int>((rows + block_rows - 1) / block_rows) : 0;
        }
        int incl = nb;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int y = __shfl_up(incl, off, 64);
            incl += lane >= off ? y : 0;
        }
        incl += running;
        const unsigned long long hit = __builtin_amdgcn_ballot_w64(incl > x);
        if (hit != 0) {
            const int first = __builtin_ctzll(hit);
            const int incl_f = __builtin_amdgcn_readlane(incl, first);
            const int nb_f = __builtin_amdgcn_readlane(nb, first);
            seq = a.num_seqs - 1 - (base + first);
            block = nb_f - 1 - (x - (incl_f - nb_f));
            span_out.q_start = __builtin_amdgcn_readlane(span.q_start, first);
            span_out.q_len = __builtin_amdgcn_readlane(span.q_len, first);
            span_out.history = __builtin_amdgcn_readlane(span.history, first);
            span_out.capacity = __builtin_amdgcn_readlane(span.capacity, first);
            span_out.kv_len = __builtin_amdgcn_readlane(span.kv_len, first);
            return true;
        }
        running = __builtin_amdgcn_readlane(incl, 63);
    }
    return false;
}

// Geometry of the 16-token tiles for keys of KHEAD and values of VHEAD elements (equal except for latent attention,
// 576 / 512). K: kLoadsK instructions of 64 16-byte chunks per tile, row r keeps its chunks XOR-swizzled by
// r mod kSwizzle (TileGeometry of the decode kernels for equal sizes). V: kLoadsV instructions, kColsV blocks of 16
// columns.
template <int KHEAD, int VHEAD>
struct PrefillGeometry {
    static_assert(KHEAD % 64 == 0 && VHEAD % 64 == 0, "whole load instructions per tile, whole blocks of four V blocks");
    static constexpr int kLoadsK = KHEAD / 32; // K load instructions per tile = K-steps of K.Q^T
    static constexpr int kChunksPerRowK = KHEAD / 8;
    static constexpr int kSwizzle = KHEAD % 128 == 0 ? 16 : 8; // stays inside a row: its chunk count is a multiple
    static constexpr int kLoadsV = VHEAD / 32;
    static constexpr int kChunksPerRowV = VHEAD / 8;
    static constexpr int kColsV = VHEAD / 16; // blocks of 16 value columns
    static __device__ __forceinline__ int kRow(int j, int lane) { return (64 * j + lane) / kChunksPerRowK; }
    static __device__ __forceinline__ int kChunk(int j, int lane) { return (64 * j + lane) % kChunksPerRowK; }
    static __device__ __forceinline__ int ldsIndex(int row, int chunk) {
        return row * kChunksPerRowK + (chunk ^ (row & (kSwizzle - 1)));
    }
};

// Tokens per step, and workgroups that share a compute unit. Up to head 128: 64 tokens, two workgroups. Head 256
// needs more than half the register file even for 64 rows, so one workgroup has the unit to itself and takes 64-token
// steps (its two K and two V buffers are 128 KiB of the 160). Head 192 fits two workgroups of 64 rows with 32-token
// steps (48 KiB each); with 128 rows it is alone on the unit and takes 64-token steps (96 KiB).
// At the Llama-3-8B chunked-prefill shape, 128 rows against 64 rows with 32-token steps: head 192 1 864 -> 1 692 us,
// head 256 4 040 -> 2 046 us (2 787 us with 64 rows and 64-token steps).
// Latent attention (keys 576): 64 rows need 200 accumulator and query registers, so one workgroup per unit, and
// 32-token steps (two K and two V buffers: 136 KiB).
template <int KHEAD, int R>
constexpr int prefillStepTokens() { return (KHEAD <= 128 || KHEAD == 256 || (KHEAD == 192 && R == 2)) ? 64 : 32; }
template <int KHEAD, int R>
constexpr int prefillWorkgroupsPerUnit() { return (KHEAD <= 128 || (KHEAD == 192 && R == 1)) ? 2 : 1; }

// PLAIN: no ALiBi and scale > 0. The running maximum is then kept in units of the raw dot product
// (a positive scale keeps the order) and each probability costs one fused multiply-add and one exp2.
template <typename T, typename Tindex, int KHEAD, int VHEAD, int R, bool PLAIN>
__global__ void __launch_bounds__(kPrefillThreads, (prefillWorkgroupsPerUnit<KHEAD, R>())) prefillTiledKernel(PrefillArgs a) {
    using S = typename T::storage;
    using G = PrefillGeometry<KHEAD, VHEAD>;
    constexpr int BM = prefillBlockRows(R);
    constexpr int BN = prefillStepTokens<KHEAD, R>();
    constexpr int TT = BN / kTileTokens;             // 16-token tiles per step: 4 or 2
    constexpr int kTileChunksK = kTileTokens * G::kChunksPerRowK, kTileChunksV = kTileTokens * G::kChunksPerRowV;
    struct Tiles {
        uint4 k[2][TT * kTileChunksK]; // [tile][token][16-byte chunk, XOR-swizzled by the token]
        uint4 v[2][TT * kTileChunksV]; // see below
    };
    __shared__ Tiles tiles;
    auto &k_lds = tiles.k;
    // V tile in LDS: [row half (8 rows)][block of 16 columns (32 bytes)][row of the half][two 16-byte chunks], i.e.
    // slot = half * 8 * chunks per row + block * 16 + (row % 8) * 2 + chunk % 2. A transposing read of one block then
    // touches two runs of 256 bytes, and 64 consecutive slots (one load instruction) are four blocks of eight rows:
    // 128 contiguous bytes of each row in global memory.
    auto &v_lds = tiles.v;

    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int c = lane & 15;
    const int g = lane >> 4;
    // KV head fastest: workgroup ids go round-robin over the 8 accelerator dies, so with 8 (or a
    // multiple of 8) KV heads every die works on its own heads and the row blocks resident on a die
    // at one time are neighbours that stream the same K/V through that die's L2.
    const int kv_head = blockIdx.x % a.num_kv_heads;
    const int block_index = blockIdx.x / a.num_kv_heads;

    int seq = 0, block = 0;
    SeqSpan span;
    if (!findRowBlock<Tindex>(a, lane, BM, block_index, seq, block, span)) {
        return;
    }
    const int total_rows = span.q_len * a.group; // > 0 here
    const int block_row0 = block * BM;
    const int last_row = min(block_row0 + BM, total_rows) - 1;
    // tokens the block's last row may see = the most any of its rows may see
    const int block_visible = __builtin_amdgcn_readfirstlane(visibleTokens(span, last_row / a.group));
    if (block_visible <= 0) {
        return;
    }
    // tokens that exist; rows beyond it are zeroed in V (they may hold anything, NaN included)
    const int kv_len = __builtin_amdgcn_readfirstlane(max(span.kv_len, block_visible));
    const int n_steps = (block_visible + BN - 1) / BN;

    // ---- this lane's columns: row c of each of the wavefront's R column groups ----
    uint4 q_reg[R][G::kLoadsK];
    int visible[R];
    float slope[R];
    int wave_max_visible = 0, wave_min_visible = 0x7fffffff;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = block_row0 + (w * R + r) * 16 + c;
        const bool valid = row < total_rows;
        const int token = valid ? row / a.group : 0;
        const int head = kv_head * a.group + (valid ? row - token * a.group : 0);
        visible[r] = valid ? visibleTokens(span, token) : 0;
        slope[r] = (a.alibi_slopes != nullptr && valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;
        const S *q_ptr = static_cast<const S *>(a.q) + (span.q_start + token) * a.q_stride + head * a.q_head_stride;
#pragma unroll
        for (int kk = 0; kk < G::kLoadsK; ++kk) {
            q_reg[r][kk] = valid ? *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
        }
        wave_max_visible = max(wave_max_visible, visible[r]);
        wave_min_visible = min(wave_min_visible, valid ? visible[r] : 0x7fffffff);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        wave_max_visible = max(wave_max_visible, __shfl_xor(wave_max_visible, off, 64));
        wave_min_visible = min(wave_min_visible, __shfl_xor(wave_min_visible, off, 64));
    }
    wave_max_visible = __builtin_amdgcn_readfirstlane(wave_max_visible);
    wave_min_visible = __builtin_amdgcn_readfirstlane(wave_min_visible);

    // ---- copy side: per step this wavefront moves one 16-token tile of K and one of V (64-token
    // steps: tile w of both), or one tile of either (32-token steps: wavefronts 0, 1 the K tiles,
    // wavefronts 2, 3 the V tiles) ----
    const bool copies_k = TT == 4 || w < 2;
    const bool copies_v = TT == 4 || w >= 2;
    const int copy_tile = TT == 4 ? w : (w & 1);
    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
    const int64_t table_row = seq * a.block_table_batch_stride;
    const int block_mask = a.block_size - 1;
    const bool small_pages = a.block_size < 16; // pages of 8 tokens: a 16-token tile spans two
    const int last_entry = (kv_len - 1) >> a.block_shift;

    // Page ids: 64 block-table entries at a time, one per lane, fetched a whole batch ahead of their
    // use with an ordinary vector load. No load in the loop waits for another load, and nothing in the
    // loop goes through the scalar cache, whose out-of-order returns would make every LDS wait a wait
    // for it too.
    auto loadIdBatch = [&](int batch) {
        const int entry = batch * 64 + lane;
        int id = 0;
        if (entry <= last_entry) {
            id = static_cast<int>(loadIndex<Tindex>(a.block_tables, table_row + entry)); // low 32 bits; clamped where used
        }
        return id;
    };
    int id_batch = 0;
    int ids_cur = loadIdBatch(0), ids_next = loadIdBatch(1);
    auto pageOfEntry = [&](int entry) {
        const int e = min(entry, last_entry);
        const int raw = (e >> 6) == id_batch ? __builtin_amdgcn_readlane(ids_cur, e & 63)
                                             : __builtin_amdgcn_readlane(ids_next, e & 63);
        return clampPage(raw, a.num_blocks);
    };

    // K goes from global memory straight into its place in LDS: slot 64 j + lane of the tile holds chunk
    // (slot % chunks per row) ^ swizzle(row) of row slot / chunks per row (PrefillGeometry::ldsIndex read backwards), so
    // that is the chunk this lane asks for with instruction j. V passes through registers (it is transposed on
    // the way).
    uint32_t k_src_off[G::kLoadsK];
#pragma unroll
    for (int j = 0; j < G::kLoadsK; ++j) {
        const int row = G::kRow(j, lane), slot = G::kChunk(j, lane);
        k_src_off[j] = row * static_cast<uint32_t>(a.k_row_stride) * sizeof(S) + 16 * (slot ^ (row & (G::kSwizzle - 1)));
    }
    // V likewise, into the layout described at v_lds
    auto vRowOfSlot = [](int slot) { return 8 * (slot / (8 * G::kChunksPerRowV)) + (slot % 16) / 2; };
    auto vChunkOfSlot = [](int slot) { return 2 * ((slot % (8 * G::kChunksPerRowV)) / 16) + slot % 2; };
    uint32_t v_src_off[G::kLoadsV];
#pragma unroll
    for (int j = 0; j < G::kLoadsV; ++j) {
        v_src_off[j] = vRowOfSlot(64 * j + lane) * static_cast<uint32_t>(a.v_row_stride) * sizeof(S) + 16 * vChunkOfSlot(64 * j + lane);
    }
    // A stage's load instructions are not issued in one burst after the barrier but one at a time between the matrix
    // instructions of the step that follows (computeStep): a wavefront cannot issue its next direct load before the
    // memory pipeline has taken the one before (each carries its LDS address in M0), and with every wavefront of the
    // compute unit issuing eight at once that cost each of them ~1 us per step. loadStage(step, true) only records
    // where the instructions of the stage read and write; issueSlot(i) issues the i-th of them (slots [0, kLoadsK)
    // are K, the rest V; a wavefront that copies one kind only has its instructions in the first slots). A slot with
    // nothing to do (no further stage, or a stage that took the lane-by-lane path) runs with no lane switched on.
    constexpr int kSlots = TT == 4 ? G::kLoadsK + G::kLoadsV : (G::kLoadsK > G::kLoadsV ? G::kLoadsK : G::kLoadsV);
    constexpr int kPendV = TT == 4 ? 1 : 0; // a wavefront that copies one kind keeps that kind's record at index 0
    uint32_t slot_off[kSlots];              // the lane's source offset for slot i
#pragma unroll
    for (int i = 0; i < kSlots; ++i) {
        if constexpr (TT == 4) {
            slot_off[i] = i < G::kLoadsK ? k_src_off[i < G::kLoadsK ? i : 0] : v_src_off[i < G::kLoadsK ? 0 : i - G::kLoadsK];
        } else {
            slot_off[i] = copies_k ? k_src_off[i < G::kLoadsK ? i : 0] : v_src_off[i < G::kLoadsV ? i : 0];
        }
    }
    const char *pend_src[2] = {k_head, v_head};
    uint4 *pend_dst[2] = {&k_lds[0][0], &v_lds[0][0]};
    unsigned long long pend_live[2] = {0ull, 0ull}; // EXEC mask of the slot's instruction: all lanes or none
    auto issueSlot = [&](int i) {
        if constexpr (TT == 4) {
            const int kind = i < G::kLoadsK ? 0 : 1, inst = kind ? i - G::kLoadsK : i;
            loadLane16ToLdsMasked(pend_src[kind], slot_off[i], pend_dst[kind] + 64 * inst, pend_live[kind]);
        } else {
            const bool exists = i < (copies_k ? G::kLoadsK : G::kLoadsV);
            loadLane16ToLdsMasked(pend_src[0], slot_off[i], pend_dst[0] + 64 * i, exists ? pend_live[0] : 0ull);
        }
    };
    auto loadStage = [&](int step, bool deferred) {
        // K and V: slots 64 j + lane of the tile; V rows past kv_len are zeroed.
        pend_live[0] = pend_live[1] = 0ull;
        const int t = step * BN + kTileTokens * copy_tile;
        const int e0 = t >> a.block_shift;
        if ((min(e0, last_entry) >> 6) > id_batch) {
            ids_cur = ids_next;
            ++id_batch;
            ids_next = loadIdBatch(id_batch + 1);
        }
        // Page ids first, loads after: reading an id out of its register waits for every vector-memory operation
        // in flight (the id batch may have been loaded in an earlier trip), the tile loads just issued included.
        const int id0 = pageOfEntry(e0), id1 = small_pages ? pageOfEntry(e0 + 1) : id0;
        if (copies_k) {
            // Rows past the end of the sequence are fetched like the others: the page they lie in exists (its id
            // is clamped to the sequence's last entry and to the pool), and whatever they hold only reaches scores
            // that the causal mask replaces.
            uint4 *k_dst = &k_lds[step & 1][copy_tile * kTileChunksK];
            if (!small_pages) {
                const char *k_tile = k_head + (id0 * a.k_batch_stride + (t & block_mask) * a.k_row_stride) * static_cast<int64_t>(sizeof(S));
                if (deferred) {
                    pend_src[0] = k_tile, pend_dst[0] = k_dst, pend_live[0] = ~0ull;
                } else {
#pragma unroll
                    for (int j = 0; j < G::kLoadsK; ++j) {
                        loadLane16ToLds(k_tile, k_src_off[j], k_dst + 64 * j);
                    }
                }
            } else { // pages of 8 tokens: rows 8..15 of the tile lie in the next page
#pragma unroll
                for (int j = 0; j < G::kLoadsK; ++j) {
                    const int row = G::kRow(j, lane), slot = G::kChunk(j, lane);
                    const int page = row >= 8 ? id1 : id0;
                    const char *src = k_head + (page * a.k_batch_stride + (row & 7) * a.k_row_stride) * static_cast<int64_t>(sizeof(S))
                                    + 16 * (slot ^ (row & (G::kSwizzle - 1)));
                    loadLane16ToLds(src, k_dst + 64 * j);
                }
            }
        }
        if (!copies_v) {
            return;
        }
        uint4 *v_dst = &v_lds[step & 1][copy_tile * kTileChunksV];
        if (t + kTileTokens <= kv_len && !small_pages) {
            const char *v_tile = v_head + (id0 * a.v_batch_stride + (t & block_mask) * a.v_row_stride) * static_cast<int64_t>(sizeof(S));
            if (deferred) {
                pend_src[kPendV] = v_tile, pend_dst[kPendV] = v_dst, pend_live[kPendV] = ~0ull;
            } else {
#pragma unroll
                for (int j = 0; j < G::kLoadsV; ++j) {
                    loadLane16ToLds(v_tile, v_src_off[j], v_dst + 64 * j);
                }
            }
            return;
        }
        // Last tile of the sequence, or two pages per tile. Rows past the sequence may hold anything (NaN included)
        // and 0 * NaN is NaN: their lanes are switched off for the load and store zeros instead.
        const int row0 = small_pages ? 0 : (t & block_mask);
#pragma unroll
        for (int j = 0; j < G::kLoadsV; ++j) {
            const int row = vRowOfSlot(64 * j + lane);
            const int page = (small_pages && row >= 8) ? id1 : id0;
            const int page_row = small_pages ? (row & 7) : row0 + row;
            const char *src = v_head + (page * a.v_batch_stride + page_row * a.v_row_stride) * static_cast<int64_t>(sizeof(S))
                            + 16 * vChunkOfSlot(64 * j + lane);
            if (t + row < kv_len) {
                loadLane16ToLds(src, v_dst + 64 * j);
            } else {
                v_dst[64 * j + lane] = make_uint4(0, 0, 0, 0);
            }
        }
    };
    // the tiles asked for by the last loadStage are in LDS
    auto awaitStage = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

    // Wavefront priorities. On a SIMD that holds wavefronts of two workgroups (heads up to 128) nothing keeps the two in
    // different phases of their steps, and a wavefront in its softmax can hold up the matrix instructions of the other
    // for as long as it has vector instructions ready. The two blocks of matrix instructions of a step therefore run at
    // a higher priority than the softmax between them (a softmax then fills the issue slots that the other wavefront's
    // matrix instructions leave free), and of two wavefronts in the same kind of phase the one in the odd hardware
    // slot goes first, which pushes the pair apart. Bit 0 of the wavefront's slot number: HW_ID bits [3:0].
    const bool odd_slot = (__builtin_amdgcn_s_getreg((3 << 11) | 4) & 1) != 0;
    auto matrixPhase = [&]() {
        if (odd_slot) {
            __builtin_amdgcn_s_setprio(3);
        } else {
            __builtin_amdgcn_s_setprio(2);
        }
    };
    auto vectorPhase = [&]() {
        if (odd_slot) {
            __builtin_amdgcn_s_setprio(1);
        } else {
            __builtin_amdgcn_s_setprio(0);
        }
    };
    // ---- softmax state ----
    // o[r][e][rr] = O[row 4g+rr of group r][column 16 e + c]; ol[r][rr] = sum of that row's probabilities
    // (computed by the matrix unit as P . 1, so it sums exactly the rounded probabilities the numerator
    // used and already sits in the accumulators' row layout); m[r] = running maximum of row c, in units
    // of the raw dot product when there is no ALiBi (scale > 0 keeps the order), else of the scaled score.
    f32x4 o[R][G::kColsV], ol[R];
    float m[R];
    float shift[R]; // -m[r] in log2 units (0 while m[r] = -inf): what the exponent of a probability adds to its score
#pragma unroll
    for (int r = 0; r < R; ++r) {
        shift[r] = 0.0f;
#pragma unroll
        for (int e = 0; e < G::kColsV; ++e) {
            o[r][e] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        ol[r] = f32x4{0.f, 0.f, 0.f, 0.f};
        m[r] = -INFINITY;
    }
    // this lane's piece of a transposing V read (see readV below), relative to block 0 of tile 0 of buffer 0
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 *LdsPiece;
    const auto v_read_base = (__attribute__((address_space(3))) char *)v_lds
                           + 16 * ((g >> 1) * 8 * G::kChunksPerRowV + (4 * (g & 1) + (c >> 2)) * 2 + ((c & 3) >> 1)) + 8 * (c & 1);
    // this lane's chunk of row c in K-step kk, within a tile (the swizzle makes it a different one per kk)
    int k_read_index[G::kLoadsK];
#pragma unroll
    for (int kk = 0; kk < G::kLoadsK; ++kk) {
        k_read_index[kk] = G::ldsIndex(c, 4 * kk + g);
    }
    const uint32_t one2 = T::pack2(1.0f, 1.0f);
    const uint4 ones = make_uint4(one2, one2, one2, one2);
    const float unit = PLAIN ? a.scale_log2 : 1.0f; // log2-domain size of one unit of m
    const float lazy = kLazyLog2 / unit;             // kLazyLog2 powers of two, in units of m

    // One step over the BN tokens in LDS buffer `buf`. masked: some score of the step lies beyond
    // what its row may see (steps on the causal diagonal); the other steps skip the comparison.
    auto computeStep = [&](int buf, int t0, bool masked) {
        f32x4 s[R][TT];
#pragma unroll
        for (int r = 0; r < R; ++r) {
#pragma unroll
            for (int tt = 0; tt < TT; ++tt) {
                s[r][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
            }
        }
        matrixPhase();
        // K.Q^T: operand idx = (tile tt, 32 dimensions kk). The scheduler groups pin the order "one LDS read, then the
        // R matrix instructions of the operand read kAheadK earlier"; the first kAheadK reads are a group of their own.
        {
            constexpr int kAheadK = kOperandsAhead;
            constexpr int kOperandsK = TT * G::kLoadsK;
            auto readK = [&](int idx) {
                const int tt = idx / G::kLoadsK, kk = idx % G::kLoadsK;
                return k_lds[buf][tt * kTileChunksK + k_read_index[kk]];
            };
            uint4 kf[kAheadK];
#pragma unroll
            for (int i = 0; i < kAheadK; ++i) {
                kf[i] = readK(i);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, kAheadK, 0);
#pragma unroll
            for (int idx = 0; idx < kOperandsK; ++idx) {
                const int tt = idx / G::kLoadsK, kk = idx % G::kLoadsK;
                const uint4 cur = kf[idx % kAheadK];
                if (idx + kAheadK < kOperandsK) {
                    kf[idx % kAheadK] = readK(idx + kAheadK);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    s[r][tt] = T::mfmaK32(cur, q_reg[r][kk], s[r][tt]);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, R, 0);
                if (idx % 2 == 1 && idx / 2 < kSlots) {
                    issueSlot(idx / 2); // one load instruction of the next stage after every second operand
                }
            }
            static_assert(kOperandsK / 2 >= kSlots, "a place in the step for every load instruction of a stage");
        }

        vectorPhase();
        uint4 p_op[R][TT / 2];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // scores in the units m[r] is kept in
            if constexpr (!PLAIN) {
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const int tok = t0 + 16 * tt + 4 * g + rr;
                        s[r][tt][rr] = s[r][tt][rr] * a.scale_log2 + slope[r] * static_cast<float>(tok - (visible[r] - 1));
                    }
                }
            }
            if (masked) {
#pragma unroll
                for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const int tok = t0 + 16 * tt + 4 * g + rr;
                        s[r][tt][rr] = tok >= visible[r] ? -INFINITY : s[r][tt][rr];
                    }
                }
            }
            // three-operand maxima: 4 TT values in 2 TT instructions
            float mx = maxOf(maxOf(s[r][0][0], s[r][0][1]), s[r][0][2]);
            mx = maxOf(maxOf(mx, s[r][0][3]), s[r][1][0]);
            mx = maxOf(maxOf(mx, s[r][1][1]), s[r][1][2]);
#pragma unroll
            for (int tt = 2; tt < TT; tt += 2) {
                mx = maxOf(maxOf(mx, s[r][tt - 1][3]), s[r][tt][0]);
                mx = maxOf(maxOf(mx, s[r][tt][1]), s[r][tt][2]);
                mx = maxOf(maxOf(mx, s[r][tt][3]), s[r][tt + 1][0]);
                mx = maxOf(maxOf(mx, s[r][tt + 1][1]), s[r][tt + 1][2]);
            }
            mx = maxOf(mx, s[r][TT - 1][3]);
            // mx: maximum over this lane's 4 x TT tokens; the row's maximum is the largest of its four lanes' (c, c + 16,
            // c + 32, c + 48) and is only formed when it is needed.
            // The reference point m[r] only has to keep the exponentials in range, it need not be the
            // exact maximum: it is moved (and the accumulators rescaled, ~70 vector instructions) only
            // when some row's maximum has grown by more than 2^kLazyLog2 since, so probabilities reach at
            // most that factor above 1. Numerator and denominator carry the same reference, the quotient
            // is unchanged.
            // (a row that has seen nothing yet has m = -inf: any finite maximum is above -inf + lazy)
            if (__builtin_amdgcn_ballot_w64(mx > m[r] + lazy) != 0) { // some lane's maximum, hence some row's
                mx = maxAcrossTokenGroups(mx);
                const float m_new = maxOf(m[r], mx);
                // rescale. Lane holds accumulators of rows 4g..4g+3, whose factors live in lanes 4g..4g+3.
                const float alpha = m_new > m[r] ? fastExp2((m[r] - m_new) * unit) : 1.0f;
                m[r] = m_new;
                // a row that has seen nothing yet keeps m = -inf: subtract 0, p = 2^-inf = 0
                shift[r] = m_new == -INFINITY ? 0.0f : -m_new * unit;
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    const float alpha_r = __shfl(alpha, 4 * g + rr, 64);
                    ol[r][rr] *= alpha_r;
#pragma unroll
                    for (int e = 0; e < G::kColsV; ++e) {
                        o[r][e][rr] *= alpha_r;
                    }
                }
            }
#pragma unroll
            for (int u = 0; u < TT / 2; ++u) {
                uint32_t wds[4];
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const f32x4 x = s[r][2 * u + h];
                    wds[2 * h] = T::pack2(fastExp2(__builtin_fmaf(x[0], unit, shift[r])), fastExp2(__builtin_fmaf(x[1], unit, shift[r])));
                    wds[2 * h + 1] = T::pack2(fastExp2(__builtin_fmaf(x[2], unit, shift[r])), fastExp2(__builtin_fmaf(x[3], unit, shift[r])));
                }
                p_op[r][u] = make_uint4(wds[0], wds[1], wds[2], wds[3]);
            }
        }

        matrixPhase();
        // P.V: the V operands run kAhead ahead as well
        constexpr int kAhead = kOperandsAhead;
        constexpr int kOperands = (TT / 2) * G::kColsV;
        // Operand (u, e) = V[32 tokens of tiles 2u, 2u + 1][columns 16 e .. 16 e + 15]: lane (g, c) needs tokens
        // 4g..4g+3 of either tile at column 16 e + c. A transposing read hands lane c of a group of 16 the element
        // c % 4 of the four 8-byte pieces that lanes c / 4, c / 4 + 4, + 8, + 12 of the group point at; so lane
        // (g, c) points at token 4g + c / 4, columns 16 e + 4 (c % 4) .. + 3.
        auto readV = [&](int idx) {
            const int u = idx / G::kColsV, e = idx % G::kColsV;
            const auto base = v_read_base + (buf * TT + 2 * u) * (kTileChunksV * 16) + 256 * e;
            const uint2 lo = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsPiece>(base)));
            const uint2 hi = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsPiece>(base + kTileChunksV * 16)));
            return make_uint4(lo.x, lo.y, hi.x, hi.y);
        };
        uint4 vf[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            vf[i] = readV(i);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0); // two reads per operand
#pragma unroll
        for (int idx = 0; idx < kOperands; ++idx) {
            const int u = idx / G::kColsV, e = idx % G::kColsV;
            const uint4 cur = vf[idx % kAhead];
            if (idx + kAhead < kOperands) {
                vf[idx % kAhead] = readV(idx + kAhead);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            if (e == 0) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    ol[r] = T::mfmaK32(p_op[r][u], ones, ol[r]);
                }
                __builtin_amdgcn_sched_group_barrier(0x008, R, 0);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                o[r][e] = T::mfmaK32(p_op[r][u], cur, o[r][e]);
            }
            __builtin_amdgcn_sched_group_barrier(0x008, R, 0);
        }
        vectorPhase();
    };

    // ---- pipeline ----
    loadStage(0, false);
    awaitStage();
    __syncthreads();
    for (int j = 0; j < n_steps; ++j) {
        const int t0 = j * BN;
        // stage j + 1 goes into the other buffer while this step computes (everybody is past step j - 1)
        if (j + 1 < n_steps) {
            loadStage(j + 1, true);
        } else {
            pend_live[0] = pend_live[1] = 0ull;
        }
        if (t0 < wave_max_visible) {
            computeStep(j & 1, t0, t0 + BN > wave_min_visible);
        } else {
#pragma unroll
            for (int i = 0; i < kSlots; ++i) {
                issueSlot(i);
            }
        }
        awaitStage();
        __syncthreads();
    }

    // ---- normalise and store. A lane holds single columns (16 e + c) of its rows; the wavefront's 16 R rows pass
    // through LDS (the tile buffers: every wavefront is past the last barrier of the loop, nothing is in flight) and go
    // out as 16-byte pieces, 64 lanes on consecutive pieces ----
    static_assert(sizeof(Tiles) >= 4 * R * 16 * VHEAD * 2, "the tile buffers hold the output rows of all four wavefronts");
    unsigned short *stage = reinterpret_cast<unsigned short *>(&tiles) + w * (R * 16 * VHEAD);
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const float inv_l = 1.0f / (ol[r][rr] + 1e-6f);
            unsigned short *row = stage + (r * 16 + 4 * g + rr) * VHEAD + c;
#pragma unroll
            for (int e = 0; e < G::kColsV; ++e) {
                row[16 * e] = static_cast<unsigned short>(T::pack2(o[r][e][rr] * inv_l, 0.0f));
            }
        }
    }
    // the wavefront's own stores have landed before its lanes read each other's columns (also keeps the compiler
    // from moving the differently typed loads below across the stores above)
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    constexpr int kPieces = R * 16 * G::kChunksPerRowV; // 16-byte pieces of the wavefront's rows
#pragma unroll
    for (int i = 0; i < kPieces / 64; ++i) {
        const int piece = 64 * i + lane;
        const int local_row = piece / G::kChunksPerRowV, chunk = piece % G::kChunksPerRowV;
        const int row = block_row0 + w * R * 16 + local_row;
        if (row >= total_rows) {
            continue;
        }
        const int token = row / a.group;
        if (visibleTokens(span, token) <= 0) {
            continue;
        }
        const int head = kv_head * a.group + (row - token * a.group);
        const uint4 x = *reinterpret_cast<const uint4 *>(stage + local_row * VHEAD + 8 * chunk);
        S *o_ptr = static_cast<S *>(a.out) + (span.q_start + token) * a.o_stride + head * a.o_head_stride;
        *reinterpret_cast<uint4 *>(o_ptr + 8 * chunk) = x;
    }
}

} // namespace op::paged_attention_prefill::amd

#endif
