// Tiled decode kernel for latent-attention caches: head_size 576 (512 latent + 64 rotary columns),
// value_size 512, the shape of the reference's dedicated kernel
// (src/infiniop/ops/paged_attention/nvidia/paged_attention_mla_hd576_v512.cu). gfx950, 64-lane wavefronts.
//
// Unit of work and arithmetic are those of the head-128 tiled kernel (decode_tiled.h): one unit = one
// (partition, KV head x 16 query heads, sequence), tiles of 16 tokens, K . Q^T and P . V on the matrix
// unit, online softmax in the log2 domain. A tile is four times as large here (K 18 KiB, V 16 KiB) and a
// single wavefront that held the 512 output columns, the query and one K and one V tile would need all
// 512 registers of its SIMD for one tile in flight. So a unit is a workgroup of TWO wavefronts:
//   * wavefront w fetches K rows 8w .. 8w+7 of the tile and puts them in the LDS tile both read
//     (two workgroup barriers per tile), so K comes from memory once; the registers are free again once
//     copied, and the next tile's rows are requested right there;
//   * both compute all 16 x 16 scores and the softmax (18 matrix instructions, cheap to duplicate);
//   * wavefront w owns value / output columns 256 w .. 256 w + 255: 64 accumulator registers and one V
//     tile of 32 registers, consumed in two strips of 128 columns; as soon as a strip of V(t) has been
//     used the same strip of V(t+1) is requested into its registers;
//   * the query rows sit in LDS next to the K tile and are read back K-step by K-step.
// That fits 256 registers per wavefront (188 as compiled), so every SIMD holds two wavefronts and a compute
// unit's LDS four units. A unit advances one tile per 1.9 - 2.5 us however many units run and whether or not
// the pages sit in cache: its pace is set by the order-preserving return of one wavefront's loads (about
// one 128-byte line per 10 - 15 ns, 136 lines per tile and wavefront) plus the part of the matrix and
// vector work that does not overlap with it, so throughput comes from the number of units. A second
// register set for K or V (two tiles in flight, one wavefront per SIMD) was measured and is slower.
// (Direct global -> LDS loads would free the K registers as well, but with one of those outstanding this
// compiler turns every wait on a vector-memory result into a wait for all of them, which serialises the
// pipeline.)
//
// Columns: within its half, the lane with c = lane % 16 owns columns 128 i + 8 c .. + 7 for i = 0, 1, so
// one load or store instruction of the wavefront covers 256 contiguous bytes of each of its rows. K rows
// (1152 bytes = 72 16-byte chunks) are fetched as flat chunks 64 j + lane, j = 0..8, of the wavefront's
// eight rows and kept in LDS with a row pitch of 73 chunks, which makes both the row-major writes and the
// column-of-16-rows reads conflict-free without a swizzle.
#ifndef INFINICORE_AMD_PA_DECODE_MLA_H
#define INFINICORE_AMD_PA_DECODE_MLA_H

#include "decode_tiled.h"

namespace op::paged_attention::amd {

constexpr int kMlaKeySize = 576;
constexpr int kMlaValueSize = 512;
constexpr int kMlaThreads = 128; // two wavefronts per unit of work

struct MlaGeometry {
    static constexpr int kSteps = kMlaKeySize / 32;       // K-steps of K.Q^T
    static constexpr int kChunksPerRow = kMlaKeySize / 8; // 16-byte chunks in one K row
    static constexpr int kLoads = 8 * kChunksPerRow / 64; // K load instructions per tile and wavefront (8 rows)
    static constexpr int kLdsPitch = kChunksPerRow + 1;   // chunks between consecutive rows in LDS
    static constexpr int kHalf = kMlaValueSize / 2;       // value columns per wavefront
    static constexpr int kStrips = kHalf / 128;           // 16-byte strips of one V row per lane
    static constexpr int kCols = kHalf / 16;              // V / output columns per lane
    // row (0..7 of the wavefront's eight) and chunk of the piece lane `lane` fetches in instruction j
    static __device__ __forceinline__ int kRow(int j, int lane) { return (64 * j + lane) / kChunksPerRow; }
    static __device__ __forceinline__ int kChunk(int j, int lane) { return (64 * j + lane) % kChunksPerRow; }
    static __device__ __forceinline__ int ldsIndex(int row, int chunk) { return row * kLdsPitch + chunk; }
};

#ifdef INFINIOP_AMD_PA_TRACE
#define MLA_STAMP(slot)                                                                                   \
    do {                                                                                                 \
        if (g_pa_trace != nullptr && threadIdx.x == 0) {                                                 \
            g_pa_trace[((static_cast<size_t>(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 8 + (slot)] = __builtin_amdgcn_s_memrealtime(); \
        }                                                                                                \
    } while (0)
#else
#define MLA_STAMP(slot) do {} while (0)
#endif

template <typename T, typename Tindex>
__global__ void __launch_bounds__(kMlaThreads, 2) decodeMlaKernel(DecodeArgs a) {
    using S = typename T::storage;
    using G = MlaGeometry;
    __shared__ uint4 k_lds[kTileTokens * G::kLdsPitch];   // one K tile
    __shared__ uint4 q_lds[kHeadsPerWave * G::kLdsPitch]; // the 16 query rows

    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int kv_head = blockIdx.y / head_chunks;
    const int chunk = blockIdx.y - kv_head * head_chunks;
    const int seq = blockIdx.z;
    // Workgroups are dealt to the eight XCDs round-robin by linear index, which follows blockIdx.x when the
    // grid's x extent is a multiple of eight. Partition p of every sequence on the same XCD would load the
    // XCDs by how many sequences reach partition p, so the partitions of sequence s are rotated by s.
    const int part = static_cast<int>((blockIdx.x + blockIdx.z) % gridDim.x);
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15; // column strip / head within the chunk / token for the K operand
    const int g = lane >> 4; // group of four tokens

    MLA_STAMP(0);
    // Everything up to the first barrier depends on the unit only, so both wavefronts leave together.
    const int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
    if (len64 <= 0) {
        return;
    }
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) << a.block_shift;
    const int len = static_cast<int>(len64 < max_len ? len64 : max_len);
    const int start = part * a.partition_tokens;
    if (start >= len) {
        return;
    }
    const int end = min(len, start + a.partition_tokens);
    const int n_tiles = (end - start + kTileTokens - 1) / kTileTokens;

    // Page ids of this partition: at most 64 table entries, one per lane, clamped into the pool.
    const int first_entry = start >> a.block_shift;
    const int last_entry = (end - 1) >> a.block_shift;
    int page_ids = 0;
    if (first_entry + lane <= last_entry) {
        page_ids = clampPage(
            loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + first_entry + lane), a.num_blocks);
    }

    // Query of head (chunk*16 + c), as the B operand of the K-steps: columns 32*kk + 8g .. +7, in LDS with
    // the layout of a K tile (row = head). Each wavefront stores half of the K-steps.
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    {
        const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
        const uint32_t keep = head_valid ? 0xffffffffu : 0u;
#pragma unroll
        for (int i = 0; i < G::kSteps / 2; ++i) {
            const int kk = wave * (G::kSteps / 2) + i;
            uint4 x = *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g);
            x.x &= keep, x.y &= keep, x.z &= keep, x.w &= keep;
            q_lds[G::ldsIndex(c, 4 * kk + g)] = x;
        }
    }
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;

    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride)
                       + wave * (G::kHalf * sizeof(S));
    const int block_mask = a.block_size - 1;

    // Byte offsets of this lane's pieces inside a tile; the same for every tile.
    uint32_t k_off[G::kLoads], v_off[4];
    {
        const uint32_t k_row_bytes = static_cast<uint32_t>(a.k_row_stride) * sizeof(S);
        const uint32_t v_row_bytes = static_cast<uint32_t>(a.v_row_stride) * sizeof(S);
#pragma unroll
        for (int j = 0; j < G::kLoads; ++j) {
            k_off[j] = (8 * wave + G::kRow(j, lane)) * k_row_bytes + 16 * G::kChunk(j, lane);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v_off[j] = (4 * g + j) * v_row_bytes + 16 * c;
        }
    }

    // Loads for a tile index past the end of the partition are issued all the same (the loop body has
    // no branch around a load) but made harmless: every lane reads the first bytes of the partition.
    auto tileAddress = [&](int t, const char *head_base, int64_t batch_stride, int64_t row_stride) -> const char * {
        const int tok0 = start + (t < n_tiles ? t : 0) * kTileTokens;
        const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
        const int row0 = tok0 & block_mask;
        return head_base + (page * batch_stride + row0 * row_stride) * static_cast<int64_t>(sizeof(S));
    };
    auto loadK = [&](int t, uint4 (&k)[G::kLoads]) {
        const uint32_t lane_mask = t < n_tiles ? 0xffffffffu : 0u;
        const char *tile = tileAddress(t, k_head, a.k_batch_stride, a.k_row_stride);
#pragma unroll
        for (int j = 0; j < G::kLoads; ++j) {
            k[j] = loadLane16(tile, k_off[j] & lane_mask);
        }
    };
    // Strip i of a V tile: v[j][4 i + w] = token row 4g + j, columns (256 wave) + 128 i + 8 c + 2 w, + 2 w + 1
    auto loadVStrip = [&](int t, int i, uint32_t (&v)[4][4 * G::kStrips]) {
        const uint32_t lane_mask = t < n_tiles ? 0xffffffffu : 0u;
        const char *tile = tileAddress(t, v_head, a.v_batch_stride, a.v_row_stride);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint4 x = loadLane16(tile + 256 * i, v_off[j] & lane_mask);
            v[j][4 * i] = x.x, v[j][4 * i + 1] = x.y, v[j][4 * i + 2] = x.z, v[j][4 * i + 3] = x.w;
        }
    };

    // o[8 i + e][r] = O[head 4g + r of the chunk][column (256 wave) + 128 i + 8 c + e]
    f32x4 o[G::kCols];
#pragma unroll
    for (int e = 0; e < G::kCols; ++e) {
        o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float m = -INFINITY; // running maximum of head c (same value in the four lanes g = 0..3)
    float l = 0.0f;      // sum of rounded probabilities of head c over this lane's tokens only

    uint4 k[G::kLoads];
    uint32_t v[4][4 * G::kStrips];
    MLA_STAMP(1);
    loadK(0, k);
#pragma unroll
    for (int i = 0; i < G::kStrips; ++i) {
        loadVStrip(0, i, v);
    }
    for (int t = 0; t < n_tiles; ++t) {
        // K: registers -> LDS -> matrix-operand layout (token c, columns 32*kk + 8g .. +7)
#pragma unroll
        for (int j = 0; j < G::kLoads; ++j) {
            k_lds[G::ldsIndex(8 * wave + G::kRow(j, lane), G::kChunk(j, lane))] = k[j];
        }
        __syncthreads(); // the tile (and, the first time, the query) is complete
        loadK(t + 1, k);
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < G::kSteps; ++kk) {
            s = T::mfmaK32(k_lds[G::ldsIndex(c, 4 * kk + g)], q_lds[G::ldsIndex(c, 4 * kk + g)], s);
        }
        __syncthreads(); // both wavefronts have read the tile: the next one may overwrite it

        const int tok0 = start + t * kTileTokens;
        const int valid = min(kTileTokens, end - tok0);
        uint2 p_op, p_lo = make_uint2(0, 0);
        softmaxStep<T, G::kCols>(o, m, l, s, g, a.scale_log2, slope, tok0 - (len - 1), valid, p_op, p_lo);
#pragma unroll
        for (int i = 0; i < G::kStrips; ++i) {
#pragma unroll
            for (int w = 4 * i; w < 4 * i + 4; ++w) {
                accumulatePair<T>(o[2 * w], o[2 * w + 1], v[0][w], v[1][w], v[2][w], v[3][w], p_op, p_lo, g, valid);
            }
            loadVStrip(t + 1, i, v); // the strip's registers are free again
        }
    }

    MLA_STAMP(2);
#ifdef INFINIOP_AMD_PA_TRACE
    if (g_pa_trace != nullptr && threadIdx.x == 0) {
        g_pa_trace[((static_cast<size_t>(blockIdx.z) * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 8 + 5] = n_tiles;
    }
#endif
    // Epilogue. Denominator of head c over all 16 token slots, then move per-head scalars to the
    // lanes that hold that head's accumulators.
    const float l_tot = sumAcrossTokenGroups(l);
    const bool single = len <= a.partition_tokens;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int hl = 4 * g + rr; // head (within the chunk) of accumulator row rr
        const float l_h = __shfl(l_tot, hl, 64);
        const float m_h = __shfl(m, hl, 64);
        const int hg = chunk * kHeadsPerWave + hl;
        if (hg >= a.group) {
            continue;
        }
        const int out_head = kv_head * a.group + hg;
        const int col0 = wave * G::kHalf + 8 * c;
        if (single) {
            const float inv_l = 1.0f / (l_h + 1e-6f);
            S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride + col0;
#pragma unroll
            for (int i = 0; i < G::kStrips; ++i) {
                uint4 w;
                w.x = T::pack2(o[8 * i + 0][rr] * inv_l, o[8 * i + 1][rr] * inv_l);
                w.y = T::pack2(o[8 * i + 2][rr] * inv_l, o[8 * i + 3][rr] * inv_l);
                w.z = T::pack2(o[8 * i + 4][rr] * inv_l, o[8 * i + 5][rr] * inv_l);
                w.w = T::pack2(o[8 * i + 6][rr] * inv_l, o[8 * i + 7][rr] * inv_l);
                *reinterpret_cast<uint4 *>(o_ptr + 128 * i) = w;
            }
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            float *dst = a.part_acc + slot * kMlaValueSize + col0;
#pragma unroll
            for (int i = 0; i < G::kStrips; ++i) {
                reinterpret_cast<float4 *>(dst + 128 * i)[0] = make_float4(o[8 * i + 0][rr], o[8 * i + 1][rr], o[8 * i + 2][rr], o[8 * i + 3][rr]);
                reinterpret_cast<float4 *>(dst + 128 * i)[1] = make_float4(o[8 * i + 4][rr], o[8 * i + 5][rr], o[8 * i + 6][rr], o[8 * i + 7][rr]);
            }
            if (c == 0 && wave == 0) {
                a.part_m[slot] = m_h;
                a.part_l[slot] = l_h;
            }
        }
    }
    MLA_STAMP(3);
}

} // namespace op::paged_attention::amd

#endif
