// Tiled decode kernels for latent-attention caches: head_size 576 (512 latent + 64 rotary columns),
// value_size 512, the shape of the reference's dedicated kernel
// (src/infiniop/ops/paged_attention/nvidia/paged_attention_mla_hd576_v512.cu). gfx950, 64-lane wavefronts.
// Four kernels: decodeMlaKernel (16 query heads per workgroup of two wavefronts, described first; with its value
// width as a parameter it also takes heads of 576 whose values are 576 wide, MlaGeometry),
// decodeMlaChunkKernel (the same 16 heads on a workgroup of eight wavefronts, for batches too small to fill the
// device with pairs), decodeMlaRowsKernel (more than 16 heads per KV head: 64 or 128 per workgroup, a wavefront per
// 16) and decodeMlaRolesKernel (64 heads per workgroup, a score and a value wavefront per SIMD); further down.
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

constexpr int kMlaThreads = 128; // two wavefronts per unit of work

// VALUE: 512 (latent attention), or 576: plain attention with heads of 576, a shape of the reference's tests
// (test/infiniop/paged_attention.py:106, nvidia/paged_attention_hd576.cu). A wavefront's half of the value columns is
// then 288 wide: the two strips of 128 and a tail of 32, of which lane c owns columns 256 + 2c and 256 + 2c + 1
// (4-byte loads and stores).
template <int VALUE>
struct MlaGeometry {
    static_assert(VALUE == kMlaValueSize || VALUE == kMlaKeySize, "values as wide as the latent part or as the keys");
    static constexpr int kSteps = kMlaKeySize / 32;       // K-steps of K.Q^T
    static constexpr int kChunksPerRow = kMlaKeySize / 8; // 16-byte chunks in one K row
    static constexpr int kLoads = 8 * kChunksPerRow / 64; // K load instructions per tile and wavefront (8 rows)
    static constexpr int kLdsPitch = kChunksPerRow + 1;   // chunks between consecutive rows in LDS
    static constexpr int kHalf = VALUE / 2;               // value columns per wavefront
    static constexpr int kStrips = kHalf / 128;           // 16-byte strips of one V row per lane
    static constexpr int kTail = kHalf - 128 * kStrips;   // columns after the strips: 0 or 32
    static constexpr int kPairs = 4 * kStrips + kTail / 32; // pairs of V / output columns per lane
    static constexpr int kCols = 2 * kPairs;              // V / output columns per lane
    // row (0..7 of the wavefront's eight) and chunk of the piece lane `lane` fetches in instruction j
    static __device__ __forceinline__ int kRow(int j, int lane) { return (64 * j + lane) / kChunksPerRow; }
    static __device__ __forceinline__ int kChunk(int j, int lane) { return (64 * j + lane) % kChunksPerRow; }
    static __device__ __forceinline__ int ldsIndex(int row, int chunk) { return row * kLdsPitch + chunk; }
};

template <typename T, typename Tindex, int VALUE>
__global__ void __launch_bounds__(kMlaThreads, 2) decodeMlaKernel(DecodeArgs a) {
    using S = typename T::storage;
    using G = MlaGeometry<VALUE>;
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
    uint32_t k_off[G::kLoads], v_off[4], v_tail_off[4];
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
            v_tail_off[j] = (4 * g + j) * v_row_bytes + 256 * G::kStrips + 4 * c;
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
    auto loadVStrip = [&](int t, int i, uint32_t (&v)[4][G::kPairs]) {
        const uint32_t lane_mask = t < n_tiles ? 0xffffffffu : 0u;
        const char *tile = tileAddress(t, v_head, a.v_batch_stride, a.v_row_stride);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint4 x = loadLane16(tile + 256 * i, v_off[j] & lane_mask);
            v[j][4 * i] = x.x, v[j][4 * i + 1] = x.y, v[j][4 * i + 2] = x.z, v[j][4 * i + 3] = x.w;
        }
    };
    // The tail: v[j][4 kStrips] = token row 4g + j, columns (kHalf wave) + 128 kStrips + 2 c, + 2 c + 1
    auto loadVTail = [&](int t, uint32_t (&v)[4][G::kPairs]) {
        if constexpr (G::kTail != 0) {
            const uint32_t lane_mask = t < n_tiles ? 0xffffffffu : 0u;
            const char *tile = tileAddress(t, v_head, a.v_batch_stride, a.v_row_stride);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v[j][4 * G::kStrips] = loadLane4(tile, v_tail_off[j] & lane_mask);
            }
        }
    };

    // o[8 i + e][r] = O[head 4g + r of the chunk][column (kHalf wave) + 128 i + 8 c + e]; the tail: o[8 kStrips + e],
    // column (kHalf wave) + 128 kStrips + 2 c + e
    f32x4 o[G::kCols];
#pragma unroll
    for (int e = 0; e < G::kCols; ++e) {
        o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float m = -INFINITY; // running maximum of head c (same value in the four lanes g = 0..3)
    float l = 0.0f;      // sum of rounded probabilities of head c over this lane's tokens only

    uint4 k[G::kLoads];
    uint32_t v[4][G::kPairs];
    loadK(0, k);
#pragma unroll
    for (int i = 0; i < G::kStrips; ++i) {
        loadVStrip(0, i, v);
    }
    loadVTail(0, v);
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
        if constexpr (G::kTail != 0) {
            constexpr int w = 4 * G::kStrips;
            accumulatePair<T>(o[2 * w], o[2 * w + 1], v[0][w], v[1][w], v[2][w], v[3][w], p_op, p_lo, g, valid);
            loadVTail(t + 1, v);
        }
    }

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
            if constexpr (G::kTail != 0) {
                constexpr int e = 8 * G::kStrips;
                *reinterpret_cast<uint32_t *>(o_ptr + 128 * G::kStrips - 6 * c) = T::pack2(o[e][rr] * inv_l, o[e + 1][rr] * inv_l);
            }
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            float *dst = a.part_acc + slot * VALUE + col0;
#pragma unroll
            for (int i = 0; i < G::kStrips; ++i) {
                reinterpret_cast<float4 *>(dst + 128 * i)[0] = make_float4(o[8 * i + 0][rr], o[8 * i + 1][rr], o[8 * i + 2][rr], o[8 * i + 3][rr]);
                reinterpret_cast<float4 *>(dst + 128 * i)[1] = make_float4(o[8 * i + 4][rr], o[8 * i + 5][rr], o[8 * i + 6][rr], o[8 * i + 7][rr]);
            }
            if constexpr (G::kTail != 0) {
                constexpr int e = 8 * G::kStrips;
                *reinterpret_cast<float2 *>(dst + 128 * G::kStrips - 6 * c) = make_float2(o[e][rr], o[e + 1][rr]);
            }
            if (c == 0 && wave == 0) {
                a.part_m[slot] = m_h;
                a.part_l[slot] = l_h;
            }
        }
    }
}

// ---- workgroups of eight wavefronts on tiles of 32 tokens ------------------------------------------------
// decodeMlaChunkKernel gives the 16 query heads of one (partition, sequence) a workgroup of EIGHT wavefronts; a K / V
// tile of 32 tokens (two halves of 16, each inside one page) goes through LDS, double-buffered.
//   * copy: wavefronts 0..3 fetch the V tile, one 128-column quarter each (lane (g, c): token rows
//     4g..4g+3 of both halves, one 8-column strip), and store it already transposed into matrix-operand
//     order (per column, the eight tokens of a lane as one 16-byte word); wavefronts 4..7 fetch the K
//     tile as flat 16-byte chunks (nine load instructions each, every one inside one half) and store it
//     row-major with a pitch of 73 chunks (conflict-free for both the row-major writes and the
//     column-of-16-rows reads).
//   * compute: wavefront w computes the partial scores of token half w % 2 over a quarter of the K-steps (5, 5, 4, 4
//     of the 18; its query slice in registers), all eight exchange them through LDS, run the same softmax, and each
//     owns 64 value columns (16 accumulator registers; P . V as 32-deep matrix instructions). Two workgroup
//     barriers per tile.
// Partial results and their merge are those of the kernel above. (More than 16 heads per KV head: decodeMlaRowsKernel,
// at the end of the file.)
constexpr int kMlaWideThreads = 512;
constexpr int kMlaWideTileTokens = 32; // two halves of 16
// K / V operands of these kernels are requested from LDS this many matrix instructions before the one that takes
// them: every operand feeds a single instruction (16 clocks) and an LDS read takes several times that.
constexpr int kMlaOperandsAhead = 6;     // decodeMlaChunkKernel
constexpr int kMlaQuadOperandsAhead = 4; // decodeMlaRowsKernel with one wavefront per SIMD (two with two)
// The kernels on 32-token tiles feed the probabilities to P.V as one term in the storage dtype, as the prefill kernel
// does. They are bound by LDS traffic and instruction issue, not by memory, and the second term that the other decode
// kernels add for bf16 (decode_tiled.h: p = hi + lo) costs 16 more matrix and ~50 more vector instructions per
// wavefront and tile while the largest error against the fp32 oracle at the 128-head shape moves from 0.96e-3 to
// 1.01e-3 (77 -> 73 us per call with the kernel of the time).
constexpr bool kMlaWideSplitProbabilities = false;

// Online-softmax step of one 32-token tile. s0 / s1 = raw scores of head c for tokens 4g..4g+3 of the
// first / second half; the rest as softmaxStep (decode_tiled.h). The probabilities come back as the A
// operand of a 32-deep matrix instruction whose k index 8g + j stands for token 4g + j of the first
// half (j < 4) or token 4g + j - 4 of the second.
// ACC_HALF: the accumulators o live in the accumulation half of the register file (where the matrix instructions of a
// kernel that may use more than 256 registers keep their results).
template <typename T, int COLS, bool ACC_HALF = false>
__device__ __forceinline__ void softmaxStepPair(f32x4 (&o)[COLS], float &m, float &l, const f32x4 s0, const f32x4 s1, int g,
                                                float scale_log2, float slope, int rel_pos0, int valid, uint4 &p_op,
                                                uint4 &p_lo) {
    float sc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        sc[i] = (i < 4 ? s0[i & 3] : s1[i & 3]) * scale_log2;
    }
    // wave-uniform branches: ALiBi is rare, and only the last tile of a partition can be short
    if (__builtin_amdgcn_ballot_w64(slope != 0.0f) != 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            sc[i] += slope * static_cast<float>(rel_pos0 + 16 * (i >> 2) + 4 * g + (i & 3));
        }
    }
    if (valid < kMlaWideTileTokens) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            sc[i] = (16 * (i >> 2) + 4 * g + (i & 3) >= valid) ? -INFINITY : sc[i];
        }
    }
    // this lane's eight tokens; the head's maximum (four lanes) is only formed when it is needed (see softmaxStep)
    const float mx_lane = maxOf(maxOf(maxOf(sc[0], sc[1]), maxOf(sc[2], sc[3])),
                                maxOf(maxOf(sc[4], sc[5]), maxOf(sc[6], sc[7])));
    if (__builtin_amdgcn_ballot_w64(mx_lane > m + kLazyRescaleLog2) != 0) {
        const float m_new = maxOf(m, maxAcrossTokenGroups(mx_lane));
        // rescale (see softmaxStep). Lane holds accumulators of heads 4g..4g+3, whose factors live in
        // lanes 4g..4g+3.
        const float alpha = fastExp2(m - m_new);
        l *= alpha;
        m = m_new;
        float alpha_r[4];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            alpha_r[rr] = __shfl(alpha, 4 * g + rr, 64);
        }
#pragma unroll
        for (int e = 0; e < COLS; ++e) {
            f32x4 x = o[e];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                x[rr] *= alpha_r[rr];
            }
            o[e] = x;
        }
    }
    uint32_t hi[4], lo[4] = {0, 0, 0, 0};
    float p_used = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float pa = fastExp2(sc[2 * i] - m), pb = fastExp2(sc[2 * i + 1] - m);
        hi[i] = T::pack2(pa, pb);
        p_used += T::unpackLo(hi[i]) + T::unpackHi(hi[i]);
        if constexpr (T::kSplitProbabilities && kMlaWideSplitProbabilities) {
            lo[i] = T::pack2(pa - T::unpackLo(hi[i]), pb - T::unpackHi(hi[i]));
            p_used += T::unpackLo(lo[i]) + T::unpackHi(lo[i]);
        }
    }
    p_op = make_uint4(hi[0], hi[1], hi[2], hi[3]);
    p_lo = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    l += p_used;
}

// One workgroup per compute unit, 32 compute units per accelerator die, workgroups dealt to the eight dies
// round-robin by linear id: 280 workgroups take as long as 512, and so do 230 if one die gets 33 of them.
// Batches of up to 256 sequences are therefore planned by every workgroup for itself from the actual
// lengths (the host only knows the width of the block table); same inputs, same answer in every wavefront,
// no LDS, no barrier:
//   * partition size of the call: among the planned size and larger ones, in steps of 64 tokens up to what
//     one page-id load covers (64 pages) or 1024 tokens, the one that needs the fewest tiles in a row,
//     i.e. (rounds of workgroups) x (tiles per partition); ties go to the larger size (fewer partial
//     results);
//   * the (sequence, partition) units are numbered densely; linear workgroup id = 8 streams (u / 8) +
//     8 stream + u % 8, so the units that exist come first, the dies get equal shares, and the workgroups
//     of one unit (one per group of head chunks) sit on the same die and meet in its L2.
struct WidePlan {
    int partition_tokens;
    int seq, part, stream; // this workgroup's unit; seq < 0: none
    int len;               // length of that sequence, clamped to [0, what its block-table row can hold]
};

template <typename Tindex>
__device__ __forceinline__ WidePlan planWide(const DecodeArgs &a, int lane, int streams, int linear_id) {
    WidePlan plan{a.partition_tokens, -1, 0, 0, 0};
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) << a.block_shift;
    // Lanes hold up to four lengths each; a batch of at most 64 sequences fills one of the four slots, and
    // the arithmetic on the empty ones (three quarters of the search below) is skipped: wave-uniform tests.
    const int slots = (a.num_seqs + 63) >> 6;
    // what an earlier call left of its search (see below), asked for in the same round trip as the lengths
    unsigned long long *const remembered = reinterpret_cast<unsigned long long *>(a.chosen_partition + 2);
    const unsigned long long seen = *remembered;
    int lens[4]; // the lengths once (one round of independent loads)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int64_t len = 0;
        if (64 * i + lane < a.num_seqs) {
            len = loadIndex<Tindex>(a.seq_lens, 64 * i + lane);
            len = len < 0 ? 0 : (len < max_len ? len : max_len);
        }
        lens[i] = static_cast<int>(len);
    }
    // The search: cost(p) = (rounds of workgroups) x (tiles per partition).
    const int cap = min(64 << a.block_shift, 1024);
    auto roundsAt = [&](int p) {
        // partitions of this lane's sequences: ceil(len / p) through the reciprocal, corrected to be exact
        // (lengths above 2^24 are rounded, which only blunts the estimate)
        const float pf = static_cast<float>(p), inv = 1.0f / pf;
        int x = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (i >= slots) {
                break;
            }
            const float lf = static_cast<float>(lens[i]);
            float q = floorf(lf * inv);
            q = q * pf > lf ? q - 1.0f : q;          // one too many
            q = (q + 1.0f) * pf <= lf ? q + 1.0f : q; // one too few
            x += static_cast<int>(q) + (q * pf < lf ? 1 : 0);
        }
        const int workgroups = __builtin_amdgcn_readlane(waveInclusiveSum(x), 63) * streams;
        return (workgroups + a.compute_units - 1) / a.compute_units;
    };
    const int first_rounds = roundsAt(a.partition_tokens);
    // (one round at the planned size: everything runs at once, larger partitions only take longer)
    if (first_rounds > 1 && a.partition_tokens + 64 <= cap) {
        // The rest of the search is the same for every call on the same lengths - the layers of a model's decode
        // step, one after the other - so its result is remembered beside the partition size left for the merge
        // kernel: one 64-bit word, a 56-bit hash of everything the search looks at above the size in units of 64
        // tokens (one word: a reader never sees the hash of one call with the size of another). Every workgroup of
        // a call takes the same branch, because those that miss all arrive at the value the first one writes. A
        // stale or colliding entry can only hold a size this search could have chosen for this shape (the hash
        // covers the shape, the checks below the range), i.e. it costs time, never correctness.
        unsigned h1 = 0, h2 = 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (i >= slots) {
                break;
            }
            unsigned x = static_cast<unsigned>(lens[i]) * 0x9E3779B1u + static_cast<unsigned>(64 * i + lane) * 0x85EBCA77u;
            x ^= x >> 15;
            h1 += x * 0x2C1B3C6Du;
            h2 += (x ^ 0x27D4EB2Fu) * 0x165667B1u;
        }
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) {
            h1 += __shfl_xor(h1, off, 64);
            h2 += __shfl_xor(h2, off, 64);
        }
        h1 += static_cast<unsigned>(a.partition_tokens) * 0x9E3779B1u + static_cast<unsigned>(streams) * 0x85EBCA77u;
        h2 += static_cast<unsigned>(a.num_seqs) * 0xC2B2AE3Du + static_cast<unsigned>(a.compute_units) * 0x27D4EB2Fu + static_cast<unsigned>(a.block_shift);
        const unsigned long long key = ((static_cast<unsigned long long>(h1) << 32) | h2) & ~0xffull;
        const int seen_steps = static_cast<int>(seen & 0xff); // remembered size = planned size + 64 x this
        if ((seen & ~0xffull) == key && a.partition_tokens + 64 * seen_steps <= cap) {
            plan.partition_tokens = a.partition_tokens + 64 * seen_steps;
        } else {
            int best_cost = first_rounds * ((a.partition_tokens + kMlaWideTileTokens - 1) / kMlaWideTileTokens);
            for (int p = a.partition_tokens + 64; p <= cap; p += 64) {
                const int cost = roundsAt(p) * ((p + kMlaWideTileTokens - 1) / kMlaWideTileTokens);
                if (cost <= best_cost) { // ties go to the larger size (fewer partial results)
                    best_cost = cost;
                    plan.partition_tokens = p;
                }
            }
            if (linear_id == 0 && lane == 0) {
                *remembered = key | static_cast<unsigned long long>((plan.partition_tokens - a.partition_tokens) / 64);
            }
        }
    }
    // dense unit of this workgroup
    const int p = plan.partition_tokens;
    const int group_of_8 = linear_id / (8 * streams), rest = linear_id - group_of_8 * (8 * streams);
    plan.stream = rest >> 3;
    const int u = 8 * group_of_8 + (rest & 7);
    int running = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (i >= slots) {
            break;
        }
        const int k = (lens[i] + p - 1) / p;
        const int incl = waveInclusiveSum(k) + running;
        const unsigned long long hit = __builtin_amdgcn_ballot_w64(incl > u);
        if (hit != 0 && plan.seq < 0) {
            const int first = __builtin_ctzll(hit);
            plan.seq = 64 * i + first;
            plan.part = u - (__builtin_amdgcn_readlane(incl, first) - __builtin_amdgcn_readlane(k, first));
            plan.len = __builtin_amdgcn_readlane(lens[i], first);
        }
        running = __builtin_amdgcn_readlane(incl, 63);
    }
    return plan;
}

// Which (sequence, partition, stream = KV head x group of head chunks) a workgroup of the 64-head kernels works on, and
// the partition size of the call. Everything depends on the workgroup only, so all its wavefronts get the same
// answer. False: no unit for this workgroup. `len` = length of the sequence, clamped to what its block-table row can
// hold.
template <typename Tindex>
__device__ __forceinline__ bool locateWideUnit(const DecodeArgs &a, int lane, int groups_of_chunks, int &seq, int &part,
                                               int &stream, int &partition_tokens, int &len) {
    if (a.chosen_partition != nullptr) {
        // planned per call (see planWide): one-dimensional grid
        const WidePlan plan = planWide<Tindex>(a, lane, a.num_kv_heads * groups_of_chunks, static_cast<int>(blockIdx.x));
        if (blockIdx.x == 0 && threadIdx.x == 0) {
            a.chosen_partition[0] = plan.partition_tokens; // for the merge kernel
        }
        if (plan.seq < 0) {
            return false;
        }
        // wave-uniform by construction; saying so keeps the address arithmetic in scalar registers
        seq = __builtin_amdgcn_readfirstlane(plan.seq);
        part = __builtin_amdgcn_readfirstlane(plan.part);
        stream = __builtin_amdgcn_readfirstlane(plan.stream);
        partition_tokens = __builtin_amdgcn_readfirstlane(plan.partition_tokens);
        len = __builtin_amdgcn_readfirstlane(plan.len); // the plan has read it already: no second round trip
        return true;
    }
    // fixed partitions on a three-dimensional grid, rotated as in decodeMlaKernel
    seq = blockIdx.z;
    part = static_cast<int>((blockIdx.x + blockIdx.z) % gridDim.x);
    stream = blockIdx.y;
    partition_tokens = a.partition_tokens;
    const int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) << a.block_shift;
    len = static_cast<int>(len64 < max_len ? len64 : max_len);
    return true;
}

template <typename T, typename Tindex>
__global__ void __launch_bounds__(kMlaWideThreads, 2) decodeMlaChunkKernel(DecodeArgs a) {
    constexpr int kOwnSteps = 5;  // K-steps of one wavefront (the last of the five may be empty)
    constexpr int kOwnBlocks = 4; // 16-column blocks of one wavefront
    using S = typename T::storage;
    constexpr int kSteps = kMlaKeySize / 32;        // 18
    constexpr int kChunksPerRow = kMlaKeySize / 8;  // 72 16-byte chunks in a K row
    constexpr int kPitch = kChunksPerRow + 1;
    constexpr int kHalfChunks = kTileTokens * kChunksPerRow; // 1152 chunks in a half
    constexpr int kLoads = 2 * kHalfChunks / 256;            // 9 load instructions per copying wavefront
    constexpr int kBlocks = kMlaValueSize / 16;              // 32 column blocks of 16
    __shared__ uint4 k_lds[2][kMlaWideTileTokens * kPitch];
    __shared__ uint4 v_lds[2][kBlocks * 64];  // [column block][token group g][lane c]: .xy first half, .zw second
    __shared__ f32x4 s_lds[8][64]; // partial scores of every wavefront

    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int groups_of_chunks = head_chunks; // a workgroup per chunk
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;

    // Which (sequence, partition, KV head x head chunk) this workgroup works on. Everything
    // up to the first barrier depends on the workgroup only, so all wavefronts leave together.
    int seq, part, stream, partition_tokens;
    int len; // of the sequence, clamped to what its block-table row can hold
    if (!locateWideUnit<Tindex>(a, lane, groups_of_chunks, seq, part, stream, partition_tokens, len)) {
        return;
    }
    const int kv_head = stream / groups_of_chunks;
    const int chunk = stream - kv_head * groups_of_chunks;
    // this wavefront's K-steps: [first_step, first_step + own_steps)
    const int first_step = (wave >> 1) * 5 - ((wave >> 1) == 3 ? 1 : 0);
    const int own_steps = (wave >> 1) < 2 ? 5 : 4;
    const int th = wave & 1; // the token half whose scores this wavefront computes

    const int start = part * partition_tokens;
    if (len <= 0 || start >= len) {
        return;
    }
    const int end = min(len, start + partition_tokens);
    const int n_tiles = (end - start + kMlaWideTileTokens - 1) / kMlaWideTileTokens;

    const int first_entry = start >> a.block_shift;
    const int last_entry = (end - 1) >> a.block_shift;
    int page_ids = 0;
    if (first_entry + lane <= last_entry) {
        page_ids = clampPage(
            loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + first_entry + lane), a.num_blocks);
    }

    // Query of head (chunk*16 + c): columns 32 (first_step + i) + 8g .. +7, the B operand of this wavefront's K-steps
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    uint4 q_reg[kOwnSteps];
    {
        const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
#pragma unroll
        for (int i = 0; i < kOwnSteps; ++i) {
            const int kk = min(first_step + i, kSteps - 1);
            const uint32_t keep = (head_valid && i < own_steps) ? 0xffffffffu : 0u; // an empty step multiplies by zero
            uint4 x = *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g);
            x.x &= keep, x.y &= keep, x.z &= keep, x.w &= keep;
            q_reg[i] = x;
        }
    }
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;

    // ---- copy side: one code path for both roles (the V wavefronts' ninth load repeats their first) ----
    const bool copies_v = wave < 4;
    const int role_wave = wave & 3;
    const char *copy_head = copies_v
        ? reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride)
        : reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const int64_t copy_batch_stride = copies_v ? a.v_batch_stride : a.k_batch_stride;
    const int64_t copy_row_stride = copies_v ? a.v_row_stride : a.k_row_stride;
    const int block_mask = a.block_size - 1;
    // Load j of a wavefront: which half of the tile (wave-uniform), this lane's byte offset inside the
    // half, and for K where the chunk goes in LDS.
    //   V: j = 4 h + i: token row 4g + i of half h, columns 128 role_wave + 8 c .. + 7
    //   K: wave-instruction 4 j + role_wave of 36; 18 per half, 64 consecutive chunks each
    uint32_t src_off[kLoads];
    int k_dst[kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
        if (copies_v) {
            const int i = j & 3;
            src_off[j] = (4 * g + i) * static_cast<uint32_t>(a.v_row_stride) * sizeof(S) + 256 * role_wave + 16 * c;
            k_dst[j] = 0;
        } else {
            const int inst = 4 * j + role_wave;
            const int ch = 64 * (inst % 18) + lane; // chunk within the half
            const int row = ch / kChunksPerRow, col = ch - row * kChunksPerRow;
            src_off[j] = row * static_cast<uint32_t>(a.k_row_stride) * sizeof(S) + 16 * col;
            k_dst[j] = (16 * (inst / 18) + row) * kPitch + col;
        }
    }
    auto halfOfLoad = [&](int j) { return copies_v ? ((j >> 2) & 1) : ((4 * j + role_wave) / 18); };

    // Register sets for tiles on their way: one (tile t + 1 while tile t is computed). A second set fits
    // the single-chunk variant (185 registers, no spills) and was measured: 38.7 vs 37.6 us at 32 sequences,
    // 139 vs 136 at 128 - one more tile in flight is not what holds that variant back. The four-chunk variant
    // (211 registers with one set) does not take a second one: 256 registers and 100 spilled, inside the loop.
    constexpr int kSets = 1;
    uint4 stage_sets[kSets][kLoads];
#pragma unroll
    for (int j = 0; j < kLoads; ++j) {
#pragma unroll
        for (int i = 0; i < kSets; ++i) {
            stage_sets[i][j] = make_uint4(0, 0, 0, 0);
        }
    }
    // Loads for a half past the end of the partition are issued all the same but read the partition's
    // first rows (the loop body has no branch around a load).
    auto loadStage = [&](int t, uint4 (&stage)[kLoads]) {
        const char *half_base[2];
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            int tok0 = start + t * kMlaWideTileTokens + 16 * h;
            tok0 = tok0 < end ? tok0 : start;
            const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
            const int row0 = tok0 & block_mask;
            half_base[h] = copy_head + (page * copy_batch_stride + row0 * copy_row_stride) * static_cast<int64_t>(sizeof(S));
        }
#pragma unroll
        for (int j = 0; j < kLoads; ++j) {
            stage[j] = loadLane16(halfOfLoad(j) ? half_base[1] : half_base[0], src_off[j]);
        }
    };
    auto storeStage = [&](int t, const uint4 (&stage)[kLoads]) {
        const int buf = t & 1;
        if (copies_v) {
            // V rows beyond the sequence may hold anything (NaN included) and 0 * NaN is NaN: zeroed here
            const bool full_tile = end - (start + t * kMlaWideTileTokens) >= kMlaWideTileTokens;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int valid = end - (start + t * kMlaWideTileTokens + 16 * h);
                uint32_t r[4][4]; // [token row i][dword]
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    r[i][0] = stage[4 * h + i].x, r[i][1] = stage[4 * h + i].y;
                    r[i][2] = stage[4 * h + i].z, r[i][3] = stage[4 * h + i].w;
                }
                if (!full_tile) { // only the last tile of a partition can be short
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        if (4 * g + i >= valid) {
                            r[i][0] = r[i][1] = r[i][2] = r[i][3] = 0u;
                        }
                    }
                }
#pragma unroll
                for (int wd = 0; wd < 4; ++wd) {
                    uint2 even, odd;
                    even.x = __builtin_amdgcn_perm(r[1][wd], r[0][wd], 0x05040100u);
                    even.y = __builtin_amdgcn_perm(r[3][wd], r[2][wd], 0x05040100u);
                    odd.x = __builtin_amdgcn_perm(r[1][wd], r[0][wd], 0x07060302u);
                    odd.y = __builtin_amdgcn_perm(r[3][wd], r[2][wd], 0x07060302u);
                    // column 128 role_wave + 8 c + 2 wd (+1) -> block 8 role_wave + 2 wd (+1), lane c
                    uint2 *dst_even = reinterpret_cast<uint2 *>(&v_lds[buf][((8 * role_wave + 2 * wd) * 4 + g) * 16 + c]) + h;
                    uint2 *dst_odd = reinterpret_cast<uint2 *>(&v_lds[buf][((8 * role_wave + 2 * wd + 1) * 4 + g) * 16 + c]) + h;
                    *dst_even = even;
                    *dst_odd = odd;
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < kLoads; ++j) {
                k_lds[buf][k_dst[j]] = stage[j];
            }
        }
    };

    // o[e][r] = O[head 4g + r][column 128 (wave / 2) + 8 c + 4 (wave % 2) + e]
    f32x4 o[kOwnBlocks];
#pragma unroll
    for (int e = 0; e < kOwnBlocks; ++e) {
        o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    const int first_block = 4 * wave;
    float m = -INFINITY; // reference point of head c's exponentials (same value in the four lanes g = 0..3)
    float l = 0.0f;      // sum of rounded probabilities of head c over this lane's tokens only

    // Tile t is computed from LDS buffer t & 1 while tile t + 1 (and, with two register sets, t + 2) is
    // on its way: set (t + 1) % kSets is stored at the start of tile t and refilled right away. With two
    // sets, two tiles per trip so that the sets are addressed statically.
    loadStage(0, stage_sets[0]);
    if constexpr (kSets == 2) {
        loadStage(1, stage_sets[1]);
    }
    storeStage(0, stage_sets[0]);
    loadStage(kSets, stage_sets[0]);
    for (int t0 = 0; t0 < n_tiles; t0 += kSets) {
#pragma unroll
    for (int d = 0; d < kSets; ++d) {
        const int t = t0 + d;
        if (t >= n_tiles) {
            break; // the same for all wavefronts: they pass the same barriers
        }
        const int buf = kSets == 2 ? d : (t & 1);
        __syncthreads(); // tile t is complete in LDS, and everybody has finished with tile t - 1
        uint4 (&next_set)[kLoads] = stage_sets[kSets == 2 ? (d ^ 1) : 0];
        if (t + 1 < n_tiles) {
            storeStage(t + 1, next_set);
        }
        loadStage(t + 1 + kSets, next_set);
        f32x4 s0, s1;
        {
            // partial scores of this wavefront's token half over its quarter of the K-steps
            f32x4 sp[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            auto readK = [&](int i) { return k_lds[buf][(16 * th + c) * kPitch + 4 * min(first_step + i, kSteps - 1) + g]; };
            constexpr int kAheadOne = kOwnSteps < kMlaOperandsAhead ? kOwnSteps : kMlaOperandsAhead;
            uint4 kf[kOwnSteps];
#pragma unroll
            for (int i = 0; i < kAheadOne; ++i) {
                kf[i] = readK(i);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, kAheadOne, 0);
#pragma unroll
            for (int i = 0; i < kOwnSteps; ++i) {
                if (i + kAheadOne < kOwnSteps) {
                    kf[i + kAheadOne] = readK(i + kAheadOne);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                sp[i & 1] = T::mfmaK32(kf[i], q_reg[i], sp[i & 1]);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            s_lds[wave][lane] = sp[0] + sp[1];
            __syncthreads(); // all eight partial tiles are there: wavefront 2 q + h holds quarter q of half h
            s0 = (s_lds[0][lane] + s_lds[2][lane]) + (s_lds[4][lane] + s_lds[6][lane]);
            s1 = (s_lds[1][lane] + s_lds[3][lane]) + (s_lds[5][lane] + s_lds[7][lane]);
        }

        const int tok0 = start + t * kMlaWideTileTokens;
        const int valid = min(kMlaWideTileTokens, end - tok0);
        uint4 p_op, p_lo;
        softmaxStepPair<T, kOwnBlocks>(o, m, l, s0, s1, g, a.scale_log2, slope, tok0 - (len - 1), valid, p_op, p_lo);
        // P.V one column block after the other, its V operand requested from LDS kMlaOperandsAhead blocks ahead;
        // the low parts of the probabilities follow two blocks behind the high parts (a matrix instruction that
        // accumulates into the result of the one before waits for it)
        constexpr int kAheadV = kOwnBlocks < kMlaOperandsAhead ? kOwnBlocks : kMlaOperandsAhead;
        constexpr int kSkew = 2; // the low part of block e goes kSkew blocks behind its high part
        auto readV = [&](int e) { return v_lds[buf][((first_block + e) * 4 + g) * 16 + c]; };
        uint4 vf[kOwnBlocks];
#pragma unroll
        for (int e = 0; e < kAheadV; ++e) {
            vf[e] = readV(e);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, kAheadV, 0);
#pragma unroll
        for (int e = 0; e < kOwnBlocks + kSkew; ++e) {
            if (e + kAheadV < kOwnBlocks) {
                vf[e + kAheadV] = readV(e + kAheadV);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            if (e < kOwnBlocks) {
                o[e] = T::mfmaK32(p_op, vf[e], o[e]);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            }
            if constexpr (T::kSplitProbabilities && kMlaWideSplitProbabilities) {
                if (e >= kSkew) {
                    o[e - kSkew] = T::mfmaK32(p_lo, vf[e - kSkew], o[e - kSkew]);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                }
            }
        }
    }
    }

    // Epilogue, as in decodeMlaKernel
    const float l_tot = sumAcrossTokenGroups(l);
    const bool single = len <= partition_tokens;
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
        const int col0 = 128 * (wave >> 1) + 8 * c + 4 * (wave & 1);
        if (single) {
            const float inv_l = 1.0f / (l_h + 1e-6f);
            S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride + col0;
            uint2 w;
            w.x = T::pack2(o[0][rr] * inv_l, o[1][rr] * inv_l);
            w.y = T::pack2(o[2][rr] * inv_l, o[3][rr] * inv_l);
            *reinterpret_cast<uint2 *>(o_ptr) = w;
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            float *dst = a.part_acc + slot * kMlaValueSize + col0;
            *reinterpret_cast<float4 *>(dst) = make_float4(o[0][rr], o[1][rr], o[2][rr], o[3][rr]);
            if (c == 0 && wave == 0) {
                a.part_m[slot] = m_h;
                a.part_l[slot] = l_h;
            }
        }
    }
}

// ---- 16 query heads per wavefront, tiles straight into LDS -------------------------------------------------
// More than 16 query heads per KV head. The unit of work is a group of WAVES head chunks of a (partition, sequence),
// units planned per call like those of decodeMlaChunkKernel; the tile pipeline is that of the prefill kernel
// (paged_attention_prefill/amd/prefill_tiled.h). WAVES = 4 (up to 64 query heads per workgroup, one wavefront per
// SIMD) or 8 (up to 128 heads, two per SIMD: a tile fetched once serves twice the heads; the faster one where the
// batch fills the device without cutting the sequences finely, decode_plan.h).
//   * Wavefront w serves head chunk w: all 18 K-steps of K . Q^T for both 16-token halves of a 32-token tile (its 16
//     query rows in 72 registers), the softmax, and all 512 value columns (128 accumulator registers; P . V as 32
//     matrix instructions of depth 32). Nothing is exchanged between wavefronts.
//   * K and V tiles go from global memory straight into LDS (16 bytes per lane, no register in between),
//     double-buffered; the first half of the wavefronts brings equal parts of the K tile, the second half of the V
//     tile, one load instruction after every few K operands of the tile before. One workgroup barrier per tile.
//   * K row-major with its 16-byte chunks XOR-swizzled by the row; V row-major in blocks of 16 columns, read back
//     through the transposing LDS read, a block of 16 tokens x 16 columns at a time (512 contiguous bytes).
//   * results leave through LDS (the tile buffers) as whole rows, 16 bytes per lane.
// ONCE: the unit has this one workgroup (all the head chunks of the KV head fit it), so nobody else asks for its tiles
// and they are fetched with the non-temporal form of the load (see loadLane16ToLds).
template <typename T, typename Tindex, int WAVES, bool ONCE>
__global__ void __launch_bounds__(64 * WAVES) decodeMlaRowsKernel(DecodeArgs a) {
    static_assert(WAVES == 4 || WAVES == 8, "one or two wavefronts per SIMD");
    using S = typename T::storage;
    constexpr int kSteps = kMlaKeySize / 32;      // 18 K-steps
    constexpr int kRowK = kMlaKeySize / 8;        // 72 16-byte chunks in a K row
    constexpr int kRowV = kMlaValueSize / 8;      // 64 in a V row
    constexpr int kSwizzle = 8;                   // stays inside a K row: 72 is a multiple of 8
    constexpr int kTileK = kTileTokens * kRowK;   // chunks of a 16-token half
    constexpr int kTileV = kTileTokens * kRowV;
    constexpr int kParts = WAVES / 4;             // wavefronts that share the copy of one half of one kind
    constexpr int kLoadsK = kTileK / 64 / kParts; // load instructions of a wavefront that copies K: 18 or 9
    constexpr int kLoadsV = kTileV / 64 / kParts; // V: 16 or 8
    constexpr int kBlocks = kMlaValueSize / 16;   // 32 column blocks of 16
    constexpr int kSlots = kLoadsK;               // load instructions of one wavefront per tile (V: the last ones empty)
    constexpr int kOutRows = kHeadsPerWave / 2;   // output rows a wavefront stages in LDS at a time
    constexpr int kOutPitch = kMlaValueSize + 4;  // floats between them (conflict-free column writes)
    constexpr int kMainK = 64;                    // chunks of a K row kept in the main region of a half; the other 8 in its tail
    constexpr int kTailK = kTileTokens * kMainK;  // first slot of the tail region
    struct Tiles {
        // [buffer][half] of {main [token][64 chunks], tail [token][8 chunks]}, chunks XOR-swizzled by token % 8: a load
        // instruction fills 64 consecutive slots, i.e. the main part of one token or the tails of eight
        uint4 k[2][2 * kTileK];
        // [buffer][half][block of 16 columns][token][two 16-byte chunks]: the 64 lanes of a transposing read of one
        // block touch 512 contiguous bytes, whichever way the hardware groups them
        uint4 v[2][2 * kTileV];
    };
    __shared__ Tiles tiles;
    static_assert(sizeof(Tiles) >= WAVES * kOutRows * kOutPitch * sizeof(float), "the tile buffers hold the staged output rows of all wavefronts");

    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int groups_of_chunks = (head_chunks + WAVES - 1) / WAVES;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;

    int seq, part, stream, partition_tokens, len;
    if (!locateWideUnit<Tindex>(a, lane, groups_of_chunks, seq, part, stream, partition_tokens, len)) {
        return;
    }
    const int kv_head = stream / groups_of_chunks;
    const int chunk = (stream - kv_head * groups_of_chunks) * WAVES + wave; // may lie beyond the last chunk: no heads
    const int start = part * partition_tokens;
    if (len <= 0 || start >= len) {
        return;
    }
    const int end = min(len, start + partition_tokens);
    const int n_tiles = (end - start + kMlaWideTileTokens - 1) / kMlaWideTileTokens;

    const int first_entry = start >> a.block_shift;
    const int last_entry = (end - 1) >> a.block_shift;
    int page_ids = 0;
    if (first_entry + lane <= last_entry) {
        page_ids = clampPage(
            loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + first_entry + lane), a.num_blocks);
    }

    // Query of head (chunk*16 + c): columns 32 kk + 8g .. +7, the B operand of K-step kk
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    uint4 q_reg[kSteps];
    {
        const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
        const uint32_t keep = head_valid ? 0xffffffffu : 0u;
#pragma unroll
        for (int kk = 0; kk < kSteps; ++kk) {
            uint4 x = *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g);
            x.x &= keep, x.y &= keep, x.z &= keep, x.w &= keep;
            q_reg[kk] = x;
        }
    }
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;

    // ---- copy side: wavefront w < WAVES / 2 brings part w of the K tile, wavefront WAVES / 2 + w part w of the V
    // tile; a part is a half (16 tokens, inside one page) or, with eight wavefronts, eight rows of one ----
    const bool copies_k = wave < WAVES / 2;
    const int copy_part = wave % (WAVES / 2);
    const int copy_half = copy_part / kParts;
    const int copy_sub = copy_part % kParts;
    const char *copy_head = copies_k
        ? reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride)
        : reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
    const int64_t copy_batch_stride = copies_k ? a.k_batch_stride : a.v_batch_stride;
    const int64_t copy_row_stride = copies_k ? a.k_row_stride : a.v_row_stride;
    const int copy_loads = copies_k ? kLoadsK : kLoadsV;
    const int block_mask = a.block_size - 1;
    // Load instruction j of a wavefront fills LDS slots [slot0(j), slot0(j) + 64) of its half, lane i the i-th, from
    // (row(j) of the half, uniform) + (this lane's piece). With R = 8 copy_sub the wavefront's first row:
    //   K, j < rows:  the main part of row R + j: slot0 = 64 (R + j); lane asks for chunk lane ^ (row % 8)
    //   K, j >= rows: the tails of rows R + 8 (j - rows) .. + 7: slot0 = tail + 8 (that row); lane asks for chunk
    //                 64 + (lane % 8 ^ row % 8) of row (that row) + lane / 8
    //   V:            slot0 = 64 (loads per wavefront x copy_sub + j), two blocks of 16 columns: row (lane % 32) / 2,
    //                 chunk 4 (that j) + 2 (lane / 32) + lane % 2 (the layout at Tiles; 64 contiguous bytes of a row)
    // so two registers hold every lane-dependent offset (lane_main, XORed with a constant per instruction, and
    // lane_tail) and the rest is scalar arithmetic.
    constexpr int kRowsK = 16 / kParts; // rows of the half this wavefront copies (K)
    const uint32_t k_row_bytes = static_cast<uint32_t>(a.k_row_stride) * sizeof(S);
    const uint32_t v_row_bytes = static_cast<uint32_t>(a.v_row_stride) * sizeof(S);
    const int copy_row0 = kRowsK * copy_sub;
    const uint32_t lane_main = copies_k ? 16u * lane : ((lane & 31) >> 1) * v_row_bytes + 16u * (2 * (lane >> 5) + (lane & 1));
    const uint32_t lane_tail = (lane >> 3) * k_row_bytes + 16u * (kMainK + ((lane & 7) ^ (lane >> 3))); // rows R + 8 q + lane / 8: same row % 8 as lane / 8
    auto slotLaneOffset = [&](int j) -> uint32_t {
        if (!copies_k) {
            return lane_main;
        }
        return j < kRowsK ? (lane_main ^ (16u * ((copy_row0 + j) & (kSwizzle - 1)))) : lane_tail;
    };
    auto slotRowOffset = [&](int j) -> uint32_t { // uniform part, bytes
        if (!copies_k) {
            return 64u * (kLoadsV * copy_sub + j);
        }
        return (j < kRowsK ? copy_row0 + j : copy_row0 + 8 * (j - kRowsK)) * k_row_bytes;
    };
    auto slotLds = [&](int j) -> int { // first slot within the half
        if (!copies_k) {
            return 64 * (kLoadsV * copy_sub + j);
        }
        return j < kRowsK ? kMainK * (copy_row0 + j) : kTailK + 8 * (copy_row0 + 8 * (j - kRowsK));
    };
    auto vRowOfLoad = [&](int) { return (lane & 31) >> 1; };
    // The load instructions of a tile are not issued in one burst after the barrier but one at a time between the
    // matrix instructions of the tile before (see the prefill kernel): stageTile records where they read and write,
    // issueSlot(i) issues the i-th. A half that ends beyond the partition takes the lane-by-lane path at once: K rows
    // beyond the end are not needed (their scores are replaced), V rows beyond it are zeroed (they may hold anything,
    // NaN included, and 0 * NaN is NaN).
    const char *pend_src = copy_head;
    uint4 *pend_dst = &tiles.k[0][0];
    unsigned long long pend_live = 0ull;
    auto issueSlot = [&](int i) {
        loadLane16ToLdsMasked<ONCE>(pend_src + slotRowOffset(i), slotLaneOffset(i), pend_dst + slotLds(i), i < copy_loads ? pend_live : 0ull);
    };
    // true: the stage is exactly copy_loads load instructions of this wavefront (what a counted wait relies on)
    auto stageTile = [&](int t, bool deferred) -> bool {
        pend_live = 0ull;
        const int tok0 = start + t * kMlaWideTileTokens + kTileTokens * copy_half;
        uint4 *dst = copies_k ? &tiles.k[t & 1][copy_half * kTileK] : &tiles.v[t & 1][copy_half * kTileV];
        if (tok0 >= end) {
            if (!copies_k) { // nothing of this half is used, but what P . V multiplies by zero has to be finite
#pragma unroll
                for (int j = 0; j < kLoadsV; ++j) {
                    dst[slotLds(j) + lane] = make_uint4(0, 0, 0, 0);
                }
            }
            return false;
        }
        const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
        const char *src = copy_head + (page * copy_batch_stride + (tok0 & block_mask) * copy_row_stride) * static_cast<int64_t>(sizeof(S));
        if (copies_k || tok0 + kTileTokens <= end) {
            if (deferred) {
                pend_src = src, pend_dst = dst, pend_live = ~0ull;
            } else {
#pragma unroll
                for (int j = 0; j < kSlots; ++j) {
                    if (j < copy_loads) {
                        loadLane16ToLds<ONCE>(src + slotRowOffset(j), slotLaneOffset(j), dst + slotLds(j));
                    }
                }
            }
            return true;
        }
#pragma unroll
        for (int j = 0; j < kLoadsV; ++j) {
            if (tok0 + vRowOfLoad(j) < end) {
                loadLane16ToLds<ONCE>(src + slotRowOffset(j) + slotLaneOffset(j), dst + slotLds(j));
            } else {
                dst[slotLds(j) + lane] = make_uint4(0, 0, 0, 0);
            }
        }
        return false;
    };

    // o[e][r] = O[head 4g + r of the chunk][column 16 e + c]
    f32x4 o[kBlocks];
#pragma unroll
    for (int e = 0; e < kBlocks; ++e) {
        o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float m = -INFINITY; // reference point of head c's exponentials (same value in the four lanes g = 0..3)
    float l = 0.0f;      // sum of rounded probabilities of head c over this lane's tokens only

    // this lane's chunk of row c in K-step kk, within a half: chunk 4 kk + g of the row, XOR-swizzled, i.e.
    // 8 (kk / 2) + ((4 (kk % 2) + g) ^ (c % 8)), in the main region up to K-step 15 and in the tail after
    const int k_read_index[2] = {c * kMainK + (g ^ (c & (kSwizzle - 1))), c * kMainK + ((4 + g) ^ (c & (kSwizzle - 1)))};
    const int k_read_tail = kTailK + c * 8 - c * kMainK; // added to k_read_index for the last two K-steps
    // this lane's piece of a transposing V read, relative to block 0 of half 0 of buffer 0: lane (g, c) points at
    // token 4g + c / 4, columns 16 e + 4 (c % 4) .. + 3 and receives tokens 4g .. 4g + 3 of column 16 e + c
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 *LdsPiece;
    const auto v_read_base = (__attribute__((address_space(3))) char *)tiles.v
                           + 16 * ((4 * g + (c >> 2)) * 2 + ((c & 3) >> 1)) + 8 * (c & 1);

    f32x4 s0, s1; // raw scores of head c for tokens 4g .. 4g + 3 of the first / second half of the tile
    auto computeScores = [&](int buf) {
        // K . Q^T: operand idx = (K-step idx / 2, half idx % 2); independent chains: four with one wavefront per SIMD,
        // two with two (the registers are needed, and the other wavefront fills the gaps)
        constexpr int kChains = WAVES == 4 ? 2 : 1; // per half
        f32x4 sp[2][2] = {{{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}, {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}}};
        {
            constexpr int kAhead = WAVES == 4 ? kMlaQuadOperandsAhead : 2;
            constexpr int kOperands = 2 * kSteps;
            constexpr int kEvery = kOperands / kSlots; // one load instruction of the next tile after every so many operands
            auto readK = [&](int idx) {
                const int kk = idx >> 1;
                const int in_half = kk < 2 * (kMainK / 8) ? 8 * (kk >> 1) + k_read_index[kk & 1] : k_read_index[kk & 1] + k_read_tail;
                return tiles.k[buf][(idx & 1) * kTileK + in_half];
            };
            uint4 kf[kAhead];
#pragma unroll
            for (int i = 0; i < kAhead; ++i) {
                kf[i] = readK(i);
            }
            __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
            for (int idx = 0; idx < kOperands; ++idx) {
                const uint4 cur = kf[idx % kAhead];
                if (idx + kAhead < kOperands) {
                    kf[idx % kAhead] = readK(idx + kAhead);
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                }
                const int kk = idx >> 1;
                sp[idx & 1][kk % kChains] = T::mfmaK32(cur, q_reg[kk], sp[idx & 1][kk % kChains]);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if (idx % kEvery == kEvery - 1) {
                    issueSlot(idx / kEvery); // V wavefronts: one load instruction of the next V tile
                }
            }
            static_assert(kOperands % kSlots == 0, "a place in the tile for every load instruction of the next");
        }
        s0 = kChains == 2 ? sp[0][0] + sp[0][1] : sp[0][0], s1 = kChains == 2 ? sp[1][0] + sp[1][1] : sp[1][0];
    };
    auto computeValues = [&](int buf, int t) {
        const int tok0 = start + t * kMlaWideTileTokens;
        const int valid = min(kMlaWideTileTokens, end - tok0);
        uint4 p_op, p_lo;
        softmaxStepPair<T, kBlocks>(o, m, l, s0, s1, g, a.scale_log2, slope, tok0 - (len - 1), valid, p_op, p_lo);

        // P . V: operand e = V[32 tokens][columns 16 e .. 16 e + 15]: two transposing reads, one per half
        constexpr int kAhead = WAVES == 4 ? kMlaQuadOperandsAhead : 2;
        constexpr int kEveryV = kBlocks / kSlots; // one load instruction after every so many operands
        auto readV = [&](int e) {
            const auto base = v_read_base + buf * (2 * kTileV * 16) + 512 * e;
            const uint2 lo = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsPiece>(base)));
            const uint2 hi = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsPiece>(base + kTileV * 16)));
            return make_uint4(lo.x, lo.y, hi.x, hi.y);
        };
        uint4 vf[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            vf[i] = readV(i);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);
#pragma unroll
        for (int e = 0; e < kBlocks; ++e) {
            const uint4 cur = vf[e % kAhead];
            if (e + kAhead < kBlocks) {
                vf[e % kAhead] = readV(e + kAhead);
                __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
            }
            o[e] = T::mfmaK32(p_op, cur, o[e]);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if (e % kEveryV == kEveryV - 1 && e / kEveryV < kSlots) {
                issueSlot(e / kEveryV); // K wavefronts: one load instruction of the K tile after the next
            }
        }
    };

    // ---- pipeline. K tiles and V tiles are double-buffered separately and a tile has two barriers:
    //   A(t): K(t) is in LDS and everybody is past P . V of tile t - 1  -> the V wavefronts ask for V(t + 1) (between
    //         the matrix instructions of K . Q^T), whose buffer P . V of tile t - 1 was the last to read;
    //   B(t): V(t) is in LDS and everybody is past K . Q^T of tile t    -> the K wavefronts ask for K(t + 2) (between
    //         the matrix instructions of P . V), whose buffer K . Q^T of tile t was the last to read.
    // A tile is thus asked for a tile and a half before it is needed. A wavefront's loads come back in the order
    // issued, so waiting until no more than the load instructions of the younger stage are outstanding means the
    // older stage has landed; where the younger stage is not exactly that many instructions (the ragged end of a
    // partition) the wait is for everything.
    auto awaitOlderStage = [&](bool younger_is_whole) {
        if (younger_is_whole) {
            if (copies_k) {
                asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kLoadsK) : "memory");
            } else {
                asm volatile("s_waitcnt vmcnt(%0)" :: "n"(kLoadsV) : "memory");
            }
        } else {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    };
    bool younger_whole = false; // of this wavefront's kind: the stage in flight behind the one it waits for next
    stageTile(0, false);
    if (copies_k && n_tiles > 1) {
        younger_whole = stageTile(1, false);
    }
    for (int t = 0; t < n_tiles; ++t) {
        if (copies_k) {
            awaitOlderStage(younger_whole); // K(t); K(t + 1) may still be on its way
        }
        __syncthreads(); // A(t)
        pend_live = 0ull;
        if (!copies_k && t + 1 < n_tiles) {
            younger_whole = stageTile(t + 1, true);
        } else if (!copies_k) {
            younger_whole = false;
        }
        computeScores(t & 1);
        if (!copies_k) {
            awaitOlderStage(younger_whole); // V(t); V(t + 1) has just been asked for
        }
        __syncthreads(); // B(t)
        pend_live = 0ull;
        if (copies_k && t + 2 < n_tiles) {
            younger_whole = stageTile(t + 2, true);
        } else if (copies_k) {
            younger_whole = false;
        }
        computeValues(t & 1, t);
    }
    __syncthreads(); // everybody is past the last tile: the buffers are free

    // ---- epilogue: a lane holds single columns (16 e + c) of heads 4g .. 4g + 3; the wavefront's 16 rows pass through
    // LDS, eight at a time (heads 4g + 2 pass + {0, 1}), and leave as 16-byte pieces, 64 lanes on consecutive pieces ----
    const float l_tot = sumAcrossTokenGroups(l);
    const bool single = len <= partition_tokens;
    float *stage = reinterpret_cast<float *>(&tiles) + wave * (kOutRows * kOutPitch);
    const int heads_here = min(kHeadsPerWave, a.group - chunk * kHeadsPerWave); // <= 0: a chunk beyond the last
    const int out_head0 = kv_head * a.group + chunk * kHeadsPerWave;
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
#pragma unroll
        for (int rr = 0; rr < 2; ++rr) {
            float *row = stage + (2 * g + rr) * kOutPitch + c;
#pragma unroll
            for (int e = 0; e < kBlocks; ++e) {
                row[16 * e] = o[e][2 * pass + rr];
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the wavefront's own stores have landed before its lanes read each other's
#pragma unroll
        for (int lr = 0; lr < kOutRows; ++lr) {
            const int r = 4 * (lr >> 1) + 2 * pass + (lr & 1); // head of the chunk in staged row lr
            if (r >= heads_here) {
                continue;
            }
            if (single) { // one row per instruction: 64 lanes x 8 columns
                const float inv_l = 1.0f / (__shfl(l_tot, r, 64) + 1e-6f);
                const float4 x = *reinterpret_cast<const float4 *>(stage + lr * kOutPitch + 8 * lane);
                const float4 y = *reinterpret_cast<const float4 *>(stage + lr * kOutPitch + 8 * lane + 4);
                uint4 w;
                w.x = T::pack2(x.x * inv_l, x.y * inv_l);
                w.y = T::pack2(x.z * inv_l, x.w * inv_l);
                w.z = T::pack2(y.x * inv_l, y.y * inv_l);
                w.w = T::pack2(y.z * inv_l, y.w * inv_l);
                S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + (out_head0 + r) * a.o_head_stride;
                *reinterpret_cast<uint4 *>(o_ptr + 8 * lane) = w;
            } else { // half a row per instruction: 64 lanes x 4 columns
                const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head0 + r) * a.max_partitions + part;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int col = 256 * h + 4 * lane;
                    *reinterpret_cast<float4 *>(a.part_acc + slot * kMlaValueSize + col) = *reinterpret_cast<const float4 *>(stage + lr * kOutPitch + col);
                }
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read back before the second pass overwrites the rows
    }
    if (!single && g == 0 && c < heads_here) {
        const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head0 + c) * a.max_partitions + part;
        a.part_m[slot] = m;
        a.part_l[slot] = l_tot;
    }
}

// ---- 64 query heads per workgroup, K . Q^T and P . V in different wavefronts ----------------------------------------
// The unit of work, its planning per call and the LDS layouts are those of decodeMlaRowsKernel with four chunks. That
// kernel runs one wavefront per SIMD, and such a wavefront does the steps of a tile one after the other: the matrix
// instructions of K . Q^T, the softmax, those of P . V, each behind the latency of its LDS operands, with two barriers;
// the 128 accumulator and 72 query registers of a chunk leave no room for a second wavefront on the SIMD. Here every
// SIMD has TWO wavefronts with different roles:
//   * score wavefront w (0..3) holds the query of chunk w (72 registers), computes K . Q^T of tile t and its softmax
//     step, and leaves in LDS the probabilities (512 bytes), the factor by which the reference point of each head
//     moved and, at the end, the sums;
//   * value wavefront w (4..7) holds the accumulators of ALL 64 heads for value columns 128 w .. 128 w + 127 (128
//     registers) and in the same period multiplies the probabilities of tile t - 1 of the four chunks by its quarter
//     of the V tile: a V operand read from LDS (a transposing read, the slow kind) serves four matrix instructions;
//     where a reference point moved it rescales first; at the end it writes its columns of the unit's result.
// Tiles are 16 tokens; K and V tiles each go round a ring of four LDS buffers (136 KiB as in the kernel above), one
// workgroup barrier per tile. In period t the score wavefronts ask for V(t + 2) and the value wavefronts for K(t + 3),
// one load instruction (global memory straight into LDS) between matrix instructions; both are first read in period
// t + 3, so before a barrier every wavefront waits until no more than its load instructions of the last two periods
// are outstanding (a wavefront's loads come back in the order issued). Every period issues whole tiles so that these
// counts are exact: rows beyond the end of the partition are fetched all the same (a tile lies inside one page), their
// scores are replaced and their V values zeroed in the operand registers; tiles beyond the last one are not needed and
// the last one is fetched again in their place.
// Measured (128 heads, 32 sequences of 512 - 4 096 tokens): 60.1 us per call against 66.5 us with a wavefront per
// chunk; a period takes 0.89 us, either role is busy for 0.8 of it. Not kept: the operands of the next tile read from
// LDS a period ahead (62.5 us), the load instructions of a period in one burst after the barrier (61.2 - 62.3 us).
template <typename T, typename Tindex, bool ONCE>
__global__ void __launch_bounds__(512) decodeMlaRolesKernel(DecodeArgs a) {
    using S = typename T::storage;
    constexpr int kChunks = 4;                    // 16-head chunks of a workgroup
    constexpr int kRing = 4;                      // LDS buffers of either kind
    constexpr int kSteps = kMlaKeySize / 32;      // 18 K-steps
    constexpr int kRowK = kMlaKeySize / 8;        // 72 16-byte chunks in a K row
    constexpr int kRowV = kMlaValueSize / 8;      // 64 in a V row
    constexpr int kSwizzle = 8;                   // stays inside a K row: 72 is a multiple of 8
    constexpr int kTileK = kTileTokens * kRowK;   // chunks of a tile
    constexpr int kTileV = kTileTokens * kRowV;
    constexpr int kBlocks = kMlaValueSize / 16;   // 32 column blocks of 16
    constexpr int kLoadsV = kTileV / 64 / kChunks; // load instructions per period of a score wavefront: 4 of the V tile
    constexpr int kLoadsKMost = 5;                // of a value wavefront: 4 main parts of K rows, and for two of them one of tails
    constexpr int kOwn = kBlocks / kChunks;       // column blocks of a value wavefront: 8
    constexpr int kOwnCols = 16 * kOwn;           // 128 columns
    constexpr int kOutRows = kChunks * kHeadsPerWave; // output rows a value wavefront stages in LDS: all 64 heads
    constexpr int kOutPitch = kOwnCols + 4;       // floats between them (conflict-free column writes)
    constexpr int kMainK = 64;                    // chunks of a K row kept in the main region of a tile; the other 8 in its tail
    constexpr int kTailK = kTileTokens * kMainK;  // first slot of the tail region
    struct Tiles {
        uint4 k[kRing][kTileK]; // {main [token][64 chunks], tail [token][8 chunks]}, chunks XOR-swizzled by token % 8
        uint4 v[kRing][kTileV]; // [block of 16 columns][token][two 16-byte chunks]
    };
    __shared__ Tiles tiles;
    __shared__ uint2 p_lds[2][kChunks][64];                 // probabilities of a tile as the A operand of P . V
    __shared__ float alpha_lds[2][kChunks][kHeadsPerWave];  // factor of head c where the reference point moved
    __shared__ __align__(16) int moved_lds[2][kChunks];     // whether any did
    __shared__ float ml_lds[kChunks][2][kHeadsPerWave];     // at the end: reference points and sums
    static_assert(sizeof(Tiles) >= kChunks * kOutRows * kOutPitch * sizeof(float), "the tile buffers hold the staged output rows");

    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int groups_of_chunks = (head_chunks + kChunks - 1) / kChunks;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool scores_role = wave < kChunks;
    const int cw = wave & (kChunks - 1); // chunk of the workgroup
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;

    int seq, part, stream, partition_tokens, len;
    if (!locateWideUnit<Tindex>(a, lane, groups_of_chunks, seq, part, stream, partition_tokens, len)) {
        return;
    }
    const int kv_head = stream / groups_of_chunks;
    const int chunk = (stream - kv_head * groups_of_chunks) * kChunks + cw; // may lie beyond the last chunk: no heads
    const int start = part * partition_tokens;
    if (len <= 0 || start >= len) {
        return;
    }
    const int end = min(len, start + partition_tokens);
    const int n_tiles = (end - start + kTileTokens - 1) / kTileTokens;

    const int first_entry = start >> a.block_shift;
    const int last_entry = (end - 1) >> a.block_shift;
    int page_ids = 0;
    if (first_entry + lane <= last_entry) {
        page_ids = clampPage(
            loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + first_entry + lane), a.num_blocks);
    }
    const int block_mask = a.block_size - 1;
    // first byte of row 0 of tile t (clamped to the last tile) of K or V
    auto tileSource = [&](int t, const char *head_base, int64_t batch_stride, int64_t row_stride) -> const char * {
        const int tok0 = start + min(t, n_tiles - 1) * kTileTokens;
        const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
        return head_base + (page * batch_stride + (tok0 & block_mask) * row_stride) * static_cast<int64_t>(sizeof(S));
    };
    const int heads_here = min(kHeadsPerWave, a.group - chunk * kHeadsPerWave); // <= 0: a chunk beyond the last
    const int n_periods = n_tiles + 1;

    if (scores_role) {
        // ================= score wavefront =================
        // Query of head (chunk*16 + c): columns 32 kk + 8g .. +7, the B operand of K-step kk
        const int head_in_group = chunk * kHeadsPerWave + c;
        const bool head_valid = head_in_group < a.group;
        const int head = kv_head * a.group + head_in_group;
        uint4 q_reg[kSteps];
        {
            const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
            const uint32_t keep = head_valid ? 0xffffffffu : 0u;
#pragma unroll
            for (int kk = 0; kk < kSteps; ++kk) {
                uint4 x = *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g);
                x.x &= keep, x.y &= keep, x.z &= keep, x.w &= keep;
                q_reg[kk] = x;
            }
        }
        const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;
        // copy: load instruction j (0..3) of this wavefront fills slots 64 (4 cw + j) .. + 63 of the V tile, two blocks of
        // 16 columns: lane -> row (lane % 32) / 2, chunk 4 (4 cw + j) + 2 (lane / 32) + lane % 2
        const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
        const uint32_t v_row_bytes = static_cast<uint32_t>(a.v_row_stride) * sizeof(S);
        const uint32_t lane_offset = ((lane & 31) >> 1) * v_row_bytes + 16u * (2 * (lane >> 5) + (lane & 1)) + 64u * (kLoadsV * cw);
        const char *pend_src = v_head;
        uint4 *pend_dst = &tiles.v[0][0];
        auto issueSlot = [&](int j) { loadLane16ToLds<ONCE>(pend_src + 64 * j, lane_offset, pend_dst + 64 * (kLoadsV * cw + j)); };
        auto stageV = [&](int t) {
            pend_src = tileSource(t, v_head, a.v_batch_stride, a.v_row_stride);
            pend_dst = &tiles.v[t % kRing][0];
        };
        // this lane's chunk of row c in K-step kk: chunk 4 kk + g of the row, XOR-swizzled, i.e.
        // 8 (kk / 2) + ((4 (kk % 2) + g) ^ (c % 8)), in the main region up to K-step 15 and in the tail after
        const int k_read_index[2] = {c * kMainK + (g ^ (c & (kSwizzle - 1))), c * kMainK + ((4 + g) ^ (c & (kSwizzle - 1)))};
        const int k_read_tail = kTailK + c * 8 - c * kMainK;

        float m = -INFINITY; // reference point of head c's exponentials (same value in the four lanes g = 0..3)
        float l = 0.0f;      // sum of rounded probabilities of head c over this lane's tokens only
#pragma unroll
        for (int t = 0; t < 2; ++t) { // V(0), V(1)
            stageV(t);
#pragma unroll
            for (int j = 0; j < kLoadsV; ++j) {
                issueSlot(j);
            }
        }
        for (int t = 0; t < n_periods; ++t) {
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * kLoadsV) : "memory"); // V(t - 1) has landed
            __syncthreads();
            if (t == n_tiles) {
                break;
            }
            stageV(t + 2);
            // K . Q^T of tile t
            f32x4 sp[2] = {{0.f, 0.f, 0.f, 0.f}, {0.f, 0.f, 0.f, 0.f}};
            {
                constexpr int kAhead = 4;
                const uint4 *k_tile = &tiles.k[t % kRing][0];
                auto readK = [&](int kk) {
                    return k_tile[kk < 2 * (kMainK / 8) ? 8 * (kk >> 1) + k_read_index[kk & 1] : k_read_index[kk & 1] + k_read_tail];
                };
                uint4 kf[kAhead];
#pragma unroll
                for (int i = 0; i < kAhead; ++i) {
                    kf[i] = readK(i);
                }
                __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
                for (int kk = 0; kk < kSteps; ++kk) {
                    const uint4 cur = kf[kk % kAhead];
                    if (kk + kAhead < kSteps) {
                        kf[kk % kAhead] = readK(kk + kAhead);
                        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    }
                    sp[kk & 1] = T::mfmaK32(cur, q_reg[kk], sp[kk & 1]);
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if (kk % 4 == 3 && kk / 4 < kLoadsV) {
                        issueSlot(kk / 4);
                    }
                }
            }
            const f32x4 s = sp[0] + sp[1]; // raw scores of head c for tokens 4g .. 4g + 3 of the tile
            // online softmax step (softmaxStep of decode_tiled.h with one-term probabilities, its rare branches
            // wave-uniform, the accumulators elsewhere)
            const int tok0 = start + t * kTileTokens;
            const int valid = min(kTileTokens, end - tok0);
            float sc[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                sc[rr] = s[rr] * a.scale_log2;
            }
            if (__builtin_amdgcn_ballot_w64(slope != 0.0f) != 0) {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    sc[rr] += slope * static_cast<float>(tok0 - (len - 1) + 4 * g + rr);
                }
            }
            if (valid < kTileTokens) {
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    sc[rr] = (4 * g + rr >= valid) ? -INFINITY : sc[rr];
                }
            }
            const float mx_lane = maxOf(maxOf(sc[0], sc[1]), maxOf(sc[2], sc[3]));
            const bool moved = __builtin_amdgcn_ballot_w64(mx_lane > m + kLazyRescaleLog2) != 0;
            if (moved) {
                const float m_new = maxOf(m, maxAcrossTokenGroups(mx_lane));
                const float alpha = fastExp2(m - m_new);
                l *= alpha;
                m = m_new;
                if (g == 0) {
                    alpha_lds[t & 1][cw][c] = alpha;
                }
            }
            if (lane == 0) {
                moved_lds[t & 1][cw] = moved ? 1 : 0;
            }
            uint2 p_op;
            p_op.x = T::pack2(fastExp2(sc[0] - m), fastExp2(sc[1] - m));
            p_op.y = T::pack2(fastExp2(sc[2] - m), fastExp2(sc[3] - m));
            l += (T::unpackLo(p_op.x) + T::unpackHi(p_op.x)) + (T::unpackLo(p_op.y) + T::unpackHi(p_op.y));
            p_lds[t & 1][cw][lane] = p_op;
        }
        // (the break above leaves after the barrier of the last period: every P . V but the last has been done)
        const float l_tot = sumAcrossTokenGroups(l);
        if (g == 0) {
            ml_lds[cw][0][c] = m;
            ml_lds[cw][1][c] = l_tot;
        }
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wavefront's last V tiles have landed: the buffers are free
        __syncthreads();
        return;
    }

    // ================= value wavefront =================
    // copy: main parts of K rows 4 cw .. 4 cw + 3 (slot 64 row, lane asks for chunk lane ^ row % 8), and for cw < 2 the
    // tails of rows 8 cw .. 8 cw + 7 (slot tail + 64 cw: lane -> row 8 cw + lane / 8, chunk 64 + (lane % 8 ^ lane / 8))
    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const uint32_t k_row_bytes = static_cast<uint32_t>(a.k_row_stride) * sizeof(S);
    const uint32_t lane_main = 16u * lane;
    const uint32_t lane_tail = (8 * cw + (lane >> 3)) * k_row_bytes + 16u * (kMainK + ((lane & 7) ^ (lane >> 3)));
    const bool copies_tail = cw < 2;
    const char *pend_src = k_head;
    uint4 *pend_dst = &tiles.k[0][0];
    auto issueSlot = [&](int j) { // j < 4: a main part; j == 4: the tails, for the wavefronts that have them
        if (j < 4) {
            const int row = 4 * cw + j;
            loadLane16ToLds<ONCE>(pend_src + row * k_row_bytes, lane_main ^ (16u * (row & (kSwizzle - 1))), pend_dst + kMainK * row);
        } else if (copies_tail) {
            loadLane16ToLds<ONCE>(pend_src, lane_tail, pend_dst + kTailK + 64 * cw);
        }
    };
    auto stageK = [&](int t) {
        pend_src = tileSource(t, k_head, a.k_batch_stride, a.k_row_stride);
        pend_dst = &tiles.k[t % kRing][0];
    };
    auto awaitPeriodBeforeLast = [&]() { // no more than the loads of the last two periods outstanding
        if (copies_tail) {
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * kLoadsKMost) : "memory");
        } else {
            asm volatile("s_waitcnt vmcnt(%0)" :: "n"(2 * (kLoadsKMost - 1)) : "memory");
        }
    };
    // o[h][e][r] = O[head 4g + r of the workgroup's chunk h][column 16 (kOwn cw + e) + c]
    f32x4 o[kChunks][kOwn];
#pragma unroll
    for (int h = 0; h < kChunks; ++h) {
#pragma unroll
        for (int e = 0; e < kOwn; ++e) {
            o[h][e] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
    }
    // this lane's piece of a transposing V read, relative to block 0 of buffer 0: lane (g, c) points at token
    // 4g + c / 4, columns 16 e + 4 (c % 4) .. + 3 and receives tokens 4g .. 4g + 3 of column 16 e + c
    typedef short s16x4 __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) s16x4 *LdsPiece;
    const auto v_read_base = (__attribute__((address_space(3))) char *)&tiles.v[0][0]
                           + 16 * ((4 * g + (c >> 2)) * 2 + ((c & 3) >> 1)) + 8 * (c & 1);
#pragma unroll
    for (int t = 0; t < 3; ++t) { // K(0), K(1), K(2)
        stageK(t);
#pragma unroll
        for (int j = 0; j < kLoadsKMost; ++j) {
            issueSlot(j);
        }
    }
    for (int t = 0; t < n_periods; ++t) {
        awaitPeriodBeforeLast(); // K(t) has landed
        __syncthreads();
        if (t == 0) {
            stageK(3);
#pragma unroll
            for (int j = 0; j < kLoadsKMost; ++j) {
                issueSlot(j);
            }
            continue;
        }
        const bool more = t < n_tiles; // the last period asks for nothing
        stageK(t + 3);
        // P . V of tile t - 1
        const int u = t - 1;
        const int valid = min(kTileTokens, end - (start + u * kTileTokens));
        uint2 p[kChunks];
#pragma unroll
        for (int h = 0; h < kChunks; ++h) {
            p[h] = p_lds[u & 1][h][lane];
        }
        const int4 moved = *reinterpret_cast<const int4 *>(&moved_lds[u & 1][0]);
        if (__builtin_amdgcn_readfirstlane(moved.x | moved.y | moved.z | moved.w) != 0) { // rare after the first tiles
            const int of_chunk[kChunks] = {moved.x, moved.y, moved.z, moved.w};
#pragma unroll
            for (int h = 0; h < kChunks; ++h) {
                if (__builtin_amdgcn_readfirstlane(of_chunk[h]) != 0) {
                    const float4 al = *reinterpret_cast<const float4 *>(&alpha_lds[u & 1][h][4 * g]);
#pragma unroll
                    for (int e = 0; e < kOwn; ++e) {
                        o[h][e][0] *= al.x, o[h][e][1] *= al.y, o[h][e][2] *= al.z, o[h][e][3] *= al.w;
                    }
                }
            }
        }
        // rows of the tile beyond the end of the sequence may hold anything, NaN included, and 0 * NaN is NaN
        const uint32_t keep_lo = (4 * g + 0 < valid ? 0x0000ffffu : 0u) | (4 * g + 1 < valid ? 0xffff0000u : 0u);
        const uint32_t keep_hi = (4 * g + 2 < valid ? 0x0000ffffu : 0u) | (4 * g + 3 < valid ? 0xffff0000u : 0u);
        constexpr int kAhead = 4;
        const auto v_tile = v_read_base + (u % kRing) * (kTileV * 16) + 512 * (kOwn * cw);
        auto readV = [&](int e) {
            return __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16(reinterpret_cast<LdsPiece>(v_tile + 512 * e)));
        };
        uint2 vf[kAhead];
#pragma unroll
        for (int i = 0; i < kAhead; ++i) {
            vf[i] = readV(i);
        }
        __builtin_amdgcn_sched_group_barrier(0x100, kChunks + 1 + kAhead, 0);
#pragma unroll
        for (int e = 0; e < kOwn; ++e) {
            uint2 cur = vf[e % kAhead];
            if (e + kAhead < kOwn) {
                vf[e % kAhead] = readV(e + kAhead);
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            }
            if (valid < kTileTokens) { // wave-uniform: only the last tile of a partition can be short
                cur.x &= keep_lo, cur.y &= keep_hi;
            }
#pragma unroll
            for (int h = 0; h < kChunks; ++h) { // the operand serves the heads of every chunk
                o[h][e] = T::mfmaK16(p[h], cur, o[h][e]);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                constexpr int kEvery = 6;
                const int done = kChunks * e + h;
                if (more && done % kEvery == kEvery - 1) {
                    issueSlot(done / kEvery); // five places: one load instruction of K(t + 3) each
                }
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // this wavefront's last K tiles have landed: the buffers are free
    __syncthreads();

    // ---- epilogue: a lane holds single columns (16 e + c of the wavefront's 128) of heads 4g .. 4g + 3 of every chunk;
    // the 64 rows pass through LDS and leave as 16-byte pieces, a row on 32 consecutive lanes ----
    const float m_c = ml_lds[cw][0][c], l_c = ml_lds[cw][1][c]; // of head c of this wavefront's own chunk
    const bool single = len <= partition_tokens;
    float *stage = reinterpret_cast<float *>(&tiles) + cw * (kOutRows * kOutPitch);
    const int chunk0 = chunk - cw; // the workgroup's first chunk
    const int out_head0 = kv_head * a.group + chunk * kHeadsPerWave;
#pragma unroll
    for (int h = 0; h < kChunks; ++h) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            float *row = stage + (kHeadsPerWave * h + 4 * g + rr) * kOutPitch + c;
#pragma unroll
            for (int e = 0; e < kOwn; ++e) {
                row[16 * e] = o[h][e][rr];
            }
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the wavefront's own stores have landed before its lanes read each other's
    constexpr int kLanesPerRow = kOwnCols / 4; // 32 lanes on one staged row
    const int col = kOwnCols * cw + 4 * (lane % kLanesPerRow);
#pragma unroll 4
    for (int i = 0; i < kOutRows * kLanesPerRow / 64; ++i) {
        const int r = (64 / kLanesPerRow) * i + lane / kLanesPerRow;  // staged row: head r % 16 of chunk r / 16
        const int head_in_group = chunk0 * kHeadsPerWave + r;         // chunks are consecutive, so are their heads
        if (head_in_group >= a.group) {
            continue;
        }
        const float4 x = *reinterpret_cast<const float4 *>(stage + r * kOutPitch + 4 * (lane % kLanesPerRow));
        const int out_head = kv_head * a.group + head_in_group;
        if (single) {
            const float inv_l = 1.0f / (ml_lds[r >> 4][1][r & 15] + 1e-6f);
            uint2 w;
            w.x = T::pack2(x.x * inv_l, x.y * inv_l);
            w.y = T::pack2(x.z * inv_l, x.w * inv_l);
            S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride;
            *reinterpret_cast<uint2 *>(o_ptr + col) = w;
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            *reinterpret_cast<float4 *>(a.part_acc + slot * kMlaValueSize + col) = x;
        }
    }
    if (!single && g == 0 && c < heads_here) {
        const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head0 + c) * a.max_partitions + part;
        a.part_m[slot] = m_c;
        a.part_l[slot] = l_c;
    }
}

} // namespace op::paged_attention::amd

#endif
