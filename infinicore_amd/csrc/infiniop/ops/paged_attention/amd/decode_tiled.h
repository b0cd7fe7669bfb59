// Tiled decode kernel for head_size = value_size = 128 on gfx950 (CDNA4, 64-lane wavefronts).
//
// Work unit: one wavefront = one (partition, KV head, sequence). All query heads that share the KV
// head (up to 16 per wavefront) are processed together, so every K and V byte is fetched from HBM
// once per KV head, not once per query head. The partition's tokens are consumed in tiles of 16.
//
// Data movement per tile (K 4 KiB + V 4 KiB when rows are packed):
//   * every global load instruction moves 16 bytes per lane and covers whole 256-byte token rows
//     (4 rows per instruction), i.e. full cache lines;
//   * K goes registers -> LDS (XOR-swizzled 16-byte chunks, conflict-free) -> registers, because the
//     matrix instruction wants lane i to hold token i while a coalesced load gives lane i column i;
//   * V needs no LDS: the lane that loads rows 4g..4g+3 of one 8-column strip is the lane that feeds
//     those four tokens to the matrix instruction; four rows are interleaved per column with byte
//     permutes.
//   * the loads of tiles t+1 and t+2 are in flight while tile t is computed; page ids of the whole partition
//     are fetched with one coalesced load up front, so no load address depends on a load in the loop.
//
// Arithmetic per tile, with lane = 16*g + c (g = 0..3, c = 0..15):
//   S[token][head] = K . Q^T   4 x v_mfma_f32_16x16x32 (A = K tile, B = Q; lane holds S[4g..4g+3][c])
//   online softmax in fp32, log2 domain; the running maximum is shared by the four lanes of a head
//   O[head][dim]  += P . V     8 x v_mfma_f32_16x16x16 (A = P rounded to the storage dtype and left
//                              in the registers S came out in, B = V strip; lane holds
//                              O[4g..4g+3][8c+e] for e = 0..7)
// The softmax denominator sums the rounded probabilities, so numerator and denominator see the same
// weights. Accumulators are rescaled only when some head's maximum actually moves.
// The math follows the reference's decode kernels (src/infiniop/ops/paged_attention/cuda/
// kernel_v2.cuh:134-336 for the recurrence, :340-554 for per-shard partial results).
#ifndef INFINICORE_AMD_PA_DECODE_TILED_H
#define INFINICORE_AMD_PA_DECODE_TILED_H

#include "decode_common.h"

namespace op::paged_attention::amd {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Matrix-instruction and packing flavours of the two storage dtypes.
struct TileBF16 : BFloat16 {
    using Base = BFloat16;
    static constexpr bool kSplitProbabilities = true; // 8-bit significand: feed p as hi + lo
    static __device__ __forceinline__ f32x4 mfmaK32(uint4 a, uint4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfmaK16(uint2 a, uint2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(s16x4, a), __builtin_bit_cast(s16x4, b), c, 0, 0, 0);
    }
    // two fp32 -> two storage values in one dword (lo in bits 0..15), round-to-nearest-even
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));
    }
    static __device__ __forceinline__ float unpackLo(uint32_t w) { return __uint_as_float(w << 16); }
    static __device__ __forceinline__ float unpackHi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
};
struct TileF16 : Half {
    using Base = Half;
    static constexpr bool kSplitProbabilities = false; // 11 bits of a value in [0, 1] are enough
    static __device__ __forceinline__ f32x4 mfmaK32(uint4 a, uint4 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ f32x4 mfmaK16(uint2 a, uint2 b, f32x4 c) {
        return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4, a), __builtin_bit_cast(f16x4, b), c, 0, 0, 0);
    }
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        f32x2 v = {lo, hi};
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
    }
    static __device__ __forceinline__ float unpackLo(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(f16x2, w)[0]);
    }
    static __device__ __forceinline__ float unpackHi(uint32_t w) {
        return static_cast<float>(__builtin_bit_cast(f16x2, w)[1]);
    }
};

constexpr int kTileTokens = 16;     // tokens per tile = rows of one matrix instruction
constexpr int kTiledHead = 128;     // head_size = value_size handled by this kernel
constexpr int kHeadsPerWave = 16;   // query heads of one KV head packed into one wavefront

// K and V rows of one 16-token tile as they come out of the global loads; kept in registers.
struct TileRegs {
    uint4 k0, k1, k2, k3; // k<j>: token row 4j+g, columns 8c..8c+7
    uint4 v0, v1, v2, v3; // v<j>: token row 4g+j, columns 8c..8c+7
};

// 16-byte load from (wave-uniform base) + (32-bit per-lane byte offset). The empty asm keeps the
// offset a value defined where it is used, so that instruction selection sees "scalar base +
// zero-extended lane offset" and emits the scalar-base form of the load, which needs no vector
// registers for addresses.
__device__ __forceinline__ uint4 loadLane16(const char *uniform_base, uint32_t lane_offset) {
    asm volatile("" : "+v"(lane_offset));
    // K and V are read exactly once per call: a non-temporal load keeps them from displacing
    // anything in the caches and measurably raises the HBM rate a gather stream reaches.
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(uniform_base + lane_offset));
    return make_uint4(v[0], v[1], v[2], v[3]);
}

// max over the four lanes {c, c+16, c+32, c+48}; every one of them gets the result (two lane swaps,
// no LDS traffic)
__device__ __forceinline__ float maxAcrossTokenGroups(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sumAcrossTokenGroups(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// Softmax state of one wavefront. o[e][r] = O[head 4g+r of the chunk][column 8c+e].
struct TileState {
    f32x4 o[8];
    float m; // running maximum of head c (same value in the four lanes g = 0..3)
    float l; // sum of rounded probabilities of head c over this lane's tokens only
};

// One tile: scores, online softmax, accumulate. `valid` = tokens of the tile that belong to the
// sequence (16 except possibly in the last tile).
template <typename T>
__device__ __forceinline__ void computeTile(TileState &st, const TileRegs r, const uint4 (&q_reg)[4], uint4 *k_lds,
                                            int c, int g, float scale_log2, float slope, int rel_pos0, int valid) {
    // K: registers -> swizzled LDS -> matrix-operand layout (token c, columns 32*kk + 8g .. +7)
    k_lds[(g) * 16 + (c ^ (g))] = r.k0;
    k_lds[(4 + g) * 16 + (c ^ (4 + g))] = r.k1;
    k_lds[(8 + g) * 16 + (c ^ (8 + g))] = r.k2;
    k_lds[(12 + g) * 16 + (c ^ (12 + g))] = r.k3;
    __builtin_amdgcn_wave_barrier();
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        s = T::mfmaK32(k_lds[c * 16 + ((4 * kk + g) ^ c)], q_reg[kk], s);
    }
    __builtin_amdgcn_wave_barrier();

    // scores of head c for tokens 4g + rr of the tile, log2 domain; rel_pos0 = position of the
    // tile's first token relative to the last token of the sequence (ALiBi distance)
    const bool tail = valid < kTileTokens;
    float sc[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        sc[rr] = s[rr] * scale_log2 + slope * static_cast<float>(rel_pos0 + 4 * g + rr);
        sc[rr] = (tail && 4 * g + rr >= valid) ? -INFINITY : sc[rr];
    }
    const float mx = maxAcrossTokenGroups(fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3])));
    const float m_new = fmaxf(st.m, mx);

    if (__builtin_amdgcn_ballot_w64(m_new > st.m) != 0) {
        // some head's maximum moved: rescale. Lane holds accumulators of heads 4g..4g+3, whose
        // factors live in lanes 4g..4g+3.
        const float alpha = fastExp2(st.m - m_new);
        st.l *= alpha;
        st.m = m_new;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const float alpha_r = __shfl(alpha, 4 * g + rr, 64);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                st.o[e][rr] *= alpha_r;
            }
        }
    }

    // Probabilities as the A operand of P.V. The matrix instruction takes them in the storage dtype;
    // fp16 keeps 11 significant bits of a value in [0, 1], bf16 only 8. For bf16 the probability is
    // therefore fed as two terms, p = hi + lo with lo = bf16(p - hi), and P.V takes two matrix
    // instructions per output tile: the product then carries ~16 bits of p, close to the fp32
    // probabilities of the reference kernel. The denominator sums exactly what the numerator used.
    const float p0 = fastExp2(sc[0] - st.m), p1 = fastExp2(sc[1] - st.m);
    const float p2 = fastExp2(sc[2] - st.m), p3 = fastExp2(sc[3] - st.m);
    uint2 p_op, p_lo;
    p_op.x = T::pack2(p0, p1);
    p_op.y = T::pack2(p2, p3);
    float p_used = (T::unpackLo(p_op.x) + T::unpackHi(p_op.x)) + (T::unpackLo(p_op.y) + T::unpackHi(p_op.y));
    if constexpr (T::kSplitProbabilities) {
        p_lo.x = T::pack2(p0 - T::unpackLo(p_op.x), p1 - T::unpackHi(p_op.x));
        p_lo.y = T::pack2(p2 - T::unpackLo(p_op.y), p3 - T::unpackHi(p_op.y));
        p_used += (T::unpackLo(p_lo.x) + T::unpackHi(p_lo.x)) + (T::unpackLo(p_lo.y) + T::unpackHi(p_lo.y));
    }
    st.l += p_used;

    // V rows beyond the sequence may hold anything (NaN included) and 0 * NaN is NaN: zero them.
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    u32x4 v0 = __builtin_bit_cast(u32x4, r.v0), v1 = __builtin_bit_cast(u32x4, r.v1);
    u32x4 v2 = __builtin_bit_cast(u32x4, r.v2), v3 = __builtin_bit_cast(u32x4, r.v3);
    if (tail) {
        const u32x4 zero = {0u, 0u, 0u, 0u};
        v0 = (4 * g + 0 >= valid) ? zero : v0;
        v1 = (4 * g + 1 >= valid) ? zero : v1;
        v2 = (4 * g + 2 >= valid) ? zero : v2;
        v3 = (4 * g + 3 >= valid) ? zero : v3;
    }

    // O += P . V, one 16-column output tile per e: column 8c+e of rows 4g..4g+3
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        uint2 even, odd;
        even.x = __builtin_amdgcn_perm(v1[w], v0[w], 0x05040100u);
        even.y = __builtin_amdgcn_perm(v3[w], v2[w], 0x05040100u);
        odd.x = __builtin_amdgcn_perm(v1[w], v0[w], 0x07060302u);
        odd.y = __builtin_amdgcn_perm(v3[w], v2[w], 0x07060302u);
        st.o[2 * w] = T::mfmaK16(p_op, even, st.o[2 * w]);
        st.o[2 * w + 1] = T::mfmaK16(p_op, odd, st.o[2 * w + 1]);
        if constexpr (T::kSplitProbabilities) {
            st.o[2 * w] = T::mfmaK16(p_lo, even, st.o[2 * w]);
            st.o[2 * w + 1] = T::mfmaK16(p_lo, odd, st.o[2 * w + 1]);
        }
    }
}

// Software pipeline over the tiles of one run. NBUF register sets rotate; NBUF-1 tiles are always
// in flight while one is computed. The body has no branch around a load, so the compiler counts
// outstanding loads exactly and each tile waits only for its own data. loadTile() must accept any
// index (it neutralises indices past the end); compute() is skipped for those.
template <int NBUF, typename Load, typename Compute>
__device__ __forceinline__ void streamTiles(int n_tiles, Load loadTile, Compute compute) {
    TileRegs buf[NBUF];
#pragma unroll
    for (int i = 0; i < NBUF - 1; ++i) {
        buf[i] = loadTile(i);
    }
    for (int t = 0; t < n_tiles; t += NBUF) {
#pragma unroll
        for (int i = 0; i < NBUF; ++i) {
            buf[(i + NBUF - 1) % NBUF] = loadTile(t + i + NBUF - 1);
            if (t + i < n_tiles) {
                compute(t + i, buf[i]);
            }
        }
    }
}

#ifndef INFINIOP_AMD_PA_GRID_BUFFERS
#define INFINIOP_AMD_PA_GRID_BUFFERS 3
#endif
#ifndef INFINIOP_AMD_PA_BALANCED_BUFFERS
#define INFINIOP_AMD_PA_BALANCED_BUFFERS 3
#endif

template <typename T, typename Tindex>
__global__ void __launch_bounds__(64) decodeTiledKernel(DecodeArgs a) {
    using S = typename T::storage;
    __shared__ uint4 k_lds[kTileTokens * kTiledHead / 8]; // one K tile, 4 KiB

    const int part = blockIdx.x;
    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int kv_head = blockIdx.y / head_chunks;
    const int chunk = blockIdx.y - kv_head * head_chunks;
    const int seq = blockIdx.z;
    const int lane = threadIdx.x;
    const int c = lane & 15; // column strip / head within the chunk / token for the K operand
    const int g = lane >> 4; // group of four tokens

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

    // Query of head (chunk*16 + c), as the B operand of the four K-steps: columns 32*kk + 8g .. +7.
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    uint4 q_reg[4];
    {
        const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            q_reg[kk] = head_valid ? *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
        }
    }
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;

    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
    const int block_mask = a.block_size - 1;
    // Byte offsets of this lane's eight 16-byte pieces inside a tile. They do not change from tile
    // to tile, so a tile's loads are "wave-uniform tile address + constant lane offset" and need no
    // per-tile vector address arithmetic.
    const uint32_t k_row_bytes = static_cast<uint32_t>(a.k_row_stride) * sizeof(S);
    const uint32_t v_row_bytes = static_cast<uint32_t>(a.v_row_stride) * sizeof(S);
    uint32_t k_off[4], v_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        k_off[j] = (4 * j + g) * k_row_bytes + 16 * c;
        v_off[j] = (4 * g + j) * v_row_bytes + 16 * c;
    }

    // The loop body is branch-free with a fixed number of loads in flight, so it also issues loads
    // for tile indices past the end of the partition. Those are made harmless: every lane reads the
    // same 16 bytes (the start of the partition's first tile), one request instead of eight KiB.
    auto loadTile = [&](int t) -> TileRegs {
        const bool real = t < n_tiles;
        const uint32_t lane_mask = real ? 0xffffffffu : 0u;
        const int tok0 = start + (real ? t : 0) * kTileTokens;
        const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
        const int row0 = tok0 & block_mask;
        const char *k_tile = k_head + (page * a.k_batch_stride + row0 * a.k_row_stride) * static_cast<int64_t>(sizeof(S));
        const char *v_tile = v_head + (page * a.v_batch_stride + row0 * a.v_row_stride) * static_cast<int64_t>(sizeof(S));
        TileRegs r;
        r.k0 = loadLane16(k_tile, k_off[0] & lane_mask);
        r.k1 = loadLane16(k_tile, k_off[1] & lane_mask);
        r.k2 = loadLane16(k_tile, k_off[2] & lane_mask);
        r.k3 = loadLane16(k_tile, k_off[3] & lane_mask);
        r.v0 = loadLane16(v_tile, v_off[0] & lane_mask);
        r.v1 = loadLane16(v_tile, v_off[1] & lane_mask);
        r.v2 = loadLane16(v_tile, v_off[2] & lane_mask);
        r.v3 = loadLane16(v_tile, v_off[3] & lane_mask);
        return r;
    };

    TileState st;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        st.o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    st.m = -INFINITY;
    st.l = 0.0f;

    auto compute = [&](int t, const TileRegs &r) {
        const int tok0 = start + t * kTileTokens;
        computeTile<T>(st, r, q_reg, k_lds, c, g, a.scale_log2, slope, tok0 - (len - 1), min(kTileTokens, end - tok0));
    };

    streamTiles<INFINIOP_AMD_PA_GRID_BUFFERS>(n_tiles, loadTile, compute);

    // Epilogue. Denominator of head c over all 16 token slots, then move per-head scalars to the
    // lanes that hold that head's accumulators.
    const float l_tot = sumAcrossTokenGroups(st.l);

    const bool single = len <= a.partition_tokens;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int hl = 4 * g + rr; // head (within the chunk) of accumulator row rr
        const float l_h = __shfl(l_tot, hl, 64);
        const float m_h = __shfl(st.m, hl, 64);
        const int hg = chunk * kHeadsPerWave + hl;
        if (hg >= a.group) {
            continue;
        }
        const int out_head = kv_head * a.group + hg;
        if (single) {
            const float inv_l = 1.0f / (l_h + 1e-6f);
            uint4 packed;
            packed.x = T::pack2(st.o[0][rr] * inv_l, st.o[1][rr] * inv_l);
            packed.y = T::pack2(st.o[2][rr] * inv_l, st.o[3][rr] * inv_l);
            packed.z = T::pack2(st.o[4][rr] * inv_l, st.o[5][rr] * inv_l);
            packed.w = T::pack2(st.o[6][rr] * inv_l, st.o[7][rr] * inv_l);
            S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride;
            *reinterpret_cast<uint4 *>(o_ptr + 8 * c) = packed;
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            float4 *pa = reinterpret_cast<float4 *>(a.part_acc + slot * kTiledHead + 8 * c);
            pa[0] = make_float4(st.o[0][rr], st.o[1][rr], st.o[2][rr], st.o[3][rr]);
            pa[1] = make_float4(st.o[4][rr], st.o[5][rr], st.o[6][rr], st.o[7][rr]);
            if (c == 0) {
                a.part_m[slot] = m_h;
                a.part_l[slot] = l_h;
            }
        }
    }
}

} // namespace op::paged_attention::amd

#endif
