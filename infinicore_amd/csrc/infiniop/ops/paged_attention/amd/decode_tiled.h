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
//   * the loads of tile t+1 are issued before tile t is computed; page ids of the whole partition
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

struct TileRegs {
    uint4 k[4]; // k[j]: token row 4j+g, columns 8c..8c+7
    uint4 v[4]; // v[j]: token row 4g+j, columns 8c..8c+7
};

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

    const S *k_head = static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride;
    const S *v_head = static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride;
    const int block_mask = a.block_size - 1;

    auto loadTile = [&](int t, TileRegs &r) {
        const int tok0 = start + t * kTileTokens;
        const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
        const int row0 = tok0 & block_mask;
        const S *k_tile = k_head + page * a.k_batch_stride + row0 * a.k_row_stride;
        const S *v_tile = v_head + page * a.v_batch_stride + row0 * a.v_row_stride;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            r.k[j] = *reinterpret_cast<const uint4 *>(k_tile + (4 * j + g) * a.k_row_stride + 8 * c);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            r.v[j] = *reinterpret_cast<const uint4 *>(v_tile + (4 * g + j) * a.v_row_stride + 8 * c);
        }
    };

    f32x4 o_acc[8]; // o_acc[e][r] = O[head 4g+r of the chunk][column 8c+e]
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        o_acc[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    float m_run = -INFINITY; // running maximum of head c (same value in the four lanes g = 0..3)
    float l_run = 0.0f;      // sum of rounded probabilities of head c over this lane's tokens only

    auto computeTile = [&](int t, TileRegs &r) {
        const int tok0 = start + t * kTileTokens;

        // K: registers -> swizzled LDS -> matrix-operand layout (token c, columns 32*kk + 8g .. +7)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = 4 * j + g;
            k_lds[row * 16 + (c ^ row)] = r.k[j];
        }
        __builtin_amdgcn_wave_barrier();
        f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            const uint4 k_op = k_lds[c * 16 + ((4 * kk + g) ^ c)];
            s = T::mfmaK32(k_op, q_reg[kk], s);
        }
        __builtin_amdgcn_wave_barrier();

        // scores of head c for tokens tok0 + 4g + r, log2 domain
        float sc[4];
        const bool tail = tok0 + kTileTokens > end;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int tok = tok0 + 4 * g + rr;
            sc[rr] = s[rr] * a.scale_log2 + slope * static_cast<float>(tok - (len - 1));
            if (tail && tok >= end) {
                sc[rr] = -INFINITY;
            }
        }
        float mx = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);

        if (__builtin_amdgcn_ballot_w64(m_new > m_run) != 0) {
            // some head's maximum moved: rescale. Lane holds accumulators of heads 4g..4g+3, whose
            // factors live in lanes 4g..4g+3.
            const float alpha = fastExp2(m_run - m_new);
            l_run *= alpha;
            m_run = m_new;
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                const float alpha_r = __shfl(alpha, 4 * g + rr, 64);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    o_acc[e][rr] *= alpha_r;
                }
            }
        }

        // probabilities, rounded to the storage dtype: A operand of P.V
        uint2 p_op;
        p_op.x = T::pack2(fastExp2(sc[0] - m_run), fastExp2(sc[1] - m_run));
        p_op.y = T::pack2(fastExp2(sc[2] - m_run), fastExp2(sc[3] - m_run));
        l_run += (T::unpackLo(p_op.x) + T::unpackHi(p_op.x)) + (T::unpackLo(p_op.y) + T::unpackHi(p_op.y));

        // V rows beyond the sequence may hold anything (NaN included): zero them, 0 * NaN is NaN.
        if (tail) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (tok0 + 4 * g + j >= end) {
                    r.v[j] = make_uint4(0, 0, 0, 0);
                }
            }
        }

        // O += P . V, one 16-column output tile per e: column 8c+e of rows 4g..4g+3
        const uint32_t v0[4] = {r.v[0].x, r.v[0].y, r.v[0].z, r.v[0].w};
        const uint32_t v1[4] = {r.v[1].x, r.v[1].y, r.v[1].z, r.v[1].w};
        const uint32_t v2[4] = {r.v[2].x, r.v[2].y, r.v[2].z, r.v[2].w};
        const uint32_t v3[4] = {r.v[3].x, r.v[3].y, r.v[3].z, r.v[3].w};
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            uint2 even, odd;
            even.x = __builtin_amdgcn_perm(v1[w], v0[w], 0x05040100u);
            even.y = __builtin_amdgcn_perm(v3[w], v2[w], 0x05040100u);
            odd.x = __builtin_amdgcn_perm(v1[w], v0[w], 0x07060302u);
            odd.y = __builtin_amdgcn_perm(v3[w], v2[w], 0x07060302u);
            o_acc[2 * w] = T::mfmaK16(p_op, even, o_acc[2 * w]);
            o_acc[2 * w + 1] = T::mfmaK16(p_op, odd, o_acc[2 * w + 1]);
        }
    };

    // Two register sets alternate so that the loads of the next tile are in flight while the
    // current one is computed.
    TileRegs ra, rb;
    loadTile(0, ra);
    for (int t = 0; t < n_tiles; t += 2) {
        if (t + 1 < n_tiles) {
            loadTile(t + 1, rb);
        }
        computeTile(t, ra);
        if (t + 1 < n_tiles) {
            if (t + 2 < n_tiles) {
                loadTile(t + 2, ra);
            }
            computeTile(t + 1, rb);
        }
    }

    // Epilogue. Denominator of head c over all 16 token slots, then move per-head scalars to the
    // lanes that hold that head's accumulators.
    float l_tot = l_run + __shfl_xor(l_run, 16, 64);
    l_tot += __shfl_xor(l_tot, 32, 64);

    const bool single = len <= a.partition_tokens;
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        const int hl = 4 * g + rr; // head (within the chunk) of accumulator row rr
        const float l_h = __shfl(l_tot, hl, 64);
        const float m_h = __shfl(m_run, hl, 64);
        const int hg = chunk * kHeadsPerWave + hl;
        if (hg >= a.group) {
            continue;
        }
        const int out_head = kv_head * a.group + hg;
        if (single) {
            const float inv_l = 1.0f / (l_h + 1e-6f);
            uint4 packed;
            packed.x = T::pack2(o_acc[0][rr] * inv_l, o_acc[1][rr] * inv_l);
            packed.y = T::pack2(o_acc[2][rr] * inv_l, o_acc[3][rr] * inv_l);
            packed.z = T::pack2(o_acc[4][rr] * inv_l, o_acc[5][rr] * inv_l);
            packed.w = T::pack2(o_acc[6][rr] * inv_l, o_acc[7][rr] * inv_l);
            S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride;
            *reinterpret_cast<uint4 *>(o_ptr + 8 * c) = packed;
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            float4 *pa = reinterpret_cast<float4 *>(a.part_acc + slot * kTiledHead + 8 * c);
            pa[0] = make_float4(o_acc[0][rr], o_acc[1][rr], o_acc[2][rr], o_acc[3][rr]);
            pa[1] = make_float4(o_acc[4][rr], o_acc[5][rr], o_acc[6][rr], o_acc[7][rr]);
            if (c == 0) {
                a.part_m[slot] = m_h;
                a.part_l[slot] = l_h;
            }
        }
    }
}

} // namespace op::paged_attention::amd

#endif
