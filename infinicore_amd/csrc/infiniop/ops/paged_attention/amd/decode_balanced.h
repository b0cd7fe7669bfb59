// Work-equalising schedule of the tiled decode kernel for ragged batches.
//
// The plain grid of decode_tiled.h gives every (sequence, KV head) its own row of fixed-size
// partitions; with ragged lengths the number of units does not match the number of wavefronts the
// device can hold, and the last, half-empty round costs as much as a full one. Here the device
// does the split itself: for one KV head (and chunk of 16 query heads) all 16-token tiles of all
// sequences form one flat range [0, T); it is cut into `waves_per_stream` equal pieces, one per
// wavefront, so every wavefront streams the same number of bytes and they all finish together in a
// single round. A piece may cover the end of one sequence and the start of the next; each
// (piece, sequence) intersection is a segment with its own softmax state.
//
// Every wavefront derives the split from seq_lens alone (a prefix sum over the batch, redone per
// wavefront, kept in LDS), so nothing is read back to the host and no wavefront waits for another.
//   * a segment that covers its whole sequence is normalised and written to `out` directly;
//   * any other segment leaves (acc, m, l) in workspace row (piece + sequence), which is unique
//     per segment because consecutive segments advance the piece, the sequence or both;
//   * decodeBalancedMergeKernel recomputes the same split and merges the rows of each sequence.
// Tile arithmetic is computeTile() of decode_tiled.h unchanged.
#ifndef INFINICORE_AMD_PA_DECODE_BALANCED_H
#define INFINICORE_AMD_PA_DECODE_BALANCED_H

#include "decode_reduce.h"
#include "decode_tiled.h"

namespace op::paged_attention::amd {

#ifdef INFINIOP_AMD_PA_TRACE
// Diagnostic build only: per-wavefront timestamps (100 MHz constant clock) of the decode phases.
__device__ unsigned long long *g_pa_trace = nullptr;
#define PA_STAMP(slot)                                                                                   \
    do {                                                                                                 \
        if (g_pa_trace != nullptr && threadIdx.x == 0) {                                                 \
            g_pa_trace[(static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x) * 8 + (slot)] = __builtin_amdgcn_s_memrealtime(); \
        }                                                                                                \
    } while (0)
#else
#define PA_STAMP(slot) do {} while (0)
#endif

constexpr int kBalancedMaxSeqs = 1024; // prefix sums of the batch live in LDS
constexpr int kBalancedMinTiles = 4;   // never cut pieces finer than 64 tokens

// Inclusive prefix sums of the per-sequence tile counts into LDS; returns the total. Executed by
// one wavefront (lanes 0..63 of the caller).
template <typename Tindex>
__device__ __forceinline__ int tilePrefixSums(const DecodeArgs &a, int lane, int *pre_incl) {
    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) << a.block_shift;
    int running = 0;
    for (int base = 0; base < a.num_seqs; base += 64) {
        const int b = base + lane;
        int x = 0;
        if (b < a.num_seqs) {
            int64_t len = loadIndex<Tindex>(a.seq_lens, b);
            len = len < max_len ? len : max_len;
            x = len > 0 ? static_cast<int>((len + kTileTokens - 1) / kTileTokens) : 0;
        }
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int y = __shfl_up(x, off, 64);
            x += lane >= off ? y : 0;
        }
        x += running;
        if (b < a.num_seqs) {
            pre_incl[b] = x;
        }
        running = __shfl(x, 63, 64);
    }
    __builtin_amdgcn_wave_barrier();
    return running;
}

// Tiles per piece: the flat range split evenly over the wavefronts of a stream, but never finer
// than kBalancedMinTiles. Decode and merge kernels must agree on this.
__device__ __forceinline__ int tilesPerPiece(int total_tiles, int waves_per_stream) {
    const int q = (total_tiles + waves_per_stream - 1) / waves_per_stream;
    return q < kBalancedMinTiles ? kBalancedMinTiles : q;
}

template <typename T, typename Tindex>
__global__ void __launch_bounds__(64) decodeBalancedKernel(DecodeArgs a, int waves_per_stream) {
    using S = typename T::storage;
    __shared__ uint4 k_lds[kTileTokens * kTiledHead / 8];
    __shared__ int pre_incl[kBalancedMaxSeqs];

    const int piece = blockIdx.x;
    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int kv_head = blockIdx.y / head_chunks;
    const int chunk = blockIdx.y - kv_head * head_chunks;
    const int lane = threadIdx.x;
    const int c = lane & 15;
    const int g = lane >> 4;

    PA_STAMP(0);
    const int total_tiles = tilePrefixSums<Tindex>(a, lane, pre_incl);
    PA_STAMP(1);
    const int q = tilesPerPiece(total_tiles, waves_per_stream);
    const int f0 = piece * q;
    const int f1 = min(total_tiles, f0 + q);
    if (f0 >= f1) {
        return;
    }
    // first sequence whose tiles reach past f0
    int seq = 0;
    for (int base = 0; base < a.num_seqs; base += 64) {
        const int b = base + lane;
        seq += __popcll(__builtin_amdgcn_ballot_w64(b < a.num_seqs && pre_incl[b] <= f0));
    }

    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) << a.block_shift;
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;
    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
    const int block_mask = a.block_size - 1;
    const uint32_t k_row_bytes = static_cast<uint32_t>(a.k_row_stride) * sizeof(S);
    const uint32_t v_row_bytes = static_cast<uint32_t>(a.v_row_stride) * sizeof(S);
    uint32_t k_off[4], v_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        k_off[j] = (4 * j + g) * k_row_bytes + 16 * c;
        v_off[j] = (4 * g + j) * v_row_bytes + 16 * c;
    }

    int f = f0;
    while (f < f1) {
        // ---- segment: tiles [t_begin, t_end) of sequence `seq` ----
        const int seq_first = seq == 0 ? 0 : pre_incl[seq - 1];
        const int seq_tiles = pre_incl[seq] - seq_first;
        const int t_begin = f - seq_first;
        const int t_end = min(seq_tiles, f1 - seq_first);
        int64_t len64 = loadIndex<Tindex>(a.seq_lens, seq);
        const int len = static_cast<int>(len64 < max_len ? len64 : max_len);

        uint4 q_reg[4];
        {
            const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                q_reg[kk] = head_valid ? *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
            }
        }
        TileState st;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            st.o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        st.m = -INFINITY;
        st.l = 0.0f;

        // The segment is walked in runs of at most 64 block-table entries (one page id per lane).
        int t_run = t_begin;
        while (t_run < t_end) {
            const int first_entry = (t_run * kTileTokens) >> a.block_shift;
            const int last_entry_all = ((t_end * kTileTokens) - 1) >> a.block_shift;
            const int last_entry = min(last_entry_all, first_entry + 63);
            // last tile of this run: the one that ends with table entry `last_entry`
            const int run_end = min(t_end, (((last_entry + 1) << a.block_shift) + kTileTokens - 1) / kTileTokens);
            int page_ids = 0;
            if (first_entry + lane <= last_entry) {
                page_ids = clampPage(
                    loadIndex<Tindex>(a.block_tables, seq * a.block_table_batch_stride + first_entry + lane), a.num_blocks);
            }
            const int n_tiles = run_end - t_run;

            // loads past the end of the run: all lanes read the run's first 16 bytes (see decode_tiled.h)
            auto loadTile = [&](int t) -> TileRegs {
                const bool real = t < n_tiles;
                const uint32_t lane_mask = real ? 0xffffffffu : 0u;
                const int tok0 = (t_run + (real ? t : 0)) * kTileTokens;
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
            auto compute = [&](int t, const TileRegs &r) {
                const int tok0 = (t_run + t) * kTileTokens;
                computeTile<T>(st, r, q_reg, k_lds, c, g, a.scale_log2, slope, tok0 - (len - 1), min(kTileTokens, len - tok0));
            };

            PA_STAMP(2);
            streamTiles<INFINIOP_AMD_PA_BALANCED_BUFFERS>(n_tiles, loadTile, compute);
            t_run = run_end;
        }
        PA_STAMP(4);

        // ---- segment epilogue ----
        const float l_tot = sumAcrossTokenGroups(st.l);
        const bool whole = t_begin == 0 && t_end == seq_tiles;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int hl = 4 * g + rr;
            const float l_h = __shfl(l_tot, hl, 64);
            const float m_h = __shfl(st.m, hl, 64);
            const int hg = chunk * kHeadsPerWave + hl;
            if (hg >= a.group) {
                continue;
            }
            const int out_head = kv_head * a.group + hg;
            if (whole) {
                const float inv_l = 1.0f / (l_h + 1e-6f);
                uint4 packed;
                packed.x = T::pack2(st.o[0][rr] * inv_l, st.o[1][rr] * inv_l);
                packed.y = T::pack2(st.o[2][rr] * inv_l, st.o[3][rr] * inv_l);
                packed.z = T::pack2(st.o[4][rr] * inv_l, st.o[5][rr] * inv_l);
                packed.w = T::pack2(st.o[6][rr] * inv_l, st.o[7][rr] * inv_l);
                S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride;
                *reinterpret_cast<uint4 *>(o_ptr + 8 * c) = packed;
            } else {
                const int64_t slot = static_cast<int64_t>(piece + seq) * a.num_heads + out_head;
                float4 *pa = reinterpret_cast<float4 *>(a.part_acc + slot * kTiledHead + 8 * c);
                pa[0] = make_float4(st.o[0][rr], st.o[1][rr], st.o[2][rr], st.o[3][rr]);
                pa[1] = make_float4(st.o[4][rr], st.o[5][rr], st.o[6][rr], st.o[7][rr]);
                if (c == 0) {
                    a.part_m[slot] = m_h;
                    a.part_l[slot] = l_h;
                }
            }
        }

        PA_STAMP(5);
        f = seq_first + t_end;
        ++seq;
        // skip sequences without tokens
        while (f < f1 && seq < a.num_seqs && pre_incl[seq] <= f) {
            ++seq;
        }
    }
}

// Merge of the segment rows of one (query head, sequence); see decode_reduce.h for the arithmetic.
// One 256-thread workgroup: thread = (row group rg = tid / 16, 8-column strip c = tid % 16).
template <typename T, typename Tindex>
__global__ void __launch_bounds__(kReduceThreads) decodeBalancedMergeKernel(DecodeArgs a, int waves_per_stream) {
    using S = typename T::storage;
    constexpr int COLS = kTiledHead / 16;
    __shared__ int pre_incl[kBalancedMaxSeqs];
    __shared__ float wave_acc[4][16][COLS];
    __shared__ float wave_m[4][16];
    __shared__ float wave_l[4][16];

    const int head = blockIdx.x;
    const int seq = blockIdx.y;
    const int tid = threadIdx.x;
    const int c = tid & 15;
    const int rg = tid >> 4;
    const int wave = tid >> 6;

    // every wavefront redoes the prefix sums (identical values land in the same LDS words)
    const int total_tiles = tilePrefixSums<Tindex>(a, tid & 63, pre_incl);
    __syncthreads();
    const int q = tilesPerPiece(total_tiles, waves_per_stream);
    const int seq_first = seq == 0 ? 0 : pre_incl[seq - 1];
    const int seq_tiles = pre_incl[seq] - seq_first;
    if (seq_tiles <= 0) {
        return;
    }
    const int piece_first = seq_first / q;
    const int piece_last = (seq_first + seq_tiles - 1) / q;
    if (piece_first == piece_last) {
        return; // one segment covered the whole sequence and wrote `out` itself
    }
    const int parts = piece_last - piece_first + 1;

    float m_loc = -INFINITY, l_loc = 0.0f;
    float acc[COLS];
#pragma unroll
    for (int i = 0; i < COLS; ++i) {
        acc[i] = 0.0f;
    }
    for (int p = rg; p < parts; p += kReduceRowGroups) {
        const int64_t slot = static_cast<int64_t>(piece_first + p + seq) * a.num_heads + head;
        const float m_p = a.part_m[slot];
        const float l_p = a.part_l[slot];
        const float4 *row = reinterpret_cast<const float4 *>(a.part_acc + slot * kTiledHead + c * COLS);
        const float4 v0 = row[0], v1 = row[1];
        const float m_new = fmaxf(m_loc, m_p);
        const float w_old = mergeWeight(m_loc, m_new), w_p = mergeWeight(m_p, m_new);
        l_loc = l_loc * w_old + l_p * w_p;
        acc[0] = acc[0] * w_old + v0.x * w_p;
        acc[1] = acc[1] * w_old + v0.y * w_p;
        acc[2] = acc[2] * w_old + v0.z * w_p;
        acc[3] = acc[3] * w_old + v0.w * w_p;
        acc[4] = acc[4] * w_old + v1.x * w_p;
        acc[5] = acc[5] * w_old + v1.y * w_p;
        acc[6] = acc[6] * w_old + v1.z * w_p;
        acc[7] = acc[7] * w_old + v1.w * w_p;
        m_loc = m_new;
    }

    const float m_w = swapMax(m_loc);
    const float fct = mergeWeight(m_loc, m_w);
    const float l_w = swapSum(l_loc * fct);
#pragma unroll
    for (int i = 0; i < COLS; ++i) {
        acc[i] = swapSum(acc[i] * fct);
    }
    if ((tid & 63) < 16) {
        wave_m[wave][c] = m_w;
        wave_l[wave][c] = l_w;
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
            wave_acc[wave][c][i] = acc[i];
        }
    }
    __syncthreads();

    if (tid < 16) {
        float m = wave_m[0][c];
#pragma unroll
        for (int w = 1; w < 4; ++w) {
            m = fmaxf(m, wave_m[w][c]);
        }
        float l = 0.0f, out_acc[COLS];
#pragma unroll
        for (int i = 0; i < COLS; ++i) {
            out_acc[i] = 0.0f;
        }
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float fw = mergeWeight(wave_m[w][c], m);
            l += wave_l[w][c] * fw;
#pragma unroll
            for (int i = 0; i < COLS; ++i) {
                out_acc[i] += wave_acc[w][c][i] * fw;
            }
        }
        const float inv_l = 1.0f / (l + 1e-6f);
        uint4 packed;
        packed.x = T::pack2(out_acc[0] * inv_l, out_acc[1] * inv_l);
        packed.y = T::pack2(out_acc[2] * inv_l, out_acc[3] * inv_l);
        packed.z = T::pack2(out_acc[4] * inv_l, out_acc[5] * inv_l);
        packed.w = T::pack2(out_acc[6] * inv_l, out_acc[7] * inv_l);
        S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride;
        *reinterpret_cast<uint4 *>(o_ptr + c * COLS) = packed;
    }
}

} // namespace op::paged_attention::amd

#endif
