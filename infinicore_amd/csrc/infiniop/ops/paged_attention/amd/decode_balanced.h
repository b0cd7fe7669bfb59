// Work-equalising schedule of the tiled decode kernel for ragged batches.
//
// The plain grid of decode_tiled.h gives every (sequence, KV head) its own row of fixed-size
// partitions; with ragged lengths the number of units does not match the number of wavefronts the
// device can hold, and the last, half-empty round costs as much as a full one. Here the device
// does the split itself: for one KV head (and chunk of 16 query heads) all 16-token tiles of all
// sequences form one flat range [0, T); it is cut into `waves_per_stream` pieces of equal cost (equal
// tile counts, less a few tiles for every sequence that starts inside the piece), one per wavefront,
// so they all finish together in a single round. A piece may cover the end of one sequence and the
// start of the next; each (piece, sequence) intersection is a segment with its own softmax state.
//
// Every wavefront derives the split from seq_lens alone (a prefix sum over the batch, redone per
// wavefront, kept in LDS), so nothing is read back to the host and no wavefront waits for another.
//   * a segment that covers its whole sequence is normalised and written to `out` directly;
//   * any other segment leaves (acc, m, l) in workspace row (piece + sequence), which is unique
//     per segment because consecutive segments advance the piece, the sequence or both;
//   * the wavefront whose piece holds a sequence's first tile records which pieces the sequence spans
//     (seq_pieces), and decodeBalancedMergeKernel merges the rows of each sequence from that.
// Tile arithmetic is computeTile() of decode_tiled.h unchanged.
#ifndef INFINICORE_AMD_PA_DECODE_BALANCED_H
#define INFINICORE_AMD_PA_DECODE_BALANCED_H

#include "decode_reduce.h"
#include "decode_tiled.h"

namespace op::paged_attention::amd {

constexpr int kBalancedMinTiles = 4;   // never cut pieces finer than 64 tokens
constexpr int kReaderSpinLimit = 1 << 22; // polls (~0.5 us each) before a reader gives up on a flag

// Inclusive prefix sum over the 64 lanes with data-parallel-primitive moves (no LDS-unit permutes: this
// runs at the head of every wavefront, before its first memory request can go out). Rows of 16 lanes are
// scanned with row shifts, then lane 15 of rows 0 and 2 is added to the next row, then lane 31 to rows 2, 3.
__device__ __forceinline__ int waveInclusiveSum(int x) {
    x += __builtin_amdgcn_update_dpp(0, x, 0x111, 0xf, 0xf, false); // row_shr:1
    x += __builtin_amdgcn_update_dpp(0, x, 0x112, 0xf, 0xf, false); // row_shr:2
    x += __builtin_amdgcn_update_dpp(0, x, 0x114, 0xf, 0xf, false); // row_shr:4
    x += __builtin_amdgcn_update_dpp(0, x, 0x118, 0xf, 0xf, false); // row_shr:8
    x += __builtin_amdgcn_update_dpp(0, x, 0x142, 0xa, 0xf, false); // row_bcast:15 into rows 1 and 3
    x += __builtin_amdgcn_update_dpp(0, x, 0x143, 0xc, 0xf, false); // row_bcast:31 into rows 2 and 3
    return x;
}

// Inclusive prefix sums of the per-sequence tile counts into LDS; returns the total. Executed by
// one wavefront (lanes 0..63 of the caller).
template <typename Tindex>
__device__ __forceinline__ int tilePrefixSums(const void *seq_lens, int num_seqs, int max_blocks_per_seq, int block_shift,
                                              int lane, int *pre_incl) {
    const int64_t max_len = static_cast<int64_t>(max_blocks_per_seq) << block_shift;
    int running = 0;
    for (int base = 0; base < num_seqs; base += 64) {
        const int b = base + lane;
        int x = 0;
        if (b < num_seqs) {
            int64_t len = loadIndex<Tindex>(seq_lens, b);
            len = len < max_len ? len : max_len;
            x = len > 0 ? static_cast<int>((len + kTileTokens - 1) / kTileTokens) : 0;
        }
        x = waveInclusiveSum(x) + running;
        if (b < num_seqs) {
            pre_incl[b] = x;
        }
        running = __builtin_amdgcn_readlane(x, 63);
    }
    __builtin_amdgcn_wave_barrier();
    // every lane holds the same total; say so, or all index arithmetic derived from it is
    // compiled as per-lane (vector) code with per-lane branches
    return __builtin_amdgcn_readfirstlane(running);
}

// Slots (tiles plus start costs) per piece: the range split evenly over the wavefronts of a stream, but
// never finer than kBalancedMinTiles.
__device__ __forceinline__ int tilesPerPiece(int total_tiles, int waves_per_stream) {
    const int q = (total_tiles + waves_per_stream - 1) / waves_per_stream;
    return q < kBalancedMinTiles ? kBalancedMinTiles : q;
}

// The prefix sums are read from LDS with a wave-uniform index; readfirstlane tells the compiler the
// value is uniform too, so everything derived from it stays in scalar registers and scalar branches.
__device__ __forceinline__ int uniformRead(const int *lds_word) {
    return __builtin_amdgcn_readfirstlane(*lds_word);
}

// Moves a loop-carried value that a load produced into the register of its consumer with an explicit
// instruction. Written as a plain assignment the move is left to the end of the block, after the
// load that refills the source has been issued; that load then cannot write the source register,
// arrives in a temporary, and the copy out of the temporary waits for every load in flight - a full
// drain of the tile pipeline at every run and segment change.
__device__ __forceinline__ unsigned handOver(unsigned v) {
    unsigned r;
    asm volatile("v_mov_b32 %0, %1" : "=v"(r) : "v"(v));
    return r;
}
__device__ __forceinline__ int handOver(int v) { return static_cast<int>(handOver(static_cast<unsigned>(v))); }

// A run = consecutive tiles of one sequence whose pages fit one page-id register (64 block-table
// entries, one per lane). All members are wave-uniform.
struct TileRun {
    int seq;
    int t0, t1;      // tiles [t0, t1) of the sequence
    int seg_end;     // end of the segment (this wavefront's share of the sequence) the run belongs to
    int first_entry; // block-table entry of tile t0
    bool valid;      // false past the end of the wavefront's piece
};

// Early arguments: the four scalars in front of the argument block are what the first memory request (the
// sequence lengths) needs. The file is compiled with -amdgpu-kernarg-preload-count=5, which has the
// dispatcher put the first five argument words into scalar registers before the wavefront starts, so that
// request goes out without waiting for the scalar load of the argument block (which proceeds beside it).
// They repeat a.seq_lens, a.num_seqs, a.max_blocks_per_seq and a.block_shift.
// Register budget: at head 128 the kernel is compiled for two wavefronts per SIMD (256 vector registers,
// no accumulation registers). It runs one per SIMD all the same (the grid has four wavefronts per compute
// unit); the point is the allocation: left alone the compiler takes 234 vector + 36 accumulation registers
// and moves values between the two files in the tile loop, with the budget it fits 230 vector registers
// without spilling (c2 57.7 -> 56.6 us, three runs each on one box). Heads 192 and 256 spill under that
// budget, head 64 fits it anyway: they are left to the compiler.
//
// FUSED: the segments of a sequence are merged by the decode kernel itself instead of by a second kernel. The
// wavefront whose piece holds a sequence's LAST segment is that sequence's reader: it keeps its own segment's
// state, and when its piece is done it waits for the rows of the sequence's earlier segments, merges them and
// writes the output. The earlier segments belong to earlier pieces of the same stream, i.e. to workgroups with
// lower linear ids, and a wavefront publishes its rows before it starts to wait for anybody else's: a reader
// only ever waits for wavefronts that were dispatched before it and that never wait before they publish, so
// the scheme cannot deadlock however few of the workgroups are resident at a time (the wait is bounded all
// the same). Rows and flags cross between accelerator dies with agent-scope accesses (decode_common.h).
template <typename T, typename Tindex, int HEAD, bool FUSED>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(HEAD == 128 ? 2 : 1, HEAD == 128 ? 2 : 8)))
decodeBalancedKernel(const void *early_seq_lens, int early_num_seqs, int early_max_blocks_per_seq, int early_block_shift,
                     DecodeArgs a, int waves_per_stream) {
    using S = typename T::storage;
    using G = TileGeometry<HEAD>;
    constexpr int NBUF = G::kBuffers;
    __shared__ uint4 k_lds[kTileTokens * G::kChunksPerRow];
    __shared__ int pre_incl[kBalancedMaxSeqs];
    // one finished segment's state (accumulators, denominator, maximum), word-major so that lane i
    // always touches bank i: written and read back by the same lane
    __shared__ float stash[(4 * G::kCols + 2) * 64];
    // FUSED: the state of the segment this wavefront is the reader of, until the end of the piece
    __shared__ float reader_stash[FUSED ? (4 * G::kCols + 2) * 64 : 1];

    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int streams = static_cast<int>(gridDim.y);
    const int piece = static_cast<int>(blockIdx.x);
    const int stream = static_cast<int>(blockIdx.y);
    const int kv_head = stream / head_chunks;
    const int chunk = stream - kv_head * head_chunks;
    const int lane = threadIdx.x;
    const int c = lane & 15;
    const int g = lane >> 4;

    // Where this wavefront's first kLead tiles were in the previous call on this workspace, as (page, first
    // row) pairs: requested beside the lengths, used further down to ask for those tiles one memory round trip
    // early (see "speculative first tiles").
    constexpr int kLead = NBUF - 1;
    static_assert(2 * kLead <= kFirstTileInts, "an entry holds the pairs of kLead tiles");
    int *const my_first_tiles = a.first_tiles + (static_cast<int64_t>(piece) * streams + stream) * kFirstTileInts;
    int guess[2 * kLead];
#pragma unroll
    for (int i = 0; i < 2 * kLead; ++i) {
        guess[i] = my_first_tiles[i];
    }
    const int total_tiles = tilePrefixSums<Tindex>(early_seq_lens, early_num_seqs, early_max_blocks_per_seq,
                                                   early_block_shift, lane, pre_incl);
    // The flat range is not cut into equal tile counts but into equal COST: a sequence that begins inside
    // a piece costs its wavefront about as much time as kStartCost more tiles would (measured: pieces with
    // such a start finish level with the others when they hold three to four tiles fewer at head 128), and they were
    // the last to finish. On a virtual axis every sequence is preceded by kStartCost empty slots; pieces are
    // equal ranges of that axis, and a piece's tiles are the real tiles its range covers: tile i of
    // sequence s sits at virtual position (tiles before s) + i + kStartCost * (s + 1).
    constexpr int kStartCost = HEAD <= 128 ? 384 / HEAD : 2;
    static_assert(kStartCost <= kBalancedMaxStartCost, "the launch plan bounds the flat axis with this");
    const int q = tilesPerPiece(total_tiles + kStartCost * a.num_seqs, waves_per_stream);
    // Pieces come in pairs (even, odd) that share 2 q slots; the even one takes q + relief of them.
    const int relief = (q * a.odd_piece_relief) >> 8;
    auto pieceOf = [&](int x) { // the piece that holds virtual slot x
        const int pair = x / (2 * q);
        return 2 * pair + (x - 2 * pair * q >= q + relief ? 1 : 0);
    };
    // Real tiles below virtual positions x0 and x1, the ends of this piece: count the sequences that lie
    // entirely below each (one pass over the prefix sums for both), then add the part of the next one.
    const int x0 = piece * q + ((piece & 1) ? relief : 0), x1 = (piece + 1) * q + ((piece & 1) ? 0 : relief);
    int s0 = 0, s1 = 0;
    int first_64 = 0; // prefix sum of sequence `lane`: the first 64 are kept in a register as well
    for (int base = 0; base < a.num_seqs; base += 64) {
        const int b = base + lane;
        const int mine = b < a.num_seqs ? pre_incl[b] : 0x3fffffff;
        first_64 = base == 0 ? mine : first_64;
        const int seq_end = mine + kStartCost * (b + 1);
        s0 += __popcll(__builtin_amdgcn_ballot_w64(seq_end <= x0));
        s1 += __popcll(__builtin_amdgcn_ballot_w64(seq_end <= x1));
    }
    s0 = __builtin_amdgcn_readfirstlane(s0);
    s1 = __builtin_amdgcn_readfirstlane(s1);
    // prefix sum of sequence s (wave-uniform s): a lane read for the first 64 sequences, which costs a few
    // clocks where the LDS round trip costs a hundred, and these reads are chained at every piece start
    // and segment switch
    auto prefixAt = [&](int s) {
        return s < 64 ? __builtin_amdgcn_readlane(first_64, s) : uniformRead(&pre_incl[s]);
    };
    auto tilesBelow = [&](int x, int s) {
        if (s >= a.num_seqs) {
            return total_tiles;
        }
        const int first = s == 0 ? 0 : prefixAt(s - 1);
        const int inside = x - (first + kStartCost * s) - kStartCost; // tiles of sequence s below x
        return first + max(0, min(inside, prefixAt(s) - first));
    };
    const int f0 = tilesBelow(x0, s0);
    const int f1 = tilesBelow(x1, s1);
    if (f0 >= f1) {
        return;
    }
    // first sequence whose tiles reach past f0: s0, or a later one if s0 has no tile at or after f0
    int seq0 = s0;
    while (prefixAt(seq0) <= f0) {
        ++seq0;
    }

    const int64_t max_len = static_cast<int64_t>(a.max_blocks_per_seq) << a.block_shift;
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;
    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
    const int block_mask = a.block_size - 1;
    const int tiles_per_entry_shift = a.block_shift - 4; // log2(block_size / 16)
    const LaneOffsets<HEAD> off(lane, static_cast<uint32_t>(a.k_row_stride) * sizeof(S),
                                static_cast<uint32_t>(a.v_row_stride) * sizeof(S));

    // ---- wave-uniform walk over the piece: sequences -> segments -> runs ----
    auto seqFirstTile = [&](int s) { return s == 0 ? 0 : prefixAt(s - 1); };
    auto seqLastTile = [&](int s) { return prefixAt(s); };
    auto makeRun = [&](int s, int t0, int seg_end) {
        TileRun r;
        r.seq = s;
        r.t0 = t0;
        r.seg_end = seg_end;
        r.first_entry = t0 >> tiles_per_entry_shift;
        const int last_entry = min((seg_end - 1) >> tiles_per_entry_shift, r.first_entry + 63);
        r.t1 = min(seg_end, (last_entry + 1) << tiles_per_entry_shift);
        r.valid = true;
        return r;
    };
    // run that starts at flat tile `flat`, which lies in sequence s
    auto runAtFlat = [&](int s, int flat) {
        const int first = seqFirstTile(s);
        return makeRun(s, flat - first, min(seqLastTile(s) - first, f1 - first));
    };
    auto nextRun = [&](const TileRun &r) {
        if (r.t1 < r.seg_end) {
            return makeRun(r.seq, r.t1, r.seg_end);
        }
        const int flat = seqFirstTile(r.seq) + r.seg_end;
        if (!r.valid || flat >= f1) {
            TileRun none = r;
            none.valid = false;
            return none;
        }
        int s = r.seq + 1;
        while (seqLastTile(s) <= flat) { // sequences without tokens
            ++s;
        }
        return runAtFlat(s, flat);
    };
    // Page ids of a run: table entries first_entry .. first_entry + 63, one per lane. The load is
    // unconditional (lanes past the run's last entry re-read that entry, a run past the end of the
    // piece re-reads its predecessor's): a predicated load reaches its loop-carried register through a
    // copy, and that copy waits for every load in flight. Low 32 bits, untouched: the value is
    // clamped where it is used, so that nothing waits for this load while tiles are in flight.
    auto loadPageIds = [&](const TileRun &r) {
        const int last_entry = (r.t1 - 1) >> tiles_per_entry_shift;
        const int entry = min(r.first_entry + lane, last_entry);
        return static_cast<int>(loadIndex<Tindex>(a.block_tables, r.seq * a.block_table_batch_stride + entry));
    };

    // ---- load side: runs NBUF-1 tiles ahead of the compute side, across runs and sequences ----
    TileRun ld_run = runAtFlat(seq0, f0);
    int ld_ids = loadPageIds(ld_run);
    TileRun ld_next = nextRun(ld_run);
    int ld_next_ids = loadPageIds(ld_next);
    int ld_t = ld_run.t0;

    auto loadNextTile = [&]() -> TileRegs<HEAD> {
        const bool real = ld_run.valid;
        const uint32_t lane_mask = real ? 0xffffffffu : 0u;
        const int entry = real ? (ld_t >> tiles_per_entry_shift) - ld_run.first_entry : 0;
        const int page = real ? clampPage(__builtin_amdgcn_readlane(ld_ids, entry), a.num_blocks) : 0;
        const int row0 = real ? (ld_t * kTileTokens) & block_mask : 0;
        const char *k_tile = k_head + (page * a.k_batch_stride + row0 * a.k_row_stride) * static_cast<int64_t>(sizeof(S));
        const char *v_tile = v_head + (page * a.v_batch_stride + row0 * a.v_row_stride) * static_cast<int64_t>(sizeof(S));
        const TileRegs<HEAD> r = loadTileRegs<HEAD>(k_tile, v_tile, off, lane_mask);
        if (real && ++ld_t == ld_run.t1) {
            // next run: its page ids were requested one run ago
            ld_run = ld_next;
            ld_ids = handOver(ld_next_ids);
            ld_t = ld_run.t0;
            ld_next = nextRun(ld_run);
            ld_next_ids = loadPageIds(ld_next);
        }
        return r;
    };

    // ---- compute side ----
    TileState<HEAD> st;
    uint4 q_reg[G::kLoads];
    int c_seq = seq0, c_t = 0, c_t_begin = 0, c_seg_end = 0, c_seq_tiles = 0, c_len = 0;

    // Query and length of the sequence that follows the current one in this piece, requested when the
    // current segment begins. A piece that crosses a sequence boundary would otherwise stop at the
    // boundary for a full memory round trip with no tile requests going out, and such pieces are the
    // last to finish.
    uint4 q_next[G::kLoads];
    int64_t len_next = 0;
    int next_seq = -1; // -1: the piece ends inside the current sequence

    // (a wavefront whose 16 lanes-heads are not all real reads head 0 for the others: valid memory,
    // and their columns are never stored - a predicated load would come back through a copy that
    // waits for every load in flight)
    auto requestQuery = [&](int s, uint4(&dst)[G::kLoads]) {
        const S *q_ptr = static_cast<const S *>(a.q) + s * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
#pragma unroll
        for (int kk = 0; kk < G::kLoads; ++kk) {
            dst[kk] = *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g);
        }
    };
    // ask for the query and length of the sequence after segment [.., flat_end) of sequence s, if the piece reaches it
    auto requestNext = [&](int s, int flat_end) {
        next_seq = -1;
        if (flat_end < f1) {
            int n = s + 1;
            while (seqLastTile(n) <= flat_end) { // sequences without tokens
                ++n;
            }
            next_seq = n;
            len_next = loadIndex<Tindex>(a.seq_lens, n);
            requestQuery(n, q_next);
        }
    };

    auto clampLength = [&](int64_t len64) {
        return __builtin_amdgcn_readfirstlane(static_cast<int>(len64 < max_len ? len64 : max_len));
    };
    // bookkeeping of a new segment: tiles [flat - first, ..) of sequence s, which has `len` tokens
    auto beginSegment = [&](int s, int flat, int len) {
        const int first = seqFirstTile(s);
        c_seq = s;
        c_seq_tiles = seqLastTile(s) - first;
        c_t_begin = flat - first;
        c_t = c_t_begin;
        c_seg_end = min(c_seq_tiles, f1 - first);
        c_len = len;
#pragma unroll
        for (int e = 0; e < G::kCols; ++e) {
            st.o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
        }
        st.m = -INFINITY;
        st.l = 0.0f;
        requestNext(s, first + c_seg_end);
    };
    // Use the query inside the rarely taken segment switch: the wait for it lands there and the
    // per-tile code keeps waiting for exactly its own tile, with the others still in flight.
    auto pinQuery = [&]() {
#pragma unroll
        for (int kk = 0; kk < G::kLoads; ++kk) {
            asm volatile("" ::"v"(q_reg[kk].x), "v"(q_reg[kk].y), "v"(q_reg[kk].z), "v"(q_reg[kk].w));
        }
    };

    // Stores the result of a finished segment of sequence `seq`: normalised output rows if the segment
    // covered the whole sequence, else the partial (acc, m, l) rows for the merge kernel.
    auto writeResult = [&](const TileState<HEAD> &state, float l_tot, int seq, bool whole) {
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const int hl = 4 * g + rr;
            const float l_h = __shfl(l_tot, hl, 64);
            const float m_h = __shfl(state.m, hl, 64);
            const int hg = chunk * kHeadsPerWave + hl;
            if (hg >= a.group) {
                continue;
            }
            const int out_head = kv_head * a.group + hg;
            if (whole) {
                S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride;
                storeOutputRow<T, HEAD>(o_ptr, c, state, rr, 1.0f / (l_h + 1e-6f));
            } else {
                const int64_t slot = static_cast<int64_t>(piece + seq) * a.num_heads + out_head;
                storePartialRow<HEAD>(a.part_acc + slot * HEAD + G::kCols * c, state, rr);
                if (c == 0) {
                    a.part_m[slot] = m_h;
                    a.part_l[slot] = l_h;
                }
            }
        }
    };
    // FUSED: partial rows of a segment for the reader of its sequence, and the flag that says they are there.
    // A row of head h is HEAD floats, stored as 16-byte chunks in the order (chunk of the lane, strip c): each
    // store instruction then writes 256 contiguous bytes per head. (m, l) of the 16 heads follow as pairs in the
    // place of the m and l arrays. Heads beyond the group lie beyond the buffers' sizes: nothing is stored.
    const int heads_here = min(kHeadsPerWave, a.group - chunk * kHeadsPerWave);
    const int first_head = kv_head * a.group + chunk * kHeadsPerWave;
    auto rowsOf = [&](int row_group) { // row_group = piece + sequence
        return agentBuffer(a.part_acc + (static_cast<int64_t>(row_group) * a.num_heads + first_head) * HEAD,
                           heads_here * HEAD * static_cast<int>(sizeof(float)));
    };
    auto pairsOf = [&](int row_group) {
        return agentBuffer(reinterpret_cast<float2 *>(a.part_m) + static_cast<int64_t>(row_group) * a.num_heads + first_head,
                           heads_here * static_cast<int>(sizeof(float2)));
    };
    auto publishSegment = [&](const TileState<HEAD> &state, float l_tot, int seq) {
        const auto rows = rowsOf(piece + seq);
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
#pragma unroll
            for (int h = 0; h < G::kCols / 4; ++h) {
                storeAgent16(rows, (4 * g + rr) * HEAD * 4 + 256 * h + 16 * c, state.o[4 * h][rr], state.o[4 * h + 1][rr],
                             state.o[4 * h + 2][rr], state.o[4 * h + 3][rr]);
            }
        }
        if (g == 0) {
            storeAgent8(pairsOf(piece + seq), 8 * c, state.m, l_tot); // lane c holds head c's maximum and sum
        }
        waitVectorMemory(); // the rows are in memory before the flag says so
        if (lane == 0) {
            storeAgent(a.seg_flags + static_cast<int64_t>(piece + seq) * streams + stream, a.token);
        }
    };

    // A segment that ends in the middle of the piece is not stored at once: stores count as outstanding
    // memory operations like the tile loads, the waits of the tile loop are fixed counts, and with a
    // few dozen stores in front of them they would wait for the stores' round trip while no tile
    // request goes out. Its state is parked in LDS instead and stored when the piece is done (or when
    // the next segment ends, if the piece holds several).
    int stash_seq = -1;
    bool stash_whole = false;
    auto flushStash = [&]() {
        TileState<HEAD> parked;
#pragma unroll
        for (int e = 0; e < G::kCols; ++e) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                parked.o[e][rr] = stash[(4 * e + rr) * 64 + lane];
            }
        }
        const float l_tot = stash[(4 * G::kCols) * 64 + lane];
        parked.m = stash[(4 * G::kCols + 1) * 64 + lane];
        parked.l = 0.0f;
        writeResult(parked, l_tot, stash_seq, stash_whole);
        stash_seq = -1;
    };
    int reader_seq = -1; // FUSED: the sequence whose last segment this piece holds next to earlier ones elsewhere
    auto parkReaderSegment = [&]() {
        const float l_tot = sumAcrossTokenGroups(st.l);
#pragma unroll
        for (int e = 0; e < G::kCols; ++e) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                reader_stash[(4 * e + rr) * 64 + lane] = st.o[e][rr];
            }
        }
        reader_stash[(4 * G::kCols) * 64 + lane] = l_tot;
        reader_stash[(4 * G::kCols + 1) * 64 + lane] = st.m;
        reader_seq = c_seq;
    };
    auto parkSegment = [&]() {
        if constexpr (FUSED) {
            if (c_t_begin > 0 && c_seg_end == c_seq_tiles) {
                parkReaderSegment(); // ends a sequence that began in an earlier piece
                return;
            }
        }
        if (stash_seq >= 0) {
            flushStash();
        }
        const float l_tot = sumAcrossTokenGroups(st.l);
#pragma unroll
        for (int e = 0; e < G::kCols; ++e) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                stash[(4 * e + rr) * 64 + lane] = st.o[e][rr];
            }
        }
        stash[(4 * G::kCols) * 64 + lane] = l_tot;
        stash[(4 * G::kCols + 1) * 64 + lane] = st.m;
        stash_seq = c_seq;
        stash_whole = c_t_begin == 0 && c_seg_end == c_seq_tiles;
    };

    auto computeNextTile = [&](const TileRegs<HEAD> &r) {
        const int tok0 = c_t * kTileTokens;
        computeTile<T, HEAD>(st, r, q_reg, k_lds, lane, c, g, a.scale_log2, slope, tok0 - (c_len - 1),
                             min(kTileTokens, c_len - tok0));
        if (++c_t == c_seg_end) {
            if (next_seq >= 0) {
                // The next sequence's query and length were asked for when this segment began.
                const int next_len = clampLength(len_next);
#pragma unroll
                for (int kk = 0; kk < G::kLoads; ++kk) {
                    q_reg[kk].x = handOver(q_next[kk].x);
                    q_reg[kk].y = handOver(q_next[kk].y);
                    q_reg[kk].z = handOver(q_next[kk].z);
                    q_reg[kk].w = handOver(q_next[kk].w);
                }
                __builtin_amdgcn_sched_barrier(0);
                const int flat = seqFirstTile(c_seq) + c_seg_end;
                parkSegment();
                beginSegment(next_seq, flat, next_len);
            }
        }
    };

    // Tell the merge kernel which pieces hold each sequence that starts in this piece (one writer per
    // sequence: the wavefront of the first stream whose piece contains the sequence's first tile).
    // Done before the first tile is requested, for the reason given at parkSegment.
    if (!FUSED && stream == 0) {
        for (int base = seq0; base < a.num_seqs; base += 64) {
            const int s = base + lane;
            bool more = false;
            if (s < a.num_seqs) {
                const int first = s == 0 ? 0 : pre_incl[s - 1];
                const int last = pre_incl[s];
                more = first < f1;
                if (last > first && first >= f0 && first < f1) {
                    a.seq_pieces[s] = make_int2(piece, pieceOf(last - 1 + kStartCost * (s + 1)) - piece + 1);
                }
            }
            if (__builtin_amdgcn_ballot_w64(more) == 0) {
                break;
            }
        }
    }
    const int n_flat = f1 - f0;
    TileRegs<HEAD> buf[NBUF];
    // The first query and length go out in front of the first tiles (results come back in the order of the
    // requests: behind the tiles they would be held up until the last tile is in).
    const int64_t first_len64 = loadIndex<Tindex>(a.seq_lens, seq0);
    requestQuery(seq0, q_reg);
    // Speculative first tiles. The page ids of this piece are one more dependent round trip away (lengths ->
    // prefix sums -> table entries -> tiles), during which the memory system would idle. The calls of one
    // decoding step (one per layer) see the same lengths and block table, so the kLead tiles the pipeline
    // starts with are most likely where they were in the previous call: they are requested now, from the
    // (page, row) pairs that call left in the workspace, next to the table entries. When the entries arrive
    // the guess is checked against them; tiles guessed right are used as they are, a wrong guess (another
    // batch, a workspace never used before: any bit pattern, forced into the pool before it is used as an
    // address) costs the bandwidth of the tiles and nothing else: their slots of the pipeline are skipped.
    int guess_page[kLead], guess_row[kLead];
#pragma unroll
    for (int i = 0; i < kLead; ++i) {
        guess_page[i] = __builtin_amdgcn_readfirstlane(guess[2 * i]);
        guess_row[i] = __builtin_amdgcn_readfirstlane(guess[2 * i + 1]);
        const int page = clampPage(guess_page[i], a.num_blocks);
        const int row0 = guess_row[i] & block_mask & ~(kTileTokens - 1);
        const char *k_tile = k_head + (page * a.k_batch_stride + row0 * a.k_row_stride) * static_cast<int64_t>(sizeof(S));
        const char *v_tile = v_head + (page * a.v_batch_stride + row0 * a.v_row_stride) * static_cast<int64_t>(sizeof(S));
        buf[i] = loadTileRegs<HEAD>(k_tile, v_tile, off, 0xffffffffu);
    }
    // (all of them go out before anything below waits for the table entries: left alone, the scheduler moves the
    // first use of the entries, and with it the wait, up between the guessed tiles)
    __builtin_amdgcn_sched_barrier(0);
    // what the table says: only pieces whose first run is longer than kLead tiles take part (no run switch
    // inside the guessed tiles); the others leave an entry that matches nothing
    int true_page[kLead], true_row[kLead];
    bool guessed = ld_run.t1 - ld_run.t0 > kLead;
#pragma unroll
    for (int i = 0; i < kLead; ++i) {
        const int t = ld_run.t0 + (guessed ? i : 0);
        true_page[i] = clampPage(__builtin_amdgcn_readlane(ld_ids, (t >> tiles_per_entry_shift) - ld_run.first_entry), a.num_blocks);
        true_row[i] = guessed ? (t * kTileTokens) & block_mask : -1;
        guessed = guessed && true_page[i] == guess_page[i] && true_row[i] == guess_row[i];
    }
    if (guessed) {
        ld_t += kLead; // those tiles are on their way
    }
    const int dead_slots = guessed ? 0 : kLead;
    pinQuery();
    beginSegment(seq0, f0, clampLength(first_len64));
    // (slot s of the pipeline holds tile s - dead_slots of the piece; the slots of a wrong guess hold nothing)
    const int n_slots = n_flat + dead_slots;
    for (int t = 0; t < n_slots; t += NBUF) {
#pragma unroll
        for (int i = 0; i < NBUF; ++i) {
            buf[(i + NBUF - 1) % NBUF] = loadNextTile();
            if (t + i < n_slots && t + i >= dead_slots) {
                computeNextTile(buf[i]);
            }
        }
    }
    // the piece's last segment, then the parked one
    {
        const bool begins = c_t_begin == 0, ends = c_seg_end == c_seq_tiles;
        if (FUSED && !begins && ends) {
            parkReaderSegment();
        } else if (FUSED && !ends) {
            publishSegment(st, sumAcrossTokenGroups(st.l), c_seq);
        } else {
            writeResult(st, sumAcrossTokenGroups(st.l), c_seq, begins && ends);
        }
    }
    if (stash_seq >= 0) {
        flushStash();
    }
    // where this piece's first tiles were, for the next call on this workspace
    if (lane < 2 * kLead) {
        int word = 0;
#pragma unroll
        for (int i = 0; i < kLead; ++i) {
            word = lane == 2 * i ? true_page[i] : (lane == 2 * i + 1 ? true_row[i] : word);
        }
        my_first_tiles[lane] = word;
    }
    if constexpr (FUSED) {
        if (reader_seq < 0) {
            return;
        }
        // ---- reader: merge the earlier segments of sequence reader_seq into the parked state ----
        const int s = reader_seq;
        const int first_piece = pieceOf(seqFirstTile(s) + kStartCost * (s + 1)); // piece of the sequence's first tile
        const int count = piece - first_piece;                                // earlier segments, >= 1
        const int64_t flag_stride = streams;
        unsigned long long *flags = a.seg_flags + static_cast<int64_t>(first_piece + s) * flag_stride + stream;
        bool arrived = true;
        for (int base = 0; base < count && arrived; base += 64) {
            const int idx = base + lane;
            int spins = 0;
            while (true) {
                const unsigned long long v = idx < count ? loadAgent(flags + idx * flag_stride) : a.token;
                if (__builtin_amdgcn_ballot_w64(v != a.token) == 0) {
                    break;
                }
                __builtin_amdgcn_s_sleep(1);
                if (++spins > kReaderSpinLimit) {
                    arrived = false; // not with in-order dispatch; never spin for ever
                    break;
                }
            }
        }
        compilerMemoryBarrier(); // the row loads below stay below the flag loads above
        // A wait that ran out must not pass for a result: the rows of this sequence are then stored as NaN
        // (and the flags cleared like any others, so that the next call starts clean).
        const int merged = arrived ? count : 0;
        const float poison = arrived ? 1.0f : __builtin_nanf("");
        if (heads_here <= 4) {
            // Up to four heads (the usual GQA ratios): the rows of a segment are heads_here x HEAD floats, and spread
            // over all 64 lanes as 16-byte chunks (lane l: chunks l, l + 64, ... of the segment, 1 KiB per load
            // instruction) they are few enough registers that eight segments are in flight at once - one round trip
            // for most sequences, where the row-per-lane-group form below needs one per four segments and keeps the
            // three lane groups without a real head idle. Chunk id of a segment = head x HEAD / 4 + q, and chunk q
            // of a row holds accumulators 4 (q / 16) .. + 3 of lane q % 16 (publishSegment); the parked state of
            // this wavefront's own segment is read from LDS in the same order, merged, and written back.
            constexpr int kChunksPerRow = HEAD / 4;
            constexpr int kMine = 4 * kChunksPerRow / 64; // chunks of a lane: 1 .. 4
            constexpr int kBatch = 8;                     // segments per round trip
            int head_of[kMine], stash_at[kMine];
            float4 mine[kMine];
            float m_run[kMine], l_run[kMine];
#pragma unroll
            for (int k = 0; k < kMine; ++k) {
                const int id = lane + 64 * k;
                head_of[k] = id / kChunksPerRow;
                const int q = id - head_of[k] * kChunksPerRow;
                stash_at[k] = (4 * (4 * (q >> 4)) + head_of[k]) * 64 + (q & 15); // accumulator 4 (q / 16), row head, lane q % 16
                mine[k] = make_float4(reader_stash[stash_at[k]], reader_stash[stash_at[k] + 4 * 64],
                                      reader_stash[stash_at[k] + 8 * 64], reader_stash[stash_at[k] + 12 * 64]);
                l_run[k] = reader_stash[(4 * G::kCols) * 64 + head_of[k]];
                m_run[k] = reader_stash[(4 * G::kCols + 1) * 64 + head_of[k]];
            }
            for (int i0 = 0; i0 < merged; i0 += kBatch) {
                float2 ml[kBatch][kMine];
                float4 v[kBatch][kMine];
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const int i = min(i0 + j, count - 1); // past the end: the last one again, merged with weight 0
                    const auto rows = rowsOf(first_piece + i + s);
                    const auto pairs = pairsOf(first_piece + i + s);
#pragma unroll
                    for (int k = 0; k < kMine; ++k) { // (chunks and pairs of heads beyond heads_here lie beyond the buffers: zeros)
                        ml[j][k] = loadAgent8(pairs, 8 * head_of[k]);
                        v[j][k] = loadAgent16(rows, 16 * (lane + 64 * k));
                    }
                }
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const bool real = i0 + j < count;
#pragma unroll
                    for (int k = 0; k < kMine; ++k) {
                        const float m_i = real ? ml[j][k].x : -INFINITY;
                        const float m_new = fmaxf(m_run[k], m_i);
                        const float w_old = mergeWeight(m_run[k], m_new), w_i = mergeWeight(m_i, m_new);
                        l_run[k] = l_run[k] * w_old + (real ? ml[j][k].y : 0.0f) * w_i;
                        mine[k].x = mine[k].x * w_old + v[j][k].x * w_i;
                        mine[k].y = mine[k].y * w_old + v[j][k].y * w_i;
                        mine[k].z = mine[k].z * w_old + v[j][k].z * w_i;
                        mine[k].w = mine[k].w * w_old + v[j][k].w * w_i;
                        m_run[k] = m_new;
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < kMine; ++k) {
                if (head_of[k] < heads_here) {
                    reader_stash[stash_at[k]] = mine[k].x;
                    reader_stash[stash_at[k] + 4 * 64] = mine[k].y;
                    reader_stash[stash_at[k] + 8 * 64] = mine[k].z;
                    reader_stash[stash_at[k] + 12 * 64] = mine[k].w;
                    if (lane + 64 * k == head_of[k] * kChunksPerRow) { // the lane with the head's first chunk
                        reader_stash[(4 * G::kCols) * 64 + head_of[k]] = l_run[k];
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // the merged state is in LDS before the lanes read each other's
            if (g == 0) { // the lanes that hold the (up to four) real heads
                TileState<HEAD> merged_state;
#pragma unroll
                for (int e = 0; e < G::kCols; ++e) {
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        merged_state.o[e][rr] = reader_stash[(4 * e + rr) * 64 + lane];
                    }
                }
#pragma unroll
                for (int rr = 0; rr < 4; ++rr) {
                    if (rr < heads_here) {
                        const float l_head = reader_stash[(4 * G::kCols) * 64 + rr];
                        S *o_ptr = static_cast<S *>(a.out) + s * a.o_stride + (first_head + rr) * a.o_head_stride;
                        storeOutputRow<T, HEAD>(o_ptr, c, merged_state, rr, poison / (l_head + 1e-6f));
                    }
                }
            }
        } else {
        TileState<HEAD> own;
#pragma unroll
        for (int e = 0; e < G::kCols; ++e) {
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                own.o[e][rr] = reader_stash[(4 * e + rr) * 64 + lane];
            }
        }
        const float own_l = reader_stash[(4 * G::kCols) * 64 + lane];
        const float own_m = reader_stash[(4 * G::kCols + 1) * 64 + lane];
        float m_run[4], l_run[4];
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            l_run[rr] = __shfl(own_l, 4 * g + rr, 64);
            m_run[rr] = __shfl(own_m, 4 * g + rr, 64);
        }
        if (4 * g < heads_here) { // lanes that hold at least one real head
            constexpr int kBatch = 4; // segments per round trip
            for (int i0 = 0; i0 < merged; i0 += kBatch) {
                float2 ml[kBatch][4];
                float4 v[kBatch][4][G::kCols / 4];
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const int i = min(i0 + j, count - 1); // past the end: the last one again, merged with weight 0
                    const auto rows = rowsOf(first_piece + i + s);
                    const auto pairs = pairsOf(first_piece + i + s);
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        ml[j][rr] = loadAgent8(pairs, 8 * (4 * g + rr));
#pragma unroll
                        for (int h = 0; h < G::kCols / 4; ++h) {
                            v[j][rr][h] = loadAgent16(rows, (4 * g + rr) * HEAD * 4 + 256 * h + 16 * c);
                        }
                    }
                }
#pragma unroll
                for (int j = 0; j < kBatch; ++j) {
                    const bool real = i0 + j < count;
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr) {
                        const float m_i = real ? ml[j][rr].x : -INFINITY;
                        const float m_new = fmaxf(m_run[rr], m_i);
                        const float w_old = mergeWeight(m_run[rr], m_new), w_i = mergeWeight(m_i, m_new);
                        l_run[rr] = l_run[rr] * w_old + (real ? ml[j][rr].y : 0.0f) * w_i;
#pragma unroll
                        for (int h = 0; h < G::kCols / 4; ++h) {
                            own.o[4 * h][rr] = own.o[4 * h][rr] * w_old + v[j][rr][h].x * w_i;
                            own.o[4 * h + 1][rr] = own.o[4 * h + 1][rr] * w_old + v[j][rr][h].y * w_i;
                            own.o[4 * h + 2][rr] = own.o[4 * h + 2][rr] * w_old + v[j][rr][h].z * w_i;
                            own.o[4 * h + 3][rr] = own.o[4 * h + 3][rr] * w_old + v[j][rr][h].w * w_i;
                        }
                        m_run[rr] = m_new;
                    }
                }
            }
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                if (4 * g + rr < heads_here) {
                    S *o_ptr = static_cast<S *>(a.out) + s * a.o_stride + (first_head + 4 * g + rr) * a.o_head_stride;
                    storeOutputRow<T, HEAD>(o_ptr, c, own, rr, poison / (l_run[rr] + 1e-6f));
                }
            }
        }
        }
        // the flags are consumed: clear them, so that a replay of this call (same token) starts clean
        for (int base = 0; base < count; base += 64) {
            const int idx = base + lane;
            if (idx < count) {
                flags[idx * flag_stride] = 0;
            }
        }
    }
}

// Merge of the segment rows of one (query head, sequence); see decode_reduce.h for the arithmetic.
// One wavefront per (head, sequence), four of them per workgroup. Lane = (row group g = lane / 16,
// strip of HEAD/16 columns c = lane % 16): row group g merges rows g, g+4, ... of the sequence, the four
// groups are then combined with lane swaps, and the lanes of group 0 store 16 bytes each. The piece
// range of the sequence was left in seq_pieces by the decode kernel, so the only dependent memory
// round trips are {length, piece range} -> rows (one trip for up to eight segments).
template <typename T, typename Tindex, int HEAD>
__global__ void __launch_bounds__(256)
decodeBalancedMergeKernel(const void *early_seq_lens, const int2 *early_seq_pieces, int early_num_heads, DecodeArgs a) {
    using S = typename T::storage;
    constexpr int kCols = TileGeometry<HEAD>::kCols;
    const int head = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int seq = blockIdx.y;
    const int lane = threadIdx.x & 63;
    const int c = lane & 15;
    const int g = lane >> 4;
    // (the early arguments repeat a.seq_lens, a.seq_pieces and a.num_heads: see decodeBalancedKernel)
    if (head >= early_num_heads) {
        return;
    }
    const int64_t len64 = loadIndex<Tindex>(early_seq_lens, seq);
    const int2 pieces = early_seq_pieces[seq]; // written by the decode kernel for every sequence with tokens
    if (len64 <= 0 || pieces.y <= 1) {
        return; // no tokens, or one segment covered the whole sequence and wrote `out` itself
    }
    const int piece_first = pieces.x;
    const int parts = pieces.y;

    float m_loc = -INFINITY, l_loc = 0.0f;
    float acc[kCols];
#pragma unroll
    for (int i = 0; i < kCols; ++i) {
        acc[i] = 0.0f;
    }
    // Two rows per row group are requested before either is used, so that a sequence of up to eight
    // segments costs one memory round trip, not two. A row past the sequence's last segment re-reads
    // segment 0 (written, finite) and enters with weight 0.
    for (int p0 = 0; p0 < parts; p0 += 8) {
        float m_p[2], l_p[2];
        float4 v[2][kCols / 4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int p = p0 + 4 * j + g;
            const bool real = p < parts;
            const int64_t slot = static_cast<int64_t>(piece_first + (real ? p : 0) + seq) * a.num_heads + head;
            const float m_row = a.part_m[slot];
            const float l_row = a.part_l[slot];
            const float4 *row = reinterpret_cast<const float4 *>(a.part_acc + slot * HEAD + kCols * c);
#pragma unroll
            for (int i = 0; i < kCols / 4; ++i) {
                v[j][i] = row[i];
            }
            m_p[j] = real ? m_row : -INFINITY;
            l_p[j] = real ? l_row : 0.0f;
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const float m_new = fmaxf(m_loc, m_p[j]);
            const float w_old = mergeWeight(m_loc, m_new), w_p = mergeWeight(m_p[j], m_new);
            l_loc = l_loc * w_old + l_p[j] * w_p;
#pragma unroll
            for (int i = 0; i < kCols / 4; ++i) {
                acc[4 * i + 0] = acc[4 * i + 0] * w_old + v[j][i].x * w_p;
                acc[4 * i + 1] = acc[4 * i + 1] * w_old + v[j][i].y * w_p;
                acc[4 * i + 2] = acc[4 * i + 2] * w_old + v[j][i].z * w_p;
                acc[4 * i + 3] = acc[4 * i + 3] * w_old + v[j][i].w * w_p;
            }
            m_loc = m_new;
        }
    }
    const float m_all = swapMax(m_loc);
    const float f = mergeWeight(m_loc, m_all);
    const float l_all = swapSum(l_loc * f);
#pragma unroll
    for (int i = 0; i < kCols; ++i) {
        acc[i] = swapSum(acc[i] * f);
    }
    if (g == 0) {
        const float inv_l = 1.0f / (l_all + 1e-6f);
        uint32_t w[kCols / 2];
#pragma unroll
        for (int i = 0; i < kCols / 2; ++i) {
            w[i] = T::pack2(acc[2 * i] * inv_l, acc[2 * i + 1] * inv_l);
        }
        S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + head * a.o_head_stride;
        storeStrip<HEAD>(o_ptr, c, w);
    }
}

} // namespace op::paged_attention::amd

#endif
