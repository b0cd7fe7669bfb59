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
// weights. Accumulators are rescaled only when some head's maximum has outgrown the reference point by 2^8.
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

// (kTileTokens = 16 tokens per tile and kHeadsPerWave = 16 query heads per wavefront: decode_plan.h)
constexpr int kTiledHead = 128;     // the head size the kernels were tuned on (others: 64, 192, 256)
constexpr float kLazyRescaleLog2 = 8.0f; // how far (in powers of two) a maximum may outgrow its reference point

// Geometry of a 16-token tile for head_size = value_size = HEAD (64, 128, 192 or 256).
//   K: 16 rows of HEAD/8 16-byte chunks; the wavefront fetches them in kLoads = HEAD/32 instructions,
//      lane i of instruction j taking flat chunk 64 j + i (so every instruction covers whole rows when
//      rows are packed). In LDS row r keeps its chunks XOR-swizzled by (r mod kSwizzle).
//   V: lane (g, c) fetches rows 4g..4g+3, columns c*kCols .. c*kCols + kCols - 1 (kCols = HEAD/16, so
//      2*kCols bytes per row): the lane that loads a strip is the lane that feeds it to the matrix unit
//      and the lane that later owns those output columns.
template <int HEAD>
struct TileGeometry {
    static_assert(HEAD == 64 || HEAD == 128 || HEAD == 192 || HEAD == 256, "head sizes of the tiled kernels");
    static constexpr int kLoads = HEAD / 32;          // K load instructions per tile = K-steps of K.Q^T
    static constexpr int kChunksPerRow = HEAD / 8;    // 16-byte chunks in one K row
    static constexpr int kSwizzle = (HEAD == 64 || HEAD == 192) ? 8 : 16;
    static constexpr int kCols = HEAD / 16;           // V / output columns per lane
    static constexpr int kWords = kCols / 2;          // dwords of one V row strip
    // Which columns a lane's strip is made of: one contiguous piece (columns kCols c ..), except at head 192,
    // where the 24 bytes of a lane are two pieces - the 16-byte chunk c of columns 0 .. 127 and the four columns
    // from 128 + 4 c - so that the 16 lanes c = 0..15 of one load or store instruction cover one contiguous run
    // of a row. (As one 24-byte piece fetched 8 bytes at a time, every instruction touched every cache line of
    // the row three times over: 90.9 us at the Llama-3-8B batch-32 shape against 79.2 us with the two pieces.
    // Head 256, two adjacent 16-byte loads per lane, gains nothing from the same split: 105.0 vs 103.1 us.)
    static constexpr int kFirstCols = HEAD == 192 ? 8 : kCols;
    static constexpr int kRestCols = kCols - kFirstCols; // 4 at head 192, else 0
    static __host__ __device__ constexpr int firstColumn(int c) { return kFirstCols * c; }
    static __host__ __device__ constexpr int restColumn(int c) { return 128 + kRestCols * c; }
    // register sets: about 16 KiB of requests in flight per wavefront (12 KiB at head 192; a third set there
    // changes nothing: 92.0 vs 90.9 us before the strips were split)
    static constexpr int kBuffers = HEAD == 64 ? 5 : (HEAD >= 192 ? 2 : 3);
    static __device__ __forceinline__ int kRow(int j, int lane) { return (64 * j + lane) / kChunksPerRow; }
    static __device__ __forceinline__ int kChunk(int j, int lane) { return (64 * j + lane) % kChunksPerRow; }
    // position (in 16-byte units) of chunk `chunk` of row `row` in the LDS tile
    static __device__ __forceinline__ int ldsIndex(int row, int chunk) {
        return row * kChunksPerRow + (chunk ^ (row & (kSwizzle - 1)));
    }
};

// K and V rows of one 16-token tile as they come out of the global loads; kept in registers.
template <int HEAD>
struct TileRegs {
    uint4 k[TileGeometry<HEAD>::kLoads];        // k[j]: flat chunk 64 j + lane of the tile
    uint32_t v[4][TileGeometry<HEAD>::kWords];  // v[j]: token row 4g+j, columns c*kCols ..
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

// IEEE-754 maximum (a NaN operand gives NaN; v_maximum3_f32). fmaxf quiets its operands first, which for values
// the compiler cannot prove quiet (matrix-unit results, lane swaps) is one more vector instruction per operand and
// keeps three-operand forms from fusing: the maximum of 16 scores is 10 instructions this way and 27 with fmaxf.
__device__ __forceinline__ float maxOf(float a, float b) { return __builtin_elementwise_maximum(a, b); }

// 16 bytes per lane from global memory straight into LDS, without a register in between (global_load_lds_dwordx4):
// lane i of the wavefront writes the 16 bytes at lds_base + 16 i (lds_base is the same for all lanes, it travels in
// M0); lanes that are switched off write nothing. The data is in LDS when the wavefront's vector-memory counter has
// counted the instruction off: the caller waits for that (s_waitcnt vmcnt) before anybody reads the bytes.
// Written as assembly on purpose. Through the compiler's builtin the instruction is known to write LDS, and every
// LDS read that follows - of any LDS address: the pass that places the waits cannot tell the buffers of a
// double-buffered tile apart - is preceded by a wait for all of these loads, which serialises the loads of the
// next tile with the arithmetic on the current one.
// Source as (wave-uniform base, 32-bit lane offset) or as a pointer per lane.
// The statements write M0 and say so in their clobber lists, so that the compiler never carries a value of its
// own in M0 across them (it uses M0 for indexed register moves, lane reads and messages). M0 is a register the
// compiler reserves, for which it warns about any clobber; the clobber is still recorded on the statement.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// ONCE: the non-temporal form, for tiles that no other workgroup asks for (where two workgroups share a tile through
// L2 it loses what the second one would have found there: latent decode with 128 heads in two workgroups 66.8 vs
// 60.1 us; one workgroup per tile: 2.5 - 5.5 % faster).
template <bool ONCE = false>
__device__ __forceinline__ void loadLane16ToLds(const char *uniform_base, uint32_t lane_offset, uint4 *lds_base) {
    const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void *)lds_base));
    if constexpr (ONCE) {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                     :: "v"(lane_offset), "s"(uniform_base), "s"(lds_address) : "memory", "m0");
    } else {
        asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                     :: "v"(lane_offset), "s"(uniform_base), "s"(lds_address) : "memory", "m0");
    }
}
// the same with the lanes of `lanes` only (an EXEC mask: all ones, or zero for an instruction that does nothing)
template <bool ONCE = false>
__device__ __forceinline__ void loadLane16ToLdsMasked(const char *uniform_base, uint32_t lane_offset, uint4 *lds_base,
                                                      unsigned long long lanes) {
    const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void *)lds_base));
    unsigned long long saved;
    if constexpr (ONCE) {
        asm volatile("s_mov_b32 m0, %3\n\ts_and_saveexec_b64 %0, %4\n\tglobal_load_lds_dwordx4 %1, %2 nt\n\ts_mov_b64 exec, %0"
                     : "=&s"(saved) : "v"(lane_offset), "s"(uniform_base), "s"(lds_address), "s"(lanes) : "memory", "scc", "m0");
    } else {
        asm volatile("s_mov_b32 m0, %3\n\ts_and_saveexec_b64 %0, %4\n\tglobal_load_lds_dwordx4 %1, %2\n\ts_mov_b64 exec, %0"
                     : "=&s"(saved) : "v"(lane_offset), "s"(uniform_base), "s"(lds_address), "s"(lanes) : "memory", "scc", "m0");
    }
}
template <bool ONCE = false>
__device__ __forceinline__ void loadLane16ToLds(const char *lane_pointer, uint4 *lds_base) {
    const uint32_t lds_address = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) void *)lds_base));
    if constexpr (ONCE) {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off nt"
                     :: "v"(lane_pointer), "s"(lds_address) : "memory", "m0");
    } else {
        asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                     :: "v"(lane_pointer), "s"(lds_address) : "memory", "m0");
    }
}
#pragma clang diagnostic pop

// max over the four lanes {c, c+16, c+32, c+48}; every one of them gets the result (two lane swaps,
// no LDS traffic)
__device__ __forceinline__ float maxAcrossTokenGroups(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = maxOf(__uint_as_float(r[0]), __uint_as_float(r[1]));
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return maxOf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sumAcrossTokenGroups(float x) {
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    u32x2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    x = __uint_as_float(r[0]) + __uint_as_float(r[1]);
    r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
    return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// 8-byte flavour of loadLane16, for row strips that are not a multiple of 16 bytes
__device__ __forceinline__ uint2 loadLane8(const char *uniform_base, uint32_t lane_offset) {
    asm volatile("" : "+v"(lane_offset));
    typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(uniform_base + lane_offset));
    return make_uint2(v[0], v[1]);
}
// and the 4-byte one (two columns)
__device__ __forceinline__ uint32_t loadLane4(const char *uniform_base, uint32_t lane_offset) {
    asm volatile("" : "+v"(lane_offset));
    return __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(uniform_base + lane_offset));
}

// This lane's strip of one V row: the first piece at uniform_base + first_offset, the rest piece (heads above
// 128) at uniform_base + rest_offset; 16-byte loads, 8-byte ones for pieces of four columns
template <int HEAD>
__device__ __forceinline__ void loadStrip(const char *uniform_base, uint32_t first_offset, uint32_t rest_offset,
                                          uint32_t (&w)[TileGeometry<HEAD>::kWords]) {
    using G = TileGeometry<HEAD>;
    static_assert(G::kFirstCols % 8 == 0 || G::kFirstCols == 4, "16-byte loads, or one 8-byte load");
    static_assert(G::kRestCols == 0 || G::kRestCols == 4, "the rest piece is one 8-byte load");
    if constexpr (G::kFirstCols % 8 == 0) {
#pragma unroll
        for (int i = 0; i < G::kFirstCols / 8; ++i) {
            const uint4 x = loadLane16(uniform_base, first_offset + 16 * i);
            w[4 * i] = x.x, w[4 * i + 1] = x.y, w[4 * i + 2] = x.z, w[4 * i + 3] = x.w;
        }
    } else {
        const uint2 x = loadLane8(uniform_base, first_offset);
        w[0] = x.x, w[1] = x.y;
    }
    if constexpr (G::kRestCols == 4) {
        const uint2 x = loadLane8(uniform_base, rest_offset);
        w[G::kFirstCols / 2] = x.x, w[G::kFirstCols / 2 + 1] = x.y;
    }
}

// The kCols output values of strip c of one row, packed two per dword, into the row that starts at `row`
// (the pieces of TileGeometry: 16-byte stores, 8-byte ones for pieces of four columns)
template <int HEAD, typename S>
__device__ __forceinline__ void storeStrip(S *row, int c, const uint32_t (&w)[TileGeometry<HEAD>::kWords]) {
    using G = TileGeometry<HEAD>;
    static_assert(sizeof(S) == 2, "two values per dword");
    if constexpr (G::kFirstCols % 8 == 0) {
#pragma unroll
        for (int i = 0; i < G::kFirstCols / 8; ++i) {
            reinterpret_cast<uint4 *>(row + G::firstColumn(c))[i] = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
        }
    } else {
        *reinterpret_cast<uint2 *>(row + G::firstColumn(c)) = make_uint2(w[0], w[1]);
    }
    if constexpr (G::kRestCols == 4) {
        *reinterpret_cast<uint2 *>(row + G::restColumn(c)) = make_uint2(w[G::kFirstCols / 2], w[G::kFirstCols / 2 + 1]);
    }
}

// Softmax state of one wavefront. o[e][r] = O[head 4g+r of the chunk][column e of strip c (TileGeometry)].
template <int HEAD>
struct TileState {
    f32x4 o[TileGeometry<HEAD>::kCols];
    float m; // running maximum of head c (same value in the four lanes g = 0..3)
    float l; // sum of rounded probabilities of head c over this lane's tokens only
};

// Row rr of the accumulators, scaled, rounded to the storage dtype and written into the output row at `row`
template <typename T, int HEAD>
__device__ __forceinline__ void storeOutputRow(typename T::storage *row, int c, const TileState<HEAD> &st, int rr, float factor) {
    uint32_t w[TileGeometry<HEAD>::kWords];
#pragma unroll
    for (int i = 0; i < TileGeometry<HEAD>::kWords; ++i) {
        w[i] = T::pack2(st.o[2 * i][rr] * factor, st.o[2 * i + 1][rr] * factor);
    }
    storeStrip<HEAD>(row, c, w);
}

// Row rr of the accumulators as fp32 partial result in column order, into the partial row at `row` (what the
// merge kernels of the fixed partitions read: value_size floats per row)
template <int HEAD>
__device__ __forceinline__ void storePartialRowInColumnOrder(float *row, int c, const TileState<HEAD> &st, int rr) {
    using G = TileGeometry<HEAD>;
#pragma unroll
    for (int i = 0; i < G::kFirstCols / 4; ++i) {
        reinterpret_cast<float4 *>(row + G::firstColumn(c))[i] = make_float4(st.o[4 * i][rr], st.o[4 * i + 1][rr], st.o[4 * i + 2][rr], st.o[4 * i + 3][rr]);
    }
#pragma unroll
    for (int i = 0; i < G::kRestCols / 4; ++i) {
        const int e = G::kFirstCols + 4 * i;
        reinterpret_cast<float4 *>(row + G::restColumn(c))[i] = make_float4(st.o[e][rr], st.o[e + 1][rr], st.o[e + 2][rr], st.o[e + 3][rr]);
    }
}

// Row rr of the accumulators as fp32 partial result, the lane's kCols floats side by side at dst (16-byte
// aligned; the layout of the work-equalising schedule, whose merge reads the rows the same way)
template <int HEAD>
__device__ __forceinline__ void storePartialRow(float *dst, const TileState<HEAD> &st, int rr) {
#pragma unroll
    for (int i = 0; i < TileGeometry<HEAD>::kCols / 4; ++i) {
        reinterpret_cast<float4 *>(dst)[i] = make_float4(st.o[4 * i][rr], st.o[4 * i + 1][rr], st.o[4 * i + 2][rr], st.o[4 * i + 3][rr]);
    }
}

// Online-softmax step of one tile. s = raw scores of head c for tokens 4g..4g+3 of the tile; rel_pos0 =
// position of the tile's first token relative to the last token of the sequence (ALiBi distance);
// `valid` = tokens of the tile that belong to the sequence (16 except possibly in the last tile).
// Updates the running maximum m, the denominator l and rescales the accumulators o when some head's
// maximum moved; returns the probabilities as the A operand of P.V.
//
// The matrix instruction takes the probabilities in the storage dtype; fp16 keeps 11 significant bits
// of a value in [0, 1], bf16 only 8. For bf16 the probability is therefore fed as two terms,
// p = hi + lo with lo = bf16(p - hi), and P.V takes two matrix instructions per output tile: the
// product then carries ~16 bits of p, close to the fp32 probabilities of the reference kernel. The
// denominator sums exactly what the numerator used.
template <typename T, int COLS>
__device__ __forceinline__ void softmaxStep(f32x4 (&o)[COLS], float &m, float &l, const f32x4 s, int g, float scale_log2,
                                            float slope, int rel_pos0, int valid, uint2 &p_op, uint2 &p_lo) {
    const bool tail = valid < kTileTokens;
    float sc[4];
#pragma unroll
    for (int rr = 0; rr < 4; ++rr) {
        sc[rr] = s[rr] * scale_log2 + slope * static_cast<float>(rel_pos0 + 4 * g + rr);
        sc[rr] = (tail && 4 * g + rr >= valid) ? -INFINITY : sc[rr];
    }
    // this lane's four tokens; a head's maximum is the largest of its four lanes' (c, c + 16, c + 32, c + 48) and
    // is only formed when it is needed
    const float mx_lane = maxOf(maxOf(sc[0], sc[1]), maxOf(sc[2], sc[3]));

    // m only has to keep the exponentials in range, it need not be the exact maximum: it is moved (and the
    // accumulators rescaled) only when some head's maximum has outgrown it by more than 2^kLazyRescaleLog2,
    // so a probability reaches at most that factor above 1. Numerator and denominator carry the same
    // reference point, the quotient is unchanged, and the partial results stay mergeable as they are.
    if (__builtin_amdgcn_ballot_w64(mx_lane > m + kLazyRescaleLog2) != 0) { // some lane's maximum, hence some head's
        const float m_new = maxOf(m, maxAcrossTokenGroups(mx_lane));
        // rescale. Lane holds accumulators of heads 4g..4g+3, whose factors live in lanes 4g..4g+3.
        const float alpha = fastExp2(m - m_new);
        l *= alpha;
        m = m_new;
#pragma unroll
        for (int rr = 0; rr < 4; ++rr) {
            const float alpha_r = __shfl(alpha, 4 * g + rr, 64);
#pragma unroll
            for (int e = 0; e < COLS; ++e) {
                o[e][rr] *= alpha_r;
            }
        }
    }

    const float p0 = fastExp2(sc[0] - m), p1 = fastExp2(sc[1] - m);
    const float p2 = fastExp2(sc[2] - m), p3 = fastExp2(sc[3] - m);
    p_op.x = T::pack2(p0, p1);
    p_op.y = T::pack2(p2, p3);
    float p_used = (T::unpackLo(p_op.x) + T::unpackHi(p_op.x)) + (T::unpackLo(p_op.y) + T::unpackHi(p_op.y));
    if constexpr (T::kSplitProbabilities) {
        p_lo.x = T::pack2(p0 - T::unpackLo(p_op.x), p1 - T::unpackHi(p_op.x));
        p_lo.y = T::pack2(p2 - T::unpackLo(p_op.y), p3 - T::unpackHi(p_op.y));
        p_used += (T::unpackLo(p_lo.x) + T::unpackHi(p_lo.x)) + (T::unpackLo(p_lo.y) + T::unpackHi(p_lo.y));
    }
    l += p_used;
}

// O += P . V for two adjacent output columns: v0..v3 hold those two columns of token rows 4g..4g+3
// (one dword per row). V rows beyond the sequence may hold anything (NaN included) and 0 * NaN is
// NaN: they are zeroed.
template <typename T>
__device__ __forceinline__ void accumulatePair(f32x4 &o_even, f32x4 &o_odd, uint32_t v0, uint32_t v1, uint32_t v2,
                                               uint32_t v3, const uint2 p_op, const uint2 p_lo, int g, int valid) {
    if (valid < kTileTokens) {
        v0 = (4 * g + 0 >= valid) ? 0u : v0;
        v1 = (4 * g + 1 >= valid) ? 0u : v1;
        v2 = (4 * g + 2 >= valid) ? 0u : v2;
        v3 = (4 * g + 3 >= valid) ? 0u : v3;
    }
    uint2 even, odd;
    even.x = __builtin_amdgcn_perm(v1, v0, 0x05040100u);
    even.y = __builtin_amdgcn_perm(v3, v2, 0x05040100u);
    odd.x = __builtin_amdgcn_perm(v1, v0, 0x07060302u);
    odd.y = __builtin_amdgcn_perm(v3, v2, 0x07060302u);
    o_even = T::mfmaK16(p_op, even, o_even);
    o_odd = T::mfmaK16(p_op, odd, o_odd);
    if constexpr (T::kSplitProbabilities) {
        o_even = T::mfmaK16(p_lo, even, o_even);
        o_odd = T::mfmaK16(p_lo, odd, o_odd);
    }
}

// One tile: scores, online softmax, accumulate.
template <typename T, int HEAD>
__device__ __forceinline__ void computeTile(TileState<HEAD> &st, const TileRegs<HEAD> r,
                                            const uint4 (&q_reg)[TileGeometry<HEAD>::kLoads], uint4 *k_lds, int lane,
                                            int c, int g, float scale_log2, float slope, int rel_pos0, int valid) {
    using G = TileGeometry<HEAD>;
    // K: registers -> swizzled LDS -> matrix-operand layout (token c, columns 32*kk + 8g .. +7)
#pragma unroll
    for (int j = 0; j < G::kLoads; ++j) {
        k_lds[G::ldsIndex(G::kRow(j, lane), G::kChunk(j, lane))] = r.k[j];
    }
    __builtin_amdgcn_wave_barrier();
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < G::kLoads; ++kk) {
        s = T::mfmaK32(k_lds[G::ldsIndex(c, 4 * kk + g)], q_reg[kk], s);
    }
    __builtin_amdgcn_wave_barrier();

    uint2 p_op, p_lo = make_uint2(0, 0);
    softmaxStep<T, G::kCols>(st.o, st.m, st.l, s, g, scale_log2, slope, rel_pos0, valid, p_op, p_lo);

    // one 16-column output tile per e: column e of strip c, rows 4g..4g+3
#pragma unroll
    for (int w = 0; w < G::kWords; ++w) {
        accumulatePair<T>(st.o[2 * w], st.o[2 * w + 1], r.v[0][w], r.v[1][w], r.v[2][w], r.v[3][w], p_op, p_lo, g, valid);
    }
}

// Software pipeline over the tiles of one run. NBUF register sets rotate; NBUF-1 tiles are always
// in flight while one is computed. The body has no branch around a load, so the compiler counts
// outstanding loads exactly and each tile waits only for its own data. loadTile() must accept any
// index (it neutralises indices past the end); compute() is skipped for those.
template <int NBUF, typename Load, typename Compute>
__device__ __forceinline__ void streamTiles(int n_tiles, Load loadTile, Compute compute) {
    decltype(loadTile(0)) buf[NBUF];
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

// Byte offsets of a lane's pieces inside a tile. They do not change from tile to tile, so a tile's
// loads are "wave-uniform tile address + constant lane offset" and need no per-tile vector address
// arithmetic.
template <int HEAD>
struct LaneOffsets {
    uint32_t k[TileGeometry<HEAD>::kLoads];
    uint32_t v[4];       // first piece of the strip of token row 4g + j
    uint32_t v_rest;     // from there to the rest piece of the same row (heads above 128)
    __device__ __forceinline__ LaneOffsets(int lane, uint32_t k_row_bytes, uint32_t v_row_bytes) {
        using G = TileGeometry<HEAD>;
#pragma unroll
        for (int j = 0; j < G::kLoads; ++j) {
            k[j] = G::kRow(j, lane) * k_row_bytes + 16 * G::kChunk(j, lane);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[j] = (4 * (lane >> 4) + j) * v_row_bytes + 2 * G::firstColumn(lane & 15);
        }
        v_rest = 2 * (G::restColumn(lane & 15) - G::firstColumn(lane & 15));
    }
};

// The eight-plus loads of one tile. lane_mask = 0 turns them into harmless reads of the first bytes
// of the tile (all lanes the same address: one request instead of a tile's worth).
template <int HEAD>
__device__ __forceinline__ TileRegs<HEAD> loadTileRegs(const char *k_tile, const char *v_tile, const LaneOffsets<HEAD> &off,
                                                       uint32_t lane_mask) {
    TileRegs<HEAD> r;
#pragma unroll
    for (int j = 0; j < TileGeometry<HEAD>::kLoads; ++j) {
        r.k[j] = loadLane16(k_tile, off.k[j] & lane_mask);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        loadStrip<HEAD>(v_tile, off.v[j] & lane_mask, (off.v[j] + off.v_rest) & lane_mask, r.v[j]);
    }
    return r;
}

template <typename T, typename Tindex, int HEAD>
__global__ void __launch_bounds__(64) decodeTiledKernel(DecodeArgs a) {
    using S = typename T::storage;
    using G = TileGeometry<HEAD>;
    __shared__ uint4 k_lds[kTileTokens * G::kChunksPerRow]; // one K tile

    const int head_chunks = (a.group + kHeadsPerWave - 1) / kHeadsPerWave;
    const int kv_head = blockIdx.y / head_chunks;
    const int chunk = blockIdx.y - kv_head * head_chunks;
    const int seq = blockIdx.z;
    // Workgroups are dealt to the eight XCDs round-robin by linear index, which follows blockIdx.x when the
    // grid's x extent is a multiple of eight. Partition p of every sequence on the same XCD would load the
    // XCDs by how many sequences reach partition p, so the partitions of sequence s are rotated by s.
    const int part = static_cast<int>((blockIdx.x + blockIdx.z) % gridDim.x);
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

    // Query of head (chunk*16 + c), as the B operand of the K-steps: columns 32*kk + 8g .. +7.
    const int head_in_group = chunk * kHeadsPerWave + c;
    const bool head_valid = head_in_group < a.group;
    const int head = kv_head * a.group + head_in_group;
    uint4 q_reg[G::kLoads];
    {
        const S *q_ptr = static_cast<const S *>(a.q) + seq * a.q_stride + (head_valid ? head : 0) * a.q_head_stride;
#pragma unroll
        for (int kk = 0; kk < G::kLoads; ++kk) {
            q_reg[kk] = head_valid ? *reinterpret_cast<const uint4 *>(q_ptr + 32 * kk + 8 * g) : make_uint4(0, 0, 0, 0);
        }
    }
    const float slope = (a.alibi_slopes != nullptr && head_valid) ? a.alibi_slopes[head] * kLog2e : 0.0f;

    const char *k_head = reinterpret_cast<const char *>(static_cast<const S *>(a.k_cache) + kv_head * a.k_head_stride);
    const char *v_head = reinterpret_cast<const char *>(static_cast<const S *>(a.v_cache) + kv_head * a.v_head_stride);
    const int block_mask = a.block_size - 1;
    const LaneOffsets<HEAD> off(lane, static_cast<uint32_t>(a.k_row_stride) * sizeof(S),
                                static_cast<uint32_t>(a.v_row_stride) * sizeof(S));

    // The loop body is branch-free with a fixed number of loads in flight, so it also issues loads
    // for tile indices past the end of the partition. Those are made harmless: every lane reads the
    // same few bytes (the start of the partition's first tile).
    auto loadTile = [&](int t) -> TileRegs<HEAD> {
        const bool real = t < n_tiles;
        const uint32_t lane_mask = real ? 0xffffffffu : 0u;
        const int tok0 = start + (real ? t : 0) * kTileTokens;
        const int page = __builtin_amdgcn_readlane(page_ids, (tok0 >> a.block_shift) - first_entry);
        const int row0 = tok0 & block_mask;
        const char *k_tile = k_head + (page * a.k_batch_stride + row0 * a.k_row_stride) * static_cast<int64_t>(sizeof(S));
        const char *v_tile = v_head + (page * a.v_batch_stride + row0 * a.v_row_stride) * static_cast<int64_t>(sizeof(S));
        return loadTileRegs<HEAD>(k_tile, v_tile, off, lane_mask);
    };

    TileState<HEAD> st;
#pragma unroll
    for (int e = 0; e < G::kCols; ++e) {
        st.o[e] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    st.m = -INFINITY;
    st.l = 0.0f;

    auto compute = [&](int t, const TileRegs<HEAD> &r) {
        const int tok0 = start + t * kTileTokens;
        computeTile<T, HEAD>(st, r, q_reg, k_lds, lane, c, g, a.scale_log2, slope, tok0 - (len - 1),
                             min(kTileTokens, end - tok0));
    };

    streamTiles<G::kBuffers>(n_tiles, loadTile, compute);

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
            S *o_ptr = static_cast<S *>(a.out) + seq * a.o_stride + out_head * a.o_head_stride;
            storeOutputRow<T, HEAD>(o_ptr, c, st, rr, 1.0f / (l_h + 1e-6f));
        } else {
            const int64_t slot = (static_cast<int64_t>(seq) * a.num_heads + out_head) * a.max_partitions + part;
            storePartialRowInColumnOrder<HEAD>(a.part_acc + slot * HEAD, c, st, rr);
            if (c == 0) {
                a.part_m[slot] = m_h;
                a.part_l[slot] = l_h;
            }
        }
    }
}

} // namespace op::paged_attention::amd

#endif
