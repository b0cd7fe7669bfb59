// Rotary position embedding of the new K vectors fused with the scatter of K and V into the paged pool, on
// AMD Instinct (gfx950): one launch for what the reference runs as two operators with a tensor in between
// (rotation: src/infiniop/ops/rope/cuda/kernel.cuh:4-118, arithmetic as in src/infiniop/ops/rope/cpu/
// rope_cpu.cc:56-98; scatter: src/infiniop/ops/paged_caching/cuda/kernel.cuh:22-89).
//
// Like the plain scatter the kernel is written for memory transactions: a workgroup is a (units of a row) x
// (heads) x (tokens) box of 256 threads, a unit being 16 bytes. A thread that rotates takes the 16 bytes
// that hold the first elements of 16 / sizeof(element) pairs and the 16 bytes that hold their partners
// (neighbouring for GPT_J, half a vector away for GPT_NEOX), plus 16 bytes of each table, and writes two
// 16-byte units of the K page row; V units are copied. Operands whose sizes, strides or addresses are not
// multiples of 16 bytes take the same kernel with one pair / one element per step.
// The decode step (one token per sequence, e.g. 32 x 8 x 128: 128 KiB in all) is a launch and three dependent
// memory round trips long; fusing saves the second launch and the round trip of the rotated K through memory.
#include "rope_paged_caching_amd.h"
#include "../../../handle.h"
#include "../../../devices/amd/amd_streaming.h"
#include "../../../../utils/check.h"
#include <cstdint>
#include <hip/hip_runtime.h>

namespace op::rope_paged_caching::amd {

namespace {

struct Args {
    void *k_cache;
    void *v_cache;
    const void *k;
    const void *v;
    const int64_t *slot_mapping;
    const void *pos_ids;
    const void *sin_table;
    const void *cos_table;
    int64_t num_tokens;
    int64_t num_slots; // num_blocks * block_size; slots at or beyond it are ignored
    int64_t table_len;
    int32_t num_kv_heads;
    int32_t block_size;
    int32_t block_shift; // log2(block_size) when it is a power of two, else -1
    int32_t head_size;
    int32_t value_size;
    int32_t pos_bytes;   // 1, 2, 4 or 8
    int32_t pos_signed;
    int32_t neox;        // pairs half a vector apart (GPT_NEOX) or neighbouring (GPT_J)
    // element strides
    int64_t k_src_token_stride, v_src_token_stride;
    int64_t k_block_stride, k_head_stride, k_slot_stride;
    int64_t v_block_stride, v_head_stride, v_slot_stride;
};

// The query rotated in the same launch: a second argument block, which the kernels without a query do not carry
// (their argument block is then no longer than the scatter alone needs; a longer one costs them 9 % at 4 096 tokens).
template <bool QUERY>
struct QueryArgs {};
template <>
struct QueryArgs<true> {
    void *q_out;
    const void *q;
    int32_t num_q_heads;
    int32_t threads_per_row; // threads of a token's box that share one query vector (a power of two)
    int64_t q_token_stride, q_head_stride, q_out_token_stride, q_out_head_stride;
};

struct F16 {
    using storage = _Float16;
};
struct BF16 {
    using storage = __bf16;
};
struct F32 {
    using storage = float;
};

__device__ __forceinline__ int64_t loadPosition(const Args &a, int64_t i) {
    switch (a.pos_bytes) {
    case 1: return a.pos_signed ? static_cast<const int8_t *>(a.pos_ids)[i] : static_cast<const uint8_t *>(a.pos_ids)[i];
    case 2: return a.pos_signed ? static_cast<const int16_t *>(a.pos_ids)[i] : static_cast<const uint16_t *>(a.pos_ids)[i];
    case 4: return a.pos_signed ? static_cast<const int32_t *>(a.pos_ids)[i] : static_cast<const uint32_t *>(a.pos_ids)[i];
    default: {
        const int64_t p = static_cast<const int64_t *>(a.pos_ids)[i];
        return (!a.pos_signed && p < 0) ? INT64_MAX : p; // an unsigned value beyond 2^63: past any table
    }
    }
}

// One pair: every product and the sum rounded to fp32 on its own (no fused multiply-add), as the reference's CPU
// statement computes it, then one rounding to the storage dtype.
template <typename S>
__device__ __forceinline__ void rotatePair(S x0, S x1, S sin_, S cos_, S &y0, S &y1) {
#pragma clang fp contract(off)
    const float a = static_cast<float>(x0), b = static_cast<float>(x1);
    const float s = static_cast<float>(sin_), c = static_cast<float>(cos_);
    const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
    y0 = static_cast<S>(ac - bs);
    y1 = static_cast<S>(as + bc);
}

template <typename S>
struct Unit16 {
    static constexpr int kElements = 16 / sizeof(S);
    S e[kElements];
};

// One vector of 2 * table_dim elements rotated from src to dst (dst may be src: a thread reads both halves of its
// pairs before it writes them). VEC: 16-byte units (see the head of the file); else one pair per step.
template <typename S, bool VEC>
__device__ __forceinline__ void rotateRow(const S *src, S *dst, const S *sin_row, const S *cos_row, int table_dim, bool neox,
                                          int step0, int step) {
    using U = Unit16<S>;
    constexpr int kPer = U::kElements;
    if constexpr (VEC) {
        // unit u of the rotation covers pairs [u * kPer, (u + 1) * kPer)
        for (int u = step0; u < table_dim / kPer; u += step) {
            const int first = neox ? u * kPer : 2 * u * kPer;                 // elements of the first unit
            const int second = neox ? table_dim + u * kPer : 2 * u * kPer + kPer;
            const U x_lo = *reinterpret_cast<const U *>(src + first);
            const U x_hi = *reinterpret_cast<const U *>(src + second);
            const U sn = *reinterpret_cast<const U *>(sin_row + u * kPer);
            const U cs = *reinterpret_cast<const U *>(cos_row + u * kPer);
            U y_lo, y_hi;
            if (neox) {
#pragma unroll
                for (int i = 0; i < kPer; ++i) {
                    rotatePair(x_lo.e[i], x_hi.e[i], sn.e[i], cs.e[i], y_lo.e[i], y_hi.e[i]);
                }
            } else {
                // the 2 kPer elements are kPer neighbouring pairs: pair i = elements 2 i, 2 i + 1
#pragma unroll
                for (int i = 0; i < kPer / 2; ++i) {
                    rotatePair(x_lo.e[2 * i], x_lo.e[2 * i + 1], sn.e[i], cs.e[i], y_lo.e[2 * i], y_lo.e[2 * i + 1]);
                    rotatePair(x_hi.e[2 * i], x_hi.e[2 * i + 1], sn.e[kPer / 2 + i], cs.e[kPer / 2 + i], y_hi.e[2 * i],
                               y_hi.e[2 * i + 1]);
                }
            }
            device::amd::storeStreamed(dst + first, y_lo);
            device::amd::storeStreamed(dst + second, y_hi);
        }
    } else {
        for (int j = step0; j < table_dim; j += step) {
            const int first = neox ? j : 2 * j;
            const int second = neox ? j + table_dim : 2 * j + 1;
            S y0, y1;
            rotatePair(src[first], src[second], sin_row[j], cos_row[j], y0, y1);
            dst[first] = y0;
            dst[second] = y1;
        }
    }
}

// Thread box: x = steps along a row, y = heads (the KV heads first, then the query heads if the query is rotated
// too: QUERY), z = tokens.
template <typename T, bool VEC, bool QUERY>
__device__ __forceinline__ void ropeScatter(const Args &a, const QueryArgs<QUERY> &qa) {
    using S = typename T::storage;
    using U = Unit16<S>;
    constexpr int kPer = U::kElements;
    const int64_t token = static_cast<int64_t>(blockIdx.x) * blockDim.z + threadIdx.z;
    if (token >= a.num_tokens) {
        return;
    }
    // the box once, up front: read inside the loops below, its extents become a memory load per head
    const int x0 = threadIdx.x, x_step = blockDim.x, y0 = threadIdx.y, y_step = blockDim.y;
    const int64_t slot = a.slot_mapping[token];
    int64_t pos = loadPosition(a, token);
    // Negative = padding (paged_caching kernel.cuh:61-63). Slots past the pool would be an out-of-bounds
    // write in the reference; here they are dropped. The query of such a token is rotated all the same.
    const bool cached = slot >= 0 && slot < a.num_slots;
    int num_q_heads = 0;
    if constexpr (QUERY) {
        num_q_heads = qa.num_q_heads;
    }
    if (!cached && num_q_heads == 0) {
        return;
    }
    pos = pos < 0 ? 0 : (pos >= a.table_len ? a.table_len - 1 : pos);
    int64_t page, row;
    if (a.block_shift >= 0) {
        page = slot >> a.block_shift;
        row = slot & (a.block_size - 1);
    } else {
        page = slot / a.block_size;
        row = slot % a.block_size;
    }
    const int table_dim = a.head_size / 2;
    const S *sin_row = static_cast<const S *>(a.sin_table) + pos * table_dim;
    const S *cos_row = static_cast<const S *>(a.cos_table) + pos * table_dim;

    if constexpr (QUERY) {
        // The query first (its loads depend on nothing the cache writes need). The token's box of x * y threads is
        // dealt anew: as many threads per vector as the rotation has steps, the others on further heads, so that
        // e.g. 32 heads of 128 bf16 elements (8 steps each) are one round of a 256-thread box.
        const int flat = y0 * x_step + x0;
        const int heads_at_once = (x_step * y_step) / qa.threads_per_row;
        for (int q_head = flat / qa.threads_per_row; q_head < num_q_heads; q_head += heads_at_once) {
            rotateRow<S, VEC>(static_cast<const S *>(qa.q) + token * qa.q_token_stride + q_head * qa.q_head_stride,
                              static_cast<S *>(qa.q_out) + token * qa.q_out_token_stride + q_head * qa.q_out_head_stride,
                              sin_row, cos_row, table_dim, a.neox != 0, flat & (qa.threads_per_row - 1), qa.threads_per_row);
        }
        if (!cached) {
            return;
        }
    }
    for (int head = y0; head < a.num_kv_heads; head += y_step) {
        const S *k_src = static_cast<const S *>(a.k) + token * a.k_src_token_stride + static_cast<int64_t>(head) * a.head_size;
        const S *v_src = static_cast<const S *>(a.v) + token * a.v_src_token_stride + static_cast<int64_t>(head) * a.value_size;
        S *k_dst = static_cast<S *>(a.k_cache) + page * a.k_block_stride + head * a.k_head_stride + row * a.k_slot_stride;
        S *v_dst = static_cast<S *>(a.v_cache) + page * a.v_block_stride + head * a.v_head_stride + row * a.v_slot_stride;
        rotateRow<S, VEC>(k_src, k_dst, sin_row, cos_row, table_dim, a.neox != 0, x0, x_step);
        if constexpr (VEC) {
            for (int u = x0; u < a.value_size / kPer; u += x_step) {
                device::amd::storeStreamed(v_dst + u * kPer, *reinterpret_cast<const U *>(v_src + u * kPer));
            }
        } else {
            for (int j = x0; j < a.value_size; j += x_step) {
                v_dst[j] = v_src[j];
            }
        }
    }
}

template <typename T, bool VEC>
__global__ void __launch_bounds__(256) ropeScatterKernel(Args a) {
    ropeScatter<T, VEC, false>(a, QueryArgs<false>{});
}
template <typename T, bool VEC>
__global__ void __launch_bounds__(256) ropeScatterQueryKernel(Args a, QueryArgs<true> qa) {
    ropeScatter<T, VEC, true>(a, qa);
}

// ---- the kernel for operands made of 16-byte units (the usual case) ----
// The box kernel above spends a token's life waiting: position -> table rows -> stores are dependent round
// trips, and the bulk of the bytes (the vectors themselves) is only requested in the second. Here a workgroup of
// 256 threads takes a few whole tokens and treats their work as one flat list of items of two 16-byte units each -
// per token the rotate items of the query heads (the unit holding the first elements of its pairs and the unit
// holding their partners), those of the KV heads, then the copy items of V (two neighbouring units) - of which
// thread t takes items t, t + 256, ... (ITEMS of them, all in registers). Straight-line code, no branch around
// a load:
//   1. the first threads ask for position and slot of the workgroup's tokens, then every thread asks for the
//      units of all its items (none of these addresses depends on the position or the slot);
//   2. positions and slots go through LDS to everybody; every item asks for its 16 bytes of each table row
//      (copy items too: one instruction stream for all lanes);
//   3. rotate (copy items pass through), store: query items to q_out, KV items to the page row the slot names.
// So a token's bytes are in flight from the first round trip on and a thread holds ITEMS x 32 bytes of them.
struct FlatShape {
    int32_t items_per_token;  // (query heads + KV heads) x rotate_steps + KV heads x copy_steps
    int32_t q_items, k_items; // query heads x rotate_steps, KV heads x rotate_steps
    int32_t rotate_steps, copy_steps; // items of one rotated vector (table_dim / elements per unit), of one V row (units / 2)
    int32_t tokens_per_group; // whole tokens per workgroup
    uint32_t inv_items, inv_rotate, inv_copy; // ceil(2^32 / x): floor(n / x) = n * inv >> 32 for n, x < 2^16
};

constexpr int kFlatThreads = 256;
constexpr int kFlatMaxTokens = 16; // tokens of one workgroup (their positions and slots sit in LDS)

__device__ __forceinline__ int divideSmall(int n, uint32_t inverse) {
    return static_cast<int>(__umulhi(static_cast<uint32_t>(n), inverse));
}

template <typename T, bool QUERY, int ITEMS>
__global__ void __launch_bounds__(kFlatThreads) ropeScatterFlatKernel(Args a, QueryArgs<QUERY> qa, FlatShape f) {
    using S = typename T::storage;
    using U = Unit16<S>;
    constexpr int kPer = U::kElements;
    __shared__ int32_t token_pos[kFlatMaxTokens];
    __shared__ int64_t token_slot[kFlatMaxTokens];
    const int tid = threadIdx.x;
    const int64_t first_token = static_cast<int64_t>(blockIdx.x) * f.tokens_per_group;
    const int tokens_here = static_cast<int>(min(static_cast<int64_t>(f.tokens_per_group), a.num_tokens - first_token));

    // 1a. position and slot of the workgroup's tokens (one thread each; the others re-read the first token's)
    const int64_t my_token = first_token + (tid < tokens_here ? tid : 0);
    const int64_t my_slot = a.slot_mapping[my_token];
    const int64_t my_pos = loadPosition(a, my_token);
    // 1b. the units of this thread's items
    const int table_dim = a.head_size / 2;
    const bool neox = a.neox != 0;
    int tok[ITEMS], kind[ITEMS], head[ITEMS], first[ITEMS], second[ITEMS], table_at[ITEMS]; // kind: 0 query, 1 key, 2 value
    bool live[ITEMS];
    uint4 lo[ITEMS], hi[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int w = tid + kFlatThreads * j;
        const int t = divideSmall(w, f.inv_items);
        live[j] = t < tokens_here;
        tok[j] = live[j] ? t : 0; // an item past the end re-reads the first token's and stores nothing
        int r = w - t * f.items_per_token;
        kind[j] = r < f.q_items ? 0 : (r < f.q_items + f.k_items ? 1 : 2);
        r -= kind[j] == 0 ? 0 : (kind[j] == 1 ? f.q_items : f.q_items + f.k_items);
        head[j] = divideSmall(r, kind[j] == 2 ? f.inv_copy : f.inv_rotate);
        const int step = r - head[j] * (kind[j] == 2 ? f.copy_steps : f.rotate_steps);
        // element offsets of the item's two units inside its vector
        first[j] = kind[j] == 2 ? 2 * step * kPer : (neox ? step * kPer : 2 * step * kPer);
        second[j] = kind[j] == 2 ? (2 * step + 1) * kPer : (neox ? table_dim + step * kPer : 2 * step * kPer + kPer);
        table_at[j] = kind[j] == 2 ? 0 : step * kPer;
        const int64_t token = first_token + tok[j];
        const S *src = static_cast<const S *>(a.v) + token * a.v_src_token_stride + static_cast<int64_t>(head[j]) * a.value_size;
        if (kind[j] == 1) {
            src = static_cast<const S *>(a.k) + token * a.k_src_token_stride + static_cast<int64_t>(head[j]) * a.head_size;
        }
        if constexpr (QUERY) {
            if (kind[j] == 0) {
                src = static_cast<const S *>(qa.q) + token * qa.q_token_stride + head[j] * qa.q_head_stride;
            }
        }
        lo[j] = *reinterpret_cast<const uint4 *>(src + first[j]);
        hi[j] = *reinterpret_cast<const uint4 *>(src + second[j]);
    }
    // 2. positions (forced into the table) and slots to everybody
    if (tid < tokens_here) {
        token_pos[tid] = static_cast<int32_t>(my_pos < 0 ? 0 : (my_pos >= a.table_len ? a.table_len - 1 : my_pos));
        token_slot[tid] = (my_slot >= 0 && my_slot < a.num_slots) ? my_slot : -1; // padding, or outside the pool: dropped
    }
    __syncthreads();
    uint4 sn[ITEMS], cs[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const int64_t at = static_cast<int64_t>(token_pos[tok[j]]) * table_dim + table_at[j];
        sn[j] = *reinterpret_cast<const uint4 *>(static_cast<const S *>(a.sin_table) + at);
        cs[j] = *reinterpret_cast<const uint4 *>(static_cast<const S *>(a.cos_table) + at);
    }
    // 3. rotate and store
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
        const U x_lo = __builtin_bit_cast(U, lo[j]), x_hi = __builtin_bit_cast(U, hi[j]);
        const U s_ = __builtin_bit_cast(U, sn[j]), c_ = __builtin_bit_cast(U, cs[j]);
        U y_lo, y_hi;
        if (neox) {
#pragma unroll
            for (int i = 0; i < kPer; ++i) {
                rotatePair(x_lo.e[i], x_hi.e[i], s_.e[i], c_.e[i], y_lo.e[i], y_hi.e[i]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kPer / 2; ++i) {
                rotatePair(x_lo.e[2 * i], x_lo.e[2 * i + 1], s_.e[i], c_.e[i], y_lo.e[2 * i], y_lo.e[2 * i + 1]);
                rotatePair(x_hi.e[2 * i], x_hi.e[2 * i + 1], s_.e[kPer / 2 + i], c_.e[kPer / 2 + i], y_hi.e[2 * i], y_hi.e[2 * i + 1]);
            }
        }
        const uint4 out_lo = kind[j] == 2 ? lo[j] : __builtin_bit_cast(uint4, y_lo);
        const uint4 out_hi = kind[j] == 2 ? hi[j] : __builtin_bit_cast(uint4, y_hi);
        const int64_t token = first_token + tok[j];
        const int64_t slot = token_slot[tok[j]];
        int64_t page, row;
        if (a.block_shift >= 0) {
            page = slot >> a.block_shift;
            row = slot & (a.block_size - 1);
        } else {
            page = slot / a.block_size;
            row = slot % a.block_size;
        }
        S *dst = static_cast<S *>(a.v_cache) + page * a.v_block_stride + head[j] * a.v_head_stride + row * a.v_slot_stride;
        if (kind[j] == 1) {
            dst = static_cast<S *>(a.k_cache) + page * a.k_block_stride + head[j] * a.k_head_stride + row * a.k_slot_stride;
        }
        bool stores = live[j] && slot >= 0;
        if constexpr (QUERY) {
            if (kind[j] == 0) {
                dst = static_cast<S *>(qa.q_out) + token * qa.q_out_token_stride + head[j] * qa.q_out_head_stride;
                stores = live[j]; // the query of a padding token is rotated all the same
            }
        }
        if (stores) {
            // streamed stores: 4 096 tokens with 32 query heads 24.5 -> 18.0 us, without a query 8.7 -> 7.95 us
            // (streamed loads on top cost 3.3 / 1.0 us: the sources are what the projection has just written)
            device::amd::storeStreamed(dst + first[j], out_lo);
            device::amd::storeStreamed(dst + second[j], out_hi);
        }
    }
}

// Smallest power of two >= x, at most 2^30.
int ceilPow2(int x) {
    int p = 1;
    while (p < x && p < (1 << 30)) {
        p <<= 1;
    }
    return p;
}

bool multipleOf16(uint64_t x) { return (x & 15u) == 0; }

uint32_t inverseOf(int x) { return static_cast<uint32_t>(((uint64_t{1} << 32) + static_cast<uint64_t>(x) - 1) / static_cast<uint64_t>(x)); }

// The flat kernel if the shape fits it (16-byte units, a token's items within one workgroup's reach): true when launched.
template <typename T>
bool launchFlat(const Args &a, const QueryArgs<true> &qa, int rotate_steps, int copy_steps, hipStream_t stream) {
    if (rotate_steps <= 0 || copy_steps <= 0) {
        return false;
    }
    if (copy_steps % 2 != 0) {
        return false; // a V row is an odd number of units: no pairs
    }
    FlatShape f{};
    f.rotate_steps = rotate_steps;
    f.copy_steps = copy_steps / 2;
    const long long q_items = static_cast<long long>(qa.num_q_heads) * rotate_steps;
    const long long k_items = static_cast<long long>(a.num_kv_heads) * rotate_steps;
    const long long items = q_items + k_items + static_cast<long long>(a.num_kv_heads) * f.copy_steps;
    constexpr int kMaxItems = 6; // per thread
    if (items > kFlatThreads * kMaxItems || a.table_len > 0x7fffffff) {
        return false;
    }
    f.q_items = static_cast<int32_t>(q_items);
    f.k_items = static_cast<int32_t>(k_items);
    f.items_per_token = static_cast<int32_t>(items);
    // Items per thread: as few as hold one token when the call is short (a decode step is one round of workgroups
    // whatever it does: latency counts), else about three (96 bytes in flight per thread).
    const int at_least = static_cast<int>((items + kFlatThreads - 1) / kFlatThreads);
    int per_thread = at_least;
    if (a.num_tokens > 1024 && per_thread < 3) {
        per_thread = 3;
    }
    per_thread = per_thread <= 3 ? per_thread : (per_thread <= 4 ? 4 : kMaxItems);
    long long tokens = static_cast<long long>(kFlatThreads) * per_thread / items;
    tokens = tokens > kFlatMaxTokens ? kFlatMaxTokens : tokens;
    f.tokens_per_group = static_cast<int32_t>(tokens);
    f.inv_items = inverseOf(f.items_per_token);
    f.inv_rotate = inverseOf(rotate_steps);
    f.inv_copy = inverseOf(f.copy_steps);
    const dim3 grid(static_cast<unsigned>((a.num_tokens + tokens - 1) / tokens));
    const bool query = qa.num_q_heads > 0;
#define LAUNCH_FLAT(N)                                                                                              \
    if (query) {                                                                                                    \
        ropeScatterFlatKernel<T, true, N><<<grid, kFlatThreads, 0, stream>>>(a, qa, f);                              \
    } else {                                                                                                        \
        ropeScatterFlatKernel<T, false, N><<<grid, kFlatThreads, 0, stream>>>(a, QueryArgs<false>{}, f);             \
    }
    switch (per_thread) {
    case 1: LAUNCH_FLAT(1) break;
    case 2: LAUNCH_FLAT(2) break;
    case 3: LAUNCH_FLAT(3) break;
    case 4: LAUNCH_FLAT(4) break;
    default: LAUNCH_FLAT(6) break;
    }
#undef LAUNCH_FLAT
    return true;
}

template <typename T>
void launch(const Args &a, QueryArgs<true> qa, bool vec, int row_steps, int rotate_steps, hipStream_t stream) {
    if (vec && launchFlat<T>(a, qa, rotate_steps, static_cast<int>(a.value_size / (16 / sizeof(typename T::storage))), stream)) {
        return;
    }
    // 256-thread box: x = steps along a row, y = heads, z = tokens
    int bx = ceilPow2(row_steps);
    bx = bx > 64 ? 64 : bx;
    int by = ceilPow2(a.num_kv_heads + qa.num_q_heads);
    by = by > 256 / bx ? 256 / bx : by;
    const int bz = 256 / (bx * by);
    const int rotate_threads = ceilPow2(rotate_steps > 0 ? rotate_steps : 1);
    qa.threads_per_row = rotate_threads < bx * by ? rotate_threads : bx * by;
    const dim3 block(bx, by, bz);
    const dim3 grid(static_cast<unsigned>((a.num_tokens + bz - 1) / bz));
    if (qa.num_q_heads > 0) {
        if (vec) {
            ropeScatterQueryKernel<T, true><<<grid, block, 0, stream>>>(a, qa);
        } else {
            ropeScatterQueryKernel<T, false><<<grid, block, 0, stream>>>(a, qa);
        }
    } else if (vec) {
        ropeScatterKernel<T, true><<<grid, block, 0, stream>>>(a);
    } else {
        ropeScatterKernel<T, false><<<grid, block, 0, stream>>>(a);
    }
}

} // namespace

struct Descriptor::Opaque {};

Descriptor::~Descriptor() { delete _opaque; }

infiniStatus_t Descriptor::create(infiniopHandle_t handle, Descriptor **desc_ptr, infiniopTensorDescriptor_t k_cache_desc,
                                  infiniopTensorDescriptor_t v_cache_desc, infiniopTensorDescriptor_t k_desc,
                                  infiniopTensorDescriptor_t v_desc, infiniopTensorDescriptor_t slot_mapping_desc,
                                  infiniopTensorDescriptor_t pos_ids_desc, infiniopTensorDescriptor_t sin_table_desc,
                                  infiniopTensorDescriptor_t cos_table_desc, infiniopRoPEAlgo_t algo, bool with_query,
                                  infiniopTensorDescriptor_t q_out_desc, infiniopTensorDescriptor_t q_desc) {
    auto info = RoPEPagedCachingInfo::create(k_cache_desc, v_cache_desc, k_desc, v_desc, slot_mapping_desc, pos_ids_desc,
                                             sin_table_desc, cos_table_desc, algo, with_query, q_out_desc, q_desc);
    CHECK_RESULT(info);
    *desc_ptr = new Descriptor(new Opaque{}, info.take(), 0, handle->device, handle->device_id);
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t Descriptor::calculate(void *workspace, size_t workspace_size, void *q_out, const void *q, void *k_cache,
                                     void *v_cache, const void *k, const void *v, const void *slot_mapping,
                                     const void *pos_ids, const void *sin_table, const void *cos_table, void *stream_) const {
    (void)workspace;
    (void)workspace_size;
    const auto &in = _info.scatter;
    const bool rotates_query = _info.has_query && _info.num_q_heads > 0 && in.head_size > 0;
    const bool caches = in.num_kv_heads > 0 && (in.head_size > 0 || in.v_head_size > 0);
    if (in.num_tokens == 0 || (!caches && !rotates_query)) {
        return INFINI_STATUS_SUCCESS;
    }
    if (rotates_query && (q_out == nullptr || q == nullptr)) {
        return INFINI_STATUS_NULL_POINTER;
    }
    // the kernel counts heads, row steps and workgroups in 32 bits
    if (in.num_kv_heads + (rotates_query ? _info.num_q_heads : 0) > 0x7fffffff || in.head_size > 0x7fffffff
        || in.v_head_size > 0x7fffffff || in.block_size > 0x7fffffff || in.num_tokens > 0x7fffffff) {
        return INFINI_STATUS_BAD_TENSOR_SHAPE;
    }
    if (k_cache == nullptr || v_cache == nullptr || k == nullptr || v == nullptr || slot_mapping == nullptr
        || pos_ids == nullptr || sin_table == nullptr || cos_table == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (_info.table_len == 0 && in.head_size > 0) {
        return INFINI_STATUS_BAD_PARAM; // no row of the tables to rotate with
    }
    int current_device = -1;
    if (hipGetDevice(&current_device) != hipSuccess || current_device != device_id) {
        return INFINI_STATUS_BAD_PARAM;
    }

    Args a{};
    a.k_cache = k_cache;
    a.v_cache = v_cache;
    a.k = k;
    a.v = v;
    a.slot_mapping = static_cast<const int64_t *>(slot_mapping);
    a.pos_ids = pos_ids;
    a.sin_table = sin_table;
    a.cos_table = cos_table;
    QueryArgs<true> qa{};
    qa.q_out = q_out;
    qa.q = q;
    qa.num_q_heads = rotates_query ? static_cast<int32_t>(_info.num_q_heads) : 0;
    qa.q_token_stride = _info.q_token_stride;
    qa.q_head_stride = _info.q_head_stride;
    qa.q_out_token_stride = _info.q_out_token_stride;
    qa.q_out_head_stride = _info.q_out_head_stride;
    a.num_tokens = static_cast<int64_t>(in.num_tokens);
    a.num_slots = static_cast<int64_t>(in.num_blocks) * static_cast<int64_t>(in.block_size);
    a.table_len = static_cast<int64_t>(_info.table_len);
    a.num_kv_heads = static_cast<int32_t>(in.num_kv_heads);
    a.block_size = static_cast<int32_t>(in.block_size);
    a.block_shift = -1;
    if (in.block_size > 0 && (in.block_size & (in.block_size - 1)) == 0) {
        a.block_shift = __builtin_ctzll(in.block_size);
    }
    a.head_size = static_cast<int32_t>(in.head_size);
    a.value_size = static_cast<int32_t>(in.v_head_size);
    a.pos_bytes = static_cast<int32_t>(infiniSizeOf(_info.pos_dtype));
    a.pos_signed = _info.pos_dtype == INFINI_DTYPE_I8 || _info.pos_dtype == INFINI_DTYPE_I16
                || _info.pos_dtype == INFINI_DTYPE_I32 || _info.pos_dtype == INFINI_DTYPE_I64;
    a.neox = _info.algo == INFINIOP_ROPE_ALGO_GPT_NEOX;
    a.k_src_token_stride = in.k_src_stride;
    a.v_src_token_stride = in.v_src_stride;
    a.k_block_stride = in.k_cache_block_stride;
    a.k_head_stride = in.k_cache_head_stride;
    a.k_slot_stride = in.k_cache_slot_stride;
    a.v_block_stride = in.v_cache_block_stride;
    a.v_head_stride = in.v_cache_head_stride;
    a.v_slot_stride = in.v_cache_slot_stride;

    // 16-byte units when every size, stride and base address allows them
    const uint64_t es = infiniSizeOf(in.dtype);
    auto bytes = [es](ptrdiff_t elements) { return static_cast<uint64_t>(elements) * es; };
    const int per = static_cast<int>(16 / es);
    bool vec = (_info.table_dim % per) == 0 && (in.v_head_size % per) == 0;
    for (uint64_t quantity : {bytes(in.head_size), bytes(in.v_head_size), bytes(in.k_src_stride), bytes(in.v_src_stride),
                              bytes(in.k_cache_block_stride), bytes(in.k_cache_head_stride), bytes(in.k_cache_slot_stride),
                              bytes(in.v_cache_block_stride), bytes(in.v_cache_head_stride), bytes(in.v_cache_slot_stride),
                              static_cast<uint64_t>(reinterpret_cast<uintptr_t>(k_cache)),
                              static_cast<uint64_t>(reinterpret_cast<uintptr_t>(v_cache)),
                              static_cast<uint64_t>(reinterpret_cast<uintptr_t>(k)),
                              static_cast<uint64_t>(reinterpret_cast<uintptr_t>(v)),
                              static_cast<uint64_t>(reinterpret_cast<uintptr_t>(sin_table)),
                              static_cast<uint64_t>(reinterpret_cast<uintptr_t>(cos_table)),
                              bytes(static_cast<ptrdiff_t>(_info.table_dim))}) {
        vec = vec && multipleOf16(quantity);
    }
    if (rotates_query) {
        for (uint64_t quantity : {bytes(_info.q_token_stride), bytes(_info.q_head_stride), bytes(_info.q_out_token_stride),
                                  bytes(_info.q_out_head_stride), static_cast<uint64_t>(reinterpret_cast<uintptr_t>(q)),
                                  static_cast<uint64_t>(reinterpret_cast<uintptr_t>(q_out))}) {
            vec = vec && multipleOf16(quantity);
        }
    }
    const int rotate_steps = static_cast<int>(vec ? _info.table_dim / per : _info.table_dim);
    const int copy_steps = static_cast<int>(vec ? in.v_head_size / per : in.v_head_size);
    const int row_steps = rotate_steps > copy_steps ? rotate_steps : copy_steps;
    auto stream = static_cast<hipStream_t>(stream_);
    switch (in.dtype) {
    case INFINI_DTYPE_F16: launch<F16>(a, qa, vec, row_steps > 0 ? row_steps : 1, rotate_steps, stream); break;
    case INFINI_DTYPE_BF16: launch<BF16>(a, qa, vec, row_steps > 0 ? row_steps : 1, rotate_steps, stream); break;
    case INFINI_DTYPE_F32: launch<F32>(a, qa, vec, row_steps > 0 ? row_steps : 1, rotate_steps, stream); break;
    default: return INFINI_STATUS_BAD_TENSOR_DTYPE;
    }
    return hipGetLastError() == hipSuccess ? INFINI_STATUS_SUCCESS : INFINI_STATUS_INTERNAL_ERROR;
}

} // namespace op::rope_paged_caching::amd
