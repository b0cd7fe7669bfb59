/*
 * CPU oracle for InfiniOP paged_attention (decode), paged_attention_prefill, paged_caching and kv_caching.
 *
 * TEST INFRASTRUCTURE ONLY. This file restates, in plain C, the algorithm of the reference's device
 * kernels so that the HIP kernels of this repository can be checked against it. Only tests/,
 * __graft_entry__.smoke() and the cpu_baseline leg of bench.py may load it; the product
 * (libinfiniop.so) never does and has no CPU path of its own.
 *
 * The reference ships no CPU implementation and no golden vectors for these two operators, and its
 * CUDA sources cannot be compiled here, so the oracle is pinned by mathematics instead (see
 * tests/test_oracle_pinning.py): an independent fp64 two-pass softmax on gathered K/V, torch's
 * scaled_dot_product_attention on the gathered sequence, closed forms (length 1, equal V rows,
 * zero query, one dominant key), invariance under page permutation, GQA == MHA on repeated heads,
 * split == unsplit, prefill row j == decode over the first history + j + 1 tokens, prefill against an
 * fp64 masked softmax, and byte-exact copy models (numpy assignment) for paged_caching and kv_caching.
 *
 * Functions and the reference code each one follows:
 *   oracle_paged_attention         src/infiniop/ops/paged_attention/cuda/kernel_v2.cuh:134-336
 *                                  (one query head at a time: fp32 dot product, score in the log2
 *                                  domain, online max/sum softmax with exp2f, out = acc / (l + 1e-6),
 *                                  round-to-nearest-even to fp16 / bf16; seq_len <= 0 leaves out untouched)
 *   oracle_paged_attention_splitkv kernel_v2.cuh:340-554 (token shards of ceil(len / splits), partial
 *                                  (m, l, acc) per shard, empty shard = (-inf, 0, 0)) and :556-616 (combine)
 *   oracle_paged_attention_prefill src/infiniop/ops/paged_attention_prefill/cuda/kernel_v2.cuh:254-472 (row ->
 *                                  sequence lookup, visible range history + j + 1, then the decode recurrence)
 *   oracle_paged_caching           src/infiniop/ops/paged_caching/cuda/kernel.cuh:22-89
 *                                  (slot < 0 skipped, page = slot / block_size, row = slot % block_size,
 *                                  source heads packed, element-wise copy)
 *   oracle_rope_paged_caching      src/infiniop/ops/rope/cpu/rope_cpu.cc:56-98 (pairs (2j, 2j + 1) or (j, j + d / 2),
 *                                  y0 = x0 cos - x1 sin, y1 = x0 sin + x1 cos in fp32, every product and sum
 *                                  rounded on its own, one rounding to the storage dtype) followed by the slot
 *                                  scatter of oracle_paged_caching, without the tensor in between
 *   oracle_rope                    the same rotation on its own, [tokens, heads, d] -> [tokens, heads, d]
 *   oracle_kv_caching              src/infiniop/ops/kv_caching/cuda/kernel.cuh:32-58
 *                                  (element (b, h, s, d) of the new tensors goes to cache position
 *                                  past_kv_lengths[b] + s; every dimension of every tensor strided)
 *
 * Build: make -C oracle   (gcc -O2 -fopenmp -shared)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_DTYPE_F16 0
#define ORACLE_DTYPE_BF16 1

/* ---- storage formats <-> float, round-to-nearest-even ---- */

static float bf16_to_float(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t float_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x0040u); /* quiet NaN */
    }
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

static float f16_to_float(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t u;
    if (exp == 0) {
        if (man == 0) {
            u = sign;
        } else { /* subnormal: normalise */
            int shift = 0;
            while ((man & 0x400u) == 0) {
                man <<= 1;
                ++shift;
            }
            man &= 0x3ffu;
            u = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        u = sign | 0x7f800000u | (man << 13);
    } else {
        u = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &u, 4);
    return f;
}

static uint16_t float_to_f16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t abs = u & 0x7fffffffu;
    if (abs > 0x7f800000u) {
        return (uint16_t)(sign | 0x7e00u); /* NaN */
    }
    if (abs >= 0x477ff000u) { /* >= 65520 rounds to inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (abs < 0x33000001u) { /* <= 2^-25 rounds to zero */
        return sign;
    }
    int32_t exp = (int32_t)(abs >> 23) - 127;
    uint32_t man = (abs & 0x7fffffu) | 0x800000u; /* 24-bit significand */
    int shift; /* bits to drop from the 24-bit significand */
    uint32_t base;
    if (exp < -14) { /* subnormal half */
        shift = 13 + (-14 - exp);
        base = 0;
    } else {
        shift = 13;
        base = ((uint32_t)(exp + 15) << 10) - 0x400u; /* the implicit bit adds the 0x400 back */
    }
    uint32_t kept = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (kept & 1u))) {
        ++kept;
    }
    return (uint16_t)(sign | (base + kept));
}

static float load_elem(const uint16_t *p, int dtype) {
    return dtype == ORACLE_DTYPE_F16 ? f16_to_float(*p) : bf16_to_float(*p);
}

static uint16_t store_elem(float f, int dtype) {
    return dtype == ORACLE_DTYPE_F16 ? float_to_f16(f) : float_to_bf16(f);
}

/* exposed so the conversion helpers themselves can be checked against numpy / torch */
float oracle_to_float(uint16_t bits, int dtype) { return load_elem(&bits, dtype); }
uint16_t oracle_from_float(float f, int dtype) { return store_elem(f, dtype); }

typedef struct {
    int dtype; /* ORACLE_DTYPE_* of q, out and both caches */
    int64_t num_seqs, num_heads, num_kv_heads, head_size, value_size, block_size, max_blocks_per_seq;
    /* element strides */
    int64_t q_stride, q_head_stride, o_stride, o_head_stride;
    int64_t k_batch_stride, k_head_stride, k_row_stride;
    int64_t v_batch_stride, v_head_stride, v_row_stride;
    int64_t block_table_stride;
    float scale;
} oracle_attention_shape;

static const float kLog2e = 1.4426950408889634f;

/* One query head of one sequence over tokens [t_begin, t_end): the recurrence of
 * kernel_v2.cuh:223-315. Leaves the un-normalised accumulator in acc[value_size] and returns m, l. */
static void attend_range(const oracle_attention_shape *s, const uint16_t *q_row, const uint16_t *k_cache,
                         const uint16_t *v_cache, const int64_t *block_table, int64_t kv_head, float alibi_slope,
                         int64_t seq_len, int64_t t_begin, int64_t t_end, float *acc, float *m_out, float *l_out) {
    const float scale_log2 = s->scale * kLog2e;
    float m = -INFINITY, l = 0.0f;
    for (int64_t d = 0; d < s->value_size; ++d) {
        acc[d] = 0.0f;
    }
    for (int64_t t = t_begin; t < t_end; ++t) {
        const int64_t page = block_table[t / s->block_size];
        const int64_t row = t % s->block_size;
        const uint16_t *k_row = k_cache + page * s->k_batch_stride + kv_head * s->k_head_stride + row * s->k_row_stride;
        const uint16_t *v_row = v_cache + page * s->v_batch_stride + kv_head * s->v_head_stride + row * s->v_row_stride;

        float qk = 0.0f;
        for (int64_t d = 0; d < s->head_size; ++d) {
            qk += load_elem(q_row + d, s->dtype) * load_elem(k_row + d, s->dtype);
        }
        float score = qk * scale_log2;
        if (alibi_slope != 0.0f) {
            score += (alibi_slope * (float)(t - (seq_len - 1))) * kLog2e;
        }
        const float m_new = fmaxf(m, score);
        const float alpha = exp2f(m - m_new);
        const float beta = exp2f(score - m_new);
        l = l * alpha + beta;
        m = m_new;
        for (int64_t d = 0; d < s->value_size; ++d) {
            acc[d] = acc[d] * alpha + beta * load_elem(v_row + d, s->dtype);
        }
    }
    *m_out = m;
    *l_out = l;
}

/* Unsplit decode, kernel_v2.cuh:134-336. Returns 0, or -1 on a bad argument.
 * out_f32 (optional, packed [num_seqs, num_heads, value_size]) receives acc / (l + 1e-6) as the fp32
 * value the kernel holds just before it rounds to the storage dtype (:320-334); comparing a device
 * result with it is free of the double rounding that comparing two rounded results carries. */
int oracle_paged_attention(void *out_, float *out_f32, const void *q_, const void *k_cache_, const void *v_cache_,
                           const int64_t *block_tables, const int64_t *seq_lens, const float *alibi_slopes,
                           const oracle_attention_shape *s, int num_threads) {
    if (s->num_kv_heads <= 0 || s->num_heads % s->num_kv_heads != 0 || s->block_size <= 0) {
        return -1;
    }
    uint16_t *out = (uint16_t *)out_;
    const uint16_t *q = (const uint16_t *)q_;
    const int64_t group = s->num_heads / s->num_kv_heads;
    const int64_t work = s->num_seqs * s->num_heads;
    if (num_threads < 1) {
        num_threads = 1;
    }
#pragma omp parallel num_threads(num_threads)
    {
        float *acc = (float *)malloc(sizeof(float) * (size_t)(s->value_size > 0 ? s->value_size : 1));
#pragma omp for schedule(dynamic, 1)
        for (int64_t w = 0; w < work; ++w) {
            const int64_t seq = w / s->num_heads, head = w % s->num_heads;
            const int64_t seq_len = seq_lens[seq];
            if (seq_len <= 0) {
                continue; /* :164-167, nothing is written */
            }
            float m, l;
            attend_range(s, q + seq * s->q_stride + head * s->q_head_stride, (const uint16_t *)k_cache_,
                         (const uint16_t *)v_cache_, block_tables + seq * s->block_table_stride, head / group,
                         alibi_slopes ? alibi_slopes[head] : 0.0f, seq_len, 0, seq_len, acc, &m, &l);
            const float inv_l = 1.0f / (l + 1e-6f);
            uint16_t *o_row = out + seq * s->o_stride + head * s->o_head_stride;
            for (int64_t d = 0; d < s->value_size; ++d) {
                o_row[d] = store_elem(acc[d] * inv_l, s->dtype);
                if (out_f32 != NULL) {
                    out_f32[(seq * s->num_heads + head) * s->value_size + d] = acc[d] * inv_l;
                }
            }
        }
        free(acc);
    }
    return 0;
}

/* Split-KV decode and combine, kernel_v2.cuh:340-616: shard i covers tokens
 * [i * ceil(len / splits), min(len, (i + 1) * ceil(len / splits))). */
int oracle_paged_attention_splitkv(void *out_, const void *q_, const void *k_cache_, const void *v_cache_,
                                   const int64_t *block_tables, const int64_t *seq_lens, const float *alibi_slopes,
                                   const oracle_attention_shape *s, int num_splits, int num_threads) {
    if (s->num_kv_heads <= 0 || s->num_heads % s->num_kv_heads != 0 || s->block_size <= 0 || num_splits < 1) {
        return -1;
    }
    uint16_t *out = (uint16_t *)out_;
    const uint16_t *q = (const uint16_t *)q_;
    const int64_t group = s->num_heads / s->num_kv_heads;
    const int64_t work = s->num_seqs * s->num_heads;
    const size_t vs = (size_t)(s->value_size > 0 ? s->value_size : 1);
    if (num_threads < 1) {
        num_threads = 1;
    }
#pragma omp parallel num_threads(num_threads)
    {
        float *part_acc = (float *)malloc(sizeof(float) * vs * (size_t)num_splits);
        float *part_m = (float *)malloc(sizeof(float) * (size_t)num_splits);
        float *part_l = (float *)malloc(sizeof(float) * (size_t)num_splits);
#pragma omp for schedule(dynamic, 1)
        for (int64_t w = 0; w < work; ++w) {
            const int64_t seq = w / s->num_heads, head = w % s->num_heads;
            const int64_t seq_len = seq_lens[seq];
            if (seq_len <= 0) {
                continue;
            }
            const int64_t shard = (seq_len + num_splits - 1) / num_splits;
            for (int i = 0; i < num_splits; ++i) {
                const int64_t t0 = (int64_t)i * shard;
                const int64_t t1 = t0 + shard < seq_len ? t0 + shard : seq_len;
                if (t0 >= t1) { /* empty shard, :676-693 */
                    part_m[i] = -INFINITY;
                    part_l[i] = 0.0f;
                    for (size_t d = 0; d < vs; ++d) {
                        part_acc[(size_t)i * vs + d] = 0.0f;
                    }
                    continue;
                }
                attend_range(s, q + seq * s->q_stride + head * s->q_head_stride, (const uint16_t *)k_cache_,
                             (const uint16_t *)v_cache_, block_tables + seq * s->block_table_stride, head / group,
                             alibi_slopes ? alibi_slopes[head] : 0.0f, seq_len, t0, t1, part_acc + (size_t)i * vs,
                             &part_m[i], &part_l[i]);
            }
            /* combine, :574-614 */
            float m = -INFINITY;
            for (int i = 0; i < num_splits; ++i) {
                m = fmaxf(m, part_m[i]);
            }
            float l = 0.0f;
            for (int i = 0; i < num_splits; ++i) {
                if (part_l[i] > 0.0f) {
                    l += part_l[i] * exp2f(part_m[i] - m);
                }
            }
            const float inv_l = 1.0f / (l + 1e-6f);
            uint16_t *o_row = out + seq * s->o_stride + head * s->o_head_stride;
            for (int64_t d = 0; d < s->value_size; ++d) {
                float acc = 0.0f;
                for (int i = 0; i < num_splits; ++i) {
                    acc += part_acc[(size_t)i * vs + (size_t)d] * exp2f(part_m[i] - m);
                }
                o_row[d] = store_elem(acc * inv_l, s->dtype);
            }
        }
        free(part_acc);
        free(part_m);
        free(part_l);
    }
    return 0;
}

/* Prefill, src/infiniop/ops/paged_attention_prefill/cuda/kernel_v2.cuh:254-472: query row i belongs to the
 * sequence s with cu_seqlens_q[s] <= i < cu_seqlens_q[s+1] (:20-38; a row no sequence owns is skipped, :297-300);
 * with q_len = cu[s+1] - cu[s] and history = kv_lens[s] - q_len, local token j = i - cu[s] attends over tokens
 * [0, history + j + 1) (:302-306, nothing is written when that range is empty) with the decode recurrence;
 * ALiBi distance is t - (history + j) (:383-386). s->num_seqs is the number of sequences, the row count of q and
 * out is total_q_tokens. rows (optional) lists the query rows to evaluate, NULL = all of them; only those rows of
 * out and out_f32 (packed [total_q_tokens, num_heads, value_size], optional) are written. */
int oracle_paged_attention_prefill(void *out_, float *out_f32, const void *q_, const void *k_cache_,
                                   const void *v_cache_, const int64_t *block_tables, const int64_t *kv_lens,
                                   const int64_t *cu_seqlens_q, const float *alibi_slopes,
                                   const oracle_attention_shape *s, int64_t total_q_tokens, const int64_t *rows,
                                   int64_t num_rows, int num_threads) {
    if (s->num_kv_heads <= 0 || s->num_heads % s->num_kv_heads != 0 || s->block_size <= 0) {
        return -1;
    }
    uint16_t *out = (uint16_t *)out_;
    const uint16_t *q = (const uint16_t *)q_;
    const int64_t group = s->num_heads / s->num_kv_heads;
    if (rows == NULL) {
        num_rows = total_q_tokens;
    }
    const int64_t work = num_rows * s->num_heads;
    if (num_threads < 1) {
        num_threads = 1;
    }
#pragma omp parallel num_threads(num_threads)
    {
        float *acc = (float *)malloc(sizeof(float) * (size_t)(s->value_size > 0 ? s->value_size : 1));
#pragma omp for schedule(dynamic, 1)
        for (int64_t w = 0; w < work; ++w) {
            const int64_t row = rows ? rows[w / s->num_heads] : w / s->num_heads;
            const int64_t head = w % s->num_heads;
            if (row < 0 || row >= total_q_tokens) {
                continue;
            }
            int64_t seq = -1;
            for (int64_t i = 0; i < s->num_seqs; ++i) {
                if (row >= cu_seqlens_q[i] && row < cu_seqlens_q[i + 1]) {
                    seq = i;
                    break;
                }
            }
            if (seq < 0) {
                continue;
            }
            const int64_t q_len = cu_seqlens_q[seq + 1] - cu_seqlens_q[seq];
            const int64_t history = kv_lens[seq] - q_len;
            const int64_t visible = history + (row - cu_seqlens_q[seq]) + 1;
            if (visible <= 0) {
                continue;
            }
            float m, l;
            attend_range(s, q + row * s->q_stride + head * s->q_head_stride, (const uint16_t *)k_cache_,
                         (const uint16_t *)v_cache_, block_tables + seq * s->block_table_stride, head / group,
                         alibi_slopes ? alibi_slopes[head] : 0.0f, visible, 0, visible, acc, &m, &l);
            const float inv_l = 1.0f / (l + 1e-6f);
            uint16_t *o_row = out + row * s->o_stride + head * s->o_head_stride;
            for (int64_t d = 0; d < s->value_size; ++d) {
                o_row[d] = store_elem(acc[d] * inv_l, s->dtype);
                if (out_f32 != NULL) {
                    out_f32[(row * s->num_heads + head) * s->value_size + d] = acc[d] * inv_l;
                }
            }
        }
        free(acc);
    }
    return 0;
}

typedef struct {
    int64_t elem_size; /* bytes per element: 2 (fp16 / bf16) or 4 (fp32) */
    int64_t num_tokens, num_kv_heads, head_size, v_head_size, block_size;
    /* element strides */
    int64_t k_src_stride, v_src_stride;
    int64_t k_cache_block_stride, v_cache_block_stride;
    int64_t k_cache_head_stride, v_cache_head_stride;
    int64_t k_cache_slot_stride, v_cache_slot_stride;
} oracle_caching_shape;

/* Slot scatter, paged_caching/cuda/kernel.cuh:52-88. */
int oracle_paged_caching(void *k_cache_, void *v_cache_, const void *k_, const void *v_, const int64_t *slot_mapping,
                         const oracle_caching_shape *s) {
    if (s->block_size <= 0 || (s->elem_size != 2 && s->elem_size != 4)) {
        return -1;
    }
    char *k_cache = (char *)k_cache_, *v_cache = (char *)v_cache_;
    const char *k = (const char *)k_, *v = (const char *)v_;
    const int64_t es = s->elem_size;
    for (int64_t tok = 0; tok < s->num_tokens; ++tok) {
        const int64_t slot = slot_mapping[tok];
        if (slot < 0) {
            continue; /* padding, :61-63 */
        }
        const int64_t page = slot / s->block_size, row = slot % s->block_size;
        for (int64_t head = 0; head < s->num_kv_heads; ++head) {
            const char *k_src = k + (tok * s->k_src_stride + head * s->head_size) * es;
            const char *v_src = v + (tok * s->v_src_stride + head * s->v_head_size) * es;
            char *k_dst = k_cache + (page * s->k_cache_block_stride + head * s->k_cache_head_stride + row * s->k_cache_slot_stride) * es;
            char *v_dst = v_cache + (page * s->v_cache_block_stride + head * s->v_cache_head_stride + row * s->v_cache_slot_stride) * es;
            for (int64_t i = 0; i < s->head_size; ++i) {
                memcpy(k_dst + i * es, k_src + i * es, (size_t)es);
            }
            for (int64_t i = 0; i < s->v_head_size; ++i) {
                memcpy(v_dst + i * es, v_src + i * es, (size_t)es);
            }
        }
    }
    return 0;
}

/* One vector of 2 * half elements rotated by row `pos` of the tables (rope_cpu.cc:71-84): pair j is elements
 * (2j, 2j + 1), or (j, j + half) for neox; four products and two sums, each rounded to fp32 on its own (no fused
 * multiply-add), one rounding to the storage dtype. dst may be src. */
static void rope_vector(char *dst, const char *src, const char *sin_table, const char *cos_table, int64_t pos,
                        int64_t half, int dtype, int neox) {
    for (int64_t j = 0; j < half; ++j) {
        const int64_t p0 = neox ? j : 2 * j, p1 = neox ? j + half : 2 * j + 1;
        float x0, x1, sn, cs;
        if (dtype == 2) {
            memcpy(&x0, src + p0 * 4, 4);
            memcpy(&x1, src + p1 * 4, 4);
            memcpy(&sn, sin_table + (pos * half + j) * 4, 4);
            memcpy(&cs, cos_table + (pos * half + j) * 4, 4);
        } else {
            x0 = load_elem((const uint16_t *)(src + p0 * 2), dtype);
            x1 = load_elem((const uint16_t *)(src + p1 * 2), dtype);
            sn = load_elem((const uint16_t *)(sin_table + (pos * half + j) * 2), dtype);
            cs = load_elem((const uint16_t *)(cos_table + (pos * half + j) * 2), dtype);
        }
        volatile float x0c = x0 * cs, x1s = x1 * sn, x0s = x0 * sn, x1c = x1 * cs;
        const float y0 = x0c - x1s, y1 = x0s + x1c;
        if (dtype == 2) {
            memcpy(dst + p0 * 4, &y0, 4);
            memcpy(dst + p1 * 4, &y1, 4);
        } else {
            const uint16_t b0 = store_elem(y0, dtype), b1 = store_elem(y1, dtype);
            memcpy(dst + p0 * 2, &b0, 2);
            memcpy(dst + p1 * 2, &b1, 2);
        }
    }
}

/* Rotary embedding of x [num_tokens, num_heads, head_size] into y (same shape; y may be x), one position per
 * token: the reference's RoPE on its own (rope_cpu.cc:56-98), which the fused operator applies to the query.
 * Strides in elements; the last dimension is packed. Positions outside the tables use the nearest row. */
int oracle_rope(void *y_, const void *x_, const int64_t *pos_ids, const void *sin_table_, const void *cos_table_,
                int64_t table_len, int dtype, int neox, int64_t num_tokens, int64_t num_heads, int64_t head_size,
                int64_t x_token_stride, int64_t x_head_stride, int64_t y_token_stride, int64_t y_head_stride) {
    const int64_t es = dtype == 2 ? 4 : 2;
    if ((head_size & 1) || table_len <= 0 || dtype < 0 || dtype > 2) {
        return -1;
    }
    for (int64_t tok = 0; tok < num_tokens; ++tok) {
        int64_t pos = pos_ids[tok];
        pos = pos < 0 ? 0 : (pos >= table_len ? table_len - 1 : pos);
        for (int64_t head = 0; head < num_heads; ++head) {
            rope_vector((char *)y_ + (tok * y_token_stride + head * y_head_stride) * es,
                        (const char *)x_ + (tok * x_token_stride + head * x_head_stride) * es,
                        (const char *)sin_table_, (const char *)cos_table_, pos, head_size / 2, dtype, neox);
        }
    }
    return 0;
}

/* Rotary embedding of K (rope_cpu.cc:56-98, one position per token) fused with the slot scatter above.
 * dtype: ORACLE_DTYPE_F16 / BF16, or 2 for fp32. neox: pairs half a vector apart, else neighbouring. A position
 * outside the tables uses the nearest row (the reference reads out of bounds); returns -1 for arguments it
 * cannot take. */
int oracle_rope_paged_caching(void *k_cache_, void *v_cache_, const void *k_, const void *v_, const int64_t *slot_mapping,
                              const int64_t *pos_ids, const void *sin_table_, const void *cos_table_, int64_t table_len,
                              int dtype, int neox, const oracle_caching_shape *s) {
    const int64_t es = dtype == 2 ? 4 : 2;
    if (s->block_size <= 0 || s->elem_size != es || (s->head_size & 1) || table_len <= 0 || dtype < 0 || dtype > 2) {
        return -1;
    }
    char *k_cache = (char *)k_cache_, *v_cache = (char *)v_cache_;
    const char *k = (const char *)k_, *v = (const char *)v_;
    const char *sin_table = (const char *)sin_table_, *cos_table = (const char *)cos_table_;
    const int64_t half = s->head_size / 2;
    for (int64_t tok = 0; tok < s->num_tokens; ++tok) {
        const int64_t slot = slot_mapping[tok];
        if (slot < 0) {
            continue;
        }
        int64_t pos = pos_ids[tok];
        pos = pos < 0 ? 0 : (pos >= table_len ? table_len - 1 : pos);
        const int64_t page = slot / s->block_size, row = slot % s->block_size;
        for (int64_t head = 0; head < s->num_kv_heads; ++head) {
            const char *k_src = k + (tok * s->k_src_stride + head * s->head_size) * es;
            const char *v_src = v + (tok * s->v_src_stride + head * s->v_head_size) * es;
            char *k_dst = k_cache + (page * s->k_cache_block_stride + head * s->k_cache_head_stride + row * s->k_cache_slot_stride) * es;
            char *v_dst = v_cache + (page * s->v_cache_block_stride + head * s->v_cache_head_stride + row * s->v_cache_slot_stride) * es;
            rope_vector(k_dst, k_src, sin_table, cos_table, pos, half, dtype, neox);
            memcpy(v_dst, v_src, (size_t)(s->v_head_size * es));
        }
    }
    return 0;
}

typedef struct {
    int64_t elem_size; /* bytes per element: 2 or 4 */
    int64_t batch_size, num_kv_heads, max_seq_len, seq_len, hidden_dim;
    /* element strides of dims 0..3 */
    int64_t k_cache_strides[4], v_cache_strides[4], k_strides[4], v_strides[4];
} oracle_kv_caching_shape;

/* Append to contiguous caches, kv_caching/cuda/kernel.cuh:32-58: one element at a time, position
 * past_kv_lengths[b] + s. A position outside the cache is an out-of-bounds write in the reference and
 * reported here (-2) without touching anything for that row. */
int oracle_kv_caching(void *k_cache_, void *v_cache_, const void *k_, const void *v_, const int64_t *past_kv_lengths,
                      const oracle_kv_caching_shape *s) {
    if (s->elem_size != 2 && s->elem_size != 4) {
        return -1;
    }
    char *k_cache = (char *)k_cache_, *v_cache = (char *)v_cache_;
    const char *k = (const char *)k_, *v = (const char *)v_;
    const int64_t es = s->elem_size;
    int rc = 0;
    for (int64_t b = 0; b < s->batch_size; ++b) {
        for (int64_t h = 0; h < s->num_kv_heads; ++h) {
            for (int64_t t = 0; t < s->seq_len; ++t) {
                const int64_t pos = past_kv_lengths[b] + t; /* :48-50 */
                if (pos < 0 || pos >= s->max_seq_len) {
                    rc = -2;
                    continue;
                }
                for (int64_t d = 0; d < s->hidden_dim; ++d) {
                    const int64_t kc = b * s->k_cache_strides[0] + h * s->k_cache_strides[1] + pos * s->k_cache_strides[2] + d * s->k_cache_strides[3];
                    const int64_t vc = b * s->v_cache_strides[0] + h * s->v_cache_strides[1] + pos * s->v_cache_strides[2] + d * s->v_cache_strides[3];
                    const int64_t ks = b * s->k_strides[0] + h * s->k_strides[1] + t * s->k_strides[2] + d * s->k_strides[3];
                    const int64_t vs = b * s->v_strides[0] + h * s->v_strides[1] + t * s->v_strides[2] + d * s->v_strides[3];
                    memcpy(k_cache + kc * es, k + ks * es, (size_t)es); /* :51-57 */
                    memcpy(v_cache + vc * es, v + vs * es, (size_t)es);
                }
            }
        }
    }
    return rc;
}
