/*
 * The framework-side adaptors of the paged operators, as a C ABI (lib/libinfinicore_ops.so).
 *
 * In the reference these are C++ functions between `infinicore::op::paged_attention_` and the InfiniOP
 * C API (src/infinicore/ops/paged_attention/paged_attention_infiniop.cc:7-79 and its siblings for
 * paged_caching, paged_attention_prefill and kv_caching): they describe the tensors, fetch an operator
 * descriptor from a thread-local LRU cache of 100 entries per device keyed by the tensors' metadata
 * (src/infinicore/ops/infiniop_impl.hpp:8-66, include/infinicore/ops/common/cache.hpp:12-83,
 * include/infinicore/common/hash.hpp:11-31), obtain a byte workspace of the size the descriptor asks
 * for, and call the operator on the current stream. They come as a plan / run / cleanup triple so that
 * a graph recorder can plan once and run many times (paged_attention_infiniop.cc:18-77).
 *
 * The same three steps are exported here over plain tensor views instead of the reference's Tensor
 * class, which belongs to a much larger framework. The device is the calling thread's current
 * InfiniRT device (infinirtSetDevice) and must be an AMD device. Nothing here has a host fallback.
 */
#ifndef INFINICORE_AMD_INFINICORE_OPS_H
#define INFINICORE_AMD_INFINICORE_OPS_H

#include "infinicore.h"
#include "infinirt.h"
#include <stdint.h>

/* What the adaptors read of a tensor: the reference's Tensor::data(), dtype(), shape(), strides()
 * (include/infinicore/tensor.hpp). `strides` are in elements; NULL means C-contiguous. */
typedef struct {
    void *data; /* device pointer */
    infiniDtype_t dtype;
    size_t ndim;
    const size_t *shape;
    const ptrdiff_t *strides;
} infinicoreTensorView_t;

/* A planned call: a shared reference to the cached operator descriptor, a workspace of its own and the
 * data pointers of the tensors it was planned on (the reference's PlannedMeta,
 * paged_attention_infiniop.cc:11-16). */
typedef struct InfinicorePlannedOp *infinicorePlannedOp_t;

typedef enum {
    INFINICORE_OP_PAGED_ATTENTION = 0,
    INFINICORE_OP_PAGED_ATTENTION_PREFILL = 1,
    INFINICORE_OP_PAGED_CACHING = 2,
    INFINICORE_OP_KV_CACHING = 3,
    INFINICORE_OP_KIND_COUNT
} infinicoreOpKind_t;

/* ---- plan: descriptor from the cache (created on a miss), workspace allocated; may not run under
 *      stream capture (it allocates). A failed plan leaves *plan_ptr NULL and returns the status of the
 *      InfiniOP call that refused the tensors. ---- */
/* paged_attention_infiniop.cc:18-46; alibi_slopes may be NULL. Unlike the reference's key
 * (paged_attention_infiniop.cc:21) the cache key includes `scale`: the descriptor stores it, and a
 * second call with the same shapes and another scale must not reuse the first one's. */
__INFINI_C __export infiniStatus_t infinicoreOpPlanPagedAttention(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *out, const infinicoreTensorView_t *q,
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *block_tables, const infinicoreTensorView_t *cache_lens,
    const infinicoreTensorView_t *alibi_slopes, float scale);
/* paged_attention_prefill_infiniop.cc:18-66 (the reference has `calculate` only; the plan form is the
 * same three steps). */
__INFINI_C __export infiniStatus_t infinicoreOpPlanPagedAttentionPrefill(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *out, const infinicoreTensorView_t *q,
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *block_tables, const infinicoreTensorView_t *total_kv_lens,
    const infinicoreTensorView_t *cum_seqlens_q, const infinicoreTensorView_t *alibi_slopes, float scale);
/* paged_caching_infiniop.cc:15-33 */
__INFINI_C __export infiniStatus_t infinicoreOpPlanPagedCaching(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *k, const infinicoreTensorView_t *v, const infinicoreTensorView_t *slot_mapping);
/* kv_caching_infiniop.cc:13-40 */
__INFINI_C __export infiniStatus_t infinicoreOpPlanKVCaching(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *k, const infinicoreTensorView_t *v, const infinicoreTensorView_t *past_kv_lengths);

/* ---- run (paged_attention_infiniop.cc:48-63): one InfiniOP call on `stream`; allocates nothing, so it
 *      may be recorded into a captured graph. Runs of one plan share its workspace: order them on one
 *      stream (or by events). The calling thread's current InfiniRT device must be the one the plan was
 *      made on, else INFINI_STATUS_BAD_PARAM. ---- */
__INFINI_C __export infiniStatus_t infinicoreOpRun(infinicorePlannedOp_t plan, infinirtStream_t stream);
/* ---- cleanup (paged_attention_infiniop.cc:65-68): frees the plan's workspace (which waits for the
 *      device), drops its reference to the descriptor, sets *plan_ptr to NULL. ---- */
__INFINI_C __export infiniStatus_t infinicoreOpCleanup(infinicorePlannedOp_t *plan_ptr);
/* Bytes of the plan's workspace (what infiniopGet...WorkspaceSize returned at plan time). */
__INFINI_C __export infiniStatus_t infinicoreOpPlannedWorkspaceSize(infinicorePlannedOp_t plan, size_t *size);

/* ---- immediate forms: `infinicore::op::paged_attention_` and friends
 *      (src/infinicore/ops/paged_attention/paged_attention.cc:38-42). Descriptor from the same cache;
 *      the workspace is the calling thread's buffer for (device, stream), which grows to the largest
 *      size asked for and is reused by every later immediate call on that stream (calls on one stream
 *      are ordered, so they can share it). Growing it allocates: not under stream capture. ---- */
__INFINI_C __export infiniStatus_t infinicoreOpPagedAttention(
    const infinicoreTensorView_t *out, const infinicoreTensorView_t *q, const infinicoreTensorView_t *k_cache,
    const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *block_tables,
    const infinicoreTensorView_t *cache_lens, const infinicoreTensorView_t *alibi_slopes, float scale,
    infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinicoreOpPagedAttentionPrefill(
    const infinicoreTensorView_t *out, const infinicoreTensorView_t *q, const infinicoreTensorView_t *k_cache,
    const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *block_tables,
    const infinicoreTensorView_t *total_kv_lens, const infinicoreTensorView_t *cum_seqlens_q,
    const infinicoreTensorView_t *alibi_slopes, float scale, infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinicoreOpPagedCaching(
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
    const infinicoreTensorView_t *v, const infinicoreTensorView_t *slot_mapping, infinirtStream_t stream);
__INFINI_C __export infiniStatus_t infinicoreOpKVCaching(
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
    const infinicoreTensorView_t *v, const infinicoreTensorView_t *past_kv_lengths, infinirtStream_t stream);

/* ---- the calling thread's descriptor caches (include/infinicore/ops/common/cache.hpp:37-69) ---- */
/* Capacity of every cache of this thread, existing and future (OpCache::setCapacity); shrinking evicts
 * from the least recently used end. 0 means unbounded, as in the reference's LRUCache
 * (include/infinicore/common/LRUCache.hpp:19-24). */
__INFINI_C __export infiniStatus_t infinicoreOpCacheSetCapacity(size_t capacity);
/* Entries held, hits and misses of one operator's cache on the current device. Any pointer may be NULL. */
__INFINI_C __export infiniStatus_t infinicoreOpCacheStats(infinicoreOpKind_t kind, size_t *entries, uint64_t *hits,
                                                         uint64_t *misses);
/* Destroys every cached descriptor no plan refers to any more (OpCache::clear), the thread's immediate
 * workspaces and its InfiniOP handles; plans stay valid. */
__INFINI_C __export infiniStatus_t infinicoreOpCacheClear(void);

#endif /* INFINICORE_AMD_INFINICORE_OPS_H */
