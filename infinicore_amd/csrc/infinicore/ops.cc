// Framework-side adaptors of the paged operators over the InfiniOP C API: tensor views -> tensor
// descriptors -> cached operator descriptor -> workspace -> one operator call. What each step replaces
// in the reference is cited at its prototype in include/infinicore_ops.h.
#include "infinicore_ops.h"

#include "infiniop.h"
#include "lru_cache.h"

#include <array>
#include <functional>
#include <map>
#include <memory>
#include <tuple>
#include <utility>
#include <vector>

namespace {

using infinicore_amd::LruCache;
using infinicore_amd::MetaKey;
using infinicore_amd::MetaKeyHash;

#define RETURN_IF_ERROR(expr)                       \
    do {                                            \
        infiniStatus_t status__ = (expr);           \
        if (status__ != INFINI_STATUS_SUCCESS) {    \
            return status__;                        \
        }                                           \
    } while (0)

// An operator descriptor owned by the cache and by every plan made from it; destroyed with the last owner
// (the reference's movable Descriptor wrapper, src/infinicore/ops/infiniop_impl.hpp:8-45).
struct Descriptor {
    InfiniopDescriptor *desc = nullptr;
    infiniStatus_t (*destroy)(InfiniopDescriptor *) = nullptr;
    size_t workspace_bytes = 0;

    Descriptor() = default;
    Descriptor(const Descriptor &) = delete;
    Descriptor &operator=(const Descriptor &) = delete;
    ~Descriptor() {
        if (desc != nullptr) {
            destroy(desc); // host memory only: safe at thread and process exit
        }
    }
};

// A tensor descriptor that lives for one create call (the operator descriptor copies what it needs).
class ScopedTensorDescriptor {
public:
    ScopedTensorDescriptor() = default;
    ScopedTensorDescriptor(const ScopedTensorDescriptor &) = delete;
    ScopedTensorDescriptor &operator=(const ScopedTensorDescriptor &) = delete;
    ~ScopedTensorDescriptor() {
        if (desc_ != nullptr) {
            infiniopDestroyTensorDescriptor(desc_);
        }
    }
    infiniStatus_t describe(const infinicoreTensorView_t *view) {
        if (view == nullptr) {
            return INFINI_STATUS_SUCCESS; // an absent optional tensor is passed on as a null descriptor
        }
        return infiniopCreateTensorDescriptor(&desc_, view->ndim, view->shape, view->strides, view->dtype);
    }
    infiniopTensorDescriptor_t get() const { return desc_; }

private:
    infiniopTensorDescriptor_t desc_ = nullptr;
};

using DescriptorCache = LruCache<MetaKey, std::shared_ptr<Descriptor>, MetaKeyHash>;

struct Workspace {
    void *ptr = nullptr;
    size_t bytes = 0;
};

// Everything the adaptors keep is per thread, as the reference's `thread_local OpCache` is
// (infiniop_impl.hpp:47-52): no locks, and a descriptor never crosses threads through the cache.
struct ThreadState {
    using DeviceKey = std::pair<int, int>; // (device type, device id)
    size_t capacity = 100;
    // one cache per operator and device (the reference's OpCache::getCache, cache.hpp:27-41)
    std::array<std::map<DeviceKey, std::unique_ptr<DescriptorCache>>, INFINICORE_OP_KIND_COUNT> caches;
    std::map<DeviceKey, infiniopHandle_t> handles;
    std::map<std::tuple<int, int, infinirtStream_t>, Workspace> arenas; // immediate calls: (device type, id, stream)

    DescriptorCache &cache(infinicoreOpKind_t kind, infiniDevice_t device, int device_id) {
        auto &slot = caches[kind][{static_cast<int>(device), device_id}];
        if (!slot) {
            slot = std::make_unique<DescriptorCache>(capacity);
        }
        return *slot;
    }

    infiniStatus_t handle(infiniDevice_t device, int device_id, infiniopHandle_t *handle_ptr) {
        infiniopHandle_t &slot = handles[{static_cast<int>(device), device_id}];
        if (slot == nullptr) {
            RETURN_IF_ERROR(infiniopCreateHandle(&slot)); // records the current device, which is (device, id)
        }
        *handle_ptr = slot;
        return INFINI_STATUS_SUCCESS;
    }

    // Device memory is deliberately not freed here: at thread or process exit the device runtime may be
    // gone already. infinicoreOpCacheClear() frees it while the runtime is alive.
    ~ThreadState() {
        for (auto &entry : handles) {
            if (entry.second != nullptr) {
                infiniopDestroyHandle(entry.second);
            }
        }
    }
};

ThreadState &state() {
    thread_local ThreadState s;
    return s;
}

infiniStatus_t currentDevice(infiniDevice_t *device, int *device_id) {
    RETURN_IF_ERROR(infinirtGetDevice(device, device_id));
    // CPU handles exist, and InfiniOP answers DEVICE_TYPE_NOT_SUPPORTED for them at create time, as the
    // reference's operator switch does: nothing to special-case here.
    return INFINI_STATUS_SUCCESS;
}

bool validView(const infinicoreTensorView_t *view) {
    return view != nullptr && (view->ndim == 0 || view->shape != nullptr);
}

void addView(MetaKey &key, const infinicoreTensorView_t *view) {
    key.addTensor(view->dtype, view->ndim, view->shape, view->strides);
}

void addOptionalView(MetaKey &key, const infinicoreTensorView_t *view) {
    key.add(view != nullptr); // include/infinicore/common/hash.hpp:35-40
    if (view != nullptr) {
        addView(key, view);
    }
}

void addScale(MetaKey &key, float scale) {
    union {
        float f;
        uint32_t u;
    } bits{scale};
    key.add(bits.u);
}

using CreateFn = std::function<infiniStatus_t(infiniopHandle_t, InfiniopDescriptor **)>;
using WorkspaceSizeFn = infiniStatus_t (*)(InfiniopDescriptor *, size_t *);
using DestroyFn = infiniStatus_t (*)(InfiniopDescriptor *);
using CallFn = std::function<infiniStatus_t(InfiniopDescriptor *, void *, size_t, infinirtStream_t)>;

// INFINIOP_CACHABLE_DESCRIPTOR_GET_OR_CREATE (infiniop_impl.hpp:54-66)
infiniStatus_t getOrCreate(infinicoreOpKind_t kind, const MetaKey &key, const CreateFn &create,
                           WorkspaceSizeFn workspace_size, DestroyFn destroy, infiniDevice_t *device_out,
                           int *device_id_out, std::shared_ptr<Descriptor> *out) {
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    RETURN_IF_ERROR(currentDevice(&device, &device_id));
    ThreadState &s = state();
    DescriptorCache &cache = s.cache(kind, device, device_id);
    std::shared_ptr<Descriptor> descriptor = cache.get(key).value_or(nullptr);
    if (!descriptor) {
        infiniopHandle_t handle = nullptr;
        RETURN_IF_ERROR(s.handle(device, device_id, &handle));
        descriptor = std::make_shared<Descriptor>();
        descriptor->destroy = destroy;
        RETURN_IF_ERROR(create(handle, &descriptor->desc));
        RETURN_IF_ERROR(workspace_size(descriptor->desc, &descriptor->workspace_bytes));
        cache.put(key, descriptor);
    }
    *device_out = device;
    *device_id_out = device_id;
    *out = std::move(descriptor);
    return INFINI_STATUS_SUCCESS;
}

} // namespace

struct InfinicorePlannedOp {
    std::shared_ptr<Descriptor> descriptor;
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    Workspace workspace;
    CallFn call; // holds the tensors' data pointers
};

namespace {

// plan = descriptor + a workspace of the plan's own (INFINIOP_WORKSPACE_TENSOR, infiniop_impl.hpp:68-76)
infiniStatus_t makePlan(infinicorePlannedOp_t *plan_ptr, std::shared_ptr<Descriptor> descriptor, infiniDevice_t device,
                        int device_id, CallFn call) {
    auto plan = std::make_unique<InfinicorePlannedOp>();
    if (descriptor->workspace_bytes != 0) {
        RETURN_IF_ERROR(infinirtMalloc(&plan->workspace.ptr, descriptor->workspace_bytes));
        plan->workspace.bytes = descriptor->workspace_bytes;
    }
    plan->descriptor = std::move(descriptor);
    plan->device = device;
    plan->device_id = device_id;
    plan->call = std::move(call);
    *plan_ptr = plan.release();
    return INFINI_STATUS_SUCCESS;
}

// immediate call: the thread's workspace for (device, stream), grown when a descriptor asks for more
infiniStatus_t runImmediate(const std::shared_ptr<Descriptor> &descriptor, infiniDevice_t device, int device_id,
                            const CallFn &call, infinirtStream_t stream) {
    Workspace &arena = state().arenas[{static_cast<int>(device), device_id, stream}];
    if (arena.bytes < descriptor->workspace_bytes) {
        if (arena.ptr != nullptr) {
            RETURN_IF_ERROR(infinirtFree(arena.ptr)); // waits for the device: earlier calls are done with it
            arena = Workspace{};
        }
        RETURN_IF_ERROR(infinirtMalloc(&arena.ptr, descriptor->workspace_bytes));
        arena.bytes = descriptor->workspace_bytes;
    }
    // the operator gets the size it asked for, not the arena's: its launch plan may depend on the size
    return call(descriptor->desc, descriptor->workspace_bytes ? arena.ptr : nullptr, descriptor->workspace_bytes, stream);
}

struct Prepared {
    std::shared_ptr<Descriptor> descriptor;
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    CallFn call;
};

infiniStatus_t preparePagedAttention(Prepared *p, const infinicoreTensorView_t *out, const infinicoreTensorView_t *q,
                                     const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
                                     const infinicoreTensorView_t *block_tables, const infinicoreTensorView_t *cache_lens,
                                     const infinicoreTensorView_t *alibi_slopes, float scale) {
    if (!validView(out) || !validView(q) || !validView(k_cache) || !validView(v_cache) || !validView(block_tables)
        || !validView(cache_lens) || (alibi_slopes != nullptr && !validView(alibi_slopes))) {
        return INFINI_STATUS_NULL_POINTER;
    }
    MetaKey key;
    for (const auto *view : {out, q, k_cache, v_cache, block_tables, cache_lens}) {
        addView(key, view);
    }
    addOptionalView(key, alibi_slopes);
    addScale(key, scale);
    auto create = [&](infiniopHandle_t handle, InfiniopDescriptor **desc) -> infiniStatus_t {
        ScopedTensorDescriptor d[7];
        const infinicoreTensorView_t *views[7] = {out, q, k_cache, v_cache, block_tables, cache_lens, alibi_slopes};
        for (int i = 0; i < 7; ++i) {
            RETURN_IF_ERROR(d[i].describe(views[i]));
        }
        return infiniopCreatePagedAttentionDescriptor(handle, desc, d[0].get(), d[1].get(), d[2].get(), d[3].get(),
                                                      d[4].get(), d[5].get(), d[6].get(), scale);
    };
    RETURN_IF_ERROR(getOrCreate(INFINICORE_OP_PAGED_ATTENTION, key, create, infiniopGetPagedAttentionWorkspaceSize,
                                infiniopDestroyPagedAttentionDescriptor, &p->device, &p->device_id, &p->descriptor));
    void *o = out->data, *qd = q->data, *k = k_cache->data, *v = v_cache->data, *bt = block_tables->data,
         *cl = cache_lens->data, *al = alibi_slopes ? alibi_slopes->data : nullptr;
    p->call = [=](InfiniopDescriptor *desc, void *ws, size_t ws_bytes, infinirtStream_t stream) {
        return infiniopPagedAttention(desc, ws, ws_bytes, o, qd, k, v, bt, cl, al, stream);
    };
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t preparePagedAttentionPrefill(Prepared *p, const infinicoreTensorView_t *out,
                                            const infinicoreTensorView_t *q, const infinicoreTensorView_t *k_cache,
                                            const infinicoreTensorView_t *v_cache,
                                            const infinicoreTensorView_t *block_tables,
                                            const infinicoreTensorView_t *total_kv_lens,
                                            const infinicoreTensorView_t *cum_seqlens_q,
                                            const infinicoreTensorView_t *alibi_slopes, float scale) {
    if (!validView(out) || !validView(q) || !validView(k_cache) || !validView(v_cache) || !validView(block_tables)
        || !validView(total_kv_lens) || !validView(cum_seqlens_q)
        || (alibi_slopes != nullptr && !validView(alibi_slopes))) {
        return INFINI_STATUS_NULL_POINTER;
    }
    MetaKey key;
    for (const auto *view : {out, q, k_cache, v_cache, block_tables, total_kv_lens, cum_seqlens_q}) {
        addView(key, view);
    }
    addOptionalView(key, alibi_slopes);
    addScale(key, scale);
    auto create = [&](infiniopHandle_t handle, InfiniopDescriptor **desc) -> infiniStatus_t {
        ScopedTensorDescriptor d[8];
        const infinicoreTensorView_t *views[8] = {out, q, k_cache, v_cache, block_tables, total_kv_lens,
                                                  cum_seqlens_q, alibi_slopes};
        for (int i = 0; i < 8; ++i) {
            RETURN_IF_ERROR(d[i].describe(views[i]));
        }
        return infiniopCreatePagedAttentionPrefillDescriptor(handle, desc, d[0].get(), d[1].get(), d[2].get(),
                                                             d[3].get(), d[4].get(), d[5].get(), d[6].get(),
                                                             d[7].get(), scale);
    };
    RETURN_IF_ERROR(getOrCreate(INFINICORE_OP_PAGED_ATTENTION_PREFILL, key, create,
                                infiniopGetPagedAttentionPrefillWorkspaceSize,
                                infiniopDestroyPagedAttentionPrefillDescriptor, &p->device, &p->device_id, &p->descriptor));
    void *o = out->data, *qd = q->data, *k = k_cache->data, *v = v_cache->data, *bt = block_tables->data,
         *sl = total_kv_lens->data, *cu = cum_seqlens_q->data, *al = alibi_slopes ? alibi_slopes->data : nullptr;
    p->call = [=](InfiniopDescriptor *desc, void *ws, size_t ws_bytes, infinirtStream_t stream) {
        return infiniopPagedAttentionPrefill(desc, ws, ws_bytes, o, qd, k, v, bt, sl, cu, al, stream);
    };
    return INFINI_STATUS_SUCCESS;
}

// paged_caching and kv_caching share their shape: two caches, two sources, one index tensor
template <typename Create, typename Call>
infiniStatus_t prepareCaching(Prepared *p, infinicoreOpKind_t kind, const infinicoreTensorView_t *k_cache,
                              const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
                              const infinicoreTensorView_t *v, const infinicoreTensorView_t *index, Create create_op,
                              WorkspaceSizeFn workspace_size, DestroyFn destroy, Call call_op) {
    if (!validView(k_cache) || !validView(v_cache) || !validView(k) || !validView(v) || !validView(index)) {
        return INFINI_STATUS_NULL_POINTER;
    }
    MetaKey key;
    for (const auto *view : {k_cache, v_cache, k, v, index}) {
        addView(key, view);
    }
    auto create = [&](infiniopHandle_t handle, InfiniopDescriptor **desc) -> infiniStatus_t {
        ScopedTensorDescriptor d[5];
        const infinicoreTensorView_t *views[5] = {k_cache, v_cache, k, v, index};
        for (int i = 0; i < 5; ++i) {
            RETURN_IF_ERROR(d[i].describe(views[i]));
        }
        return create_op(handle, desc, d[0].get(), d[1].get(), d[2].get(), d[3].get(), d[4].get());
    };
    RETURN_IF_ERROR(getOrCreate(kind, key, create, workspace_size, destroy, &p->device, &p->device_id, &p->descriptor));
    void *kc = k_cache->data, *vc = v_cache->data, *kd = k->data, *vd = v->data, *ix = index->data;
    p->call = [=](InfiniopDescriptor *desc, void *ws, size_t ws_bytes, infinirtStream_t stream) {
        return call_op(desc, ws, ws_bytes, kc, vc, kd, vd, ix, stream);
    };
    return INFINI_STATUS_SUCCESS;
}

infiniStatus_t preparePagedCaching(Prepared *p, const infinicoreTensorView_t *k_cache,
                                   const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
                                   const infinicoreTensorView_t *v, const infinicoreTensorView_t *slot_mapping) {
    return prepareCaching(p, INFINICORE_OP_PAGED_CACHING, k_cache, v_cache, k, v, slot_mapping,
                          infiniopCreatePagedCachingDescriptor, infiniopGetPagedCachingWorkspaceSize,
                          infiniopDestroyPagedCachingDescriptor, infiniopPagedCaching);
}

infiniStatus_t prepareKVCaching(Prepared *p, const infinicoreTensorView_t *k_cache,
                                const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
                                const infinicoreTensorView_t *v, const infinicoreTensorView_t *past_kv_lengths) {
    return prepareCaching(p, INFINICORE_OP_KV_CACHING, k_cache, v_cache, k, v, past_kv_lengths,
                          infiniopCreateKVCachingDescriptor, infiniopGetKVCachingWorkspaceSize,
                          infiniopDestroyKVCachingDescriptor, infiniopKVCaching);
}

infiniStatus_t finishPlan(infinicorePlannedOp_t *plan_ptr, infiniStatus_t prepared, Prepared &p) {
    RETURN_IF_ERROR(prepared);
    return makePlan(plan_ptr, std::move(p.descriptor), p.device, p.device_id, std::move(p.call));
}

infiniStatus_t finishImmediate(infiniStatus_t prepared, const Prepared &p, infinirtStream_t stream) {
    RETURN_IF_ERROR(prepared);
    return runImmediate(p.descriptor, p.device, p.device_id, p.call, stream);
}

} // namespace

// ---------------------------------------------------------------------------------------------------------
// plan
// ---------------------------------------------------------------------------------------------------------
#define PLAN_PROLOGUE()                        \
    if (plan_ptr == nullptr) {                 \
        return INFINI_STATUS_NULL_POINTER;     \
    }                                          \
    *plan_ptr = nullptr;                       \
    Prepared p

__INFINI_C infiniStatus_t infinicoreOpPlanPagedAttention(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *out, const infinicoreTensorView_t *q,
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *block_tables, const infinicoreTensorView_t *cache_lens,
    const infinicoreTensorView_t *alibi_slopes, float scale) {
    PLAN_PROLOGUE();
    return finishPlan(plan_ptr,
                      preparePagedAttention(&p, out, q, k_cache, v_cache, block_tables, cache_lens, alibi_slopes, scale),
                      p);
}

__INFINI_C infiniStatus_t infinicoreOpPlanPagedAttentionPrefill(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *out, const infinicoreTensorView_t *q,
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *block_tables, const infinicoreTensorView_t *total_kv_lens,
    const infinicoreTensorView_t *cum_seqlens_q, const infinicoreTensorView_t *alibi_slopes, float scale) {
    PLAN_PROLOGUE();
    return finishPlan(plan_ptr,
                      preparePagedAttentionPrefill(&p, out, q, k_cache, v_cache, block_tables, total_kv_lens,
                                                   cum_seqlens_q, alibi_slopes, scale),
                      p);
}

__INFINI_C infiniStatus_t infinicoreOpPlanPagedCaching(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *k, const infinicoreTensorView_t *v, const infinicoreTensorView_t *slot_mapping) {
    PLAN_PROLOGUE();
    return finishPlan(plan_ptr, preparePagedCaching(&p, k_cache, v_cache, k, v, slot_mapping), p);
}

__INFINI_C infiniStatus_t infinicoreOpPlanKVCaching(
    infinicorePlannedOp_t *plan_ptr, const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache,
    const infinicoreTensorView_t *k, const infinicoreTensorView_t *v, const infinicoreTensorView_t *past_kv_lengths) {
    PLAN_PROLOGUE();
    return finishPlan(plan_ptr, prepareKVCaching(&p, k_cache, v_cache, k, v, past_kv_lengths), p);
}

// ---------------------------------------------------------------------------------------------------------
// run / cleanup
// ---------------------------------------------------------------------------------------------------------
__INFINI_C infiniStatus_t infinicoreOpRun(infinicorePlannedOp_t plan, infinirtStream_t stream) {
    if (plan == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    // the plan's workspace, tensors and stream belong to the device it was planned on: that device must be
    // the calling thread's current one (the reference's graph runs on the context's current device too)
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    RETURN_IF_ERROR(infinirtGetDevice(&device, &device_id));
    if (device != plan->device || device_id != plan->device_id) {
        return INFINI_STATUS_BAD_PARAM;
    }
    return plan->call(plan->descriptor->desc, plan->workspace.ptr, plan->workspace.bytes, stream);
}

__INFINI_C infiniStatus_t infinicoreOpCleanup(infinicorePlannedOp_t *plan_ptr) {
    if (plan_ptr == nullptr || *plan_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    std::unique_ptr<InfinicorePlannedOp> plan(*plan_ptr);
    *plan_ptr = nullptr;
    if (plan->workspace.ptr != nullptr) {
        RETURN_IF_ERROR(infinirtFree(plan->workspace.ptr));
    }
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infinicoreOpPlannedWorkspaceSize(infinicorePlannedOp_t plan, size_t *size) {
    if (plan == nullptr || size == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    *size = plan->workspace.bytes;
    return INFINI_STATUS_SUCCESS;
}

// ---------------------------------------------------------------------------------------------------------
// immediate
// ---------------------------------------------------------------------------------------------------------
__INFINI_C infiniStatus_t infinicoreOpPagedAttention(
    const infinicoreTensorView_t *out, const infinicoreTensorView_t *q, const infinicoreTensorView_t *k_cache,
    const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *block_tables,
    const infinicoreTensorView_t *cache_lens, const infinicoreTensorView_t *alibi_slopes, float scale,
    infinirtStream_t stream) {
    Prepared p;
    return finishImmediate(
        preparePagedAttention(&p, out, q, k_cache, v_cache, block_tables, cache_lens, alibi_slopes, scale), p, stream);
}

__INFINI_C infiniStatus_t infinicoreOpPagedAttentionPrefill(
    const infinicoreTensorView_t *out, const infinicoreTensorView_t *q, const infinicoreTensorView_t *k_cache,
    const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *block_tables,
    const infinicoreTensorView_t *total_kv_lens, const infinicoreTensorView_t *cum_seqlens_q,
    const infinicoreTensorView_t *alibi_slopes, float scale, infinirtStream_t stream) {
    Prepared p;
    return finishImmediate(preparePagedAttentionPrefill(&p, out, q, k_cache, v_cache, block_tables, total_kv_lens,
                                                        cum_seqlens_q, alibi_slopes, scale),
                           p, stream);
}

__INFINI_C infiniStatus_t infinicoreOpPagedCaching(
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
    const infinicoreTensorView_t *v, const infinicoreTensorView_t *slot_mapping, infinirtStream_t stream) {
    Prepared p;
    return finishImmediate(preparePagedCaching(&p, k_cache, v_cache, k, v, slot_mapping), p, stream);
}

__INFINI_C infiniStatus_t infinicoreOpKVCaching(
    const infinicoreTensorView_t *k_cache, const infinicoreTensorView_t *v_cache, const infinicoreTensorView_t *k,
    const infinicoreTensorView_t *v, const infinicoreTensorView_t *past_kv_lengths, infinirtStream_t stream) {
    Prepared p;
    return finishImmediate(prepareKVCaching(&p, k_cache, v_cache, k, v, past_kv_lengths), p, stream);
}

// ---------------------------------------------------------------------------------------------------------
// caches
// ---------------------------------------------------------------------------------------------------------
__INFINI_C infiniStatus_t infinicoreOpCacheSetCapacity(size_t capacity) {
    ThreadState &s = state();
    s.capacity = capacity;
    for (auto &by_device : s.caches) {
        for (auto &entry : by_device) {
            entry.second->setCapacity(capacity);
        }
    }
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infinicoreOpCacheStats(infinicoreOpKind_t kind, size_t *entries, uint64_t *hits,
                                                 uint64_t *misses) {
    if (kind < 0 || kind >= INFINICORE_OP_KIND_COUNT) {
        return INFINI_STATUS_BAD_PARAM;
    }
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    RETURN_IF_ERROR(currentDevice(&device, &device_id));
    DescriptorCache &cache = state().cache(kind, device, device_id);
    if (entries != nullptr) {
        *entries = cache.size();
    }
    if (hits != nullptr) {
        *hits = cache.hits();
    }
    if (misses != nullptr) {
        *misses = cache.misses();
    }
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infinicoreOpCacheClear(void) {
    ThreadState &s = state();
    for (auto &by_device : s.caches) {
        by_device.clear();
    }
    // The arenas belong to devices: make each one current to free its memory (OpCache::clear does the
    // same for descriptors, cache.hpp:54-76), then restore the caller's device.
    infiniDevice_t device = INFINI_DEVICE_CPU;
    int device_id = 0;
    RETURN_IF_ERROR(infinirtGetDevice(&device, &device_id));
    infiniStatus_t first_error = INFINI_STATUS_SUCCESS;
    for (auto &entry : s.arenas) {
        if (entry.second.ptr == nullptr) {
            continue;
        }
        infiniStatus_t status = infinirtSetDevice(static_cast<infiniDevice_t>(std::get<0>(entry.first)),
                                                  std::get<1>(entry.first));
        if (status == INFINI_STATUS_SUCCESS) {
            status = infinirtFree(entry.second.ptr);
        }
        if (status != INFINI_STATUS_SUCCESS && first_error == INFINI_STATUS_SUCCESS) {
            first_error = status;
        }
    }
    s.arenas.clear();
    RETURN_IF_ERROR(infinirtSetDevice(device, device_id));
    for (auto &entry : s.handles) {
        if (entry.second != nullptr) {
            infiniopDestroyHandle(entry.second);
        }
    }
    s.handles.clear();
    return first_error;
}
