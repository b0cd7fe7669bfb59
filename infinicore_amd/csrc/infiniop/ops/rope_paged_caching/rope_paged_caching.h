// Shape of a backend descriptor class for the fused rotary-embedding + paged_caching operator. A backend
// instantiates it in its own namespace with DESCRIPTOR(ns) and defines create/calculate/~Descriptor (the
// pattern of the reference's per-operator headers, e.g. src/infiniop/ops/paged_caching/paged_caching.h:7-47).
#ifndef INFINICORE_AMD_ROPE_PAGED_CACHING_H
#define INFINICORE_AMD_ROPE_PAGED_CACHING_H

#include "../../operator.h"
#include "info.h"

#define DESCRIPTOR(NAMESPACE)                                                                                   \
    namespace op::rope_paged_caching::NAMESPACE {                                                               \
    class Descriptor final : public InfiniopDescriptor {                                                        \
        struct Opaque;                                                                                          \
        Opaque *_opaque;                                                                                        \
        RoPEPagedCachingInfo _info;                                                                             \
        size_t _workspace_size;                                                                                 \
                                                                                                                \
        Descriptor(Opaque *opaque, const RoPEPagedCachingInfo &info, size_t workspace_size,                     \
                   infiniDevice_t device_type, int device_id)                                                   \
            : InfiniopDescriptor{device_type, device_id}, _opaque(opaque), _info(info),                         \
              _workspace_size(workspace_size) {}                                                                \
                                                                                                                \
    public:                                                                                                     \
        ~Descriptor();                                                                                          \
        size_t workspaceSize() const { return _workspace_size; }                                                \
        static infiniStatus_t create(infiniopHandle_t handle, Descriptor **desc_ptr,                            \
                                     infiniopTensorDescriptor_t k_cache_desc,                                   \
                                     infiniopTensorDescriptor_t v_cache_desc,                                   \
                                     infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc,      \
                                     infiniopTensorDescriptor_t slot_mapping_desc,                              \
                                     infiniopTensorDescriptor_t pos_ids_desc,                                   \
                                     infiniopTensorDescriptor_t sin_table_desc,                                 \
                                     infiniopTensorDescriptor_t cos_table_desc, infiniopRoPEAlgo_t algo,        \
                                     bool with_query, infiniopTensorDescriptor_t q_out_desc,                    \
                                     infiniopTensorDescriptor_t q_desc);                                        \
        bool hasQuery() const { return _info.has_query; }                                                       \
        /* q_out / q: used by descriptors created with a query only */                                          \
        infiniStatus_t calculate(void *workspace, size_t workspace_size, void *q_out, const void *q,            \
                                 void *k_cache, void *v_cache,                                                  \
                                 const void *k, const void *v, const void *slot_mapping, const void *pos_ids,   \
                                 const void *sin_table, const void *cos_table, void *stream) const;             \
    };                                                                                                          \
    }

#endif
