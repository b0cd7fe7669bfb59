// Shape of a backend descriptor class for paged_attention. A backend instantiates it in its own
// namespace with DESCRIPTOR(ns) and defines create/calculate/~Descriptor (same pattern as the
// reference's src/infiniop/ops/paged_attention/paged_attention.h:7-51).
#ifndef INFINICORE_AMD_PAGED_ATTENTION_H
#define INFINICORE_AMD_PAGED_ATTENTION_H

#include "../../operator.h"
#include "info.h"

#define DESCRIPTOR(NAMESPACE)                                                                                \
    namespace op::paged_attention::NAMESPACE {                                                               \
    class Descriptor final : public InfiniopDescriptor {                                                     \
        struct Opaque;                                                                                       \
        Opaque *_opaque;                                                                                     \
        PagedAttentionInfo _info;                                                                            \
        size_t _workspace_size;                                                                              \
                                                                                                             \
        Descriptor(Opaque *opaque, const PagedAttentionInfo &info, size_t workspace_size,                    \
                   infiniDevice_t device_type, int device_id)                                                \
            : InfiniopDescriptor{device_type, device_id}, _opaque(opaque), _info(info),                      \
              _workspace_size(workspace_size) {}                                                             \
                                                                                                             \
    public:                                                                                                  \
        ~Descriptor();                                                                                       \
        size_t workspaceSize() const { return _workspace_size; }                                             \
        static infiniStatus_t create(infiniopHandle_t handle, Descriptor **desc_ptr,                         \
                                     infiniopTensorDescriptor_t out_desc, infiniopTensorDescriptor_t q_desc, \
                                     infiniopTensorDescriptor_t k_cache_desc,                                \
                                     infiniopTensorDescriptor_t v_cache_desc,                                \
                                     infiniopTensorDescriptor_t block_tables_desc,                           \
                                     infiniopTensorDescriptor_t seq_lens_desc,                               \
                                     infiniopTensorDescriptor_t alibi_slopes_desc, float scale);             \
        infiniStatus_t calculate(void *workspace, size_t workspace_size, void *out, const void *q,           \
                                 const void *k_cache, const void *v_cache, const void *block_tables,         \
                                 const void *seq_lens, const void *alibi_slopes, void *stream) const;        \
        /* same call with the partial results in the library's own per-device scratch array */               \
        infiniStatus_t calculateNoAlloc(void *out, const void *q, const void *k_cache, const void *v_cache,  \
                                        const void *block_tables, const void *seq_lens,                      \
                                        const void *alibi_slopes, void *stream) const;                       \
                                                                                                             \
    private:                                                                                                 \
        infiniStatus_t launch(void *workspace, void *out, const void *q, const void *k_cache,                \
                              const void *v_cache, const void *block_tables, const void *seq_lens,           \
                              const void *alibi_slopes, void *stream) const;                                 \
    };                                                                                                       \
    }

#endif
