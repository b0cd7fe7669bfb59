// C entry points of paged_attention: pick the backend from the handle's / descriptor's device type.
// Replaces the reference's src/infiniop/ops/paged_attention/operator.cc:21-190; the only backend in
// this build is amd, every other device type answers DEVICE_TYPE_NOT_SUPPORTED.
#include "../../handle.h"
#include "../../operator.h"
#include "amd/paged_attention_amd.h"
#include "infiniop/ops/paged_attention.h"

using AmdDescriptor = op::paged_attention::amd::Descriptor;

__INFINI_C infiniStatus_t infiniopCreatePagedAttentionDescriptor(infiniopHandle_t handle,
                                                                 infiniopPagedAttentionDescriptor_t *desc_ptr,
                                                                 infiniopTensorDescriptor_t out_desc,
                                                                 infiniopTensorDescriptor_t q_desc,
                                                                 infiniopTensorDescriptor_t k_cache_desc,
                                                                 infiniopTensorDescriptor_t v_cache_desc,
                                                                 infiniopTensorDescriptor_t block_tables_desc,
                                                                 infiniopTensorDescriptor_t seq_lens_desc,
                                                                 infiniopTensorDescriptor_t alibi_slopes_desc,
                                                                 float scale) {
    if (handle == nullptr || desc_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (handle->device) {
    case INFINI_DEVICE_AMD:
        return AmdDescriptor::create(handle, reinterpret_cast<AmdDescriptor **>(desc_ptr), out_desc, q_desc,
                                     k_cache_desc, v_cache_desc, block_tables_desc, seq_lens_desc, alibi_slopes_desc,
                                     scale);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopGetPagedAttentionWorkspaceSize(infiniopPagedAttentionDescriptor_t desc, size_t *size) {
    if (desc == nullptr || size == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        *size = reinterpret_cast<AmdDescriptor *>(desc)->workspaceSize();
        return INFINI_STATUS_SUCCESS;
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopPagedAttention(infiniopPagedAttentionDescriptor_t desc, void *workspace,
                                                 size_t workspace_size, void *out, const void *q, const void *k_cache,
                                                 const void *v_cache, const void *block_tables, const void *seq_lens,
                                                 const void *alibi_slopes, void *stream) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        return reinterpret_cast<AmdDescriptor *>(desc)->calculate(workspace, workspace_size, out, q, k_cache, v_cache,
                                                                  block_tables, seq_lens, alibi_slopes, stream);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopPagedAttentionNoAlloc(infiniopPagedAttentionDescriptor_t desc, void *out, const void *q,
                                                        const void *k_cache, const void *v_cache,
                                                        const void *block_tables, const void *seq_lens,
                                                        const void *alibi_slopes, void *stream) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        return reinterpret_cast<AmdDescriptor *>(desc)->calculateNoAlloc(out, q, k_cache, v_cache, block_tables,
                                                                         seq_lens, alibi_slopes, stream);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopDestroyPagedAttentionDescriptor(infiniopPagedAttentionDescriptor_t desc) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        delete reinterpret_cast<AmdDescriptor *>(desc);
        return INFINI_STATUS_SUCCESS;
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}
