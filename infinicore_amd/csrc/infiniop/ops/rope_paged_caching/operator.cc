// C entry points of the fused rotary-embedding + paged_caching operator: pick the backend from the handle's /
// descriptor's device type. The reference has the two halves as separate operators
// (src/infiniop/ops/rope/operator.cc, src/infiniop/ops/paged_caching/operator.cc:21-197); the only backend of
// the fused one is amd, every other device type answers DEVICE_TYPE_NOT_SUPPORTED.
#include "../../handle.h"
#include "../../operator.h"
#include "amd/rope_paged_caching_amd.h"
#include "infiniop/ops/rope_paged_caching.h"

using AmdDescriptor = op::rope_paged_caching::amd::Descriptor;

__INFINI_C infiniStatus_t infiniopCreateRoPEPagedCachingDescriptor(
    infiniopHandle_t handle, infiniopRoPEPagedCachingDescriptor_t *desc_ptr, infiniopTensorDescriptor_t k_cache_desc,
    infiniopTensorDescriptor_t v_cache_desc, infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc,
    infiniopTensorDescriptor_t slot_mapping_desc, infiniopTensorDescriptor_t pos_ids_desc,
    infiniopTensorDescriptor_t sin_table_desc, infiniopTensorDescriptor_t cos_table_desc, infiniopRoPEAlgo_t algo) {
    if (handle == nullptr || desc_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (handle->device) {
    case INFINI_DEVICE_AMD:
        return AmdDescriptor::create(handle, reinterpret_cast<AmdDescriptor **>(desc_ptr), k_cache_desc, v_cache_desc,
                                     k_desc, v_desc, slot_mapping_desc, pos_ids_desc, sin_table_desc, cos_table_desc, algo,
                                     false, nullptr, nullptr);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopCreateRoPEQKPagedCachingDescriptor(
    infiniopHandle_t handle, infiniopRoPEPagedCachingDescriptor_t *desc_ptr, infiniopTensorDescriptor_t q_out_desc,
    infiniopTensorDescriptor_t q_desc, infiniopTensorDescriptor_t k_cache_desc, infiniopTensorDescriptor_t v_cache_desc,
    infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc, infiniopTensorDescriptor_t slot_mapping_desc,
    infiniopTensorDescriptor_t pos_ids_desc, infiniopTensorDescriptor_t sin_table_desc,
    infiniopTensorDescriptor_t cos_table_desc, infiniopRoPEAlgo_t algo) {
    if (handle == nullptr || desc_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (handle->device) {
    case INFINI_DEVICE_AMD:
        return AmdDescriptor::create(handle, reinterpret_cast<AmdDescriptor **>(desc_ptr), k_cache_desc, v_cache_desc,
                                     k_desc, v_desc, slot_mapping_desc, pos_ids_desc, sin_table_desc, cos_table_desc, algo,
                                     true, q_out_desc, q_desc);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopGetRoPEPagedCachingWorkspaceSize(infiniopRoPEPagedCachingDescriptor_t desc, size_t *size) {
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

__INFINI_C infiniStatus_t infiniopRoPEPagedCaching(infiniopRoPEPagedCachingDescriptor_t desc, void *workspace,
                                                   size_t workspace_size, void *k_cache, void *v_cache, const void *k,
                                                   const void *v, const void *slot_mapping, const void *pos_ids,
                                                   const void *sin_table, const void *cos_table, void *stream) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        if (reinterpret_cast<AmdDescriptor *>(desc)->hasQuery()) {
            return INFINI_STATUS_BAD_PARAM; // created with a query: run it with infiniopRoPEQKPagedCaching
        }
        return reinterpret_cast<AmdDescriptor *>(desc)->calculate(workspace, workspace_size, nullptr, nullptr, k_cache,
                                                                  v_cache, k, v, slot_mapping, pos_ids, sin_table,
                                                                  cos_table, stream);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopRoPEQKPagedCaching(infiniopRoPEPagedCachingDescriptor_t desc, void *workspace,
                                                     size_t workspace_size, void *q_out, const void *q, void *k_cache,
                                                     void *v_cache, const void *k, const void *v, const void *slot_mapping,
                                                     const void *pos_ids, const void *sin_table, const void *cos_table,
                                                     void *stream) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        if (!reinterpret_cast<AmdDescriptor *>(desc)->hasQuery()) {
            return INFINI_STATUS_BAD_PARAM; // created without a query: run it with infiniopRoPEPagedCaching
        }
        return reinterpret_cast<AmdDescriptor *>(desc)->calculate(workspace, workspace_size, q_out, q, k_cache, v_cache, k,
                                                                  v, slot_mapping, pos_ids, sin_table, cos_table, stream);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopDestroyRoPEPagedCachingDescriptor(infiniopRoPEPagedCachingDescriptor_t desc) {
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
