// C entry points of paged_caching: pick the backend from the handle's / descriptor's device type.
// Replaces the reference's src/infiniop/ops/paged_caching/operator.cc:21-197; the only backend in
// this build is amd, every other device type answers DEVICE_TYPE_NOT_SUPPORTED.
#include "../../handle.h"
#include "../../operator.h"
#include "amd/paged_caching_amd.h"
#include "infiniop/ops/paged_caching.h"

using AmdDescriptor = op::paged_caching::amd::Descriptor;

__INFINI_C infiniStatus_t infiniopCreatePagedCachingDescriptor(infiniopHandle_t handle,
                                                               infiniopPagedCachingDescriptor_t *desc_ptr,
                                                               infiniopTensorDescriptor_t k_cache_desc,
                                                               infiniopTensorDescriptor_t v_cache_desc,
                                                               infiniopTensorDescriptor_t k_desc,
                                                               infiniopTensorDescriptor_t v_desc,
                                                               infiniopTensorDescriptor_t slot_mapping_desc) {
    if (handle == nullptr || desc_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (handle->device) {
    case INFINI_DEVICE_AMD:
        return AmdDescriptor::create(handle, reinterpret_cast<AmdDescriptor **>(desc_ptr), k_cache_desc, v_cache_desc,
                                     k_desc, v_desc, slot_mapping_desc);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopGetPagedCachingWorkspaceSize(infiniopPagedCachingDescriptor_t desc, size_t *size) {
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

__INFINI_C infiniStatus_t infiniopPagedCaching(infiniopPagedCachingDescriptor_t desc, void *workspace,
                                               size_t workspace_size, void *k_cache, void *v_cache, const void *k,
                                               const void *v, const void *slot_mapping, void *stream) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        return reinterpret_cast<AmdDescriptor *>(desc)->calculate(workspace, workspace_size, k_cache, v_cache, k, v,
                                                                  slot_mapping, stream);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopDestroyPagedCachingDescriptor(infiniopPagedCachingDescriptor_t desc) {
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
