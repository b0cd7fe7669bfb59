// C entry points of kv_caching: pick the backend from the handle's / descriptor's device type.
// Replaces the reference's src/infiniop/ops/kv_caching/operator.cc:12-176; the only backend in
// this build is amd, every other device type answers DEVICE_TYPE_NOT_SUPPORTED.
#include "../../handle.h"
#include "../../operator.h"
#include "amd/kv_caching_amd.h"
#include "infiniop/ops/kv_caching.h"

using AmdDescriptor = op::kv_caching::amd::Descriptor;

__INFINI_C infiniStatus_t infiniopCreateKVCachingDescriptor(infiniopHandle_t handle,
                                                               infiniopKVCachingDescriptor_t *desc_ptr,
                                                               infiniopTensorDescriptor_t k_cache_d,
                                                               infiniopTensorDescriptor_t v_cache_d,
                                                               infiniopTensorDescriptor_t k_d,
                                                               infiniopTensorDescriptor_t v_d,
                                                               infiniopTensorDescriptor_t past_kv_lengths) {
    if (handle == nullptr || desc_ptr == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (handle->device) {
    case INFINI_DEVICE_AMD:
        return AmdDescriptor::create(handle, reinterpret_cast<AmdDescriptor **>(desc_ptr), k_cache_d, v_cache_d,
                                     k_d, v_d, past_kv_lengths);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopGetKVCachingWorkspaceSize(infiniopKVCachingDescriptor_t desc, size_t *size) {
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

__INFINI_C infiniStatus_t infiniopKVCaching(infiniopKVCachingDescriptor_t desc, void *workspace,
                                               size_t workspace_size, void *k_cache, void *v_cache, const void *k,
                                               const void *v, const void *past_kv_lengths, void *stream) {
    if (desc == nullptr) {
        return INFINI_STATUS_NULL_POINTER;
    }
    switch (desc->device_type) {
    case INFINI_DEVICE_AMD:
        return reinterpret_cast<AmdDescriptor *>(desc)->calculate(workspace, workspace_size, k_cache, v_cache, k, v,
                                                                  past_kv_lengths, stream);
    default:
        return INFINI_STATUS_DEVICE_TYPE_NOT_SUPPORTED;
    }
}

__INFINI_C infiniStatus_t infiniopDestroyKVCachingDescriptor(infiniopKVCachingDescriptor_t desc) {
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
