#include "tensor.h"

// strides == NULL means a C-contiguous tensor (reference src/infiniop/tensor_descriptor.cc:8-24).
__INFINI_C infiniStatus_t infiniopCreateTensorDescriptor(infiniopTensorDescriptor_t *desc_ptr, size_t ndim,
                                                         const size_t *shape, const ptrdiff_t *strides,
                                                         infiniDtype_t dtype) {
    if (desc_ptr == nullptr || (ndim > 0 && shape == nullptr)) {
        return INFINI_STATUS_NULL_POINTER;
    }
    if (strides != nullptr) {
        *desc_ptr = new InfiniopTensorDescriptor(dtype, ndim, shape, strides);
        return INFINI_STATUS_SUCCESS;
    }
    std::vector<ptrdiff_t> packed(ndim);
    ptrdiff_t running = 1;
    for (size_t i = ndim; i-- > 0;) {
        packed[i] = running;
        running *= static_cast<ptrdiff_t>(shape[i]);
    }
    *desc_ptr = new InfiniopTensorDescriptor(dtype, ndim, shape, packed.data());
    return INFINI_STATUS_SUCCESS;
}

__INFINI_C infiniStatus_t infiniopDestroyTensorDescriptor(infiniopTensorDescriptor_t desc) {
    delete desc;
    return INFINI_STATUS_SUCCESS;
}
