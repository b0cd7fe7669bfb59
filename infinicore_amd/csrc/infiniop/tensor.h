// Tensor descriptor object: dtype + shape + element strides, nothing else
// (reference src/infiniop/tensor.h and tensor_descriptor.cc:31-83).
#ifndef INFINICORE_AMD_INFINIOP_TENSOR_IMPL_H
#define INFINICORE_AMD_INFINIOP_TENSOR_IMPL_H

#include "infiniop/tensor_descriptor.h"
#include <vector>

struct InfiniopTensorDescriptor {
    infiniDtype_t _dtype;
    std::vector<size_t> _shape;
    std::vector<ptrdiff_t> _strides;

    InfiniopTensorDescriptor(infiniDtype_t dtype, size_t ndim, const size_t *shape, const ptrdiff_t *strides)
        : _dtype(dtype), _shape(shape, shape + ndim), _strides(strides, strides + ndim) {}

    infiniDtype_t dtype() const { return _dtype; }
    size_t ndim() const { return _shape.size(); }
    const std::vector<size_t> &shape() const { return _shape; }
    size_t dim(size_t i) const { return _shape[i]; }
    const std::vector<ptrdiff_t> &strides() const { return _strides; }
    ptrdiff_t stride(size_t i) const { return _strides[i]; }
    // packed row-major strides (dimensions of extent 1 may carry any stride)
    bool isContiguous() const {
        ptrdiff_t expected = 1;
        for (size_t i = _shape.size(); i-- > 0;) {
            if (_shape[i] != 1 && _strides[i] != expected) {
                return false;
            }
            expected *= static_cast<ptrdiff_t>(_shape[i]);
        }
        return true;
    }
    size_t numel() const {
        size_t n = 1;
        for (size_t d : _shape) {
            n *= d;
        }
        return n;
    }
};

// Bytes per element of a dtype (0 for INVALID).
inline size_t infiniSizeOf(infiniDtype_t dtype) {
    switch (dtype) {
    case INFINI_DTYPE_BYTE: case INFINI_DTYPE_BOOL: case INFINI_DTYPE_I8: case INFINI_DTYPE_U8: case INFINI_DTYPE_F8:
        return 1;
    case INFINI_DTYPE_I16: case INFINI_DTYPE_U16: case INFINI_DTYPE_F16: case INFINI_DTYPE_BF16:
        return 2;
    case INFINI_DTYPE_I32: case INFINI_DTYPE_U32: case INFINI_DTYPE_F32: case INFINI_DTYPE_C16:
        return 4;
    case INFINI_DTYPE_I64: case INFINI_DTYPE_U64: case INFINI_DTYPE_F64: case INFINI_DTYPE_C32:
        return 8;
    case INFINI_DTYPE_C64:
        return 16;
    case INFINI_DTYPE_C128:
        return 32;
    default:
        return 0;
    }
}

#endif
