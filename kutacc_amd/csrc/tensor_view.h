// Non-owning strided tensor descriptor behind kutacc_tensor_h.
// Same information content as reference src/tensor/tensor.h:21-53 (data pointer, sizes, strides in
// elements, rank, dtype); a handle is a heap-allocated TensorView owned by a TensorWrapper.
#pragma once
#include <cstdint>
#include <vector>

#include "kutacc.h"

namespace kutacc {
struct TensorView {
    void *data = nullptr;
    std::vector<int64_t> sizes;
    std::vector<int64_t> strides;
    int64_t dim = 0;
    DType dtype = kBF16;

    int64_t numel() const
    {
        if (dim == 0) {
            return 0;
        }
        int64_t n = 1;
        for (int64_t i = 0; i < dim; ++i) {
            n *= sizes[(size_t)i];
        }
        return n;
    }
    int64_t size(int64_t i) const { return sizes[(size_t)i]; }
    int64_t stride(int64_t i) const { return strides[(size_t)i]; }
};

inline TensorView *as_view(kutacc_tensor_h h) { return static_cast<TensorView *>(h); }

inline size_t dtype_bytes(DType t)
{
    switch (t) {
        case kInt64: return 8;
        case kBF16: return 2;
        case kFP32: return 4;
        default: return 0;
    }
}
} // namespace kutacc
