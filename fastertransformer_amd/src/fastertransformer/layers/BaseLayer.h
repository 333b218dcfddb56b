// Common base of the decode layers: stream, allocator and buffer-lifetime flags.
// Public surface of the reference's src/fastertransformer/layers/BaseLayer.h:26-66; the cuBLAS
// wrapper and device-properties pointers are kept as opaque, never-dereferenced arguments because
// the sampling path does not use them.
#pragma once
#include "src/fastertransformer/utils/Tensor.h"
#include "src/fastertransformer/utils/allocator.h"

namespace fastertransformer {

class cublasMMWrapper;   // opaque: accepted for signature compatibility, never dereferenced
struct cudaDeviceProp;   // opaque, same reason

class BaseLayer {
public:
    BaseLayer(hipStream_t stream, cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
              bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop = nullptr, bool sparse = false):
        stream_(stream),
        cublas_wrapper_(cublas_wrapper),
        allocator_(allocator),
        cuda_device_prop_(cuda_device_prop),
        is_free_buffer_after_forward_(is_free_buffer_after_forward),
        sparse_(sparse)
    {
    }
    virtual ~BaseLayer() = default;

    virtual hipStream_t getStream()
    {
        return stream_;
    }
    virtual void setStream(hipStream_t stream)
    {
        stream_ = stream;
    }

protected:
    virtual void allocateBuffer() = 0;
    virtual void freeBuffer()     = 0;

    hipStream_t      stream_;
    cublasMMWrapper* cublas_wrapper_;
    IAllocator*      allocator_;
    cudaDeviceProp*  cuda_device_prop_ = nullptr;
    bool             is_free_buffer_after_forward_;
    bool             is_allocate_buffer_ = false;
    bool             sparse_;
};

}  // namespace fastertransformer
