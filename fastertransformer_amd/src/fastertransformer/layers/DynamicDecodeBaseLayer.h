// Interface shared by the per-step decode layers
// (reference: src/fastertransformer/layers/DynamicDecodeBaseLayer.h:25-47).
#pragma once
#include <string>
#include <unordered_map>

#include "src/fastertransformer/layers/BaseLayer.h"

namespace fastertransformer {

class DynamicDecodeBaseLayer: public BaseLayer {
public:
    DynamicDecodeBaseLayer(hipStream_t stream, cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                           bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop):
        BaseLayer(stream, cublas_wrapper, allocator, is_free_buffer_after_forward, cuda_device_prop)
    {
    }
    ~DynamicDecodeBaseLayer() override = default;
    DynamicDecodeBaseLayer(DynamicDecodeBaseLayer const& other): BaseLayer(other) {}

    virtual void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args) = 0;
    virtual void forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors) = 0;
    virtual void forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                         const std::unordered_map<std::string, Tensor>* input_tensors)           = 0;
    virtual void forward(TensorMap* output_tensors, TensorMap* input_tensors)                     = 0;
};

}  // namespace fastertransformer
