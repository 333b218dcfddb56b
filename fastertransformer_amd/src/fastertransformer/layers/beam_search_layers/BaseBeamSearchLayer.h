// One beam-search step on the logits of a window of the batch: penalties, the step itself (left to the derived
// class), the key / value cache indirection of the surviving beams. Public surface of the reference's
// src/fastertransformer/layers/beam_search_layers/BaseBeamSearchLayer.h:27-71.
#pragma once
#include "src/fastertransformer/kernels/sampling_kernels.h"
#include "src/fastertransformer/layers/DynamicDecodeBaseLayer.h"

namespace fastertransformer {

template<typename T>
class BaseBeamSearchLayer: public DynamicDecodeBaseLayer {
protected:
    size_t vocab_size_;
    size_t vocab_size_padded_;

    size_t topk_softmax_workspace_size_ = 0;  // bytes
    void*  topk_softmax_workspace_      = nullptr;

    void         allocateBuffer() override;
    virtual void allocateBuffer(size_t batch_size, size_t beam_width) = 0;
    void         freeBuffer() override;

    virtual void invokeSoftMax(TensorMap* output_tensors, TensorMap* input_tensors) = 0;

public:
    BaseBeamSearchLayer(size_t max_batch_size, size_t head_num, size_t size_per_head, size_t beam_width,
                        size_t vocab_size, size_t vocab_size_padded, int end_id, float diversity_rate,
                        float temperature, float len_penalty, float repetition_penalty, hipStream_t stream,
                        cublasMMWrapper* cublas_wrapper, IAllocator* allocator, bool is_free_buffer_after_forward);
    BaseBeamSearchLayer(BaseBeamSearchLayer<T> const& beam_search_layer);
    ~BaseBeamSearchLayer() override;

    void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args) override;
    void forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors) override;
    void forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                 const std::unordered_map<std::string, Tensor>* input_tensors) override;
    void forward(TensorMap* output_tensors, TensorMap* input_tensors) override;
};

}  // namespace fastertransformer
