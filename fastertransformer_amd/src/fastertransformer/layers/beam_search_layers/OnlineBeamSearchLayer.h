// The beam-search step itself: log-softmax, candidates, hypotheses, the beams' bookkeeping. Public surface of the
// reference's src/fastertransformer/layers/beam_search_layers/OnlineBeamSearchLayer.h:24-64.
#pragma once
#include "src/fastertransformer/layers/beam_search_layers/BaseBeamSearchLayer.h"

namespace fastertransformer {

template<typename T>
class OnlineBeamSearchLayer: public BaseBeamSearchLayer<T> {
private:
    void allocateBuffer() override;
    void allocateBuffer(size_t batch_size, size_t beam_width) override;

    using BaseBeamSearchLayer<T>::vocab_size_;
    using BaseBeamSearchLayer<T>::vocab_size_padded_;
    using BaseBeamSearchLayer<T>::topk_softmax_workspace_size_;
    using BaseBeamSearchLayer<T>::topk_softmax_workspace_;
    using BaseBeamSearchLayer<T>::stream_;
    using BaseBeamSearchLayer<T>::allocator_;
    using BaseBeamSearchLayer<T>::is_allocate_buffer_;

protected:
    void invokeSoftMax(TensorMap* output_tensors, TensorMap* input_tensors) override;

public:
    OnlineBeamSearchLayer(size_t max_batch_size, size_t head_num, size_t size_per_head, size_t beam_width,
                          size_t vocab_size, size_t vocab_size_padded, int end_id, float diversity_rate,
                          float temperature, float len_penalty, float repetition_penalty, hipStream_t stream,
                          cublasMMWrapper* cublas_wrapper, IAllocator* allocator, bool is_free_buffer_after_forward);
    OnlineBeamSearchLayer(OnlineBeamSearchLayer<T> const& beam_search_layer);
    ~OnlineBeamSearchLayer() override;
};

}  // namespace fastertransformer
