// Top-k (optionally top-k then top-p) sampling layer. Public surface of the reference's
// src/fastertransformer/layers/sampling_layers/TopKSamplingLayer.h:26-72.
#pragma once
#include "src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.h"

namespace fastertransformer {

template<typename T>
class TopKSamplingLayer: public BaseSamplingLayer<T> {
    uint runtime_max_top_k_ = 1;
    // the two environment switches of the layer as setup() found them
    bool fused_disabled_           = false;
    int  fused_log_probs_min_rows_ = 0;

    void allocateBuffer() override;
    void allocateBuffer(size_t batch_size, Tensor top_k, Tensor top_p) override;
    void freeBuffer() override;
    void runSampling(TensorMap* output_tensors, TensorMap* input_tensors, T* logits) override;
    bool runFused(TensorMap* output_tensors, TensorMap* input_tensors) override;
    void ensureWorkspace(int local_batch_size);

    using BaseSamplingLayer<T>::vocab_size_;
    using BaseSamplingLayer<T>::vocab_size_padded_;
    using BaseSamplingLayer<T>::sampling_workspace_size_;
    using BaseSamplingLayer<T>::sampling_workspace_;
    using BaseSamplingLayer<T>::curandstate_buf_;
    using BaseSamplingLayer<T>::skip_decode_buf_;
    using BaseSamplingLayer<T>::skip_decode_;
    using BaseSamplingLayer<T>::runtime_top_k_buf_;
    using BaseSamplingLayer<T>::runtime_top_p_buf_;
    using BaseSamplingLayer<T>::runtime_top_k_;
    using BaseSamplingLayer<T>::runtime_top_p_;
    using BaseSamplingLayer<T>::stream_;
    using BaseSamplingLayer<T>::allocator_;
    using BaseSamplingLayer<T>::is_allocate_buffer_;

public:
    TopKSamplingLayer(size_t max_batch_size, size_t vocab_size, size_t vocab_size_padded, int end_id, size_t top_k,
                      unsigned long long random_seed, float temperature, float len_penalty, float repetition_penalty,
                      hipStream_t stream, cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                      bool is_free_buffer_after_forward);
    TopKSamplingLayer(TopKSamplingLayer<T> const& top_k_sampling_layer);
    ~TopKSamplingLayer() override;

    void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args) override;
};

}  // namespace fastertransformer
