// Top-p (nucleus) sampling layer with top_p decay / minimum / reset ids. Public surface of the
// reference's src/fastertransformer/layers/sampling_layers/TopPSamplingLayer.h:25-82.
#pragma once
#include "src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.h"

namespace fastertransformer {

template<typename T>
class TopPSamplingLayer: public BaseSamplingLayer<T> {
    float    runtime_max_top_p_   = 0.0f;
    bool     keep_probabilities_  = false;  // FT_SAMPLING_DISABLE_FUSED=1, read once per setup()
    float*   initial_top_p_buf_   = nullptr;
    float*   top_p_decay_buf_     = nullptr;
    float*   top_p_min_buf_       = nullptr;
    int32_t* top_p_reset_ids_buf_ = nullptr;
    size_t   cub_temp_storage_size_ = 0;

    void allocateBuffer() override;
    void allocateBuffer(size_t batch_size, Tensor top_k, Tensor top_p) override;
    void freeBuffer() override;
    void runSampling(TensorMap* output_tensors, TensorMap* input_tensors, T* logits) override;

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
    using BaseSamplingLayer<T>::cuda_device_prop_;

public:
    TopPSamplingLayer(size_t max_batch_size, size_t vocab_size, size_t vocab_size_padded, int end_id, float top_p,
                      unsigned long long random_seed, float temperature, float len_penalty, float repetition_penalty,
                      hipStream_t stream, cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                      bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop);
    TopPSamplingLayer(TopPSamplingLayer<T> const& top_p_sampling_layer);
    ~TopPSamplingLayer() override;

    void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args) override;
};

}  // namespace fastertransformer
