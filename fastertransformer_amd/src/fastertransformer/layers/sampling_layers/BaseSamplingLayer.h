// Shared machinery of the top-k and top-p sampling layers: per-row runtime arguments, generator
// state, the penalty pipeline and the skip logic that routes each row to exactly one of the two
// layers. Public surface of the reference's
// src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.h:27-88.
#pragma once
#include <vector>

#include "src/fastertransformer/kernels/sampling_kernels.h"
#include "src/fastertransformer/layers/DynamicDecodeBaseLayer.h"

namespace fastertransformer {

template<typename T>
class BaseSamplingLayer: public DynamicDecodeBaseLayer {
protected:
    size_t vocab_size_;
    size_t vocab_size_padded_;

    size_t sampling_workspace_size_ = 0;
    void*  sampling_workspace_      = nullptr;

    // device buffers, [batch]
    curandState_t* curandstate_buf_         = nullptr;
    float*         temperature_buf_         = nullptr;
    float*         repetition_penalty_buf_  = nullptr;
    float*         frequency_penalty_buf_   = nullptr;  // extension
    int*           min_lengths_buf_         = nullptr;
    bool*          skip_decode_buf_         = nullptr;
    uint*          runtime_top_k_buf_       = nullptr;
    float*         runtime_top_p_buf_       = nullptr;
    // private copy of the logits window, only ever allocated for batches that mix top-k and top-p rows
    T*     runtime_logits_buf_      = nullptr;
    size_t runtime_logits_capacity_ = 0;

    // host mirrors
    std::vector<float>   temperature_;
    std::vector<float>   repetition_penalty_;
    std::vector<float>   frequency_penalty_;
    std::vector<int>     min_lengths_;
    std::vector<uint8_t> skip_decode_;
    std::vector<uint>    runtime_top_k_;
    std::vector<float>   runtime_top_p_;

    RepetitionPenaltyType repetition_penalty_type_ = RepetitionPenaltyType::None;
    bool                  has_frequency_penalty_   = false;
    bool                  skip_any_                = false;
    size_t                setup_batch_size_        = 0;

    void         allocateBuffer() override;
    virtual void allocateBuffer(size_t batch_size, Tensor top_k, Tensor top_p);
    void         freeBuffer() override;

    // the rows this layer owns in the window [ite*local, (ite+1)*local), after the penalty pipeline
    virtual void runSampling(TensorMap* output_tensors, TensorMap* input_tensors, T* logits) = 0;
    // a layer may handle the whole step in fused kernels; returns true when it did
    virtual bool runFused(TensorMap* output_tensors, TensorMap* input_tensors)
    {
        (void)output_tensors;
        (void)input_tensors;
        return false;
    }

    template<typename V>
    void fillFromArg(std::vector<V>& host, V* device, const Tensor& arg, size_t batch_size);

public:
    BaseSamplingLayer(size_t max_batch_size, size_t vocab_size, size_t vocab_size_padded, int end_id, size_t top_k,
                      float top_p, unsigned long long random_seed, float temperature, float len_penalty,
                      float repetition_penalty, hipStream_t stream, cublasMMWrapper* cublas_wrapper,
                      IAllocator* allocator, bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop);
    BaseSamplingLayer(BaseSamplingLayer const& sampling_layer);
    ~BaseSamplingLayer() override;

    void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args) override;
    void forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors) override;
    void forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                 const std::unordered_map<std::string, Tensor>* input_tensors) override;
    void forward(TensorMap* output_tensors, TensorMap* input_tensors) override;

    // host view of the routing decided in setup (true = row not handled by this layer)
    const std::vector<uint8_t>& skipDecode() const
    {
        return skip_decode_;
    }
};

}  // namespace fastertransformer
