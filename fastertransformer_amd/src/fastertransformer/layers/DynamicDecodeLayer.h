// Per-step decode orchestrator: bad words -> top-k / top-p sampling -> stop words -> length criterion, or, for
// logits with more than one beam per entry, bad words -> the beam-search layer -> stop words -> length criterion.
// Public surface of the reference's src/fastertransformer/layers/DynamicDecodeLayer.h:29-75.
#pragma once
#include <string>
#include <unordered_map>

#include "src/fastertransformer/layers/beam_search_layers/OnlineBeamSearchLayer.h"
#include "src/fastertransformer/layers/sampling_layers/TopKSamplingLayer.h"
#include "src/fastertransformer/layers/sampling_layers/TopPSamplingLayer.h"

namespace fastertransformer {

template<typename T>
class DynamicDecodeLayer: public BaseLayer {
public:
    using NamedTensors = std::unordered_map<std::string, Tensor>;

    DynamicDecodeLayer(size_t vocab_size, size_t vocab_size_padded, int end_id, hipStream_t stream,
                       cublasMMWrapper* cublas_wrapper, IAllocator* allocator, bool is_free_buffer_after_forward,
                       cudaDeviceProp* cuda_device_prop);
    DynamicDecodeLayer(DynamicDecodeLayer const& other);
    ~DynamicDecodeLayer() override;

    void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args);
    void forward(TensorMap* output_tensors, TensorMap* input_tensors);
    void forward(NamedTensors* output_tensors, const NamedTensors* input_tensors);
    void setStream(hipStream_t stream) override;

protected:
    // sizes first: the three layers below are built from them
    size_t vocab_size_;
    size_t vocab_size_padded_;
    // one step goes to the two sampling layers (every row belongs to exactly one of them) or to the beam-search layer
    TopKSamplingLayer<T>*     topk_decode_              = nullptr;
    TopPSamplingLayer<T>*     topp_decode_              = nullptr;
    OnlineBeamSearchLayer<T>* online_beamsearch_decode_ = nullptr;
    // setup() saw per-entry values that differ: beam search then takes the entries of a window one by one
    bool has_diff_runtime_args_ = false;
    // pinned host word the length criterion reports through
    int* h_pinned_finished_sum_ = nullptr;

    void initialize();
    void allocateBuffer() override;
    void freeBuffer() override;
    // the parts of a step around the layers; `first` / `rows`: the micro-batch window in entries
    void banBadWords(TensorMap* output_tensors, TensorMap* input_tensors, size_t first, size_t rows, int step);
    void stopCriteria(TensorMap* output_tensors, TensorMap* input_tensors, size_t first, size_t rows, int step);
    // the step for logits [batch, beam_width > 1, vocab_padded]
    void forwardBeams(TensorMap* output_tensors, TensorMap* input_tensors, int ite, size_t rows);
};

}  // namespace fastertransformer
