// The two host classes of beam search, over the kernels of csrc/beam_kernels.hip. They keep the reference's names,
// constructors and tensor keys (layers/beam_search_layers/BaseBeamSearchLayer.h:27-71 and
// OnlineBeamSearchLayer.h:24-64) and nothing between steps except a workspace:
//   BaseBeamSearchLayer<T>::forward   - penalties on the window's logits, the step (invokeSoftMax of the derived
//                                       class), the key / value cache indirection of the surviving beams
//   OnlineBeamSearchLayer<T>          - the step: log-softmax, candidates, hypotheses, then the split of the
//                                       chosen ids into token and parent beam
// Tensors of a call (reference: BaseBeamSearchLayer.cu:177-207). Inputs: logits [local_batch, beam_width,
// vocab_padded], step, ite, max_input_length (host), end_id [local_batch], src_cache_indirection [local_batch,
// beam_width, max_seq_len]; optional embedding_bias [vocab_padded], input_lengths [local_batch * beam_width] and,
// on the host, temperature, len_penalty, beam_search_diversity_rate, repetition_penalty or presence_penalty,
// min_length. Outputs: output_ids [max_seq_len, batch, beam_width], parent_ids (same shape), finished,
// cum_log_probs, sequence_length [local_batch * beam_width], tgt_cache_indirection; optional output_log_probs
// [max_seq_len, batch, beam_width] and beam_hyps (a host pointer to a BeamHypotheses).
#pragma once
#include "src/fastertransformer/kernels/sampling_kernels.h"
#include "src/fastertransformer/layers/DynamicDecodeBaseLayer.h"

namespace fastertransformer {

// Sizes and positions one call works with, read once from its tensor maps.
struct BeamStepShape {
    int    batch, beams, local_batch, max_seq_len, step, ite;
    size_t window;   // first beam of this window among batch * beams
    size_t at_step;  // offset of this window's beams in row `step` of a [max_seq_len, batch * beams] array
    BeamStepShape(const TensorMap& outputs, const TensorMap& inputs);
};

template<typename T>
class BaseBeamSearchLayer: public DynamicDecodeBaseLayer {
public:
    // only the sizes, the stream and the allocator are used; the other arguments are deprecated in the reference
    // as well (every step reads its values from its inputs)
    BaseBeamSearchLayer(size_t, size_t, size_t, size_t, size_t vocab_size, size_t vocab_size_padded, int, float, float,
                        float, float, hipStream_t stream, cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                        bool is_free_buffer_after_forward);
    BaseBeamSearchLayer(BaseBeamSearchLayer<T> const& other);
    ~BaseBeamSearchLayer() override;

    void setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args) override;
    void forward(TensorMap* output_tensors, TensorMap* input_tensors) override;
    void forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors) override;
    void forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                 const std::unordered_map<std::string, Tensor>* input_tensors) override;

protected:
    virtual void invokeSoftMax(TensorMap* output_tensors, TensorMap* input_tensors) = 0;
    virtual void allocateBuffer(size_t batch_size, size_t beam_width)               = 0;
    void         allocateBuffer() override;
    void         freeBuffer() override;

    size_t vocab_size_;
    size_t vocab_size_padded_;
    void*  topk_softmax_workspace_      = nullptr;
    size_t topk_softmax_workspace_size_ = 0;  // bytes
};

template<typename T>
class OnlineBeamSearchLayer: public BaseBeamSearchLayer<T> {
public:
    OnlineBeamSearchLayer(size_t, size_t, size_t, size_t, size_t vocab_size, size_t vocab_size_padded, int, float,
                          float, float, float, hipStream_t stream, cublasMMWrapper* cublas_wrapper,
                          IAllocator* allocator, bool is_free_buffer_after_forward);
    OnlineBeamSearchLayer(OnlineBeamSearchLayer<T> const& other);
    ~OnlineBeamSearchLayer() override = default;

protected:
    void invokeSoftMax(TensorMap* output_tensors, TensorMap* input_tensors) override;
    void allocateBuffer(size_t batch_size, size_t beam_width) override;
    void allocateBuffer() override;
};

}  // namespace fastertransformer
