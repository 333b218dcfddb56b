#include "src/fastertransformer/layers/beam_search_layers/BaseBeamSearchLayer.h"

namespace fastertransformer {

template<typename T>
BaseBeamSearchLayer<T>::BaseBeamSearchLayer(size_t max_batch_size, size_t head_num, size_t size_per_head,
                                            size_t beam_width, size_t vocab_size, size_t vocab_size_padded,
                                            int end_id, float diversity_rate, float temperature, float len_penalty,
                                            float repetition_penalty, hipStream_t stream,
                                            cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                            bool is_free_buffer_after_forward):
    DynamicDecodeBaseLayer(stream, cublas_wrapper, allocator, is_free_buffer_after_forward, nullptr),
    vocab_size_(vocab_size),
    vocab_size_padded_(vocab_size_padded)
{
    // the remaining arguments are deprecated in the reference as well: every step reads them from its inputs
    (void)max_batch_size;
    (void)head_num;
    (void)size_per_head;
    (void)beam_width;
    (void)end_id;
    (void)diversity_rate;
    (void)temperature;
    (void)len_penalty;
    (void)repetition_penalty;
}

template<typename T>
BaseBeamSearchLayer<T>::BaseBeamSearchLayer(BaseBeamSearchLayer<T> const& other):
    DynamicDecodeBaseLayer(other), vocab_size_(other.vocab_size_), vocab_size_padded_(other.vocab_size_padded_)
{
}

template<typename T>
BaseBeamSearchLayer<T>::~BaseBeamSearchLayer()
{
    freeBuffer();
}

template<typename T>
void BaseBeamSearchLayer<T>::allocateBuffer()
{
    FT_CHECK(false);  // sizes come with the step (reference: OnlineBeamSearchLayer.cu:181-185)
}

template<typename T>
void BaseBeamSearchLayer<T>::freeBuffer()
{
    if (is_allocate_buffer_) {
        allocator_->free((void**)(&topk_softmax_workspace_));
        topk_softmax_workspace_size_ = 0;
        is_allocate_buffer_          = false;
    }
}

template<typename T>
void BaseBeamSearchLayer<T>::setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args)
{
    // nothing is kept between steps (reference: BaseBeamSearchLayer.cu:132-136)
    (void)batch_size;
    (void)beam_width;
    (void)runtime_args;
}

// reference: BaseBeamSearchLayer.cu:138-175 (positional and unordered_map forms)
template<typename T>
void BaseBeamSearchLayer<T>::forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors)
{
    TensorMap in({{"logits", input_tensors->at(0)},
                  {"embedding_bias", input_tensors->at(1)},
                  {"step", input_tensors->at(2)},
                  {"src_cache_indirection", input_tensors->at(4)},
                  {"max_input_length", input_tensors->at(5)},
                  {"input_lengths", input_tensors->at(6)},
                  {"ite", input_tensors->at(7)}});
    TensorMap out({{"output_ids", output_tensors->at(0)},
                   {"finished", output_tensors->at(1)},
                   {"cum_log_probs", output_tensors->at(2)},
                   {"parent_ids", output_tensors->at(3)},
                   {"sequence_length", output_tensors->at(4)},
                   {"tgt_cache_indirection", output_tensors->at(5)}});
    forward(&out, &in);
}

template<typename T>
void BaseBeamSearchLayer<T>::forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                                     const std::unordered_map<std::string, Tensor>* input_tensors)
{
    TensorMap in(*input_tensors);
    TensorMap out(*output_tensors);
    forward(&out, &in);
}

// reference: BaseBeamSearchLayer.cu:177-284. Inputs: logits [local_batch, beam_width, vocab_padded], embedding_bias
// (optional), step, src_cache_indirection [local_batch, beam_width, max_seq_len], end_id [local_batch],
// max_input_length, input_lengths (optional), ite, and on the host, optional: beam_search_diversity_rate,
// temperature, len_penalty, repetition_penalty or presence_penalty, min_length. Outputs: output_ids
// [max_seq_len, batch, beam_width], finished, cum_log_probs, parent_ids, sequence_length, tgt_cache_indirection,
// output_log_probs (optional), beam_hyps (optional).
template<typename T>
void BaseBeamSearchLayer<T>::forward(TensorMap* output_tensors, TensorMap* input_tensors)
{
    FT_CHECK(input_tensors->size() >= 7);
    FT_CHECK(output_tensors->size() >= 5);
    const int batch_size = output_tensors->at("output_ids").shape[1];
    const int beam_width = output_tensors->at("output_ids").shape[2];
    allocateBuffer(batch_size, beam_width);

    const int step             = input_tensors->at("step").template getVal<int>();
    const int ite              = input_tensors->at("ite").template getVal<int>();
    const int local_batch_size = input_tensors->at("logits").shape[0];

    const float temperature    = input_tensors->template getVal<float>("temperature", 1.0f);
    const T*    embedding_bias = input_tensors->template getPtr<const T>("embedding_bias", nullptr);

    RepetitionPenaltyType penalty_type = RepetitionPenaltyType::None;
    float                 penalty      = getDefaultPenaltyValue(penalty_type);
    const bool            has_rep      = input_tensors->isExist("repetition_penalty");
    const bool            has_pres     = input_tensors->isExist("presence_penalty");
    if (has_rep || has_pres) {
        FT_CHECK_WITH_INFO(!(has_rep && has_pres),
                           "Found ambiguous parameters repetition_penalty and presence_penalty which are mutually "
                           "exclusive. Please provide one of repetition_penalty or presence_penalty.");
        penalty_type = has_rep ? RepetitionPenaltyType::Multiplicative : RepetitionPenaltyType::Additive;
        penalty      = has_rep ? input_tensors->template getVal<float>("repetition_penalty") :
                                 input_tensors->template getVal<float>("presence_penalty");
    }

    const size_t window = (size_t)ite * local_batch_size * beam_width;
    invokeAddBiasApplyPenalties(
        step, input_tensors->at("logits").template getPtr<T>(),
        step > 0 ? output_tensors->at("output_ids")
                       .template getPtrWithOffset<const int>((size_t)(step - 1) * batch_size * beam_width + window) :
                   (const int*)nullptr,
        output_tensors->template getPtr<const int>("output_ids"),
        output_tensors->template getPtr<const int>("parent_ids"),
        input_tensors->template getPtr<const int>("input_lengths", nullptr),
        output_tensors->template getPtr<const int>("sequence_length", nullptr), embedding_bias, ite,
        input_tensors->template getVal<int>("max_input_length"), local_batch_size, batch_size, beam_width,
        (int)vocab_size_, (int)vocab_size_padded_, input_tensors->template getPtr<const int>("end_id", nullptr),
        temperature, penalty, penalty_type, input_tensors->template getVal<int>("min_length", 0), stream_);
    sync_check_hip_error();

    invokeSoftMax(output_tensors, input_tensors);

    if (beam_width > 1) {
        const int max_seq_len = output_tensors->at("output_ids").shape[0];
        update_indir_cache_kernelLauncher(
            output_tensors->at("tgt_cache_indirection").template getPtr<int>(),
            input_tensors->at("src_cache_indirection").template getPtr<const int>(),
            output_tensors->at("parent_ids")
                .template getPtrWithOffset<const int>((size_t)step * beam_width * batch_size + window),
            output_tensors->at("finished").template getPtr<const bool>(), batch_size, local_batch_size, beam_width,
            max_seq_len, step, stream_);
        sync_check_hip_error();
    }
    if (is_free_buffer_after_forward_) {
        freeBuffer();
    }
}

template class BaseBeamSearchLayer<float>;
template class BaseBeamSearchLayer<half>;
template class BaseBeamSearchLayer<bfloat16>;

}  // namespace fastertransformer
