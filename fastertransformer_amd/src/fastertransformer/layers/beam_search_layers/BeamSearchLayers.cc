#include "src/fastertransformer/layers/beam_search_layers/BeamSearchLayers.h"

namespace fastertransformer {

BeamStepShape::BeamStepShape(const TensorMap& outputs, const TensorMap& inputs)
{
    const Tensor& ids = outputs.at("output_ids");
    FT_CHECK_WITH_INFO(ids.shape.size() == 3, "output_ids must be [max_seq_len, batch, beam_width]");
    max_seq_len = (int)ids.shape[0];
    batch       = (int)ids.shape[1];
    beams       = (int)ids.shape[2];
    local_batch = (int)inputs.at("logits").shape[0];
    step        = inputs.at("step").getVal<int>();
    ite         = inputs.at("ite").getVal<int>();
    window      = (size_t)ite * local_batch * beams;
    at_step     = (size_t)step * batch * beams + window;
}

namespace {

// host scalar of a step, or its default
template<typename V>
V hostValue(const TensorMap& inputs, const char* key, V fallback)
{
    return inputs.isExist(key) ? inputs.at(key).getVal<V>() : fallback;
}

// positional argument lists of the oldest forward() form (reference: BaseBeamSearchLayer.cu:138-164); slot 3 of the
// inputs is not used
const char* const kPositionalInputs[]  = {"logits", "embedding_bias", "step", nullptr, "src_cache_indirection",
                                          "max_input_length", "input_lengths", "ite"};
const char* const kPositionalOutputs[] = {"output_ids", "finished", "cum_log_probs", "parent_ids", "sequence_length",
                                          "tgt_cache_indirection"};

}  // namespace

// ---- BaseBeamSearchLayer ---------------------------------------------------------------------------------------
template<typename T>
BaseBeamSearchLayer<T>::BaseBeamSearchLayer(size_t, size_t, size_t, size_t, size_t vocab_size,
                                            size_t vocab_size_padded, int, float, float, float, float,
                                            hipStream_t stream, cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                            bool is_free_buffer_after_forward):
    DynamicDecodeBaseLayer(stream, cublas_wrapper, allocator, is_free_buffer_after_forward, nullptr),
    vocab_size_(vocab_size),
    vocab_size_padded_(vocab_size_padded)
{
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
    FT_CHECK_WITH_INFO(false, "the workspace is sized by the step: allocateBuffer(batch_size, beam_width)");
}

template<typename T>
void BaseBeamSearchLayer<T>::freeBuffer()
{
    if (topk_softmax_workspace_ != nullptr) {
        allocator_->free((void**)(&topk_softmax_workspace_));
    }
    topk_softmax_workspace_size_ = 0;
    is_allocate_buffer_          = false;
}

template<typename T>
void BaseBeamSearchLayer<T>::setup(const size_t, const size_t, TensorMap*)
{
    // a beam-search step takes all of its values from its inputs
}

template<typename T>
void BaseBeamSearchLayer<T>::forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors)
{
    TensorMap in, out;
    for (size_t i = 0; i < sizeof(kPositionalInputs) / sizeof(kPositionalInputs[0]); ++i) {
        if (kPositionalInputs[i] != nullptr) {
            in.insert({kPositionalInputs[i], input_tensors->at(i)});
        }
    }
    for (size_t i = 0; i < sizeof(kPositionalOutputs) / sizeof(kPositionalOutputs[0]); ++i) {
        out.insert({kPositionalOutputs[i], output_tensors->at(i)});
    }
    forward(&out, &in);
}

template<typename T>
void BaseBeamSearchLayer<T>::forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                                     const std::unordered_map<std::string, Tensor>* input_tensors)
{
    TensorMap in(*input_tensors), out(*output_tensors);
    forward(&out, &in);
}

// reference: BaseBeamSearchLayer<T>::forward, layers/beam_search_layers/BaseBeamSearchLayer.cu:177-284
template<typename T>
void BaseBeamSearchLayer<T>::forward(TensorMap* output_tensors, TensorMap* input_tensors)
{
    FT_CHECK(input_tensors->size() >= 7);
    FT_CHECK(output_tensors->size() >= 5);
    const BeamStepShape s(*output_tensors, *input_tensors);
    allocateBuffer((size_t)s.batch, (size_t)s.beams);

    // one of the two penalties at most; which one decides how it is applied
    const bool multiplicative = input_tensors->isExist("repetition_penalty");
    const bool additive       = input_tensors->isExist("presence_penalty");
    FT_CHECK_WITH_INFO(!(multiplicative && additive),
                       "Found ambiguous parameters repetition_penalty and presence_penalty which are mutually "
                       "exclusive. Please provide one of repetition_penalty or presence_penalty.");
    const RepetitionPenaltyType kind = multiplicative ? RepetitionPenaltyType::Multiplicative :
                                       additive       ? RepetitionPenaltyType::Additive :
                                                        RepetitionPenaltyType::None;
    const float penalty = multiplicative ? input_tensors->at("repetition_penalty").template getVal<float>() :
                          additive       ? input_tensors->at("presence_penalty").template getVal<float>() :
                                           getDefaultPenaltyValue(kind);

    const Tensor& ids     = output_tensors->at("output_ids");
    const int*    history = ids.template getPtr<const int>();
    // the tokens chosen one step ago, for this window (none before the first step)
    const int* newest = s.step > 0 ? history + (s.at_step - (size_t)s.batch * s.beams) : nullptr;
    invokeAddBiasApplyPenalties(s.step, input_tensors->at("logits").template getPtr<T>(), newest, history,
                                output_tensors->at("parent_ids").template getPtr<const int>(),
                                input_tensors->at("input_lengths", Tensor()).template getPtr<const int>(),
                                output_tensors->at("sequence_length", Tensor()).template getPtr<const int>(),
                                input_tensors->at("embedding_bias", Tensor()).template getPtr<const T>(), s.ite,
                                input_tensors->at("max_input_length").template getVal<int>(), s.local_batch, s.batch,
                                s.beams, (int)vocab_size_, (int)vocab_size_padded_,
                                input_tensors->at("end_id", Tensor()).template getPtr<const int>(),
                                hostValue<float>(*input_tensors, "temperature", 1.0f), penalty, kind,
                                hostValue<int>(*input_tensors, "min_length", 0), stream_);
    sync_check_hip_error();

    invokeSoftMax(output_tensors, input_tensors);

    if (s.beams > 1) {
        // positions up to `step` of every live beam's cache follow the beam it continues
        update_indir_cache_kernelLauncher(output_tensors->at("tgt_cache_indirection").template getPtr<int>(),
                                          input_tensors->at("src_cache_indirection").template getPtr<const int>(),
                                          output_tensors->at("parent_ids").template getPtr<const int>() + s.at_step,
                                          output_tensors->at("finished").template getPtr<const bool>(), s.batch,
                                          s.local_batch, s.beams, s.max_seq_len, s.step, stream_);
        sync_check_hip_error();
    }
    if (is_free_buffer_after_forward_) {
        freeBuffer();
    }
}

// ---- OnlineBeamSearchLayer -------------------------------------------------------------------------------------
template<typename T>
OnlineBeamSearchLayer<T>::OnlineBeamSearchLayer(size_t a, size_t b, size_t c, size_t d, size_t vocab_size,
                                                size_t vocab_size_padded, int e, float f, float g, float h, float i,
                                                hipStream_t stream, cublasMMWrapper* cublas_wrapper,
                                                IAllocator* allocator, bool is_free_buffer_after_forward):
    BaseBeamSearchLayer<T>(a, b, c, d, vocab_size, vocab_size_padded, e, f, g, h, i, stream, cublas_wrapper, allocator,
                           is_free_buffer_after_forward)
{
}

template<typename T>
OnlineBeamSearchLayer<T>::OnlineBeamSearchLayer(OnlineBeamSearchLayer<T> const& other): BaseBeamSearchLayer<T>(other)
{
}

template<typename T>
void OnlineBeamSearchLayer<T>::allocateBuffer()
{
    BaseBeamSearchLayer<T>::allocateBuffer();
}

// The reference reserves a fixed worst case (OnlineBeamSearchLayer.cu:187-199); here the size the kernels report for
// this batch, kept and grown on demand.
template<typename T>
void OnlineBeamSearchLayer<T>::allocateBuffer(size_t batch_size, size_t beam_width)
{
    const size_t need = topkSoftMaxWorkspaceBytes<T>((int)batch_size, (int)beam_width, (int)this->vocab_size_padded_);
    if (this->topk_softmax_workspace_ == nullptr || need > this->topk_softmax_workspace_size_) {
        this->topk_softmax_workspace_      = this->allocator_->reMalloc(this->topk_softmax_workspace_, need, true);
        this->topk_softmax_workspace_size_ = need;
    }
    this->is_allocate_buffer_ = true;
}

// reference: OnlineBeamSearchLayer<T>::invokeSoftMax, layers/beam_search_layers/OnlineBeamSearchLayer.cu:87-176
template<typename T>
void OnlineBeamSearchLayer<T>::invokeSoftMax(TensorMap* output_tensors, TensorMap* input_tensors)
{
    const BeamStepShape s(*output_tensors, *input_tensors);
    const float         length_penalty = hostValue<float>(*input_tensors, "len_penalty", 0.0f);
    const int*          end_ids        = input_tensors->at("end_id").template getPtr<const int>();
    bool*               finished       = output_tensors->at("finished").template getPtr<bool>();
    int*                lengths        = output_tensors->at("sequence_length").template getPtr<int>();
    int*                all_ids        = output_tensors->at("output_ids").template getPtr<int>();
    int*                all_parents    = output_tensors->at("parent_ids").template getPtr<int>();
    float*              all_log_probs  = output_tensors->at("output_log_probs", Tensor()).template getPtr<float>();

    // the caller's hypotheses structure travels as a host pointer; the fields that describe this step are filled in
    BeamHypotheses hyps{};
    if (output_tensors->isExist("beam_hyps")) {
        hyps                      = *static_cast<const BeamHypotheses*>(output_tensors->at("beam_hyps").template getPtr<void>());
        hyps.step                 = s.step;
        hyps.ite                  = s.ite;
        hyps.batch_size           = s.batch;
        hyps.local_batch_size     = s.local_batch;
        hyps.max_seq_len          = s.max_seq_len;
        hyps.length_penalty       = length_penalty;
        hyps.output_ids_src       = all_ids;
        hyps.parent_ids_src       = all_parents;
        hyps.sequence_lengths_src = lengths;
        hyps.log_probs_src        = all_log_probs;
        hyps.end_ids              = end_ids;
    }

    int* chosen = all_ids + s.at_step;  // absolute ids first, tokens after the update
    check_ftk(ftk_invoke_topk_softmax(FtkDType<T>::value, input_tensors->at("logits").template getPtr<T>(), nullptr,
                                      finished, lengths, output_tensors->at("cum_log_probs").template getPtr<float>(),
                                      all_log_probs != nullptr ? all_log_probs + s.at_step : nullptr, chosen,
                                      this->topk_softmax_workspace_, &this->topk_softmax_workspace_size_, &hyps,
                                      s.local_batch, s.beams, (int)this->vocab_size_padded_, end_ids,
                                      hostValue<float>(*input_tensors, "beam_search_diversity_rate", 0.0f),
                                      length_penalty, this->stream_));
    sync_check_hip_error();
    invokeUpdate(finished, all_parents + s.at_step, lengths, chosen, chosen, &hyps, s.local_batch, s.beams,
                 (int)this->vocab_size_padded_, end_ids, this->stream_);
    sync_check_hip_error();
}

template class BaseBeamSearchLayer<float>;
template class BaseBeamSearchLayer<half>;
template class BaseBeamSearchLayer<bfloat16>;
template class OnlineBeamSearchLayer<float>;
template class OnlineBeamSearchLayer<half>;
template class OnlineBeamSearchLayer<bfloat16>;

}  // namespace fastertransformer
