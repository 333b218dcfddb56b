#include "src/fastertransformer/layers/beam_search_layers/OnlineBeamSearchLayer.h"

namespace fastertransformer {

// reference: OnlineBeamSearchLayer<T>::invokeSoftMax, layers/beam_search_layers/OnlineBeamSearchLayer.cu:87-176
template<typename T>
void OnlineBeamSearchLayer<T>::invokeSoftMax(TensorMap* output_tensors, TensorMap* input_tensors)
{
    FT_CHECK(input_tensors->size() >= 7);
    FT_CHECK(output_tensors->size() >= 6);

    const int   batch_size       = output_tensors->at("output_ids").shape[1];
    const int   beam_width       = output_tensors->at("output_ids").shape[2];
    const int   step             = input_tensors->at("step").template getVal<int>();
    const int   ite              = input_tensors->at("ite").template getVal<int>();
    const int   local_batch_size = input_tensors->at("logits").shape[0];
    const float diversity_rate   = input_tensors->template getVal<float>("beam_search_diversity_rate", 0.0f);
    const float length_penalty   = input_tensors->template getVal<float>("len_penalty", 0.0f);

    const size_t id_offset = (size_t)step * batch_size * beam_width + (size_t)local_batch_size * ite * beam_width;

    BeamHypotheses beam_hyps{};
    if (output_tensors->isExist("beam_hyps")) {
        beam_hyps = *((BeamHypotheses*)(output_tensors->at("beam_hyps").template getPtr<void>()));
        beam_hyps.step                 = step;
        beam_hyps.ite                  = ite;
        beam_hyps.local_batch_size     = local_batch_size;
        beam_hyps.batch_size           = output_tensors->at("output_ids").shape[1];
        beam_hyps.max_seq_len          = output_tensors->at("output_ids").shape[0];
        beam_hyps.output_ids_src       = output_tensors->at("output_ids").template getPtr<int>();
        beam_hyps.parent_ids_src       = output_tensors->at("parent_ids").template getPtr<int>();
        beam_hyps.sequence_lengths_src = output_tensors->at("sequence_length").template getPtr<int>();
        beam_hyps.log_probs_src        = output_tensors->template getPtr<float>("output_log_probs", nullptr);
        beam_hyps.length_penalty       = length_penalty;
        beam_hyps.end_ids              = input_tensors->at("end_id").template getPtr<int>();
    }

    float* output_log_probs = output_tensors->isExist("output_log_probs") ?
                                  output_tensors->template getPtrWithOffset<float>("output_log_probs", id_offset) :
                                  nullptr;
    int*   ids              = output_tensors->at("output_ids").template getPtrWithOffset<int>(id_offset);
    check_ftk(ftk_invoke_topk_softmax(FtkDType<T>::value, input_tensors->at("logits").template getPtr<T>(), nullptr,
                                      output_tensors->at("finished").template getPtr<bool>(),
                                      output_tensors->at("sequence_length").template getPtr<int>(),
                                      output_tensors->at("cum_log_probs").template getPtr<float>(), output_log_probs,
                                      ids, topk_softmax_workspace_, &topk_softmax_workspace_size_, &beam_hyps,
                                      local_batch_size, beam_width, (int)vocab_size_padded_,
                                      input_tensors->at("end_id").template getPtr<int>(), diversity_rate,
                                      length_penalty, stream_));
    sync_check_hip_error();

    invokeUpdate(output_tensors->at("finished").template getPtr<bool>(),
                 output_tensors->at("parent_ids").template getPtrWithOffset<int>(id_offset),
                 output_tensors->at("sequence_length").template getPtr<int>(), ids, ids, &beam_hyps, local_batch_size,
                 beam_width, (int)vocab_size_padded_, input_tensors->at("end_id").template getPtr<const int>(),
                 stream_);
    sync_check_hip_error();
}

template<typename T>
void OnlineBeamSearchLayer<T>::allocateBuffer()
{
    FT_CHECK(false);
}

// reference: OnlineBeamSearchLayer.cu:187-199 (a fixed worst-case count of floats there; the queried size of
// this batch here, grown on demand)
template<typename T>
void OnlineBeamSearchLayer<T>::allocateBuffer(size_t batch_size, size_t beam_width)
{
    const size_t need = topkSoftMaxWorkspaceBytes<T>((int)batch_size, (int)beam_width, (int)vocab_size_padded_);
    if (need > topk_softmax_workspace_size_ || topk_softmax_workspace_ == nullptr) {
        topk_softmax_workspace_      = allocator_->reMalloc(topk_softmax_workspace_, need, true);
        topk_softmax_workspace_size_ = need;
    }
    is_allocate_buffer_ = true;
}

template<typename T>
OnlineBeamSearchLayer<T>::OnlineBeamSearchLayer(size_t max_batch_size, size_t head_num, size_t size_per_head,
                                                size_t beam_width, size_t vocab_size, size_t vocab_size_padded,
                                                int end_id, float diversity_rate, float temperature,
                                                float len_penalty, float repetition_penalty, hipStream_t stream,
                                                cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                                bool is_free_buffer_after_forward):
    BaseBeamSearchLayer<T>(max_batch_size, head_num, size_per_head, beam_width, vocab_size, vocab_size_padded, end_id,
                           diversity_rate, temperature, len_penalty, repetition_penalty, stream, cublas_wrapper,
                           allocator, is_free_buffer_after_forward)
{
}

template<typename T>
OnlineBeamSearchLayer<T>::OnlineBeamSearchLayer(OnlineBeamSearchLayer<T> const& other): BaseBeamSearchLayer<T>(other)
{
}

template<typename T>
OnlineBeamSearchLayer<T>::~OnlineBeamSearchLayer()
{
}

template class OnlineBeamSearchLayer<float>;
template class OnlineBeamSearchLayer<half>;
template class OnlineBeamSearchLayer<bfloat16>;

}  // namespace fastertransformer
