#include "src/fastertransformer/layers/DynamicDecodeLayer.h"

namespace fastertransformer {

template<typename T>
void DynamicDecodeLayer<T>::allocateBuffer()
{
    // one pinned int: the finished-row count the length criterion hands back to the host
    h_pinned_finished_sum_ = (int*)allocator_->reMalloc(h_pinned_finished_sum_, sizeof(int), true, true);
}

template<typename T>
void DynamicDecodeLayer<T>::freeBuffer()
{
    allocator_->free((void**)(&h_pinned_finished_sum_), true);
}

template<typename T>
void DynamicDecodeLayer<T>::initialize()
{
    // every argument except sizes / stream / allocator is deprecated in the reference constructors
    // (layers/DynamicDecodeLayer.cc:80-107); runtime values arrive through setup()
    topk_decode_ = new TopKSamplingLayer<T>(0, vocab_size_, vocab_size_padded_, 0, 0, 0, 1.0f, 0.0f, 1.0f, stream_,
                                            cublas_wrapper_, allocator_, false);
    topp_decode_ = new TopPSamplingLayer<T>(0, vocab_size_, vocab_size_padded_, 0, 0.0f, 0, 1.0f, 0.0f, 1.0f, stream_,
                                            cublas_wrapper_, allocator_, false, cuda_device_prop_);
    allocateBuffer();
}

template<typename T>
DynamicDecodeLayer<T>::DynamicDecodeLayer(size_t vocab_size, size_t vocab_size_padded, int end_id, hipStream_t stream,
                                          cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                          bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop):
    BaseLayer(stream, cublas_wrapper, allocator, is_free_buffer_after_forward, cuda_device_prop),
    vocab_size_(vocab_size),
    vocab_size_padded_(vocab_size_padded)
{
    (void)end_id;
    FT_CHECK_WITH_INFO(vocab_size_ > 0 && vocab_size_ <= vocab_size_padded_,
                       "vocab_size must be in (0, vocab_size_padded]");
    initialize();
}

template<typename T>
DynamicDecodeLayer<T>::~DynamicDecodeLayer()
{
    delete topk_decode_;
    delete topp_decode_;
    freeBuffer();
}

template<typename T>
DynamicDecodeLayer<T>::DynamicDecodeLayer(DynamicDecodeLayer const& other):
    BaseLayer(other), vocab_size_(other.vocab_size_), vocab_size_padded_(other.vocab_size_padded_)
{
    initialize();
}

template<typename T>
void DynamicDecodeLayer<T>::setStream(hipStream_t stream)
{
    BaseLayer::setStream(stream);
    topk_decode_->setStream(stream);
    topp_decode_->setStream(stream);
}

// reference: DynamicDecodeLayer<T>::setup, layers/DynamicDecodeLayer.cc:153-178
template<typename T>
void DynamicDecodeLayer<T>::setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args)
{
    FT_CHECK_WITH_INFO(beam_width == 1, "this engine implements the sampling path only (beam_width must be 1)");
    topk_decode_->setup(batch_size, beam_width, runtime_args);
    topp_decode_->setup(batch_size, beam_width, runtime_args);
}

template<typename T>
void DynamicDecodeLayer<T>::forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                                    const std::unordered_map<std::string, Tensor>* input_tensors)
{
    TensorMap input_map(*input_tensors);
    TensorMap output_map(*output_tensors);
    forward(&output_map, &input_map);
}

// reference: DynamicDecodeLayer<T>::forward, layers/DynamicDecodeLayer.cc:191-474 (tensor names and
// shapes are documented there, :193-235). Extension: input "uniform_draws" [batch] float on the GPU,
// one draw in (0, 1] per row, replaces the generator for this step.
template<typename T>
void DynamicDecodeLayer<T>::forward(TensorMap* output_tensors, TensorMap* input_tensors)
{
    const int ite  = (int)input_tensors->at("ite").getVal<uint>();
    const int step = input_tensors->at("step").getVal<int>();
    FT_CHECK(input_tensors->at("logits").shape.size() == 3);

    const size_t batch_size       = input_tensors->at("logits").shape[0];
    const size_t beam_width       = input_tensors->at("logits").shape[1];
    const size_t local_batch_size = (size_t)input_tensors->at("local_batch_size").getVal<int>();
    FT_CHECK_WITH_INFO(beam_width == 1, "this engine implements the sampling path only (beam_width must be 1)");
    FT_CHECK_WITH_INFO((ite + 1) * local_batch_size <= batch_size, "ite / local_batch_size window exceeds the batch");
    const size_t local_batch_offset = ite * local_batch_size;

    if (input_tensors->isExist("bad_words_list")) {
        const auto& bad_words = input_tensors->at("bad_words_list");
        FT_CHECK_WITH_INFO(bad_words.shape.size() == 2 || bad_words.shape.size() == 3,
                           "Bad words dimension must be 2 or 3.");
        const bool is_matrix = bad_words.shape.size() == 2;
        if (!is_matrix) {
            FT_CHECK_WITH_INFO(bad_words.shape[0] == batch_size,
                               fmtstr("Shape of dim 0 of bad words is invalid. It must be equal to batch size."
                                      " However, it is %d and the batch size is %d.",
                                      (int)bad_words.shape[0], (int)batch_size));
        }
        const bool   shared_bad_words = is_matrix || bad_words.shape[0] == 1;
        const size_t bad_words_len    = bad_words.shape[is_matrix ? 1 : 2];
        invokeBanBadWords((T*)input_tensors->at("logits").getPtrWithOffset(local_batch_offset * vocab_size_padded_),
                          output_tensors->at("output_ids").getPtr<const int>(), (const int*)nullptr, (int)batch_size,
                          (int)local_batch_size, (int)beam_width,
                          shared_bad_words ?
                              bad_words.getPtr<const int>() :
                              bad_words.getPtrWithOffset<const int>(local_batch_offset * 2 * bad_words_len),
                          shared_bad_words, bad_words_len, (int)local_batch_offset, (int)vocab_size_padded_,
                          (size_t)step, stream_);
    }

    {
        Tensor logits = input_tensors->at("logits");
        Tensor end_id = input_tensors->at("end_id");

        TensorMap decode_input_tensors(
            {{"logits", logits.slice({local_batch_size, beam_width, logits.shape[2]},
                                     local_batch_offset * logits.shape[2])},
             {"step", input_tensors->at("step")},
             {"max_input_length", input_tensors->at("max_input_length")},
             {"end_id", end_id.slice({local_batch_size}, local_batch_offset)},
             {"ite", Tensor{MEMORY_CPU, TYPE_INT32, {1}, &ite}}});
        if (input_tensors->isExist("embedding_bias")) {
            decode_input_tensors.insert({"embedding_bias", input_tensors->at("embedding_bias")});
        }
        if (input_tensors->isExist("input_lengths")) {
            Tensor input_lengths = input_tensors->at("input_lengths");
            decode_input_tensors.insert(
                {"input_lengths", input_lengths.slice({local_batch_size, beam_width}, local_batch_offset)});
        }
        if (input_tensors->isExist("uniform_draws")) {
            Tensor draws = input_tensors->at("uniform_draws");
            decode_input_tensors.insert({"uniform_draws", draws.slice({local_batch_size}, local_batch_offset)});
        }

        TensorMap decode_output_tensors({{"output_ids", output_tensors->at("output_ids")}});
        if (output_tensors->isExist("sequence_length")) {
            Tensor sequence_length = output_tensors->at("sequence_length");
            decode_output_tensors.insert(
                {"sequence_length", sequence_length.slice({local_batch_size * beam_width}, local_batch_offset)});
        }
        if (output_tensors->isExist("finished")) {
            Tensor finished = output_tensors->at("finished");
            decode_output_tensors.insert(
                {"finished", finished.slice({local_batch_size * beam_width}, local_batch_offset)});
        }
        if (output_tensors->isExist("cum_log_probs")) {
            Tensor cum_log_probs = output_tensors->at("cum_log_probs");
            decode_output_tensors.insert(
                {"cum_log_probs", cum_log_probs.slice({local_batch_size * beam_width}, local_batch_offset)});
        }
        if (output_tensors->isExist("output_log_probs")) {
            Tensor       output_log_probs = output_tensors->at("output_log_probs");
            const int    max_input_length = input_tensors->at("max_input_length").getVal<int>();
            const size_t step_offset      = (size_t)(step - max_input_length) * batch_size * beam_width;
            decode_output_tensors.insert(
                {"output_log_probs",
                 output_log_probs.slice({output_log_probs.shape[0] - (step - max_input_length),
                                         local_batch_size * beam_width},
                                        step_offset + local_batch_offset)});
        }
        // every row belongs to exactly one of the two layers (k > 0 or greedy: top-k; k == 0 && p > 0: top-p)
        topk_decode_->forward(&decode_output_tensors, &decode_input_tensors);
        topp_decode_->forward(&decode_output_tensors, &decode_input_tensors);
    }

    if (input_tensors->isExist("stop_words_list")) {
        const size_t stop_words_length = input_tensors->at("stop_words_list").shape[2];
        FT_CHECK_WITH_INFO(output_tensors->at("finished", Tensor()).getPtr<bool>() != nullptr,
                           "stop_words_list needs the finished output");
        // only the rows of this window are examined
        check_ftk(ftk_invoke_stop_words_criterion_rows(
            output_tensors->at("output_ids").getPtr<const int>(), nullptr,
            input_tensors->at("stop_words_list").getPtrWithOffset<const int>(local_batch_offset * 2 * stop_words_length),
            output_tensors->at("finished").getPtrWithOffset<bool>(local_batch_offset), local_batch_offset,
            stop_words_length, (int)batch_size, (int)local_batch_size, (int)beam_width, step, stream_));
    }

    if (input_tensors->isExist("sequence_limit_length")) {
        invokeLengthCriterion(output_tensors->at("finished").getPtr<bool>(),
                              output_tensors->at("should_stop").getPtr<bool>(), h_pinned_finished_sum_,
                              input_tensors->at("sequence_limit_length").getPtr<const uint32_t>(), (int)batch_size,
                              (int)beam_width, step, stream_);
    }
}

template class DynamicDecodeLayer<float>;
template class DynamicDecodeLayer<half>;
template class DynamicDecodeLayer<bfloat16>;

}  // namespace fastertransformer
