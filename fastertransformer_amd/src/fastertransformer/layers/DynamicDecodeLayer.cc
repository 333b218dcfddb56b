#include "src/fastertransformer/layers/DynamicDecodeLayer.h"

#include <cstring>

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
    online_beamsearch_decode_ =
        new OnlineBeamSearchLayer<T>(0, 0, 0, 0, vocab_size_, vocab_size_padded_, 0, 0.0f, 1.0f, 0.0f, 1.0f, stream_,
                                     cublas_wrapper_, allocator_, is_free_buffer_after_forward_);
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
    delete online_beamsearch_decode_;
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
    online_beamsearch_decode_->setStream(stream);
}

// reference: DynamicDecodeLayer<T>::setup, layers/DynamicDecodeLayer.cc:153-178
template<typename T>
void DynamicDecodeLayer<T>::setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args)
{
    // reference: hasDiffRuntimeArgs, layers/DynamicDecodeLayer.cc:476-514
    has_diff_runtime_args_ = false;
    for (const char* key : {"beam_search_diversity_rate", "temperature", "len_penalty", "repetition_penalty",
                            "presence_penalty", "min_length"}) {
        if (!runtime_args->isExist(key)) {
            continue;
        }
        const Tensor& t = runtime_args->at(key);
        FT_CHECK(t.shape.size() == 1);
        FT_CHECK_WITH_INFO(t.type == TYPE_FP32 || t.type == TYPE_INT32 || t.type == TYPE_UINT32
                               || t.type == TYPE_UINT64,
                           std::string(key) + ": " + t.toString() + " is invalid.");
        const size_t width = Tensor::getTypeSize(t.type);
        const char*  data  = (const char*)t.data;
        for (size_t j = 1; j < t.shape[0]; ++j) {
            has_diff_runtime_args_ = has_diff_runtime_args_ || memcmp(data, data + j * width, width) != 0;
        }
    }
    if (beam_width == 1) {
        topk_decode_->setup(batch_size, beam_width, runtime_args);
        topp_decode_->setup(batch_size, beam_width, runtime_args);
    }
}

template<typename T>
void DynamicDecodeLayer<T>::forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                                    const std::unordered_map<std::string, Tensor>* input_tensors)
{
    TensorMap input_map(*input_tensors);
    TensorMap output_map(*output_tensors);
    forward(&output_map, &input_map);
}

namespace {

// The rows [first, first + count) of a tensor whose leading dimension is the batch: a view, no copy.
Tensor rowWindow(const Tensor& t, size_t first, size_t count)
{
    std::vector<size_t> shape = t.shape;
    size_t              inner = 1;
    for (size_t d = 1; d < shape.size(); ++d) {
        inner *= shape[d];
    }
    shape[0] = count;
    return t.slice(shape, first * inner);
}

// What the two sampling layers see of a step: tensors with one entry per row are cut to the micro-batch window,
// the others are handed over as they are. (Key names: layers/DynamicDecodeLayer.cc:193-235 of the reference.)
const char* const kRowInputs[]   = {"logits", "end_id", "input_lengths", "uniform_draws"};
const char* const kWholeInputs[] = {"step", "max_input_length", "embedding_bias"};
const char* const kRowOutputs[]  = {"sequence_length", "finished", "cum_log_probs"};

}  // namespace

// reference: DynamicDecodeLayer<T>::forward, layers/DynamicDecodeLayer.cc:191-474 (tensor names and
// shapes are documented there, :193-235). Extension: input "uniform_draws" [batch] float on the GPU,
// one draw in (0, 1] per row, replaces the generator for this step.
template<typename T>
void DynamicDecodeLayer<T>::forward(TensorMap* output_tensors, TensorMap* input_tensors)
{
    const Tensor& logits = input_tensors->at("logits");
    FT_CHECK(logits.shape.size() == 3);
    const int    ite   = (int)input_tensors->at("ite").getVal<uint>();
    const int    step  = input_tensors->at("step").getVal<int>();
    const size_t batch = logits.shape[0];
    const size_t rows  = (size_t)input_tensors->at("local_batch_size").getVal<int>();
    const size_t first = (size_t)ite * rows;  // the window: rows [first, first + rows) of the batch
    FT_CHECK_WITH_INFO(first + rows <= batch, "ite / local_batch_size window exceeds the batch");
    if (logits.shape[1] > 1) {
        banBadWords(output_tensors, input_tensors, first, rows, step);
        forwardBeams(output_tensors, input_tensors, ite, rows);
        stopCriteria(output_tensors, input_tensors, first, rows, step);
        return;
    }

    banBadWords(output_tensors, input_tensors, first, rows, step);

    // Every row belongs to exactly one of the two layers (k > 0 or greedy: top-k; k == 0 && p > 0: top-p);
    // both get the same window.
    TensorMap window_in({{"ite", Tensor{MEMORY_CPU, TYPE_INT32, {1}, &ite}}});
    for (const char* key : kWholeInputs) {
        if (input_tensors->isExist(key)) {
            window_in.insert({key, input_tensors->at(key)});
        }
    }
    for (const char* key : kRowInputs) {
        if (input_tensors->isExist(key)) {
            window_in.insert({key, rowWindow(input_tensors->at(key), first, rows)});
        }
    }
    TensorMap window_out({{"output_ids", output_tensors->at("output_ids")}});
    for (const char* key : kRowOutputs) {
        if (output_tensors->isExist(key)) {
            window_out.insert({key, rowWindow(output_tensors->at(key), first, rows)});
        }
    }
    if (output_tensors->isExist("output_log_probs")) {
        // [generated length, batch]: the layers write row 0 of what they are given, so the view starts at this
        // step's row and this window's column (layers/DynamicDecodeLayer.cc:427-435)
        const Tensor& lp        = output_tensors->at("output_log_probs");
        const size_t  generated = (size_t)(step - input_tensors->at("max_input_length").getVal<int>());
        window_out.insert({"output_log_probs", lp.slice({lp.shape[0] - generated, rows}, generated * batch + first)});
    }
    topk_decode_->forward(&window_out, &window_in);
    topp_decode_->forward(&window_out, &window_in);

    stopCriteria(output_tensors, input_tensors, first, rows, step);
}

// reference: the beam_width > 1 branch of DynamicDecodeLayer<T>::forward, layers/DynamicDecodeLayer.cc:286-385. The
// entries of the window go to the beam-search layer together, or one by one when setup() saw per-entry runtime
// values that differ; per-beam state is cut to the sub-window, everything else is handed over whole (including
// the cache indirections, which the layer indexes from the sub-window's first entry, as the reference's does).
template<typename T>
void DynamicDecodeLayer<T>::forwardBeams(TensorMap* output_tensors, TensorMap* input_tensors, int ite, size_t rows)
{
    const Tensor& logits = input_tensors->at("logits");
    const size_t  beams  = logits.shape[1];
    const size_t  group  = has_diff_runtime_args_ ? 1 : rows;  // entries per call of the layer
    const size_t  calls  = rows / group;
    FT_CHECK_WITH_INFO(output_tensors->isExist("cum_log_probs"), "cum_log_probs should be provided in beam search.");
    for (uint sub = (uint)(ite * calls); sub < (uint)((ite + 1) * calls); ++sub) {
        const size_t first_entry = (size_t)sub * group;
        const size_t first_beam  = first_entry * beams;
        TensorMap    in({{"logits", rowWindow(logits, first_entry, group)},
                         {"end_id", rowWindow(input_tensors->at("end_id"), first_entry, group)},
                         {"ite", Tensor{MEMORY_CPU, TYPE_UINT32, {1}, &sub}}});
        if (input_tensors->isExist("input_lengths")) {
            // [batch, beam_width], or the same values as one flat list: one length per beam either way
            const Tensor& t = input_tensors->at("input_lengths");
            in.insert({"input_lengths", Tensor{t.where, t.type, {group, beams}, t.getPtrWithOffset(first_beam)}});
        }
        for (auto it = input_tensors->begin(); it != input_tensors->end(); ++it) {
            // step, max_input_length, embedding_bias, src_cache_indirection and the runtime values of the step
            if (!in.isExist(it->first) && it->first.find("random_seed") == std::string::npos) {
                in.insert({it->first, it->second});
            }
        }
        TensorMap out;
        for (const char* key : {"output_ids", "parent_ids", "tgt_cache_indirection", "output_log_probs", "beam_hyps"}) {
            if (output_tensors->isExist(key)) {
                out.insert({key, output_tensors->at(key)});
            }
        }
        for (const char* key : kRowOutputs) {
            if (output_tensors->isExist(key)) {
                const Tensor& t = output_tensors->at(key);  // [batch * beam_width]
                out.insert({key, Tensor{t.where, t.type, {group * beams}, t.getPtrWithOffset(first_beam)}});
            }
        }
        online_beamsearch_decode_->forward(&out, &in);
    }
}

// Bad words are masked on the caller's logits before either layer looks at them (layers/DynamicDecodeLayer.cc:
// 248-281): a [2, L] list serves every row (so does [1, 2, L] at batch 1); [batch, 2, L] has a list per row.
template<typename T>
void DynamicDecodeLayer<T>::banBadWords(TensorMap* output_tensors, TensorMap* input_tensors, size_t first, size_t rows,
                                        int step)
{
    if (!input_tensors->isExist("bad_words_list")) {
        return;
    }
    const Tensor& words = input_tensors->at("bad_words_list");
    const size_t  rank  = words.shape.size();
    const size_t  batch = input_tensors->at("logits").shape[0];
    FT_CHECK_WITH_INFO(rank == 2 || rank == 3, "Bad words dimension must be 2 or 3.");
    FT_CHECK_WITH_INFO(rank == 2 || words.shape[0] == batch,
                       fmtstr("Shape of dim 0 of bad words is invalid. It must be equal to batch size."
                              " However, it is %d and the batch size is %d.",
                              (int)words.shape[0], (int)batch));
    const bool   one_list = rank == 2 || words.shape[0] == 1;
    const size_t length   = words.shape[rank - 1];
    const int*   lists    = one_list ? words.getPtr<const int>() : words.getPtrWithOffset<const int>(first * 2 * length);
    // The window starts `first` entries, that is first * beams rows of logits and columns of the history, into the
    // batch. (The reference offsets both by `first` whatever the beam width, layers/DynamicDecodeLayer.cc:261-280:
    // with beams, a later window's bans then land on other beams' rows and follow other beams' histories. Not
    // reproduced; the stop-word launch of the reference, :449-462, already counts in beams.)
    const size_t beams = input_tensors->at("logits").shape[1];
    invokeBanBadWords((T*)input_tensors->at("logits").getPtrWithOffset(first * beams * vocab_size_padded_),
                      output_tensors->at("output_ids").getPtr<const int>(),
                      beams > 1 ? output_tensors->at("parent_ids").getPtr<const int>() : (const int*)nullptr,
                      (int)batch, (int)rows, (int)beams, lists, one_list, length, (int)(first * beams),
                      (int)vocab_size_padded_, (size_t)step, stream_);
}

// After sampling: stop words on the rows of this window (layers/DynamicDecodeLayer.cc:449-462; the reference
// examines `batch` rows from the window's start, which runs past the window), then the length criterion on the
// whole batch, which also tells the host whether every row is finished (:464-473).
template<typename T>
void DynamicDecodeLayer<T>::stopCriteria(TensorMap* output_tensors, TensorMap* input_tensors, size_t first,
                                         size_t rows, int step)
{
    const size_t batch = input_tensors->at("logits").shape[0];
    const size_t beams = input_tensors->at("logits").shape[1];
    if (input_tensors->isExist("stop_words_list")) {
        const Tensor& words  = input_tensors->at("stop_words_list");
        const size_t  length = words.shape[2];
        FT_CHECK_WITH_INFO(output_tensors->at("finished", Tensor()).getPtr<bool>() != nullptr,
                           "stop_words_list needs the finished output");
        check_ftk(ftk_invoke_stop_words_criterion_rows(
            output_tensors->at("output_ids").getPtr<const int>(),
            beams > 1 ? output_tensors->at("parent_ids").getPtr<const int>() : nullptr,
            words.getPtrWithOffset<const int>(first * 2 * length),
            output_tensors->at("finished").getPtrWithOffset<bool>(first * beams), first * beams, length, (int)batch,
            (int)rows, (int)beams, step, stream_));
    }
    if (input_tensors->isExist("sequence_limit_length")) {
        invokeLengthCriterion(output_tensors->at("finished").getPtr<bool>(),
                              output_tensors->at("should_stop").getPtr<bool>(), h_pinned_finished_sum_,
                              input_tensors->at("sequence_limit_length").getPtr<const uint32_t>(), (int)batch,
                              (int)beams, step, stream_);
    }
}

template class DynamicDecodeLayer<float>;
template class DynamicDecodeLayer<half>;
template class DynamicDecodeLayer<bfloat16>;

}  // namespace fastertransformer
