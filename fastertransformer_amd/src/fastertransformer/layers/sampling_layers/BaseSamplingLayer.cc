#include "src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.h"

#include <algorithm>

namespace fastertransformer {

template<typename T>
void BaseSamplingLayer<T>::allocateBuffer()
{
    FT_CHECK(false);
}

template<typename T>
void BaseSamplingLayer<T>::allocateBuffer(size_t batch_size, Tensor top_k, Tensor top_p)
{
    (void)top_k;
    (void)top_p;
    auto dev = [&](auto* ptr, size_t bytes) { return allocator_->reMalloc(ptr, bytes, false); };
    curandstate_buf_        = (curandState_t*)dev(curandstate_buf_, sizeof(curandState_t) * batch_size);
    temperature_buf_        = (float*)dev(temperature_buf_, sizeof(float) * batch_size);
    repetition_penalty_buf_ = (float*)dev(repetition_penalty_buf_, sizeof(float) * batch_size);
    frequency_penalty_buf_  = (float*)dev(frequency_penalty_buf_, sizeof(float) * batch_size);
    min_lengths_buf_        = (int*)dev(min_lengths_buf_, sizeof(int) * batch_size);
    skip_decode_buf_        = (bool*)dev(skip_decode_buf_, sizeof(bool) * batch_size);
    runtime_top_k_buf_      = (uint*)dev(runtime_top_k_buf_, sizeof(uint) * batch_size);
    runtime_top_p_buf_      = (float*)dev(runtime_top_p_buf_, sizeof(float) * batch_size);
    temperature_.resize(batch_size);
    repetition_penalty_.resize(batch_size);
    frequency_penalty_.resize(batch_size);
    min_lengths_.resize(batch_size);
    skip_decode_.resize(batch_size);
    runtime_top_k_.resize(batch_size);
    runtime_top_p_.resize(batch_size);
    is_allocate_buffer_ = true;
}

template<typename T>
void BaseSamplingLayer<T>::freeBuffer()
{
    if (is_allocate_buffer_) {
        allocator_->free((void**)(&curandstate_buf_));
        allocator_->free((void**)(&temperature_buf_));
        allocator_->free((void**)(&repetition_penalty_buf_));
        allocator_->free((void**)(&frequency_penalty_buf_));
        allocator_->free((void**)(&min_lengths_buf_));
        allocator_->free((void**)(&skip_decode_buf_));
        allocator_->free((void**)(&runtime_top_k_buf_));
        allocator_->free((void**)(&runtime_top_p_buf_));
        if (runtime_logits_buf_ != nullptr) {
            allocator_->free((void**)(&runtime_logits_buf_));
            runtime_logits_capacity_ = 0;
        }
        if (sampling_workspace_ != nullptr) {
            allocator_->free((void**)(&sampling_workspace_));
        }
        is_allocate_buffer_ = false;
    }
}

template<typename T>
BaseSamplingLayer<T>::BaseSamplingLayer(size_t max_batch_size, size_t vocab_size, size_t vocab_size_padded, int end_id,
                                        size_t top_k, float top_p, unsigned long long random_seed, float temperature,
                                        float len_penalty, float repetition_penalty, hipStream_t stream,
                                        cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                        bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop):
    DynamicDecodeBaseLayer(stream, cublas_wrapper, allocator, is_free_buffer_after_forward, cuda_device_prop),
    vocab_size_(vocab_size),
    vocab_size_padded_(vocab_size_padded)
{
    // the remaining constructor arguments are deprecated in the reference as well; runtime values
    // arrive through setup()
    (void)max_batch_size;
    (void)end_id;
    (void)top_k;
    (void)top_p;
    (void)random_seed;
    (void)temperature;
    (void)len_penalty;
    (void)repetition_penalty;
}

template<typename T>
BaseSamplingLayer<T>::BaseSamplingLayer(BaseSamplingLayer const& other):
    DynamicDecodeBaseLayer(other), vocab_size_(other.vocab_size_), vocab_size_padded_(other.vocab_size_padded_)
{
}

template<typename T>
BaseSamplingLayer<T>::~BaseSamplingLayer()
{
}

// Broadcast a [1] or copy a [batch] host argument into the host mirror and the device buffer.
template<typename T>
template<typename V>
void BaseSamplingLayer<T>::fillFromArg(std::vector<V>& host, V* device, const Tensor& arg, size_t batch_size)
{
    FT_CHECK_WITH_INFO(arg.size() == 1 || arg.size() == batch_size,
                       fmtstr("runtime argument must be of shape [1] or [batch_size(%ld)], got %s", batch_size,
                              vec2str(arg.shape).c_str()));
    if (arg.size() == 1) {
        std::fill_n(host.begin(), batch_size, arg.getVal<V>());
    }
    else {
        std::copy_n(arg.getPtr<V>(), batch_size, host.begin());
    }
    check_hip_error(hipMemcpyAsync(device, host.data(), sizeof(V) * batch_size, hipMemcpyHostToDevice, stream_));
}

// reference: BaseSamplingLayer<T>::setup, layers/sampling_layers/BaseSamplingLayer.cc:112-206
template<typename T>
void BaseSamplingLayer<T>::setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args)
{
    (void)beam_width;
    Tensor runtime_top_k = runtime_args->isExist("runtime_top_k") ? runtime_args->at("runtime_top_k") : Tensor();
    Tensor runtime_top_p = runtime_args->isExist("runtime_top_p") ? runtime_args->at("runtime_top_p") : Tensor();
    allocateBuffer(batch_size, runtime_top_k, runtime_top_p);
    setup_batch_size_ = batch_size;

    // generator: one seed for all rows, one per row, or seed 0
    if (runtime_args->isExist("random_seed")) {
        Tensor random_seeds = runtime_args->at("random_seed");
        FT_CHECK_WITH_INFO(random_seeds.shape.size() == 1
                               && (random_seeds.size() == 1 || random_seeds.size() == batch_size),
                           fmtstr("random_seeds must be of shape [1] or [batch_size(%ld)], got random_seeds.shape=%s",
                                  batch_size, vec2str(random_seeds.shape).c_str()));
        std::vector<ftk_rng_state> states(batch_size);
        for (size_t i = 0; i < batch_size; ++i) {
            states[i].seed   = random_seeds.getVal<unsigned long long>(random_seeds.size() == 1 ? 0 : i);
            states[i].offset = 0;
        }
        // on the layer's stream, so that it is ordered against steps still queued there; `states` is a
        // temporary, so the copy is waited for
        check_hip_error(hipMemcpyAsync(curandstate_buf_, states.data(), sizeof(ftk_rng_state) * batch_size,
                                       hipMemcpyHostToDevice, stream_));
        check_hip_error(hipStreamSynchronize(stream_));
    }
    else {
        invokeCurandInitialize(curandstate_buf_, batch_size, 0, stream_);
    }

    const float default_temperature = 1.0f;
    Tensor      temperature = runtime_args->at("temperature", Tensor(MEMORY_CPU, TYPE_FP32, {1}, &default_temperature));
    fillFromArg(temperature_, temperature_buf_, temperature, batch_size);

    const bool has_rep  = runtime_args->isExist("repetition_penalty");
    const bool has_pres = runtime_args->isExist("presence_penalty");
    const bool has_freq = runtime_args->isExist("frequency_penalty");
    FT_CHECK_WITH_INFO(!(has_rep && (has_pres || has_freq)),
                       "Found ambiguous parameters repetition_penalty and presence_penalty which are mutually "
                       "exclusive. Please provide one of repetition_penalty or presence_penalty.");
    has_frequency_penalty_ = has_freq;
    if (has_rep || has_pres || has_freq) {
        repetition_penalty_type_ = has_rep ? RepetitionPenaltyType::Multiplicative : RepetitionPenaltyType::Additive;
        const float zero         = 0.0f;
        Tensor      penalty      = has_rep  ? runtime_args->at("repetition_penalty") :
                                   has_pres ? runtime_args->at("presence_penalty") :
                                              Tensor(MEMORY_CPU, TYPE_FP32, {1}, &zero);
        fillFromArg(repetition_penalty_, repetition_penalty_buf_, penalty, batch_size);
        if (has_freq) {
            fillFromArg(frequency_penalty_, frequency_penalty_buf_, runtime_args->at("frequency_penalty"), batch_size);
        }
    }
    else {
        repetition_penalty_type_ = RepetitionPenaltyType::None;
    }

    const int default_min_length = 0;
    Tensor    min_lengths = runtime_args->at("min_length", Tensor(MEMORY_CPU, TYPE_INT32, {1}, &default_min_length));
    fillFromArg(min_lengths_, min_lengths_buf_, min_lengths, batch_size);
}

template<typename T>
void BaseSamplingLayer<T>::forward(std::vector<Tensor>* output_tensors, const std::vector<Tensor>* input_tensors)
{
    (void)output_tensors;
    (void)input_tensors;
    FT_CHECK(false);  // positional overload is dead in the reference too (BaseSamplingLayer.cc:226)
}

template<typename T>
void BaseSamplingLayer<T>::forward(std::unordered_map<std::string, Tensor>*       output_tensors,
                                   const std::unordered_map<std::string, Tensor>* input_tensors)
{
    TensorMap input_map(*input_tensors);
    TensorMap output_map(*output_tensors);
    forward(&output_map, &input_map);
}

// reference: BaseSamplingLayer<T>::forward, layers/sampling_layers/BaseSamplingLayer.cc:255-359
template<typename T>
void BaseSamplingLayer<T>::forward(TensorMap* output_tensors, TensorMap* input_tensors)
{
    FT_CHECK(input_tensors->size() >= 4);
    FT_CHECK(output_tensors->size() >= 1);
    const int batch_size       = output_tensors->at("output_ids").shape[1];
    const int local_batch_size = input_tensors->at("logits").shape[0];
    const int step             = input_tensors->at("step").getVal<int>();
    const int ite              = input_tensors->at("ite").getVal<int>();
    const int max_input_length = input_tensors->at("max_input_length").getVal<int>();
    T*        logits           = input_tensors->at("logits").getPtr<T>();
    const int off              = ite * local_batch_size;
    FT_CHECK_WITH_INFO((size_t)(off + local_batch_size) <= setup_batch_size_,
                       "forward() window exceeds the batch size given to setup()");

    const uint8_t* skip = skip_decode_.data() + off;
    if (std::all_of(skip, skip + local_batch_size, [](uint8_t s) { return s != 0; })) {
        return;  // no row of this window belongs to this layer
    }
    skip_any_ = std::any_of(skip, skip + local_batch_size, [](uint8_t s) { return s != 0; });

    if (runFused(output_tensors, input_tensors)) {
        if (is_free_buffer_after_forward_) {
            freeBuffer();
        }
        return;
    }

    if (skip_any_) {
        // both layers run on this window: work on a private copy so the other layer still sees the
        // caller's logits
        const size_t n = input_tensors->at("logits").size();
        FT_CHECK(n == (size_t)local_batch_size * vocab_size_padded_);
        if (runtime_logits_capacity_ < n) {
            runtime_logits_buf_      = (T*)allocator_->reMalloc(runtime_logits_buf_, sizeof(T) * n, false);
            runtime_logits_capacity_ = n;
        }
        check_hip_error(hipMemcpyAsync(runtime_logits_buf_, logits, sizeof(T) * n, hipMemcpyDeviceToDevice, stream_));
        logits = runtime_logits_buf_;
    }

    const T* embedding_bias =
        input_tensors->isExist("embedding_bias") ? input_tensors->at("embedding_bias").getPtr<T>() : nullptr;
    const float* temps = temperature_.data() + off;
    if (embedding_bias != nullptr
        || !std::all_of(temps, temps + local_batch_size, [](float t) { return t == 1.0f; })) {
        invokeBatchApplyTemperaturePenalty(logits, embedding_bias, temperature_buf_ + off, local_batch_size,
                                           (int)vocab_size_, (int)vocab_size_padded_, stream_);
    }
    sync_check_hip_error();

    if (step > 1 && repetition_penalty_type_ != RepetitionPenaltyType::None) {
        const float  default_value = getDefaultPenaltyValue(repetition_penalty_type_);
        const float* pens          = repetition_penalty_.data() + off;
        bool all_default = std::all_of(pens, pens + local_batch_size, [&](float x) { return x == default_value; });
        if (has_frequency_penalty_) {
            const float* fr = frequency_penalty_.data() + off;
            all_default     = all_default && std::all_of(fr, fr + local_batch_size, [](float x) { return x == 0.0f; });
        }
        if (!all_default) {
            const int* history       = output_tensors->at("output_ids").getPtrWithOffset<int>(off);
            const int* input_lengths = input_tensors->at("input_lengths", Tensor{MEMORY_GPU, TYPE_INT32, {}, nullptr})
                                           .template getPtr<int>();
            if (has_frequency_penalty_) {
                invokeBatchApplyFrequencyPenalty(logits, repetition_penalty_buf_ + off, frequency_penalty_buf_ + off,
                                                 history, batch_size, local_batch_size, (int)vocab_size_padded_,
                                                 input_lengths, max_input_length, step, stream_);
            }
            else {
                invokeBatchApplyRepetitionPenalty(logits, repetition_penalty_buf_ + off, history, batch_size,
                                                  local_batch_size, (int)vocab_size_padded_, input_lengths,
                                                  max_input_length, step, repetition_penalty_type_, stream_);
            }
            sync_check_hip_error();
        }
    }

    const int  num_generated_tokens = step - max_input_length;
    const int* min_lengths          = min_lengths_.data() + off;
    if (std::any_of(min_lengths, min_lengths + local_batch_size,
                    [&](int min_length) { return min_length > num_generated_tokens; })) {
        FT_CHECK_WITH_INFO(input_tensors->isExist("end_id"), "Need end_id to apply min length penlaty");
        invokeMinLengthPenalty(logits, min_lengths_buf_ + off, input_tensors->getPtr<const int>("end_id"),
                               output_tensors->getPtr<const int>("sequence_length"), max_input_length,
                               local_batch_size, (int)vocab_size_padded_, stream_);
        sync_check_hip_error();
    }

    runSampling(output_tensors, input_tensors, logits);

    if (is_free_buffer_after_forward_) {
        freeBuffer();
    }
    sync_check_hip_error();
}

template class BaseSamplingLayer<float>;
template class BaseSamplingLayer<half>;
template class BaseSamplingLayer<bfloat16>;

}  // namespace fastertransformer
