#include "src/fastertransformer/layers/sampling_layers/TopKSamplingLayer.h"

#include <algorithm>
#include <cstdlib>

namespace fastertransformer {

// Row routing and clipping of (k, p): what the reference computes on the device in
// setup_topk_runtime_args (layers/sampling_layers/TopKSamplingLayer.cu:28-77) and then copies back.
// Done on the host here; the normalised arrays go to the device once.
static void normaliseTopKArgs(size_t batch_size, uint top_k, std::vector<uint>& top_ks, size_t top_ks_size,
                              float top_p, std::vector<float>& top_ps, size_t top_ps_size,
                              std::vector<uint8_t>& skip_decode)
{
    const uint TOP_K_MAX = 1024;
    for (size_t i = 0; i < batch_size; ++i) {
        uint  k = top_ks_size > 1 ? top_ks[i] : top_k;
        float p = top_ps_size > 1 ? top_ps[i] : top_p;
        if (k == 0 && p == 0.0f) {
            k = 1;  // top_p == 0 without top_k means greedy
        }
        if (k > 0 && p == 0.0f) {
            p = 1.0f;  // plain top-k
        }
        if (k > TOP_K_MAX) {
            FT_LOG_WARNING("topk (%u) is larger than max supported number (%u) for token %zu clip to max supported "
                           "number %u.",
                           k, TOP_K_MAX, i, TOP_K_MAX);
            k = TOP_K_MAX;
        }
        if (p < 0.0f || p > 1.0f) {
            const float clipped = p < 0.0f ? 0.0f : 1.0f;
            FT_LOG_WARNING("topp (%f) is out of range ([0.0, 1.0f]) for token %zu clip to closest number %f.", p, i,
                           clipped);
            p = clipped;
        }
        top_ks[i]      = k;
        top_ps[i]      = p;
        skip_decode[i] = k == 0 ? 1 : 0;
    }
}

template<typename T>
void TopKSamplingLayer<T>::allocateBuffer()
{
    FT_CHECK(false);
}

template<typename T>
void TopKSamplingLayer<T>::allocateBuffer(size_t batch_size, Tensor top_k, Tensor top_p)
{
    BaseSamplingLayer<T>::allocateBuffer(batch_size, top_k, top_p);
    uint max_top_k = top_k.size() > 0 ? top_k.max<uint>() : 1;
    if (max_top_k == 0) {
        max_top_k = 1;  // k == 0 && p == 0 is served as greedy (k = 1)
    }
    if (max_top_k > 1024) {
        max_top_k = 1024;
    }
    // workspace query: null workspace returns the size and launches nothing
    invokeTopKSampling<T>(nullptr, sampling_workspace_size_, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                          nullptr, (int)max_top_k, 1.0f, (int)vocab_size_padded_, nullptr, stream_, (int)batch_size,
                          skip_decode_buf_);
    sampling_workspace_ = allocator_->reMalloc(sampling_workspace_, sampling_workspace_size_, false);
    is_allocate_buffer_ = true;
}

template<typename T>
void TopKSamplingLayer<T>::freeBuffer()
{
    BaseSamplingLayer<T>::freeBuffer();
}

// Two environment switches, read once per setup() (not per step: getenv is neither free nor safe against a
// concurrent setenv in a serving process).
// FT_SAMPLING_DISABLE_FUSED=1 forces the kernel-by-kernel sequence of the reference.
static bool fusedDisabledByEnvironment()
{
    const char* env = std::getenv("FT_SAMPLING_DISABLE_FUSED");
    return env != nullptr && env[0] == '1';
}

// With log-prob outputs the fused step reads the logits twice in one launch (1024 threads per row up to 256 rows, 512
// beyond): measured on MI355X it is ahead of the kernel sequence at every batch from 1 row on (8 x 50257 fp32: 28 us
// against 69 us), so every window takes it. FT_SAMPLING_FUSED_LOGPROBS_MIN_ROWS sets a smallest window that does;
// smaller ones then run the kernel sequence.
static int fusedLogProbsMinRowsFromEnvironment()
{
    const char* env = std::getenv("FT_SAMPLING_FUSED_LOGPROBS_MIN_ROWS");
    return env != nullptr && env[0] != '\0' ? std::atoi(env) : 0;
}

// reference: TopKSamplingLayer<T>::setup, layers/sampling_layers/TopKSamplingLayer.cu:134-186
template<typename T>
void TopKSamplingLayer<T>::setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args)
{
    BaseSamplingLayer<T>::setup(batch_size, beam_width, runtime_args);
    fused_disabled_           = fusedDisabledByEnvironment();
    fused_log_probs_min_rows_ = fusedLogProbsMinRowsFromEnvironment();

    uint         tmp_top_k     = 0;
    const Tensor runtime_top_k = runtime_args->isExist("runtime_top_k") ?
                                     runtime_args->at("runtime_top_k") :
                                     Tensor(MEMORY_CPU, TYPE_UINT32, {1}, &tmp_top_k);
    const Tensor runtime_top_p = runtime_args->isExist("runtime_top_p") ? runtime_args->at("runtime_top_p") : Tensor();
    const size_t runtime_top_k_size = runtime_top_k.size();
    const size_t runtime_top_p_size = runtime_top_p.size();

    const uint  top_k = runtime_top_k.max<uint>();
    const float top_p = runtime_top_p_size == 0 ? 0.0f : runtime_top_p.getVal<float>();

    if (runtime_top_k_size > 1) {
        FT_CHECK_WITH_INFO(runtime_top_k.size() == batch_size,
                           fmtstr("runtime_top_k.size() (%d) == batch_size (%d) is not satisfied!",
                                  (int)runtime_top_k.size(), (int)batch_size));
        std::copy_n(runtime_top_k.getPtr<uint>(), batch_size, runtime_top_k_.begin());
    }
    if (runtime_top_p_size > 1) {
        FT_CHECK_WITH_INFO(runtime_top_p.size() == batch_size,
                           fmtstr("runtime_top_p.size() (%d) == batch_size (%d) is not satisfied!",
                                  (int)runtime_top_p.size(), (int)batch_size));
        std::copy_n(runtime_top_p.getPtr<float>(), batch_size, runtime_top_p_.begin());
    }
    normaliseTopKArgs(batch_size, top_k, runtime_top_k_, runtime_top_k_size, top_p, runtime_top_p_,
                      runtime_top_p_size, skip_decode_);
    runtime_max_top_k_ = *std::max_element(runtime_top_k_.begin(), runtime_top_k_.begin() + batch_size);
    if (runtime_max_top_k_ == 0) {
        runtime_max_top_k_ = 1;  // every row belongs to the top-p layer
    }
    check_hip_error(hipMemcpyAsync(runtime_top_k_buf_, runtime_top_k_.data(), sizeof(uint) * batch_size,
                                   hipMemcpyHostToDevice, stream_));
    check_hip_error(hipMemcpyAsync(runtime_top_p_buf_, runtime_top_p_.data(), sizeof(float) * batch_size,
                                   hipMemcpyHostToDevice, stream_));
    check_hip_error(hipMemcpyAsync(skip_decode_buf_, skip_decode_.data(), sizeof(bool) * batch_size,
                                   hipMemcpyHostToDevice, stream_));
    // the host vectors are read by the copies above: make them safe to modify on return
    check_hip_error(hipStreamSynchronize(stream_));
}

// The chunking of a row depends on the number of rows in the call, so a window smaller than the
// setup batch can need a slightly larger workspace: grow on demand.
template<typename T>
void TopKSamplingLayer<T>::ensureWorkspace(int local_batch_size)
{
    size_t need = 0;
    invokeTopKSampling<T>(nullptr, need, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                          (int)runtime_max_top_k_, 1.0f, (int)vocab_size_padded_, nullptr, stream_, local_batch_size,
                          nullptr);
    if (need > sampling_workspace_size_) {
        sampling_workspace_      = allocator_->reMalloc(sampling_workspace_, need, false);
        sampling_workspace_size_ = need;
    }
}

// One streaming pass over the logits for the whole penalty + mask + top-k pipeline - two passes when log-prob
// outputs are requested, which need the probabilities of the whole row. Not taken for the configurations the fused
// step reports as unsupported (log-probs with a bias or a large k, the frequency-penalty extension outside the
// one-launch step), nor for log-probs on small windows.
template<typename T>
bool TopKSamplingLayer<T>::runFused(TensorMap* output_tensors, TensorMap* input_tensors)
{
    float* cum_log_probs    = output_tensors->at("cum_log_probs", Tensor()).template getPtr<float>();
    float* output_log_probs = output_tensors->at("output_log_probs", Tensor()).template getPtr<float>();
    if (fused_disabled_) {
        return false;
    }
    const int batch_size       = output_tensors->at("output_ids").shape[1];
    const int local_batch_size = input_tensors->at("logits").shape[0];
    const int ite              = input_tensors->at("ite").template getVal<int>();
    const int step             = input_tensors->at("step").template getVal<int>();
    const int max_input_length = input_tensors->at("max_input_length").template getVal<int>();
    const int off              = ite * local_batch_size;
    if ((cum_log_probs != nullptr || output_log_probs != nullptr) && local_batch_size < fused_log_probs_min_rows_) {
        return false;
    }

    ftk_fused_topk_args a{};
    a.dtype             = FtkDType<T>::value;
    a.logits            = input_tensors->at("logits").template getPtr<T>();
    a.embedding_bias    = input_tensors->at("embedding_bias", Tensor()).template getPtr<T>();
    a.vocab_size        = (int)vocab_size_;
    a.vocab_size_padded = (int)vocab_size_padded_;
    a.batch_size        = batch_size;
    a.local_batch_size  = local_batch_size;
    a.step              = step;
    a.max_input_length  = max_input_length;

    const float* temps = this->temperature_.data() + off;
    const bool   temp_active =
        a.embedding_bias != nullptr || !std::all_of(temps, temps + local_batch_size, [](float t) { return t == 1.0f; });
    a.temperatures = temp_active ? this->temperature_buf_ + off : nullptr;

    a.penalty_type = FTK_PENALTY_NONE;
    if (step > 1 && this->repetition_penalty_type_ != RepetitionPenaltyType::None) {
        const float  dflt = getDefaultPenaltyValue(this->repetition_penalty_type_);
        const float* pens = this->repetition_penalty_.data() + off;
        if (!std::all_of(pens, pens + local_batch_size, [&](float x) { return x == dflt; })) {
            a.penalty_type = toFtkPenalty(this->repetition_penalty_type_);
            a.penalties    = this->repetition_penalty_buf_ + off;
        }
        if (this->has_frequency_penalty_) {
            const float* fr = this->frequency_penalty_.data() + off;
            if (!std::all_of(fr, fr + local_batch_size, [](float x) { return x == 0.0f; })) {
                // (x - presence - frequency * count: the presence array goes along even when it is all zeros)
                a.penalty_type        = FTK_PENALTY_ADDITIVE;
                a.penalties           = this->repetition_penalty_buf_ + off;
                a.frequency_penalties = this->frequency_penalty_buf_ + off;
            }
        }
    }
    const int  num_generated_tokens = step - max_input_length;
    const int* min_lengths          = this->min_lengths_.data() + off;
    if (std::any_of(min_lengths, min_lengths + local_batch_size,
                    [&](int m) { return m > num_generated_tokens; })) {
        FT_CHECK_WITH_INFO(input_tensors->isExist("end_id"), "Need end_id to apply min length penlaty");
        a.min_lengths = this->min_lengths_buf_ + off;
        FT_CHECK(output_tensors->template getPtr<const int>("sequence_length") != nullptr);
    }
    a.end_ids       = input_tensors->at("end_id").template getPtr<const int>();
    a.input_lengths = input_tensors->at("input_lengths", Tensor()).template getPtr<const int>();
    a.output_ids    = output_tensors->at("output_ids").template getPtrWithOffset<int>(off);
    a.top_ks        = (const int*)(runtime_top_k_buf_ + off);
    a.top_ps        = runtime_top_p_buf_ + off;
    a.max_top_k     = (int)runtime_max_top_k_;
    a.skip_decode   = skip_decode_buf_ + off;
    a.rng_state     = curandstate_buf_ + off;
    a.uniform_draws = input_tensors->at("uniform_draws", Tensor()).template getPtr<const float>();
    a.ids = output_tensors->at("output_ids").template getPtrWithOffset<int>((size_t)step * batch_size + off);
    a.sequence_length = output_tensors->at("sequence_length", Tensor()).template getPtr<int>();
    a.finished        = output_tensors->at("finished", Tensor()).template getPtr<bool>();
    a.cum_log_probs    = cum_log_probs;
    a.output_log_probs = output_log_probs;
    // size query (null workspace), grow if this window needs more than setup() reserved
    a.workspace = nullptr;
    const int query = ftk_fused_topk_step(&a, stream_);
    if (query == FTK_ERR_UNSUPPORTED) {
        return false;  // log-probs with a bias, a large k or a tiny vocabulary, a frequency penalty outside the
                       // one-launch step: the kernel sequence
    }
    check_ftk(query);
    if (a.workspace_size > sampling_workspace_size_) {
        sampling_workspace_      = allocator_->reMalloc(sampling_workspace_, a.workspace_size, false);
        sampling_workspace_size_ = a.workspace_size;
    }
    a.workspace      = sampling_workspace_;
    a.workspace_size = sampling_workspace_size_;
    check_ftk(ftk_fused_topk_step(&a, stream_));
    sync_check_hip_error();
    return true;
}

// reference: TopKSamplingLayer<T>::runSampling, layers/sampling_layers/TopKSamplingLayer.cu:189-268
template<typename T>
void TopKSamplingLayer<T>::runSampling(TensorMap* output_tensors, TensorMap* input_tensors, T* logits)
{
    const int batch_size       = output_tensors->at("output_ids").shape[1];
    const int local_batch_size = input_tensors->at("logits").shape[0];
    const int ite              = input_tensors->at("ite").template getVal<int>();
    const int step             = input_tensors->at("step").template getVal<int>();
    const int off              = ite * local_batch_size;

    const int* end_ids  = input_tensors->at("end_id").template getPtr<const int>();
    bool*      finished = output_tensors->at("finished", Tensor()).template getPtr<bool>();
    float* cum_log_probs    = output_tensors->at("cum_log_probs", Tensor()).template getPtr<float>();
    float* output_log_probs = output_tensors->at("output_log_probs", Tensor()).template getPtr<float>();
    if (cum_log_probs != nullptr || output_log_probs != nullptr) {
        // The reference masks pads and finished rows (invokeAddBiasEndMask) and then takes the softmax of the
        // result (TopKSamplingLayer.cu:220-245). The softmax applies the very same mask to what it reads
        // (pad columns -> -MAX_T, finished rows -> +-MAX_T by end id), so the first pass over the logits
        // changes nothing in its result and is left out.
        invokeAddBiasSoftMax(logits, (T*)nullptr, end_ids, finished, local_batch_size, (int)vocab_size_padded_,
                             (int)vocab_size_, stream_);
        sync_check_hip_error();
    }
    else {
        invokeAddBiasEndMask(logits, (T*)nullptr, end_ids, finished, local_batch_size, (int)vocab_size_,
                             (int)vocab_size_padded_, stream_);
        sync_check_hip_error();
    }
    ensureWorkspace(local_batch_size);
    invokeBatchTopKSampling(
        sampling_workspace_, sampling_workspace_size_, logits,
        output_tensors->at("output_ids").template getPtrWithOffset<int>((size_t)step * batch_size + off),
        output_tensors->at("sequence_length", Tensor()).template getPtr<int>(), finished, cum_log_probs,
        output_log_probs, curandstate_buf_ + off, (int)runtime_max_top_k_, (const int*)(runtime_top_k_buf_ + off), 1.0f,
        runtime_top_p_buf_ + off, (int)vocab_size_padded_, end_ids, stream_, local_batch_size, skip_decode_buf_ + off,
        input_tensors->at("uniform_draws", Tensor()).template getPtr<const float>());
    sync_check_hip_error();
}

template<typename T>
TopKSamplingLayer<T>::TopKSamplingLayer(size_t max_batch_size, size_t vocab_size, size_t vocab_size_padded, int end_id,
                                        size_t top_k, unsigned long long random_seed, float temperature,
                                        float len_penalty, float repetition_penalty, hipStream_t stream,
                                        cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                        bool is_free_buffer_after_forward):
    BaseSamplingLayer<T>(max_batch_size, vocab_size, vocab_size_padded, end_id, top_k, 0.0f, random_seed, temperature,
                         len_penalty, repetition_penalty, stream, cublas_wrapper, allocator,
                         is_free_buffer_after_forward, nullptr)
{
}

template<typename T>
TopKSamplingLayer<T>::TopKSamplingLayer(TopKSamplingLayer<T> const& other): BaseSamplingLayer<T>(other)
{
}

template<typename T>
TopKSamplingLayer<T>::~TopKSamplingLayer()
{
    freeBuffer();
}

template class TopKSamplingLayer<float>;
template class TopKSamplingLayer<half>;
template class TopKSamplingLayer<bfloat16>;

}  // namespace fastertransformer
