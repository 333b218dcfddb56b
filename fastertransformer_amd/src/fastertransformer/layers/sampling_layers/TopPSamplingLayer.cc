#include <cstdlib>
#include "src/fastertransformer/layers/sampling_layers/TopPSamplingLayer.h"

#include <algorithm>

namespace fastertransformer {

template<typename T>
void TopPSamplingLayer<T>::allocateBuffer()
{
    FT_CHECK(false);
}

template<typename T>
void TopPSamplingLayer<T>::allocateBuffer(size_t batch_size, Tensor top_k, Tensor top_p)
{
    BaseSamplingLayer<T>::allocateBuffer(batch_size, top_k, top_p);
    auto dev = [&](auto* ptr, size_t bytes) { return allocator_->reMalloc(ptr, bytes, false); };
    initial_top_p_buf_   = (float*)dev(initial_top_p_buf_, sizeof(float) * batch_size);
    top_p_decay_buf_     = (float*)dev(top_p_decay_buf_, sizeof(float) * batch_size);
    top_p_min_buf_       = (float*)dev(top_p_min_buf_, sizeof(float) * batch_size);
    top_p_reset_ids_buf_ = (int32_t*)dev(top_p_reset_ids_buf_, sizeof(int32_t) * batch_size);
    is_allocate_buffer_  = true;
}

template<typename T>
void TopPSamplingLayer<T>::freeBuffer()
{
    if (is_allocate_buffer_) {
        allocator_->free((void**)(&initial_top_p_buf_));
        allocator_->free((void**)(&top_p_decay_buf_));
        allocator_->free((void**)(&top_p_min_buf_));
        allocator_->free((void**)(&top_p_reset_ids_buf_));
    }
    BaseSamplingLayer<T>::freeBuffer();
}

// reference: TopPSamplingLayer<T>::setup (layers/sampling_layers/TopPSamplingLayer.cu:184-253) and its
// device-side set_topp_runtime_args (:30-109); the normalisation runs on the host here.
// top_p_decay / top_p_min / top_p_reset_ids arrive as [batch] device tensors, as in the reference.
template<typename T>
void TopPSamplingLayer<T>::setup(const size_t batch_size, const size_t beam_width, TensorMap* runtime_args)
{
    BaseSamplingLayer<T>::setup(batch_size, beam_width, runtime_args);
    {
        // The reference leaves the probabilities in the logits buffer (TopPSamplingLayer.cu:287-297); nothing in its
        // decode loop reads them again, so by default the step samples straight from the logits and leaves them
        // alone. FT_SAMPLING_DISABLE_FUSED=1 (the switch that makes the top-k layer mutate the logits like the
        // reference, read once per setup() as there) keeps that side effect.
        const char* env     = std::getenv("FT_SAMPLING_DISABLE_FUSED");
        keep_probabilities_ = env != nullptr && env[0] == '1';
    }
    const Tensor runtime_top_p = runtime_args->isExist("runtime_top_p") ? runtime_args->at("runtime_top_p") : Tensor();
    const size_t runtime_top_p_size = runtime_top_p.size();
    if (runtime_top_p_size == 0) {
        std::fill_n(skip_decode_.begin(), batch_size, (uint8_t)1);
        return;
    }
    uint         tmp_top_k          = 0;
    const Tensor runtime_top_k      = runtime_args->isExist("runtime_top_k") ?
                                          runtime_args->at("runtime_top_k") :
                                          Tensor(MEMORY_CPU, TYPE_UINT32, {1}, &tmp_top_k);
    const size_t runtime_top_k_size = runtime_top_k.size();
    const uint   top_k              = runtime_top_k.getVal<uint>();
    const float  top_p              = runtime_top_p.getVal<float>();
    if (runtime_top_k_size > 1) {
        FT_CHECK(runtime_top_k.size() == batch_size);
        std::copy_n(runtime_top_k.getPtr<uint>(), batch_size, runtime_top_k_.begin());
    }
    if (runtime_top_p_size > 1) {
        FT_CHECK(runtime_top_p.size() == batch_size);
        std::copy_n(runtime_top_p.getPtr<float>(), batch_size, runtime_top_p_.begin());
    }

    std::vector<float>   decay(batch_size, 1.0f), pmin(batch_size, 1e-6f);
    std::vector<int32_t> reset(batch_size, -1);
    auto fetch = [&](const char* key, void* dst, size_t elem) {
        if (!runtime_args->isExist(key)) {
            return;
        }
        const Tensor t = runtime_args->at(key);
        FT_CHECK_WITH_INFO(t.size() == batch_size, fmtstr("%s must be of shape [batch_size]", key));
        // ordered after whatever produced the tensor on this layer's stream, then waited for
        check_hip_error(hipMemcpyAsync(dst, t.data, elem * batch_size,
                                       t.where == MEMORY_GPU ? hipMemcpyDeviceToHost : hipMemcpyHostToHost, stream_));
        check_hip_error(hipStreamSynchronize(stream_));
    };
    fetch("top_p_decay", decay.data(), sizeof(float));
    fetch("top_p_min", pmin.data(), sizeof(float));
    fetch("top_p_reset_ids", reset.data(), sizeof(int32_t));

    for (size_t i = 0; i < batch_size; ++i) {
        uint  k = runtime_top_k_size > 1 ? runtime_top_k_[i] : top_k;
        float p = runtime_top_p_size > 1 ? runtime_top_p_[i] : top_p;
        if (k == 0 && p == 0.0f) {
            k = 1;  // greedy rows belong to the top-k layer
        }
        if (p < 0.0f || p > 1.0f) {
            const float clipped = p < 0.0f ? 0.0f : 1.0f;
            FT_LOG_WARNING("topp (%f) is out of range ([0.0, 1.0f]) for token %zu clip to closest number %f.", p, i,
                           clipped);
            p = clipped;
        }
        runtime_top_k_[i] = k;
        runtime_top_p_[i] = p;
        skip_decode_[i]   = k > 0 ? 1 : 0;
        if (decay[i] > 1.0f || decay[i] <= 0.0f) {
            FT_LOG_WARNING("top_p_decay_buf (%f) is out of range ([0.0, 1.0f]) for token %zu, change to 1.0f.",
                           decay[i], i);
            decay[i] = 1.0f;
        }
        if (pmin[i] > 1.0f || pmin[i] <= 0.0f) {
            FT_LOG_WARNING("top_p_min_buf (%f) is out of range ([0.0, 1.0f]) for token %zu, change to 0.5f.", pmin[i],
                           i);
            pmin[i] = 0.5f;
        }
    }
    runtime_max_top_p_ = *std::max_element(runtime_top_p_.begin(), runtime_top_p_.begin() + batch_size);
    auto h2d = [&](void* dst, const void* src, size_t bytes) {
        check_hip_error(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream_));
    };
    h2d(runtime_top_k_buf_, runtime_top_k_.data(), sizeof(uint) * batch_size);
    h2d(runtime_top_p_buf_, runtime_top_p_.data(), sizeof(float) * batch_size);
    h2d(initial_top_p_buf_, runtime_top_p_.data(), sizeof(float) * batch_size);
    h2d(skip_decode_buf_, skip_decode_.data(), sizeof(bool) * batch_size);
    h2d(top_p_decay_buf_, decay.data(), sizeof(float) * batch_size);
    h2d(top_p_min_buf_, pmin.data(), sizeof(float) * batch_size);
    h2d(top_p_reset_ids_buf_, reset.data(), sizeof(int32_t) * batch_size);
    check_hip_error(hipStreamSynchronize(stream_));  // sources are host temporaries

    // fallback-sort workspace (only rows that draw deep into a flat distribution touch it)
    const bool any_row = std::any_of(skip_decode_.begin(), skip_decode_.begin() + batch_size,
                                     [](uint8_t s) { return s == 0; });
    if (any_row) {
        cub_temp_storage_size_ = 0;
        invokeFusedTopPStep<T>(nullptr, sampling_workspace_size_, nullptr, nullptr, (int)vocab_size_,
                               vocab_size_padded_, (int)batch_size, nullptr, nullptr, nullptr, nullptr, nullptr,
                               nullptr, nullptr, nullptr, 0.0f, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                               stream_);
        sampling_workspace_ = allocator_->reMalloc(sampling_workspace_, sampling_workspace_size_, false);
    }
}

// reference: TopPSamplingLayer<T>::runSampling, layers/sampling_layers/TopPSamplingLayer.cu:256-343
// (invokeTopPInitialize is not needed: no id table is ever read)
template<typename T>
void TopPSamplingLayer<T>::runSampling(TensorMap* output_tensors, TensorMap* input_tensors, T* logits)
{
    const int batch_size       = output_tensors->at("output_ids").shape[1];
    const int local_batch_size = input_tensors->at("logits").shape[0];
    const int step             = input_tensors->at("step").template getVal<int>();
    const int ite              = input_tensors->at("ite").template getVal<int>();
    const int off              = ite * local_batch_size;

    const int* end_ids  = input_tensors->at("end_id").template getPtr<const int>();
    bool*      finished = output_tensors->at("finished", Tensor()).template getPtr<bool>();
    float* cum_log_probs    = output_tensors->at("cum_log_probs", Tensor()).template getPtr<float>();
    float* output_log_probs = output_tensors->at("output_log_probs", Tensor()).template getPtr<float>();
    int*   ids = output_tensors->at("output_ids").template getPtrWithOffset<int>((size_t)step * batch_size + off);

    // The reference's three launches per step (softmax, sampler, decay) go out as one call: the sampler's first
    // pass over the row rides on the softmax's last one and the decay on the sampler's last kernel. The chunking
    // of a row depends on the number of rows in the call, so a window smaller than the setup batch can need a
    // slightly larger workspace: ask for this window's size and grow on demand.
    size_t need = 0;
    invokeFusedTopPStep<T>(nullptr, need, nullptr, nullptr, (int)vocab_size_, vocab_size_padded_, local_batch_size,
                           nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0.0f, nullptr,
                           nullptr, nullptr, nullptr, nullptr, nullptr, stream_);
    if (need > sampling_workspace_size_) {
        sampling_workspace_      = allocator_->reMalloc(sampling_workspace_, need, false);
        sampling_workspace_size_ = need;
    }
    if (!keep_probabilities_
        && invokeFusedTopPSampleStep<T>(
            sampling_workspace_, sampling_workspace_size_, logits, (int)vocab_size_, vocab_size_padded_,
            local_batch_size, end_ids, finished,
            output_tensors->at("sequence_length", Tensor()).template getPtr<int>(), ids, cum_log_probs,
            output_log_probs, curandstate_buf_ + off,
            input_tensors->at("uniform_draws", Tensor()).template getPtr<const float>(), runtime_max_top_p_,
            runtime_top_p_buf_ + off, initial_top_p_buf_ + off, top_p_decay_buf_ + off, top_p_min_buf_ + off,
            top_p_reset_ids_buf_ + off, skip_decode_buf_ + off, stream_)) {
        sync_check_hip_error();
        return;
    }
    invokeFusedTopPStep<T>(sampling_workspace_, sampling_workspace_size_, logits, (const T*)nullptr, (int)vocab_size_,
                           vocab_size_padded_, local_batch_size, end_ids, finished,
                           output_tensors->at("sequence_length", Tensor()).template getPtr<int>(), ids, cum_log_probs,
                           output_log_probs, curandstate_buf_ + off,
                           input_tensors->at("uniform_draws", Tensor()).template getPtr<const float>(),
                           runtime_max_top_p_, runtime_top_p_buf_ + off, initial_top_p_buf_ + off,
                           top_p_decay_buf_ + off, top_p_min_buf_ + off, top_p_reset_ids_buf_ + off,
                           skip_decode_buf_ + off, stream_);
    sync_check_hip_error();
}

template<typename T>
TopPSamplingLayer<T>::TopPSamplingLayer(size_t max_batch_size, size_t vocab_size, size_t vocab_size_padded, int end_id,
                                        float top_p, unsigned long long random_seed, float temperature,
                                        float len_penalty, float repetition_penalty, hipStream_t stream,
                                        cublasMMWrapper* cublas_wrapper, IAllocator* allocator,
                                        bool is_free_buffer_after_forward, cudaDeviceProp* cuda_device_prop):
    BaseSamplingLayer<T>(max_batch_size, vocab_size, vocab_size_padded, end_id, 0, top_p, random_seed, temperature,
                         len_penalty, repetition_penalty, stream, cublas_wrapper, allocator,
                         is_free_buffer_after_forward, cuda_device_prop)
{
}

template<typename T>
TopPSamplingLayer<T>::TopPSamplingLayer(TopPSamplingLayer<T> const& other): BaseSamplingLayer<T>(other)
{
}

template<typename T>
TopPSamplingLayer<T>::~TopPSamplingLayer()
{
    freeBuffer();
}

template class TopPSamplingLayer<float>;
template class TopPSamplingLayer<half>;
template class TopPSamplingLayer<bfloat16>;

}  // namespace fastertransformer
