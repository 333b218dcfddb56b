// C++ launchers with the reference's names and parameter order, forwarding to the C ABI of
// libftk_sampling.so (include/ftk_sampling.h). They replace the declarations of the reference's
//   src/fastertransformer/kernels/sampling_topk_kernels.h
//   src/fastertransformer/kernels/sampling_topp_kernels.h
//   src/fastertransformer/kernels/sampling_penalty_kernels.h
//   src/fastertransformer/kernels/ban_bad_words.h
//   src/fastertransformer/kernels/stop_criteria_kernels.h
// Differences: hipStream_t for cudaStream_t; ftk_rng_state* for curandState_t* followed by an
// optional `uniform_draws` device array (defaulted, so reference call sites compile unchanged apart
// from the state type); C-ABI return codes are re-thrown as the exceptions the reference throws.
#pragma once
#include "src/fastertransformer/kernels/penalty_types.h"
#include "src/fastertransformer/utils/Tensor.h"

namespace fastertransformer {

typedef ftk_rng_state curandState_t;  // call sites keep the reference's spelling

template<typename T>
struct FtkDType;
template<>
struct FtkDType<float> {
    static constexpr int value = FTK_DTYPE_F32;
};
template<>
struct FtkDType<half> {
    static constexpr int value = FTK_DTYPE_F16;
};
template<>
struct FtkDType<bfloat16> {
    static constexpr int value = FTK_DTYPE_BF16;
};

inline int toFtkPenalty(RepetitionPenaltyType t)
{
    return t == RepetitionPenaltyType::Additive ? FTK_PENALTY_ADDITIVE :
           t == RepetitionPenaltyType::Multiplicative ? FTK_PENALTY_MULTIPLICATIVE : FTK_PENALTY_NONE;
}

// ---- sampling_topk_kernels.h ----------------------------------------------------------------
inline void invokeCurandInitialize(curandState_t* state, const size_t batch_size, unsigned long long random_seed,
                                   hipStream_t stream)
{
    check_ftk(ftk_invoke_curand_initialize(state, batch_size, random_seed, stream));
}

inline void invokeCurandBatchInitialize(curandState_t* states, const size_t batch_size,
                                        const unsigned long long* random_seeds, hipStream_t stream)
{
    check_ftk(ftk_invoke_curand_batch_initialize(states, batch_size, random_seeds, stream));
}

template<typename T>
void invokeAddBiasEndMask(T* logits, const T* bias, const int* end_ids, const bool* finished, const int batch_size,
                          const int vocab_size, const int vocab_size_padded, hipStream_t stream)
{
    check_ftk(ftk_invoke_add_bias_end_mask(FtkDType<T>::value, logits, bias, end_ids, finished, batch_size, vocab_size,
                                           vocab_size_padded, stream));
}

template<typename T>
void invokeBatchTopKSampling(void* workspace, size_t& workspace_size, const T* log_probs, int* ids,
                             int* sequence_length, bool* finished, float* cum_log_probs, float* output_log_probs,
                             curandState_t* curandstate, const int max_top_k, const int* top_ks, const float top_p,
                             const float* top_ps, const int vocab_size_padded, const int* end_ids, hipStream_t stream,
                             const int batch_size, const bool* skip_decode, const float* uniform_draws = nullptr)
{
    check_ftk(ftk_invoke_batch_topk_sampling(FtkDType<T>::value, workspace, &workspace_size, log_probs, ids,
                                             sequence_length, finished, cum_log_probs, output_log_probs, curandstate,
                                             uniform_draws, max_top_k, top_ks, top_p, top_ps, vocab_size_padded,
                                             end_ids, stream, batch_size, skip_decode));
}

template<typename T>
void invokeTopKSampling(void* workspace, size_t& workspace_size, const T* log_probs, int* ids, int* sequence_length,
                        bool* finished_buf, float* cum_log_probs, float* output_log_probs, curandState_t* curandstate,
                        const int top_k, const float top_p, const int vocab_size_padded, const int* end_ids,
                        hipStream_t stream, const int batch_size, const bool* skip_decode,
                        const float* uniform_draws = nullptr)
{
    invokeBatchTopKSampling(workspace, workspace_size, log_probs, ids, sequence_length, finished_buf, cum_log_probs,
                            output_log_probs, curandstate, top_k, (const int*)nullptr, top_p, (const float*)nullptr,
                            vocab_size_padded, end_ids, stream, batch_size, skip_decode, uniform_draws);
}

template<typename T>
void invokeTopKTopPSampling(void* workspace, size_t& workspace_size, int* output_ids, const T* logits,
                            int* sequence_length, bool* finished_buf, float* cum_log_probs, float* output_log_probs,
                            curandState_t* curandstate, const int batch_size, const int top_k, const float top_p,
                            const int vocab_size_padded, const int* end_ids, hipStream_t stream,
                            const float* uniform_draws = nullptr)
{
    invokeTopKSampling(workspace, workspace_size, logits, output_ids, sequence_length, finished_buf, cum_log_probs,
                       output_log_probs, curandstate, top_k, top_p, vocab_size_padded, end_ids, stream, batch_size,
                       (const bool*)nullptr, uniform_draws);
}

// ---- sampling_topp_kernels.h ----------------------------------------------------------------
inline void invokeTopPInitialize(int* topp_id_val_buf, int* topp_offset_buf, int* begin_topp_offset_buf_,
                                 const size_t batch_size, const int n, hipStream_t stream)
{
    check_ftk(ftk_invoke_topp_initialize(topp_id_val_buf, topp_offset_buf, begin_topp_offset_buf_, batch_size, n,
                                         stream));
}

template<typename T>
void invokeAddBiasSoftMax(T* logits, const T* bias, const int* end_ids, const bool* finished, const int m,
                          const int n_padded, const int n, hipStream_t stream)
{
    check_ftk(ftk_invoke_add_bias_softmax(FtkDType<T>::value, logits, bias, end_ids, finished, m, n_padded, n, stream));
}

template<typename T>
void invokeBatchTopPSampling(void* workspace, size_t& workspace_size, size_t& cub_temp_storage_size, int* output_ids,
                             int* sequence_length, bool* finished_buf, float* cum_log_probs, float* output_log_probs,
                             const T* log_probs, const int* id_vals, int* offset_buf, int* begin_offset_buf,
                             curandState_t* curandstate, const int batch_size, const size_t vocab_size_padded,
                             const int* end_ids, const float max_top_p, const float* top_ps, hipStream_t stream,
                             void* device_prop, const bool* skip_decode, const float* uniform_draws = nullptr)
{
    (void)device_prop;
    check_ftk(ftk_invoke_batch_topp_sampling(FtkDType<T>::value, workspace, &workspace_size, &cub_temp_storage_size,
                                             output_ids, sequence_length, finished_buf, cum_log_probs,
                                             output_log_probs, log_probs, id_vals, offset_buf, begin_offset_buf,
                                             curandstate, uniform_draws, batch_size, vocab_size_padded, end_ids,
                                             max_top_p, top_ps, stream, skip_decode));
}

template<typename T>
void invokeTopPSampling(void* workspace, size_t& workspace_size, size_t& cub_temp_storage_size, int* output_ids,
                        int* sequence_length, bool* finished_buf, float* cum_log_probs, float* output_log_probs,
                        const T* log_probs, const int* id_vals, int* offset_buf, int* begin_offset_buf,
                        curandState_t* curandstate, const int batch_size, const size_t vocab_size_padded,
                        const int* end_ids, const float top_p, hipStream_t stream, void* device_prop,
                        const bool* skip_decode, const float* uniform_draws = nullptr)
{
    invokeBatchTopPSampling(workspace, workspace_size, cub_temp_storage_size, output_ids, sequence_length,
                            finished_buf, cum_log_probs, output_log_probs, log_probs, id_vals, offset_buf,
                            begin_offset_buf, curandstate, batch_size, vocab_size_padded, end_ids, top_p,
                            (const float*)nullptr, stream, device_prop, skip_decode, uniform_draws);
}

// One call for the softmax, the top-p sampler and the decay of a step (TopPSamplingLayer<T>::runSampling,
// layers/sampling_layers/TopPSamplingLayer.cu:256-343); workspace == nullptr asks for the size.
template<typename T>
void invokeFusedTopPStep(void* workspace, size_t& workspace_size, T* logits, const T* bias, const int vocab_size,
                         const size_t vocab_size_padded, const int batch_size, const int* end_ids, bool* finished,
                         int* sequence_length, int* output_ids, float* cum_log_probs, float* output_log_probs,
                         curandState_t* curandstate, const float* uniform_draws, const float max_top_p,
                         float* runtime_top_p, const float* initial_top_p, const float* top_p_decay,
                         const float* top_p_min, const int32_t* top_p_reset_ids, const bool* skip_decode,
                         hipStream_t stream)
{
    check_ftk(ftk_fused_topp_step(FtkDType<T>::value, workspace, &workspace_size, logits, bias, vocab_size,
                                  vocab_size_padded, batch_size, end_ids, finished, sequence_length, output_ids,
                                  cum_log_probs, output_log_probs, curandstate, uniform_draws, max_top_p,
                                  runtime_top_p, initial_top_p, top_p_decay, top_p_min, top_p_reset_ids, skip_decode,
                                  stream));
}

// The same step for a caller that does not need the probabilities afterwards: `logits` is only read. False when
// the step does not take this shape (fewer than 1024 columns): the caller then uses invokeFusedTopPStep. The
// workspace is invokeFusedTopPStep's.
template<typename T>
bool invokeFusedTopPSampleStep(void* workspace, size_t workspace_size, const T* logits, const int vocab_size,
                               const size_t vocab_size_padded, const int batch_size, const int* end_ids, bool* finished,
                               int* sequence_length, int* output_ids, float* cum_log_probs, float* output_log_probs,
                               curandState_t* curandstate, const float* uniform_draws, const float max_top_p,
                               float* runtime_top_p, const float* initial_top_p, const float* top_p_decay,
                               const float* top_p_min, const int32_t* top_p_reset_ids, const bool* skip_decode,
                               hipStream_t stream)
{
    const int rc = ftk_fused_topp_sample_step(FtkDType<T>::value, workspace, &workspace_size, logits, vocab_size,
                                              vocab_size_padded, batch_size, end_ids, finished, sequence_length,
                                              output_ids, cum_log_probs, output_log_probs, curandstate, uniform_draws,
                                              max_top_p, runtime_top_p, initial_top_p, top_p_decay, top_p_min,
                                              top_p_reset_ids, skip_decode, stream);
    if (rc == FTK_ERR_UNSUPPORTED) {
        return false;
    }
    check_ftk(rc);
    return true;
}

inline void invokeComputeToppDecay(float* runtime_top_p, const float* runtime_initial_top_p, const int* output_ids,
                                   const float* top_p_decay, const float* top_p_min, const int32_t* top_p_reset_ids,
                                   const int local_batch_size, hipStream_t stream)
{
    check_ftk(ftk_invoke_compute_topp_decay(runtime_top_p, runtime_initial_top_p, output_ids, top_p_decay, top_p_min,
                                            top_p_reset_ids, local_batch_size, stream));
}

// ---- sampling_penalty_kernels.h -------------------------------------------------------------
template<typename T>
void invokeApplyRepetitionPenalty(T* logits, const float penalty, const int* start_ids, int* output_ids,
                                  const int batch_size, const int local_batch_size, const int vocab_size,
                                  const int vocab_size_padd, const int* input_lengths, const int max_input_len,
                                  const int step, const RepetitionPenaltyType penalty_type, hipStream_t stream)
{
    check_ftk(ftk_invoke_apply_repetition_penalty(FtkDType<T>::value, logits, penalty, start_ids, output_ids,
                                                  batch_size, local_batch_size, vocab_size, vocab_size_padd,
                                                  input_lengths, max_input_len, step, toFtkPenalty(penalty_type),
                                                  stream));
}

template<typename T>
void invokeBatchApplyRepetitionPenalty(T* logits, const float* penalties, const int* output_ids, const int batch_size,
                                       const int local_batch_size, const int vocab_size, const int* input_lengths,
                                       const int max_input_length, const int step,
                                       const RepetitionPenaltyType penalty_type, hipStream_t stream)
{
    check_ftk(ftk_invoke_batch_apply_repetition_penalty(FtkDType<T>::value, logits, penalties, output_ids, batch_size,
                                                        local_batch_size, vocab_size, input_lengths,
                                                        max_input_length, step, toFtkPenalty(penalty_type), stream));
}

template<typename T>
void invokeBatchApplyFrequencyPenalty(T* logits, const float* presence, const float* frequency, const int* output_ids,
                                      const int batch_size, const int local_batch_size, const int vocab_size,
                                      const int* input_lengths, const int max_input_length, const int step,
                                      hipStream_t stream)
{
    check_ftk(ftk_invoke_batch_apply_frequency_penalty(FtkDType<T>::value, logits, presence, frequency, output_ids,
                                                       batch_size, local_batch_size, vocab_size, input_lengths,
                                                       max_input_length, step, stream));
}

template<typename T>
void invokeApplyTemperaturePenalty(T* logits, const T* bias, const float temperature, const int batch_size,
                                   const int vocab_size, const int vocab_size_padd, hipStream_t stream)
{
    check_ftk(ftk_invoke_apply_temperature_penalty(FtkDType<T>::value, logits, bias, temperature, batch_size,
                                                   vocab_size, vocab_size_padd, stream));
}

template<typename T>
void invokeBatchApplyTemperaturePenalty(T* logits, const T* bias, const float* temperatures, const int batch_size,
                                        const int vocab_size, const int vocab_size_padd, hipStream_t stream)
{
    check_ftk(ftk_invoke_batch_apply_temperature_penalty(FtkDType<T>::value, logits, bias, temperatures, batch_size,
                                                         vocab_size, vocab_size_padd, stream));
}

template<typename T>
void invokeMinLengthPenalty(T* logits, const int* min_lengths, const int* end_ids, const int* sequnece_lengths,
                            const int max_input_length, const int batch_size, const int vocab_size_padded,
                            hipStream_t stream)
{
    check_ftk(ftk_invoke_min_length_penalty(FtkDType<T>::value, logits, min_lengths, end_ids, sequnece_lengths,
                                            max_input_length, batch_size, vocab_size_padded, stream));
}

// ---- ban_bad_words.h, stop_criteria_kernels.h ---------------------------------------------------
template<typename T>
void invokeBanBadWords(T* logits, const int* output_ids_buf, const int* parent_ids_buf, int batch_size,
                       int local_batch_size, int beam_width, const int* bad_words, bool share_words,
                       size_t bad_words_len, int id_offset, int vocab_size_padded, size_t step, hipStream_t stream)
{
    check_ftk(ftk_invoke_ban_bad_words(FtkDType<T>::value, logits, output_ids_buf, parent_ids_buf, batch_size,
                                       local_batch_size, beam_width, bad_words, share_words, bad_words_len, id_offset,
                                       vocab_size_padded, step, stream));
}

inline void invokeStopWordsCriterion(const int* output_ids, const int* parent_ids, const int* stop_words,
                                     bool* finished, size_t id_offset, size_t stop_words_len, int batch_size,
                                     int beam_width, int step, hipStream_t stream)
{
    check_ftk(ftk_invoke_stop_words_criterion(output_ids, parent_ids, stop_words, finished, id_offset, stop_words_len,
                                              batch_size, beam_width, step, stream));
}

inline void invokeLengthCriterion(bool* finished, bool* should_stop, int* h_pinned_finished_sum_,
                                  const uint32_t* sequence_limit_length, int batch_size, int beam_width, int step,
                                  hipStream_t stream)
{
    check_ftk(ftk_invoke_length_criterion(finished, should_stop, h_pinned_finished_sum_, sequence_limit_length,
                                          batch_size, beam_width, step, stream));
}

// ---- logprob_kernels.h, decoding_kernels.h, gpt_kernels.h (the steps either side of the sampling path) ----
template<typename T>
void invokeLogProbFromLogits(float* cum_log_probs, const T* logits, const int* input_ids, const int* input_lengths,
                             const size_t max_input_length, const size_t batch_size, const size_t vocab_size,
                             const size_t vocab_size_padded, void* workspace, const size_t workspace_size,
                             hipStream_t stream, const bool batch_first = false)
{
    check_ftk(ftk_invoke_log_prob_from_logits(FtkDType<T>::value, cum_log_probs, logits, input_ids, input_lengths,
                                              max_input_length, batch_size, vocab_size, vocab_size_padded, workspace,
                                              workspace_size, stream, batch_first));
}

template<typename T>
void invokeDecodingInitialize(bool* finished, int* sequence_length, int* word_ids, T* cum_log_probs,
                              const int* sentence_ids, const int batch_size, const int beam_width,
                              const int max_input_length, hipStream_t stream)
{
    check_ftk(ftk_invoke_decoding_initialize(FtkDType<T>::value, finished, sequence_length, word_ids, cum_log_probs,
                                             sentence_ids, batch_size, beam_width, max_input_length, stream));
}

inline void invokePlusScalar(int* buf, const int val, const int size, hipStream_t stream)
{
    check_ftk(ftk_invoke_plus_scalar(buf, val, size, stream));
}

inline void invokeTransposeAxis01(int* out, int* in, const int* in_skipping_dim1, const int dim0, const int dim1,
                                  hipStream_t stream)
{
    check_ftk(ftk_invoke_transpose_axis01(out, in, in_skipping_dim1, dim0, dim1, stream));
}

// kernels/decoding_kernels.cu:787-813
inline void invokeFinalize(int* output_ids, int* sequence_lengths, float* cum_log_probs, float* output_log_probs,
                           const int* topk_output_ids, const int* topk_sequence_lengths, const float* scores,
                           const float* topk_cum_log_probs, const float* topk_log_probs, const int* num_beams,
                           const int beam_width, const int max_seq_len, const int batch_size, hipStream_t stream)
{
    check_ftk(ftk_invoke_finalize(output_ids, sequence_lengths, cum_log_probs, output_log_probs, topk_output_ids,
                                  topk_sequence_lengths, scores, topk_cum_log_probs, topk_log_probs, num_beams,
                                  beam_width, max_seq_len, batch_size, stream));
}

// ---- beam_search_topk_kernels.h / online_softmax_beamsearch_kernels.h -----------------------------------
typedef ftk_beam_hypotheses BeamHypotheses;  // kernels/beam_search_topk_kernels.h:31-58, the same fields

// Bytes of temp_storage a call with these sizes needs (the reference's layer computes a count of floats itself,
// layers/beam_search_layers/OnlineBeamSearchLayer.cu:201-207).
template<typename T>
size_t topkSoftMaxWorkspaceBytes(const int batch_size, const int beam_width, const int vocab_size)
{
    size_t bytes = 0;
    check_ftk(ftk_invoke_topk_softmax(FtkDType<T>::value, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                                      nullptr, nullptr, &bytes, nullptr, batch_size, beam_width, vocab_size, nullptr,
                                      0.0f, 0.0f, nullptr));
    return bytes;
}

// kernels/online_softmax_beamsearch_kernels.cu:671-701; temp_storage_size counts 4-byte elements as there
template<typename T>
void invokeTopkSoftMax(const T* log_probs, const T* bias, const bool* finished, const int* sequence_lengths,
                       float* cum_log_probs, float* output_log_probs, int* ids, void* temp_storage,
                       const int temp_storage_size, BeamHypotheses* beam_hyps, const int batch_size,
                       const int beam_width, const int vocab_size, const int* end_ids, const float diversity_rate,
                       const float length_penalty, hipStream_t stream)
{
    size_t bytes = (size_t)temp_storage_size * sizeof(float);
    check_ftk(ftk_invoke_topk_softmax(FtkDType<T>::value, log_probs, bias, finished, sequence_lengths, cum_log_probs,
                                      output_log_probs, ids, temp_storage, &bytes, beam_hyps, batch_size, beam_width,
                                      vocab_size, end_ids, diversity_rate, length_penalty, stream));
}

// kernels/beam_search_penalty_kernels.cu:175-267
template<typename T>
void invokeAddBiasApplyPenalties(int step, T* logits, const int* current_ids, const int* previous_ids,
                                 const int* parent_ids, const int* input_lengths, const int* sequence_lengths,
                                 const T* bias, const int ite, const int max_input_length, const int local_batch_size,
                                 const int batch_size, const int beam_width, const int vocab_size,
                                 const int vocab_size_padded, const int* end_ids, const float temperature,
                                 const float repetition_penalty, const RepetitionPenaltyType repetition_penalty_type,
                                 const int min_length, hipStream_t stream)
{
    check_ftk(ftk_invoke_add_bias_apply_penalties(FtkDType<T>::value, step, logits, current_ids, previous_ids,
                                                  parent_ids, input_lengths, sequence_lengths, bias, ite,
                                                  max_input_length, local_batch_size, batch_size, beam_width,
                                                  vocab_size, vocab_size_padded, end_ids, temperature,
                                                  repetition_penalty, toFtkPenalty(repetition_penalty_type),
                                                  min_length, stream));
}

// layers/beam_search_layers/OnlineBeamSearchLayer.cu:63-85
inline void invokeUpdate(bool* finished, int* parent_ids, int* sequence_length, int* word_ids, int* output_ids,
                         BeamHypotheses* beam_hyps, const int local_batch_size, const int beam_width,
                         const int vocab_size_padded, const int* end_ids, hipStream_t stream)
{
    check_ftk(ftk_invoke_beam_update(finished, parent_ids, sequence_length, word_ids, output_ids, beam_hyps,
                                     local_batch_size, beam_width, vocab_size_padded, end_ids, stream));
}

// layers/beam_search_layers/BaseBeamSearchLayer.cu:51-77
inline void update_indir_cache_kernelLauncher(int* tgt_indir_cache, const int* src_indir_cache, const int* beam_ids,
                                              const bool* finished, int batch_dim, int local_batch_size,
                                              int beam_width, int max_seq_len, int step, hipStream_t stream)
{
    check_ftk(ftk_invoke_update_indir_cache(tgt_indir_cache, src_indir_cache, beam_ids, finished, batch_dim,
                                            local_batch_size, beam_width, max_seq_len, step, stream));
}

}  // namespace fastertransformer
