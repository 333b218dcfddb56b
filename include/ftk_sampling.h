/*
 * C ABI of the MI355X (gfx950) decode-step sampling engine: libftk_sampling.so.
 *
 * Every entry point replaces one `invoke*` kernel launcher of NVIDIA/FasterTransformer's sampling
 * path (paths below are relative to the FasterTransformer source tree). Parameter order and meaning
 * follow the reference launcher; the differences are mechanical:
 *   - the C++ template parameter T becomes the leading `dtype` argument (FTK_DTYPE_*);
 *   - `cudaStream_t` becomes `ftk_stream_t` (a `hipStream_t` passed as void*);
 *   - `curandState_t*` becomes `ftk_rng_state*` (counter-based Philox-4x32-10 state) followed by an
 *     optional `const float* uniform_draws`: when non-null, row b uses uniform_draws[b] in (0, 1]
 *     instead of drawing, which makes a step reproducible bit for bit;
 *   - `size_t&` workspace-size out-parameters become `size_t*`;
 *   - errors are return codes: 0 = success, > 0 = hipError_t, < 0 = FTK_ERR_*.
 * All pointers are device pointers unless stated otherwise. No entry point allocates memory; all
 * scratch comes in through `workspace`. Calls are asynchronous on `stream` unless stated otherwise.
 */
#ifndef FTK_SAMPLING_H
#define FTK_SAMPLING_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void* ftk_stream_t;

enum { FTK_DTYPE_F32 = 0, FTK_DTYPE_F16 = 1, FTK_DTYPE_BF16 = 2 };

/* kernels/penalty_types.h:26-30 (same enumerator order) */
enum { FTK_PENALTY_ADDITIVE = 0, FTK_PENALTY_MULTIPLICATIVE = 1, FTK_PENALTY_NONE = 2 };

enum {
    FTK_ERR_DTYPE       = -1, /* unknown dtype */
    FTK_ERR_TOPK_DOMAIN = -2, /* top-k outside [1, 1024]: std::domain_error in sampling_topk_kernels.cu:393-394 */
    FTK_ERR_ARGUMENT    = -3, /* null / inconsistent argument */
    FTK_ERR_WORKSPACE   = -4, /* workspace smaller than the queried size */
    FTK_ERR_STATIC_WORKSPACE = -5, /* ftk_fused_topk_step_static: the step needs more than the library's fixed array */
    FTK_ERR_UNSUPPORTED = -6 /* ftk_fused_topk_step: log-prob outputs for a configuration the fused step does not cover */
};

/* Per-row generator state; replaces curandState_t (48 bytes) in every signature. Row b draws
 * Philox-4x32-10(key = seed, counter = {offset, 0, 0, 0}).x mapped to (0, 1], then offset++. */
typedef struct ftk_rng_state {
    uint64_t seed;
    uint64_t offset;
} ftk_rng_state;

const char* ftk_error_string(int code);

/* ---- kernels/sampling_topk_kernels.h ----------------------------------------------------- */

/* invokeCurandInitialize, kernels/sampling_topk_kernels.cu:39-47 */
int ftk_invoke_curand_initialize(ftk_rng_state* state, size_t batch_size, unsigned long long random_seed,
                                 ftk_stream_t stream);

/* invokeCurandBatchInitialize, kernels/sampling_topk_kernels.cu:57-65 */
int ftk_invoke_curand_batch_initialize(ftk_rng_state* states, size_t batch_size,
                                       const unsigned long long* random_seeds, ftk_stream_t stream);

/* invokeAddBiasEndMask<T>, kernels/sampling_topk_kernels.cu:96-110 */
int ftk_invoke_add_bias_end_mask(int dtype, void* logits, const void* bias, const int* end_ids, const bool* finished,
                                 int batch_size, int vocab_size, int vocab_size_padded, ftk_stream_t stream);

/* invokeBatchTopKSampling<T>, kernels/sampling_topk_kernels.cu:345-396.
 * workspace == NULL: writes the required size to *workspace_size and launches nothing.
 * invokeTopKSampling (:438-474) is this call with top_ks == NULL and top_ps == NULL;
 * invokeTopKTopPSampling (:510-544) additionally passes skip_decode == NULL. */
int ftk_invoke_batch_topk_sampling(int dtype, void* workspace, size_t* workspace_size, const void* log_probs, int* ids,
                                   int* sequence_length, bool* finished, float* cum_log_probs,
                                   float* output_log_probs, ftk_rng_state* rng_state, const float* uniform_draws,
                                   int max_top_k, const int* top_ks, float top_p, const float* top_ps,
                                   int vocab_size_padded, const int* end_ids, ftk_stream_t stream, int batch_size,
                                   const bool* skip_decode);

/* ---- kernels/sampling_topp_kernels.h ----------------------------------------------------- */

/* invokeTopPInitialize, kernels/sampling_topp_kernels.cu:790-799. Kept for callers that own such
 * buffers; this engine's top-p never reads the id table, so any of the pointers may be NULL. */
int ftk_invoke_topp_initialize(int* topp_id_val_buf, int* topp_offset_buf, int* begin_topp_offset_buf,
                               size_t batch_size, int n, ftk_stream_t stream);

/* invokeAddBiasSoftMax<T>, kernels/sampling_topp_kernels.cu:1347-1361 */
int ftk_invoke_add_bias_softmax(int dtype, void* logits, const void* bias, const int* end_ids, const bool* finished,
                                int m, int n_padded, int n, ftk_stream_t stream);

/* invokeBatchTopPSampling<T>, kernels/sampling_topp_kernels.cu:1006-1161 (`log_probs` holds
 * probabilities). workspace == NULL: size query (cub_temp_storage_size is reported as 0).
 * id_vals / offset_buf / begin_offset_buf are accepted and ignored. invokeTopPSampling
 * (:1207-1250) is this call with top_ps == NULL. cudaDeviceProp* is dropped (only the reference's
 * disabled single-pass branch read it). */
int ftk_invoke_batch_topp_sampling(int dtype, void* workspace, size_t* workspace_size, size_t* cub_temp_storage_size,
                                   int* output_ids, int* sequence_length, bool* finished, float* cum_log_probs,
                                   float* output_log_probs, const void* log_probs, const int* id_vals,
                                   int* offset_buf, int* begin_offset_buf, ftk_rng_state* rng_state,
                                   const float* uniform_draws, int batch_size, size_t vocab_size_padded,
                                   const int* end_ids, float max_top_p, const float* top_ps, ftk_stream_t stream,
                                   const bool* skip_decode);

/* invokeComputeToppDecay, kernels/sampling_topp_kernels.cu:1414-1427 */
int ftk_invoke_compute_topp_decay(float* runtime_top_p, const float* runtime_initial_top_p, const int* output_ids,
                                  const float* top_p_decay, const float* top_p_min, const int32_t* top_p_reset_ids,
                                  int local_batch_size, ftk_stream_t stream);

/* One call for what TopPSamplingLayer<T>::runSampling issues per step
 * (layers/sampling_layers/TopPSamplingLayer.cu:256-343): invokeAddBiasSoftMax on `logits` ([batch_size,
 * vocab_size_padded], left holding the probabilities exactly as ftk_invoke_add_bias_softmax leaves them),
 * invokeBatchTopPSampling on the result with `runtime_top_p` as top_ps (NULL: max_top_p for every row), and, when
 * top_p_decay is not NULL, invokeComputeToppDecay on the ids just written. Results are those of the three calls
 * in sequence; the row is read once less and the histogram of the sampler is taken while the probabilities are
 * written. workspace == NULL: size query (slightly above ftk_invoke_batch_topp_sampling's). */
int ftk_fused_topp_step(int dtype, void* workspace, size_t* workspace_size, void* logits, const void* bias,
                        int vocab_size, size_t vocab_size_padded, int batch_size, const int* end_ids, bool* finished,
                        int* sequence_length, int* output_ids, float* cum_log_probs, float* output_log_probs,
                        ftk_rng_state* rng_state, const float* uniform_draws, float max_top_p, float* runtime_top_p,
                        const float* initial_top_p, const float* top_p_decay, const float* top_p_min,
                        const int32_t* top_p_reset_ids, const bool* skip_decode, ftk_stream_t stream);

/* ftk_fused_topp_step for callers that do not need the probabilities: same arguments without the bias, same ids,
 * log-probs, lengths, finished flags and decayed top-p values, but `logits` is only read (the reference leaves the
 * probabilities there, layers/sampling_layers/TopPSamplingLayer.cu:287-297; nothing in its decode loop reads them
 * again). Every probability that is needed is worked out from the logits on the way, with the arithmetic of
 * ftk_invoke_add_bias_softmax, so the row is read three times and never written. FTK_ERR_UNSUPPORTED (also from
 * the size query) when vocab_size < 1024; a step with an embedding bias takes ftk_fused_topp_step.
 * workspace == NULL: size query (ftk_fused_topp_step's). */
int ftk_fused_topp_sample_step(int dtype, void* workspace, size_t* workspace_size, const void* logits,
                               int vocab_size, size_t vocab_size_padded, int batch_size, const int* end_ids,
                               bool* finished, int* sequence_length, int* output_ids, float* cum_log_probs,
                               float* output_log_probs, ftk_rng_state* rng_state, const float* uniform_draws,
                               float max_top_p, float* runtime_top_p, const float* initial_top_p,
                               const float* top_p_decay, const float* top_p_min, const int32_t* top_p_reset_ids,
                               const bool* skip_decode, ftk_stream_t stream);

/* ---- kernels/sampling_penalty_kernels.h -------------------------------------------------- */

/* invokeApplyTemperaturePenalty<T>, kernels/sampling_penalty_kernels.cu:75-99 */
int ftk_invoke_apply_temperature_penalty(int dtype, void* logits, const void* bias, float temperature, int batch_size,
                                         int vocab_size, int vocab_size_padd, ftk_stream_t stream);

/* invokeBatchApplyTemperaturePenalty<T>, kernels/sampling_penalty_kernels.cu:181-206 */
int ftk_invoke_batch_apply_temperature_penalty(int dtype, void* logits, const void* bias, const float* temperatures,
                                               int batch_size, int vocab_size, int vocab_size_padd,
                                               ftk_stream_t stream);

/* invokeApplyRepetitionPenalty<T>, kernels/sampling_penalty_kernels.cu:288-337 (start_ids is unused there too) */
int ftk_invoke_apply_repetition_penalty(int dtype, void* logits, float penalty, const int* start_ids,
                                        const int* output_ids, int batch_size, int local_batch_size, int vocab_size,
                                        int vocab_size_padd, const int* input_lengths, int max_input_len, int step,
                                        int penalty_type, ftk_stream_t stream);

/* invokeBatchApplyRepetitionPenalty<T>, kernels/sampling_penalty_kernels.cu:426-459
 * (`vocab_size` is the row stride, as in the reference) */
int ftk_invoke_batch_apply_repetition_penalty(int dtype, void* logits, const float* penalties, const int* output_ids,
                                              int batch_size, int local_batch_size, int vocab_size,
                                              const int* input_lengths, int max_input_length, int step,
                                              int penalty_type, ftk_stream_t stream);

/* Extension without a reference counterpart: additive presence + frequency penalty,
 * logit <- T(float(logit) - presence[b] - frequency[b] * count), count = occurrences of the id in
 * the non-padding history; with frequency == 0 it equals the additive penalty above. */
int ftk_invoke_batch_apply_frequency_penalty(int dtype, void* logits, const float* presence, const float* frequency,
                                             const int* output_ids, int batch_size, int local_batch_size,
                                             int vocab_size, const int* input_lengths, int max_input_length,
                                             int step, ftk_stream_t stream);

/* invokeMinLengthPenalty<T>, kernels/sampling_penalty_kernels.cu:502-517 */
int ftk_invoke_min_length_penalty(int dtype, void* logits, const int* min_lengths, const int* end_ids,
                                  const int* sequence_lengths, int max_input_length, int batch_size,
                                  int vocab_size_padded, ftk_stream_t stream);

/* ---- kernels/ban_bad_words.h, kernels/stop_criteria_kernels.h ------------------------------ */

/* invokeBanBadWords<T>, kernels/ban_bad_words.cu:88-120. With beam_width > 1 the logits are
 * [local_batch_size * beam_width, vocab_size_padded], a word list belongs to a batch entry, and a beam's history is
 * followed back through parent_ids_buf ([max_seq_len, batch_size * beam_width], required then). */
int ftk_invoke_ban_bad_words(int dtype, void* logits, const int* output_ids_buf, const int* parent_ids_buf,
                             int batch_size, int local_batch_size, int beam_width, const int* bad_words,
                             bool share_words, size_t bad_words_len, int id_offset, int vocab_size_padded,
                             size_t step, ftk_stream_t stream);

/* invokeStopWordsCriterion, kernels/stop_criteria_kernels.cu:83-104 (with beam_width > 1: finished
 * [batch_size * beam_width], histories followed back through parent_ids) */
int ftk_invoke_stop_words_criterion(const int* output_ids, const int* parent_ids, const int* stop_words,
                                    bool* finished, size_t id_offset, size_t stop_words_len, int batch_size,
                                    int beam_width, int step, ftk_stream_t stream);

/* The same kernel over the first `num_rows` rows only, `batch_size` staying the row stride of
 * output_ids. DynamicDecodeLayer::forward needs it for micro-batch windows: the reference passes its
 * window through offset pointers yet still examines `batch_size` rows (layers/DynamicDecodeLayer.cc:451-461),
 * which runs past the window; this entry point examines the window only. */
int ftk_invoke_stop_words_criterion_rows(const int* output_ids, const int* parent_ids, const int* stop_words,
                                         bool* finished, size_t id_offset, size_t stop_words_len, int batch_size,
                                         int num_rows, int beam_width, int step, ftk_stream_t stream);

/* invokeLengthCriterion, kernels/stop_criteria_kernels.cu:135-157. `should_stop` is a host bool and
 * `h_pinned_finished_sum` one pinned host int; like the reference the call returns only when
 * *should_stop is valid. */
int ftk_invoke_length_criterion(bool* finished, bool* should_stop, int* h_pinned_finished_sum,
                                const uint32_t* sequence_limit_length, int batch_size, int beam_width, int step,
                                ftk_stream_t stream);

/* ---- fused decode step ---------------------------------------------------------------------
 * One call = the kernel sequence BaseSamplingLayer<T>::forward + TopKSamplingLayer<T>::runSampling
 * issue for the rows a top-k layer owns (layers/sampling_layers/BaseSamplingLayer.cc:255-359,
 * layers/sampling_layers/TopKSamplingLayer.cu:189-268): temperature(+bias), repetition/presence penalty,
 * min-length, end/pad mask, (softmax when log-probs are requested,) top-k selection and sampling, with the
 * logits read from HBM once - twice with log-probs or a k above 192 - and never written (the reference leaves them penalised,
 * or turned into probabilities). Bad words are
 * not part of it: DynamicDecodeLayer masks them on the logits before the sampling layers run
 * (ftk_invoke_ban_bad_words), here as in the reference. */
typedef struct ftk_fused_topk_args {
    int         dtype;
    const void* logits;         /* [local_batch, vocab_size_padded], not modified */
    const void* embedding_bias; /* [vocab_size_padded] or NULL */
    int         vocab_size, vocab_size_padded;
    int         batch_size;       /* stride of output_ids rows */
    int         local_batch_size; /* rows in this call */
    int         step, max_input_length;
    /* per-row arguments, already offset to the local window */
    const float* temperatures;   /* NULL = 1.0 */
    const float* penalties;      /* NULL or [local] */
    int          penalty_type;   /* FTK_PENALTY_* */
    const int*   min_lengths;    /* NULL = no min-length mask */
    const int*   end_ids;        /* [local] */
    const int*   input_lengths;  /* [local] or NULL */
    const int*   output_ids;     /* history base + window offset: element (t, row) at output_ids[t*batch_size+row] */
    const int*   top_ks;    /* [local] */
    const float* top_ps;    /* [local] */
    int          max_top_k;
    const bool*  skip_decode; /* [local] or NULL */
    ftk_rng_state* rng_state; /* [local] */
    const float*   uniform_draws; /* [local] or NULL */
    /* outputs */
    int*  ids;             /* [local]: output_ids + step*batch_size + window offset */
    int*  sequence_length; /* [local] or NULL */
    bool* finished;        /* [local] or NULL */
    /* Log-prob outputs (both NULL: none). With either one the step takes the probabilities of the whole row as
     * the reference does (softmax after the penalties, top-k on probabilities): cum_log_probs[b] += log p,
     * output_log_probs[b] = log p - log(sum of the k probabilities). Covered for launches without embedding
     * bias, largest k <= 128 and vocab_size >= 1024 (rows of any pitch, starting on any element boundary);
     * anything else returns FTK_ERR_UNSUPPORTED (also for the size query) and launches nothing: run the kernel
     * sequence instead. Every row goes to one workgroup here, which pays from a few hundred rows on. */
    float* cum_log_probs;    /* [local] or NULL */
    float* output_log_probs; /* [local] or NULL: the row of this step */
    void*  workspace;
    size_t workspace_size;
    /* Frequency penalty, an extension without reference code: with it a column that occurs `count` times in the row's
     * history gets x - penalties[b] - frequency_penalties[b] * count (penalty_type must be FTK_PENALTY_ADDITIVE and
     * `penalties` hold the presence term, zeros if there is none). [local] or NULL. Covered where the step runs as one
     * launch of one workgroup per row (no log-probs, no bias, largest k <= 192, rows on 16-byte boundaries, up to
     * 256 rows of a small launch or nearly full rounds of 256 rows, history up to 4096 positions, vocabulary up to
     * 2^18); anything else returns FTK_ERR_UNSUPPORTED: run ftk_invoke_batch_apply_frequency_penalty and the rest of
     * the kernel sequence instead. */
    const float* frequency_penalties;
} ftk_fused_topk_args;

/* workspace == NULL in args: writes the required size into args->workspace_size, launches nothing. */
int ftk_fused_topk_step(ftk_fused_topk_args* args, ftk_stream_t stream);

/* ---- the fused step over vocabulary shards (producer hand-over) --------------------------------------
 * The reference writes a step's logits from its last GEMM - one vocabulary shard per rank under tensor parallelism,
 * gathered afterwards - and reads them back in DynamicDecodeLayer::forward
 * (src/fastertransformer/models/multi_gpu_gpt/ParallelGpt.cc:1374-1433, :1436-1501). These two entry points let a
 * producer (a GEMM epilogue working through column tiles, or a rank that holds one shard) hand over columns
 * [col_offset, col_offset + args->vocab_size) of every row on their own:
 *   gather: args->logits points at the shard's first column of the first row, args->vocab_size is the number of the
 *           shard's columns that lie inside the vocabulary, args->vocab_size_padded the pitch of its rows in
 *           elements; token ids (history, end ids) are global. Leaves, per row and shard, candidate lists that hold
 *           every element at or above a lower bound of the k-th largest value of the shard's columns (column numbers
 *           global), and in `partials`, when given, the shard's (maximum, sum of exp(x - maximum)) over the final
 *           values (after temperature, penalties and masks). Samples nothing.
 *   merge:  after every shard's gather: the selection of ftk_fused_topk_step over the lists of all shards. ids, lengths
 *           and flags are those of ftk_fused_topk_step on the whole rows, bit for bit. args->vocab_size /
 *           vocab_size_padded are the whole vocabulary's; args->logits are the whole rows, or NULL when nobody holds
 *           them (a row whose lists overflowed - thousands of candidates tied around the k-th value - then gets id -1).
 *           `row_stats`, when given (with `partials`), receives the rows' (maximum, sum of exp(x - maximum)) combined
 *           over the shards: log p of the sampled token = x - maximum - log(sum), within 1e-5 of the reference's
 *           softmax but not in its summation order.
 * Both calls take the same workspace (size query: workspace == NULL, from either call with the same n_shards,
 * shard_width and batch) and the same per-row arguments. Largest k <= 192, no embedding bias, no log-prob outputs
 * (FTK_ERR_UNSUPPORTED otherwise); with a history penalty the step must not exceed 8192. What a rank would send
 * instead of its shard of the row is its lists: typically a few hundred entries of 8 bytes per row. */
typedef struct ftk_topk_shards {
    int    n_shards;                 /* shards a row is cut into, 1 .. 16 */
    int    shard_width;              /* columns of the widest shard: fixes the workspace layout for every call */
    int    global_vocab_size_padded; /* of the whole rows (sizes the merge's recovery bitmaps) */
    int    shard;                    /* gather: which shard this call reads */
    int    col_offset;               /* gather: global number of the shard's first column */
    float* partials;                 /* [local_batch][n_shards][2] or NULL */
    float* row_stats;                /* merge: [local_batch][2] or NULL */
} ftk_topk_shards;
int ftk_fused_topk_shard_gather(ftk_fused_topk_args* args, const ftk_topk_shards* shards, ftk_stream_t stream);
int ftk_fused_topk_shard_merge(ftk_fused_topk_args* args, const ftk_topk_shards* shards, ftk_stream_t stream);

/* The fused step for callers that cannot allocate device memory (code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc). It has no counterpart in the reference. Same arguments and results as
 * ftk_fused_topk_step, except that args->workspace is ignored: the workspace is a fixed array of
 * FTK_FUSED_STATIC_WORKSPACE_BYTES inside the library's device code, one copy per GPU, held until the process
 * ends. The call allocates and frees nothing. On return args->workspace_size holds the size the step needed;
 * a step that needs more than the array returns FTK_ERR_STATIC_WORKSPACE and launches nothing (the headline
 * step, 256 rows x 128256 fp32 with a history penalty, needs about 21 MB). All calls on one GPU share that
 * GPU's array: calls that overlap in time on one GPU (different streams or threads) race; calls on one stream
 * are safe back to back. The array is the current device's (make the stream's device current, as for any launch),
 * and its address is looked up on the first call on a device (hipGetDevice + hipGetSymbolAddress): make that first
 * call outside any graph capture. Every process that loads the library holds the 32 MiB on every GPU it touches,
 * whether or not it calls this entry point. */
#define FTK_FUSED_STATIC_WORKSPACE_BYTES (32u << 20)
int ftk_fused_topk_step_static(ftk_fused_topk_args* args, ftk_stream_t stream);

/* Measurement aid without a counterpart in the reference: reads `bytes` (16-byte aligned, a multiple of 16 is
 * used) once with the launch shape and load instructions of the fused step's streaming kernel and nothing else
 * (one maximum per 16 bytes; one float per wave goes to `sink`, which needs at least 4096 floats). It is the
 * yardstick the streaming kernel's duration is compared with. elapsed_ms != NULL: the launch carries a pair of
 * events, the call waits for the kernel and returns its duration. A measurement aid, not a serving entry point:
 * with elapsed_ms it creates and destroys the two events (hipEventCreate, which may allocate) and blocks the
 * calling thread, so it belongs neither under a graph capture nor in code that must not allocate. */
int ftk_measure_plain_read(const void* data, size_t bytes, float* sink, size_t sink_floats, ftk_stream_t stream,
                           float* elapsed_ms);

/* ---- the steps either side of the sampling path -------------------------------------------- */
/* kernels/logprob_kernels.cu:137-183 invokeLogProbFromLogits<T>: cum_log_probs[b] = sum over step < lengths[b]-1 of
 * log softmax(logits[step, b, :vocab_size])[input_ids[step+1, b]]. logits [max_input_length, batch, Vp] or, with
 * batch_first, [batch, max_input_length, Vp]; input_ids laid out the same way; workspace >= 4 * max_input_length *
 * batch bytes (FTK_ERR_WORKSPACE otherwise; the reference asserts). Results agree with the reference within
 * rounding (1e-5 relative), not bit for bit. */
int ftk_invoke_log_prob_from_logits(int dtype, float* cum_log_probs, const void* logits, const int* input_ids,
                                    const int* input_lengths, size_t max_input_length, size_t batch_size,
                                    size_t vocab_size, size_t vocab_size_padded, void* workspace,
                                    size_t workspace_size, ftk_stream_t stream, bool batch_first);

/* kernels/decoding_kernels.cu:49-65 invokeDecodingInitialize<T>: finished = false, sequence_length =
 * max_input_length, word_ids = sentence_ids[batch] (when word_ids != NULL), cum_log_probs = 0 for the first beam of a
 * batch entry and -MAX_T_VAL (65504 for half, 1e20 otherwise) for the others; cum_log_probs is a T array. */
int ftk_invoke_decoding_initialize(int dtype, bool* finished, int* sequence_length, int* word_ids, void* cum_log_probs,
                                   const int* sentence_ids, int batch_size, int beam_width, int max_input_length,
                                   ftk_stream_t stream);

/* kernels/decoding_kernels.cu:688-696 invokePlusScalar<int>: buf[i] += val */
int ftk_invoke_plus_scalar(int* buf, int val, int size, ftk_stream_t stream);

/* kernels/gpt_kernels.cu:347-357 invokeTransposeAxis01<int>(out, in, in_skipping_dim1, dim0, dim1): out [dim1, dim0],
 * in [dim0, dim1]; with in_skipping_dim1 != NULL column i1 is read at an extra offset in_skipping_dim1[i1] * dim1.
 * This is how the time-major output ids [max_seq, batch] become [batch, max_seq]. out must not alias in. */
int ftk_invoke_transpose_axis01(int* out, const int* in, const int* in_skipping_dim1, int dim0, int dim1,
                                ftk_stream_t stream);

/* kernels/decoding_kernels.cu:697-813 invokeFinalize: per batch entry, the (at most 2 * beam_width, num_beams[b]
 * valid) finished hypotheses ranked by score - largest first, the smaller index among equal scores - and the best
 * beam_width of them copied out: sequence_lengths, cum_log_probs (optional), and ids / log-probs (optional) without
 * their first position. Shapes: output_ids [batch, beam_width, max_seq_len], sequence_lengths and cum_log_probs
 * [batch, beam_width], output_log_probs like output_ids; topk_output_ids and topk_log_probs
 * [batch, 2 * beam_width, max_seq_len + 1], topk_sequence_lengths, scores, topk_cum_log_probs
 * [batch, 2 * beam_width], num_beams [batch]. Hypotheses beyond num_beams[b] count as the lowest score (the
 * reference reads uninitialised shared memory for them). */
int ftk_invoke_finalize(int* output_ids, int* sequence_lengths, float* cum_log_probs, float* output_log_probs,
                        const int* topk_output_ids, const int* topk_sequence_lengths, const float* scores,
                        const float* topk_cum_log_probs, const float* topk_log_probs, const int* num_beams,
                        int beam_width, int max_seq_len, int batch_size, ftk_stream_t stream);

/* BeamHypotheses, kernels/beam_search_topk_kernels.h:31-58, field for field (sequence_lengths_src,
 * length_penalty and is_return_normed_score are carried for callers that fill the reference's struct; the kernels
 * of this call do not read them, like the reference's). */
typedef struct ftk_beam_hypotheses {
    int*         output_ids_tgt;
    int*         sequence_lengths_tgt;
    float*       cum_log_probs;
    float*       normed_scores;
    float*       log_probs;
    float*       min_normed_scores;
    int*         num_beams;
    bool*        is_done;
    const int*   output_ids_src;
    const int*   parent_ids_src;
    const int*   sequence_lengths_src;
    const int*   end_ids;
    const float* log_probs_src;
    int          step;
    int          ite;
    int          batch_size;
    int          local_batch_size;
    int          max_seq_len;
    float        length_penalty;
    bool         early_stopping;
    bool         is_return_normed_score;
} ftk_beam_hypotheses;

/* invokeTopkSoftMax<T>, kernels/online_softmax_beamsearch_kernels.cu:671-701: one beam-search step over
 * log_probs [batch_size * beam_width, vocab_size]. Per row the log-softmax and its 2 * beam_width best tokens; per
 * batch entry the candidates ranked by cum_log_probs + log-softmax (length penalty and diversity term applied as
 * the reference does); end tokens among the first beam_width go to the hypotheses, the others become the next beams:
 * ids [batch_size, beam_width] receives row * vocab_size + token (the reference's absolute ids), cum_log_probs is
 * updated in place, output_log_probs (optional) gets the step's log-probs. beam_hyps may be NULL or carry
 * num_beams == NULL (no hypotheses kept). beam_width 2..64 and vocab_size >= 2 * beam_width, else
 * FTK_ERR_ARGUMENT. temp_storage == NULL: size query in bytes (the reference takes a size in elements from its
 * layer). Sums of exponentials are accumulated in double precision in no particular order, so log-probs agree with
 * the reference's pairwise (max, sum) merges within 1e-5 relative, not bit for bit. */
int ftk_invoke_topk_softmax(int dtype, const void* log_probs, const void* bias, const bool* finished,
                            const int* sequence_lengths, float* cum_log_probs, float* output_log_probs, int* ids,
                            void* temp_storage, size_t* temp_storage_size, const ftk_beam_hypotheses* beam_hyps,
                            int batch_size, int beam_width, int vocab_size, const int* end_ids, float diversity_rate,
                            float length_penalty, ftk_stream_t stream);

/* invokeAddBiasApplyPenalties<T>, kernels/beam_search_penalty_kernels.cu:175-267: what BaseBeamSearchLayer applies
 * to logits [local_batch_size * beam_width, vocab_size_padded] before the step above: bias and temperature with
 * pad columns masked (when there is a bias, a temperature other than 1 or padding), the repetition
 * (multiplicative) or presence (additive) penalty over each beam's own history, followed back through parent_ids
 * (when step > 0 and the penalty is not the neutral value), and the min-length mask of the end id (when
 * step - max_input_length < min_length; needs sequence_lengths and end_ids). current_ids = the ids of step - 1 of
 * this window; previous_ids / parent_ids = the [max_seq_len, batch_size * beam_width] arrays from their start
 * (parent_ids is offset by `ite` windows inside, previous_ids is not, as in the reference). Histories of more than
 * 8192 steps return FTK_ERR_ARGUMENT. */
int ftk_invoke_add_bias_apply_penalties(int dtype, int step, void* logits, const int* current_ids,
                                        const int* previous_ids, const int* parent_ids, const int* input_lengths,
                                        const int* sequence_lengths, const void* bias, int ite, int max_input_length,
                                        int local_batch_size, int batch_size, int beam_width, int vocab_size,
                                        int vocab_size_padded, const int* end_ids, float temperature,
                                        float repetition_penalty, int repetition_penalty_type, int min_length,
                                        ftk_stream_t stream);

/* invokeUpdate, layers/beam_search_layers/OnlineBeamSearchLayer.cu:24-85: splits the absolute ids the step wrote
 * (word_ids, [local_batch_size, beam_width]) into token (word_ids, output_ids: may be the same array) and parent
 * beam (parent_ids), sets finished where the token is the end id, and gives every row the length of the beam it
 * continues plus its own token. An entry whose hypotheses are complete (beam_hyps->num_beams == beam_width) gets
 * all its beams finished. The reference's threads read and write other rows of their batch entry within one launch;
 * here every row first counts its token, then takes the length of its parent (what a warp in lockstep does).
 * beam_width <= 64. */
int ftk_invoke_beam_update(bool* finished, int* parent_ids, int* sequence_length, int* word_ids, int* output_ids,
                           const ftk_beam_hypotheses* beam_hyps, int local_batch_size, int beam_width,
                           int vocab_size_padded, const int* end_ids, ftk_stream_t stream);

/* update_indir_cache_kernelLauncher, layers/beam_search_layers/BaseBeamSearchLayer.cu:22-77: the key / value cache
 * indirection [local_batch_size, beam_width, max_seq_len] of the beams after a step: position `step` points at
 * the beam itself, earlier positions are copied from the parent beam (beam_ids = the step's parent_ids); rows of
 * finished beams are left as they are. batch_dim is accepted and unused, as in the reference. */
int ftk_invoke_update_indir_cache(int* tgt_indir_cache, const int* src_indir_cache, const int* beam_ids,
                                  const bool* finished, int batch_dim, int local_batch_size, int beam_width,
                                  int max_seq_len, int step, ftk_stream_t stream);

/* ---- per-kernel timing of the fused step (the reference's counterpart is its CudaTimer / NVTX ranges,
 * utils/cuda_utils.h:247-258, utils/nvtx_utils.h:37-49) ------------------------------------------
 * ftk_profile_enable(n) makes the next n fused steps bracket each of their kernels with HIP events on
 * the caller's stream (n = 0 switches it off); ftk_profile_read sums them (it synchronises on the
 * events) and resets the count. kernel: 0 = history bitmap, 1 = gather (the streaming pass; the whole step where
 * one launch does it), 2 = select, 3 = the first of two reads a launch with a large k makes (the maxima that bound
 * the row's k-th largest).
 * Measurement aids, not serving entry points: ftk_profile_enable destroys the events of the last call and creates
 * 2 * n new ones per kernel slot (hipEventCreate, which may allocate); steps that run with profiling on launch
 * with those events and do not belong under a graph capture; the
 * event slots and counters are process-wide and unsynchronised, so ftk_profile_enable / ftk_profile_read and
 * the steps they observe must not run concurrently from several threads. With profiling off (the default) the
 * fused steps touch none of this. */
int ftk_profile_enable(int max_launches);
int ftk_profile_read(int kernel, double* total_ms, int* launches);

#ifdef __cplusplus
}
#endif
#endif /* FTK_SAMPLING_H */
