// Bad-word masking, stop-word / length stop criteria, generator initialisation and the small test
// probes of the C ABI.
#include <chrono>
#include <string.h>

#include "ftk_device.cuh"
#include "ftk_sampling.h"
#ifdef FTK_TEST_HOOKS
#include "ftk_test_hooks.h"
#endif
#include "ftk_words.cuh"

namespace ftk {

// src/fastertransformer/kernels/ban_bad_words.cu:22-86. grid (ceil(L/block), rows); one thread per word slot.
// `id_offset`: the window's first row in the batch (the column of row r's history is id_offset + r).
template<int DT>
__global__ void ban_bad_words_kernel(typename Storage<DT>::T* __restrict__ logits, const int* __restrict__ output_ids,
                                     int batch_size, const int* __restrict__ bad_words, int bad_words_len,
                                     bool share_words, int id_offset, int vocab_size_padded, int step)
{
    typedef Storage<DT> S;
    const int           w   = blockIdx.x * blockDim.x + threadIdx.x;
    const int           row = blockIdx.y;
    if (w >= bad_words_len) {
        return;
    }
    const WordList words = word_list(share_words ? bad_words : bad_words + (size_t)row * 2 * bad_words_len, bad_words_len);
    const int      tok   = banned_token(words, w, output_ids + id_offset + row, (size_t)batch_size, step);
    if (0 < tok && tok < vocab_size_padded) {  // token 0 is never banned, as in the reference
        logits[(size_t)row * vocab_size_padded + tok] = S::st(-__builtin_inff());
    }
}

// src/fastertransformer/kernels/stop_criteria_kernels.cu:24-81
__global__ void stop_words_kernel(const int* __restrict__ output_ids, const int* __restrict__ stop_words,
                                  bool* __restrict__ finished, int id_offset, int stop_words_len, int batch_size,
                                  int step)
{
    const int w   = blockIdx.x * blockDim.x + threadIdx.x;
    const int row = blockIdx.y;
    if (w >= stop_words_len) {
        return;
    }
    const WordList words = word_list(stop_words + (size_t)row * 2 * stop_words_len, stop_words_len);
    if (stop_word_matches(words, w, output_ids + id_offset + row, (size_t)batch_size, step)) {
        finished[row] = true;
    }
}

// The two kernels above for beam search: grid (ceil(L/block), rows * beams); the history is followed through
// parent_ids (ftk_words.cuh). `id_offset` is added to the column index as given, like the reference does.
template<int DT>
__global__ void ban_bad_words_beams_kernel(typename Storage<DT>::T* __restrict__ logits,
                                           const int* __restrict__ output_ids, const int* __restrict__ parent_ids,
                                           int batch_size, int beams, const int* __restrict__ bad_words,
                                           int bad_words_len, bool share_words, int id_offset, int vocab_size_padded,
                                           int step)
{
    typedef Storage<DT> S;
    const int           w     = blockIdx.x * blockDim.x + threadIdx.x;
    const int           row   = blockIdx.y;
    const int           entry = row / beams;
    if (w >= bad_words_len) {
        return;
    }
    const WordList words =
        word_list(share_words ? bad_words : bad_words + (size_t)entry * 2 * bad_words_len, bad_words_len);
    const int* first;
    int        count;
    if (!words.ngram(w, &first, &count) || count < 1) {
        return;
    }
    const size_t base = (size_t)id_offset + (size_t)entry * beams;
    const bool   ban  = count == 1
                     || beam_history_ends_with(first, count - 1, output_ids + base, parent_ids + base,
                                               (size_t)batch_size * beams, row % beams, beams, step - 1);
    const int tok = first[count - 1];
    if (ban && 0 < tok && tok < vocab_size_padded) {
        logits[(size_t)row * vocab_size_padded + tok] = S::st(-__builtin_inff());
    }
}

__global__ void stop_words_beams_kernel(const int* __restrict__ output_ids, const int* __restrict__ parent_ids,
                                        const int* __restrict__ stop_words, bool* __restrict__ finished, int id_offset,
                                        int stop_words_len, int batch_size, int beams, int step)
{
    const int w     = blockIdx.x * blockDim.x + threadIdx.x;
    const int row   = blockIdx.y;
    const int entry = row / beams;
    if (w >= stop_words_len) {
        return;
    }
    const WordList words = word_list(stop_words + (size_t)entry * 2 * stop_words_len, stop_words_len);
    const int*     first;
    int            count;
    if (!words.ngram(w, &first, &count)) {
        return;
    }
    const size_t base = (size_t)id_offset + (size_t)entry * beams;
    if (beam_history_ends_with(first, count, output_ids + base, parent_ids + base, (size_t)batch_size * beams,
                               row % beams, beams, step)) {
        finished[row] = true;
    }
}

// src/fastertransformer/kernels/stop_criteria_kernels.cu:106-133: one workgroup; the count goes to
// pinned host memory with a system-scope release so the waiting host thread sees it.
__global__ void __launch_bounds__(512)
length_criterion_kernel(bool* __restrict__ finished, int* finished_sum, const uint32_t* __restrict__ limit, int n,
                        int beam_width, int step)
{
    __shared__ int smem[16];
    int            count = 0;
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
        const bool f = finished[i] || ((uint32_t)step >= limit[i / beam_width]);
        finished[i]  = f;
        count += f ? 1 : 0;
    }
    count = block_sum_i(count, smem);
    if (threadIdx.x == 0) {
        __hip_atomic_store(finished_sum, count, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

__global__ void rng_init_kernel(RngState* states, int n, unsigned long long seed,
                                const unsigned long long* __restrict__ seeds)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        states[i].seed   = seeds != nullptr ? seeds[i] : seed;
        states[i].offset = 0;
    }
}

#ifdef FTK_TEST_HOOKS
__global__ void test_math_kernel(int kind, const float* __restrict__ in, float* __restrict__ out, size_t n)
{
    for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const float x = in[i];
        float       y;
        switch (kind) {
            case 0: y = det_expf(x); break;
            case 1: y = det_logf(x); break;
            case 2: y = half_bits_to_float(float_to_half_bits(x)); break;
            case 3: y = bf16_bits_to_float(float_to_bf16_bits(x)); break;
            case 4: y = 1.0f / (x + 1e-6f); break;             // correctly rounded division
            case 5: y = x * 1.1754944e-38f + x * 0.5f * 1.1754944e-38f; break;  // subnormal arithmetic
            case 6: y = det_expf_nonpos(x); break;
            case 7: {
                // pairs (numerator, denominator): the short division into the even slot, `/` into the odd one
                const float      other = in[i ^ 1];
                const RowDivisor div((i & 1) ? x : other);
                y = (i & 1) ? other / x : (div.ok ? div.divide(x) : x / other);
            } break;
            default: y = x;
        }
        out[i] = y;
    }
}

__global__ void test_rng_kernel(RngState* states, float* out, int batch, int n_draws)
{
    const int b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b < batch) {
        for (int i = 0; i < n_draws; ++i) {
            out[(size_t)b * n_draws + i] = rng_next_uniform(states + b);
        }
    }
}
#endif  // FTK_TEST_HOOKS

}  // namespace ftk

using namespace ftk;

extern "C" {

const char* ftk_error_string(int code)
{
    switch (code) {
        case 0: return "success";
        case FTK_ERR_DTYPE: return "unsupported logits dtype";
        case FTK_ERR_TOPK_DOMAIN: return "top-k kernel supports 1<=k<=1024";
        case FTK_ERR_ARGUMENT: return "invalid argument";
        case FTK_ERR_WORKSPACE: return "workspace too small";
        case FTK_ERR_UNSUPPORTED:
            return "log-prob outputs are not covered by the fused step for this configuration: run the kernel sequence";
        case FTK_ERR_STATIC_WORKSPACE:
            return "the step needs more workspace than the library's fixed array (FTK_FUSED_STATIC_WORKSPACE_BYTES): "
                   "use ftk_fused_topk_step with a caller workspace";
        default: break;
    }
    if (code > 0) {
        return hipGetErrorString((hipError_t)code);
    }
    return "unknown error";
}

int ftk_invoke_curand_initialize(ftk_rng_state* state, size_t batch_size, unsigned long long random_seed,
                                 ftk_stream_t stream)
{
    if (batch_size == 0) {
        return 0;
    }
    rng_init_kernel<<<(int)((batch_size + 255) / 256), 256, 0, (hipStream_t)stream>>>((RngState*)state, (int)batch_size,
                                                                                    random_seed, nullptr);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_curand_batch_initialize(ftk_rng_state* states, size_t batch_size,
                                       const unsigned long long* random_seeds, ftk_stream_t stream)
{
    if (batch_size == 0) {
        return 0;
    }
    rng_init_kernel<<<(int)((batch_size + 255) / 256), 256, 0, (hipStream_t)stream>>>((RngState*)states,
                                                                                    (int)batch_size, 0ull, random_seeds);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_ban_bad_words(int dtype, void* logits, const int* output_ids_buf, const int* parent_ids_buf,
                             int batch_size, int local_batch_size, int beam_width, const int* bad_words,
                             bool share_words, size_t bad_words_len, int id_offset, int vocab_size_padded,
                             size_t step, ftk_stream_t stream)
{
    if (bad_words_len == 0 || local_batch_size <= 0) {
        return 0;
    }
    if (beam_width < 1 || (beam_width > 1 && parent_ids_buf == nullptr)
        || (long long)local_batch_size * beam_width > 65535) {
        return FTK_ERR_ARGUMENT;
    }
    const int block = (int)min((size_t)256, ((bad_words_len + 63) / 64) * 64);
    if (beam_width > 1) {
        dim3 beams_grid((unsigned)((bad_words_len + block - 1) / block), (unsigned)(local_batch_size * beam_width));
        FTK_DISPATCH_DTYPE(dtype, ban_bad_words_beams_kernel<DT><<<beams_grid, block, 0, (hipStream_t)stream>>>(
                                      (Storage<DT>::T*)logits, output_ids_buf, parent_ids_buf, batch_size, beam_width,
                                      bad_words, (int)bad_words_len, share_words, id_offset, vocab_size_padded,
                                      (int)step));
        FTK_LAUNCH_CHECK();
        return 0;
    }
    dim3      grid((unsigned)((bad_words_len + block - 1) / block), (unsigned)local_batch_size);
    FTK_DISPATCH_DTYPE(dtype, ban_bad_words_kernel<DT><<<grid, block, 0, (hipStream_t)stream>>>(
                                  (Storage<DT>::T*)logits, output_ids_buf, batch_size, bad_words, (int)bad_words_len,
                                  share_words, id_offset, vocab_size_padded, (int)step));
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_stop_words_criterion_rows(const int* output_ids, const int* parent_ids, const int* stop_words,
                                         bool* finished, size_t id_offset, size_t stop_words_len, int batch_size,
                                         int num_rows, int beam_width, int step, ftk_stream_t stream)
{
    if (stop_words_len == 0 || num_rows <= 0) {
        return 0;
    }
    if (beam_width < 1 || (beam_width > 1 && parent_ids == nullptr) || (long long)num_rows * beam_width > 65535) {
        return FTK_ERR_ARGUMENT;
    }
    const int block = (int)min((size_t)256, ((stop_words_len + 63) / 64) * 64);
    if (beam_width > 1) {
        dim3 beams_grid((unsigned)((stop_words_len + block - 1) / block), (unsigned)(num_rows * beam_width));
        stop_words_beams_kernel<<<beams_grid, block, 0, (hipStream_t)stream>>>(
            output_ids, parent_ids, stop_words, finished, (int)id_offset, (int)stop_words_len, batch_size, beam_width,
            step);
        FTK_LAUNCH_CHECK();
        return 0;
    }
    dim3      grid((unsigned)((stop_words_len + block - 1) / block), (unsigned)num_rows);
    stop_words_kernel<<<grid, block, 0, (hipStream_t)stream>>>(output_ids, stop_words, finished, (int)id_offset,
                                                               (int)stop_words_len, batch_size, step);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_stop_words_criterion(const int* output_ids, const int* parent_ids, const int* stop_words,
                                    bool* finished, size_t id_offset, size_t stop_words_len, int batch_size,
                                    int beam_width, int step, ftk_stream_t stream)
{
    // the reference launcher examines `batch_size` rows starting at the given pointers
    return ftk_invoke_stop_words_criterion_rows(output_ids, parent_ids, stop_words, finished, id_offset,
                                                stop_words_len, batch_size, batch_size, beam_width, step, stream);
}

int ftk_invoke_length_criterion(bool* finished, bool* should_stop, int* h_pinned_finished_sum,
                                const uint32_t* sequence_limit_length, int batch_size, int beam_width, int step,
                                ftk_stream_t stream)
{
    if (should_stop == nullptr || h_pinned_finished_sum == nullptr || batch_size <= 0) {
        return FTK_ERR_ARGUMENT;
    }
    const int n     = batch_size * beam_width;
    const int block = min(512, ((n + 63) / 64) * 64);
    __atomic_store_n(h_pinned_finished_sum, -1, __ATOMIC_RELEASE);
    length_criterion_kernel<<<1, block, 0, (hipStream_t)stream>>>(finished, h_pinned_finished_sum,
                                                                  sequence_limit_length, n, beam_width, step);
    FTK_LAUNCH_CHECK();
    // Wait for the kernel's store to pinned memory (the reference spins the same way,
    // stop_criteria_kernels.cu:153), but bounded: after 2 ms fall back to a stream synchronise so a
    // failed launch can never hang the caller.
    const auto t0 = std::chrono::steady_clock::now();
    while (__atomic_load_n(h_pinned_finished_sum, __ATOMIC_ACQUIRE) == -1) {
        if (std::chrono::steady_clock::now() - t0 > std::chrono::milliseconds(2)) {
            const hipError_t e = hipStreamSynchronize((hipStream_t)stream);
            if (e != hipSuccess) {
                return (int)e;
            }
            break;
        }
    }
    const int sum = __atomic_load_n(h_pinned_finished_sum, __ATOMIC_ACQUIRE);
    if (sum == -1) {
        return FTK_ERR_ARGUMENT;  // h_pinned_finished_sum is not host memory the device can write
    }
    *should_stop = sum == n;
    return 0;
}

#ifdef FTK_TEST_HOOKS
// ---- test hooks (declared in include/ftk_test_hooks.h; only the hooks build of the library has them)
float ftk_host_expf(float x)
{
    return det_expf(x);
}

float ftk_host_logf(float x)
{
    return det_logf(x);
}

void ftk_host_philox4x32_10(const uint32_t counter[4], const uint32_t key[2], uint32_t out[4])
{
    philox4x32_10(counter[0], counter[1], counter[2], counter[3], key[0], key[1], out);
}

int ftk_test_device_math(int kind, const float* in, float* out, size_t n, ftk_stream_t stream)
{
    if (n == 0) {
        return 0;
    }
    const int grid = (int)min((size_t)2048, (n + 255) / 256);
    test_math_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(kind, in, out, n);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_test_rng_uniform(ftk_rng_state* states, float* out, int batch_size, int n_draws, ftk_stream_t stream)
{
    if (batch_size <= 0) {
        return 0;
    }
    test_rng_kernel<<<(batch_size + 255) / 256, 256, 0, (hipStream_t)stream>>>((RngState*)states, out, batch_size,
                                                                             n_draws);
    FTK_LAUNCH_CHECK();
    return 0;
}
#endif  // FTK_TEST_HOOKS

}  // extern "C"
