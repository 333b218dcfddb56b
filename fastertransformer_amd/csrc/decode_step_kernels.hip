// The steps either side of the sampling path: context log-probs of given tokens and the small state
// kernels of a decode loop.
//   src/fastertransformer/kernels/logprob_kernels.cu:35-183    invokeLogProbFromLogits
//   src/fastertransformer/kernels/decoding_kernels.cu:26-65    invokeDecodingInitialize
//   src/fastertransformer/kernels/decoding_kernels.cu:680-696  invokePlusScalar
//   src/fastertransformer/kernels/gpt_kernels.cu:329-357       invokeTransposeAxis01 (2-D, optional offsets)
#include "ftk_device.cuh"
#include "ftk_sampling.h"

namespace ftk {

// ---- log-probs -----------------------------------------------------------------------------------
// log_probs[step, b] = logits[step, b, ids[step+1, b]] - max - log(sum exp(logits - max) + 1e-9) for
// step < lengths[b] - 1. The reference reads every row twice (max, then sum); here a row is read once:
// each thread keeps a running (max, sum of exp relative to that max) over 16-byte vectors and the pairs are
// merged across the workgroup. The result is a float within rounding of the reference's, not bit-equal.
constexpr int LP_THREADS = 256;

struct MaxSum {
    float m, s;
};

__device__ __forceinline__ MaxSum merge(MaxSum a, MaxSum b)
{
    const float M = __builtin_fmaxf(a.m, b.m);
    if (M == -__builtin_inff()) {
        return MaxSum{M, 0.0f};
    }
    return MaxSum{M, a.s * __expf(a.m - M) + b.s * __expf(b.m - M)};
}

template<int DT>
__global__ void __launch_bounds__(LP_THREADS)
log_probs_kernel(float* __restrict__ log_probs, const typename Storage<DT>::T* __restrict__ logits,
                 const int* __restrict__ ids, const int* __restrict__ lengths, int max_len, int batch, int V,
                 size_t Vp, bool batch_first)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    __shared__ MaxSum     sh[LP_THREADS / WAVE];
    const int             t    = threadIdx.x;
    const int             step = batch_first ? (int)(blockIdx.x % (unsigned)(max_len - 1)) : (int)(blockIdx.x / (unsigned)batch);
    const int             b    = batch_first ? (int)(blockIdx.x / (unsigned)(max_len - 1)) : (int)(blockIdx.x % (unsigned)batch);
    if (step >= lengths[b] - 1) {
        return;
    }
    const size_t off = batch_first ? ((size_t)b * max_len + step) * Vp : ((size_t)step * batch + b) * Vp;
    const T*     row = logits + off;
    const float  NEG = -__builtin_inff();
    MaxSum       acc{NEG, 0.0f};

    auto add_block = [&](const float* x, int n) {
        float vm = NEG;
        for (int j = 0; j < n; ++j) {
            vm = __builtin_fmaxf(vm, x[j]);
        }
        if (vm == NEG) {
            return;
        }
        if (vm > acc.m) {
            acc.s *= __expf(acc.m - vm);  // exp(-inf) = 0 for the first block
            acc.m = vm;
        }
        float add = 0.0f;
        for (int j = 0; j < n; ++j) {
            add += __expf(x[j] - acc.m);
        }
        acc.s += add;
    };

    // columns before the first 16-byte boundary and after the last whole vector go one by one
    const int a     = (int)(((16u - ((uintptr_t)row & 15u)) & 15u) / sizeof(T));
    const int head  = a < V ? a : V;
    const int nvec  = (V - head) / EPV;
    const int tail0 = head + nvec * EPV;
    if (t < head) {
        const float x = S::ld(row[t]);
        add_block(&x, 1);
    }
    const uint4* vec = reinterpret_cast<const uint4*>(row + head);
    constexpr int U  = 4;  // vectors in flight per thread
    for (int i0 = t; i0 < nvec; i0 += U * LP_THREADS) {
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * LP_THREADS;
            raw[u]      = i < nvec ? vec[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            if (i0 + u * LP_THREADS < nvec) {
                float    x[EPV];
                const T* e = reinterpret_cast<const T*>(&raw[u]);
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    x[j] = S::ld(e[j]);
                }
                add_block(x, EPV);
            }
        }
    }
    if (tail0 + t < V) {
        const float x = S::ld(row[tail0 + t]);
        add_block(&x, 1);
    }

#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        MaxSum other;
        other.m = __shfl_xor(acc.m, o, WAVE);
        other.s = __shfl_xor(acc.s, o, WAVE);
        acc     = merge(acc, other);
    }
    if (lane_id() == 0) {
        sh[wave_id()] = acc;
    }
    __syncthreads();
    if (t == 0) {
        MaxSum all = sh[0];
        for (int w = 1; w < LP_THREADS / WAVE; ++w) {
            all = merge(all, sh[w]);
        }
        const int idx = batch_first ? step + b * (max_len - 1) : step * batch + b;
        const int tok = batch_first ? step + 1 + b * max_len : (step + 1) * batch + b;
        log_probs[idx] = S::ld(row[ids[tok]]) - all.m - det_logf(all.s + 1e-9f);
    }
}

__global__ void __launch_bounds__(LP_THREADS)
accumulate_log_probs_kernel(float* __restrict__ cum_log_probs, const float* __restrict__ log_probs,
                            const int* __restrict__ lengths, int max_len, int batch, bool batch_first)
{
    __shared__ float sh[LP_THREADS / WAVE];
    const int        b      = blockIdx.x;
    const int        length = lengths[b];
    const float*     lp     = log_probs + (batch_first ? (size_t)b * (max_len - 1) : (size_t)b);
    const size_t     stride = batch_first ? 1 : (size_t)batch;
    float            acc    = 0.0f;
    for (int step = threadIdx.x; step < length - 1; step += LP_THREADS) {
        acc += lp[step * stride];
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        acc += __shfl_xor(acc, o, WAVE);
    }
    if (lane_id() == 0) {
        sh[wave_id()] = acc;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        float total = 0.0f;
        for (int w = 0; w < LP_THREADS / WAVE; ++w) {
            total += sh[w];
        }
        cum_log_probs[b] = total;
    }
}

// ---- decode-loop state ---------------------------------------------------------------------------
template<int DT>
__global__ void decoding_initialize_kernel(bool* __restrict__ finished, int* __restrict__ sequence_length,
                                           int* __restrict__ word_ids, typename Storage<DT>::T* __restrict__ cum_log_probs,
                                           const int* __restrict__ sentence_ids, int n, int beam_width,
                                           int max_input_length)
{
    typedef Storage<DT> S;
    // the reference's "minus infinity" of the beam scores: HALF_FLT_MAX for half, 1e20 otherwise
    const float max_t = DT == DT_F16 ? 65504.0f : 1e20f;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += blockDim.x * gridDim.x) {
        finished[i]        = false;
        sequence_length[i] = max_input_length;
        if (word_ids != nullptr) {
            word_ids[i] = sentence_ids[i / beam_width];
        }
        cum_log_probs[i] = S::st((i % beam_width == 0) ? 0.0f : -max_t);
    }
}

// The hypotheses of a batch entry (at most 2 * beam_width of them, num_beams valid) ranked by score, the best
// beam_width copied out without their first token. One workgroup per batch entry; a rank is the hypothesis with
// the largest remaining score, the smallest index among equals (the reference scans from index 0).
constexpr int FIN_THREADS = 256;

__global__ void __launch_bounds__(FIN_THREADS)
finalize_kernel(int* __restrict__ output_ids, int* __restrict__ sequence_lengths, float* __restrict__ cum_log_probs,
                float* __restrict__ output_log_probs, const int* __restrict__ topk_output_ids,
                const int* __restrict__ topk_sequence_lengths, const float* __restrict__ scores,
                const float* __restrict__ topk_cum_log_probs, const float* __restrict__ topk_log_probs,
                const int* __restrict__ num_beams, int beam_width, int max_seq_len)
{
    extern __shared__ int        fin_shared[];  // rank [beam_width], scores [2 * beam_width]
    __shared__ unsigned long long red[16];
    int*                         rank     = fin_shared;
    float*                       s_scores = reinterpret_cast<float*>(fin_shared + beam_width);
    const int                    b        = blockIdx.x;
    const int                    t        = threadIdx.x;
    const int                    hyps     = 2 * beam_width;
    const int                    valid    = min(num_beams[b], hyps);
    for (int j = t; j < hyps; j += FIN_THREADS) {
        s_scores[j] = j < valid ? scores[(size_t)b * hyps + j] : -3.402823466e+38f;
    }
    __syncthreads();
    for (int i = 0; i < beam_width; ++i) {
        // largest score, then smallest index: one 64-bit maximum over (order-preserving score, ~index)
        unsigned long long best = 0ull;
        for (int j = t; j < hyps; j += FIN_THREADS) {
            const unsigned long long key = ((unsigned long long)order_key(s_scores[j]) << 32) | (uint32_t)(~j);
            best                         = key > best ? key : best;
        }
        best = block_max<unsigned long long, FIN_THREADS / WAVE>(best, red, 0ull);
        if (t == 0) {
            const int j = (int)~(uint32_t)best;
            rank[i]     = j;
            s_scores[j] = -3.402823466e+38f;
        }
        __syncthreads();
    }
    for (int i = t; i < beam_width; i += FIN_THREADS) {
        const size_t src                             = (size_t)b * hyps + rank[i];
        sequence_lengths[(size_t)b * beam_width + i] = topk_sequence_lengths[src];
        if (cum_log_probs != nullptr) {
            cum_log_probs[(size_t)b * beam_width + i] = topk_cum_log_probs[src];
        }
    }
    for (int beam = 0; beam < beam_width; ++beam) {
        const size_t src = ((size_t)b * hyps + rank[beam]) * (max_seq_len + 1) + 1;  // (+1: the start token is dropped)
        const size_t dst = ((size_t)b * beam_width + beam) * max_seq_len;
        const int    len = topk_sequence_lengths[(size_t)b * hyps + rank[beam]];
        for (int i = t; i < len; i += FIN_THREADS) {
            output_ids[dst + i] = topk_output_ids[src + i];
            if (output_log_probs != nullptr) {
                output_log_probs[dst + i] = topk_log_probs[src + i];
            }
        }
    }
}

__global__ void plus_scalar_kernel(int* __restrict__ buf, int val, int size)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < size; i += blockDim.x * gridDim.x) {
        buf[i] += val;
    }
}

// out[i1, i0] = in[offset(i1) + i0 * dim1 + i1]: 32 x 32 tiles through LDS so that both sides are coalesced
constexpr int TR_TILE = 32;

__global__ void __launch_bounds__(TR_TILE * 8)
transpose_axis01_kernel(int* __restrict__ out, const int* __restrict__ in, const int* __restrict__ in_skipping_dim1,
                        int dim0, int dim1)
{
    __shared__ int tile[TR_TILE][TR_TILE + 1];
    const int      tx = threadIdx.x % TR_TILE, ty = threadIdx.x / TR_TILE;  // 32 x 8
    const int      b0 = blockIdx.y * TR_TILE, b1 = blockIdx.x * TR_TILE;
    for (int r = ty; r < TR_TILE; r += 8) {
        const int i0 = b0 + r, i1 = b1 + tx;
        if (i0 < dim0 && i1 < dim1) {
            const size_t offset = in_skipping_dim1 == nullptr ? 0 : (size_t)in_skipping_dim1[i1] * dim1;
            tile[r][tx]         = in[offset + (size_t)i0 * dim1 + i1];
        }
    }
    __syncthreads();
    for (int r = ty; r < TR_TILE; r += 8) {
        const int i1 = b1 + r, i0 = b0 + tx;
        if (i0 < dim0 && i1 < dim1) {
            out[(size_t)i1 * dim0 + i0] = tile[tx][r];
        }
    }
}

}  // namespace ftk

using namespace ftk;

extern "C" {

int ftk_invoke_log_prob_from_logits(int dtype, float* cum_log_probs, const void* logits, const int* input_ids,
                                    const int* input_lengths, size_t max_input_length, size_t batch_size,
                                    size_t vocab_size, size_t vocab_size_padded, void* workspace,
                                    size_t workspace_size, ftk_stream_t stream, bool batch_first)
{
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (batch_size == 0) {
        return 0;
    }
    if (cum_log_probs == nullptr || logits == nullptr || input_ids == nullptr || input_lengths == nullptr
        || vocab_size == 0 || vocab_size > vocab_size_padded || max_input_length == 0) {
        return FTK_ERR_ARGUMENT;
    }
    if (workspace == nullptr || workspace_size < sizeof(float) * max_input_length * batch_size) {
        return FTK_ERR_WORKSPACE;  // the reference asserts the same bound (logprob_kernels.cu:161)
    }
    hipStream_t st        = (hipStream_t)stream;
    float*      log_probs = (float*)workspace;
    if (max_input_length > 1) {
        const size_t rows = (max_input_length - 1) * batch_size;
        if (rows > 0x7FFFFFFFull) {
            return FTK_ERR_ARGUMENT;
        }
        FTK_DISPATCH_DTYPE(dtype, log_probs_kernel<DT><<<(unsigned)rows, LP_THREADS, 0, st>>>(
                                      log_probs, (const Storage<DT>::T*)logits, input_ids, input_lengths,
                                      (int)max_input_length, (int)batch_size, (int)vocab_size, vocab_size_padded,
                                      batch_first));
        FTK_LAUNCH_CHECK();
    }
    accumulate_log_probs_kernel<<<(unsigned)batch_size, LP_THREADS, 0, st>>>(
        cum_log_probs, log_probs, input_lengths, (int)max_input_length, (int)batch_size, batch_first);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_decoding_initialize(int dtype, bool* finished, int* sequence_length, int* word_ids, void* cum_log_probs,
                                   const int* sentence_ids, int batch_size, int beam_width, int max_input_length,
                                   ftk_stream_t stream)
{
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    const int n = batch_size * beam_width;
    if (n <= 0) {
        return 0;
    }
    if (finished == nullptr || sequence_length == nullptr || cum_log_probs == nullptr
        || (word_ids != nullptr && sentence_ids == nullptr) || beam_width < 1) {
        return FTK_ERR_ARGUMENT;
    }
    FTK_DISPATCH_DTYPE(dtype, decoding_initialize_kernel<DT><<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(
                                  finished, sequence_length, word_ids, (Storage<DT>::T*)cum_log_probs, sentence_ids, n,
                                  beam_width, max_input_length));
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_plus_scalar(int* buf, int val, int size, ftk_stream_t stream)
{
    if (size <= 0) {
        return 0;
    }
    if (buf == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    plus_scalar_kernel<<<min(1024, (size + 255) / 256), 256, 0, (hipStream_t)stream>>>(buf, val, size);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_transpose_axis01(int* out, const int* in, const int* in_skipping_dim1, int dim0, int dim1,
                                ftk_stream_t stream)
{
    if (dim0 <= 0 || dim1 <= 0) {
        return 0;
    }
    if (out == nullptr || in == nullptr || out == in) {
        return FTK_ERR_ARGUMENT;
    }
    dim3 grid((dim1 + TR_TILE - 1) / TR_TILE, (dim0 + TR_TILE - 1) / TR_TILE);
    transpose_axis01_kernel<<<grid, TR_TILE * 8, 0, (hipStream_t)stream>>>(out, in, in_skipping_dim1, dim0, dim1);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_finalize(int* output_ids, int* sequence_lengths, float* cum_log_probs, float* output_log_probs,
                        const int* topk_output_ids, const int* topk_sequence_lengths, const float* scores,
                        const float* topk_cum_log_probs, const float* topk_log_probs, const int* num_beams,
                        int beam_width, int max_seq_len, int batch_size, ftk_stream_t stream)
{
    if (batch_size <= 0) {
        return 0;
    }
    if (output_ids == nullptr || sequence_lengths == nullptr || topk_output_ids == nullptr
        || topk_sequence_lengths == nullptr || scores == nullptr || num_beams == nullptr
        || (cum_log_probs != nullptr && topk_cum_log_probs == nullptr)
        || (output_log_probs != nullptr && topk_log_probs == nullptr) || beam_width < 1 || beam_width * 2 >= 1024
        || max_seq_len < 0) {
        return FTK_ERR_ARGUMENT;  // (the reference asserts 2 * beam_width < 1024)
    }
    const size_t smem = (size_t)beam_width * sizeof(int) + (size_t)beam_width * 2 * sizeof(float);
    finalize_kernel<<<batch_size, FIN_THREADS, smem, (hipStream_t)stream>>>(
        output_ids, sequence_lengths, cum_log_probs, output_log_probs, topk_output_ids, topk_sequence_lengths, scores,
        topk_cum_log_probs, topk_log_probs, num_beams, beam_width, max_seq_len);
    FTK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
