// Stand-alone logit penalty / mask kernels (in place on the logits, like the reference launchers
// in src/fastertransformer/kernels/sampling_penalty_kernels.cu and the end-id mask of
// src/fastertransformer/kernels/sampling_topk_kernels.cu:67-110).
//
// These are the drop-in `invoke*` entry points. The decode layer's hot path does not call them:
// it folds the same arithmetic (the `*_value` helpers of ftk_transform.cuh) into the single
// streaming pass of the fused kernel.
#include "ftk_device.cuh"
#include "ftk_sampling.h"
#include "ftk_transform.cuh"

namespace ftk {

constexpr int EW_THREADS = 256;

// ---- temperature (+ bias) ------------------------------------------------------------------
// One 16-byte vector per thread and iteration when rows are 16-byte aligned, scalar otherwise.
template<int DT, bool VEC16>
__global__ void __launch_bounds__(EW_THREADS)
temperature_kernel(typename Storage<DT>::T* __restrict__ logits, const typename Storage<DT>::T* __restrict__ bias,
                   const float* __restrict__ temperatures, float scalar_temperature, int V, int Vp, bool scalar_variant)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = VEC16 ? (int)(16 / sizeof(T)) : 1;
    const int             row = blockIdx.y;
    const float           temp = temperatures != nullptr ? temperatures[row] : scalar_temperature;
    const TemperatureCtx<DT> ctx(temp, V, Vp, scalar_variant);
    T*                    rowp = logits + (size_t)row * Vp;
    const int             nvec = Vp / EPV;
    for (int i = blockIdx.x * EW_THREADS + threadIdx.x; i < nvec; i += gridDim.x * EW_THREADS) {
        if constexpr (VEC16) {
            uint4 raw = reinterpret_cast<const uint4*>(rowp)[i];
            T*    e   = reinterpret_cast<T*>(&raw);
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                const int v = i * EPV + j;
                e[j]        = ctx.apply(e[j], bias, v);
            }
            reinterpret_cast<uint4*>(rowp)[i] = raw;
        }
        else {
            rowp[i] = ctx.apply(rowp[i], bias, i);
        }
    }
}

template<int DT>
static int launch_temperature(void* logits, const void* bias, const float* temperatures, float scalar_temperature,
                              int batch, int V, int Vp, bool scalar_variant, hipStream_t stream)
{
    typedef typename Storage<DT>::T T;
    if (batch <= 0 || Vp <= 0) {
        return 0;
    }
    const bool vec = ((size_t)Vp * sizeof(T)) % 16 == 0 && ((uintptr_t)logits % 16) == 0;
    const int  epv = vec ? (int)(16 / sizeof(T)) : 1;
    const int  gx  = max(1, min((Vp / epv + EW_THREADS - 1) / EW_THREADS, 64));
    dim3       grid(gx, batch);
    if (vec) {
        temperature_kernel<DT, true><<<grid, EW_THREADS, 0, stream>>>((T*)logits, (const T*)bias, temperatures,
                                                                      scalar_temperature, V, Vp, scalar_variant);
    }
    else {
        temperature_kernel<DT, false><<<grid, EW_THREADS, 0, stream>>>((T*)logits, (const T*)bias, temperatures,
                                                                       scalar_temperature, V, Vp, scalar_variant);
    }
    FTK_LAUNCH_CHECK();
    return 0;
}

// ---- repetition / presence penalty -----------------------------------------------------------
// One workgroup per row. Every distinct history id must be penalised once from its pre-penalty
// value; an LDS bitmap over the vocabulary elects one owner per id (atomicOr), and only the owner
// touches that logit, so no second phase is needed. The vocabulary is walked in windows of
// BITMAP_BITS ids when it exceeds the bitmap.
constexpr int REP_THREADS  = 256;
constexpr int BITMAP_WORDS = 8192;  // 262144 ids per window, 32 KB of LDS
constexpr int BITMAP_BITS  = BITMAP_WORDS * 32;

template<int DT>
__global__ void __launch_bounds__(REP_THREADS)
repetition_kernel(typename Storage<DT>::T* __restrict__ logits, const float* __restrict__ penalties,
                  float scalar_penalty, const int* __restrict__ output_ids, int batch_size, int vocab_stride,
                  int id_limit, const int* __restrict__ input_lengths, int max_input_length, int step, int type)
{
    typedef Storage<DT>   S;
    __shared__ uint32_t   bitmap[BITMAP_WORDS];
    const int             row          = blockIdx.x;
    const float           pen          = penalties != nullptr ? penalties[row] : scalar_penalty;
    const int             input_length = input_lengths != nullptr ? input_lengths[row] : max_input_length;
    typename S::T*        rowp         = logits + (size_t)row * vocab_stride;
    for (int base = 0; base < id_limit; base += BITMAP_BITS) {
        const int words = min(BITMAP_WORDS, (id_limit - base + 31) / 32);
        for (int i = threadIdx.x; i < words; i += REP_THREADS) {
            bitmap[i] = 0u;
        }
        __syncthreads();
        for (int t = threadIdx.x; t < step; t += REP_THREADS) {
            if (t >= input_length && t < max_input_length) {
                continue;  // padding between a short prompt and max_input_length
            }
            const int id = output_ids[(size_t)t * batch_size + row];
            if (id < base || id >= id_limit || id >= base + BITMAP_BITS) {
                continue;
            }
            const int      rel = id - base;
            const uint32_t bit = 1u << (rel & 31);
            const uint32_t old = atomicOr(&bitmap[rel >> 5], bit);
            if ((old & bit) == 0u) {
                rowp[id] = S::st(repetition_value(S::ld(rowp[id]), pen, type));
            }
        }
        __syncthreads();
    }
}

// ---- presence + frequency penalty (extension) -----------------------------------------------
// One workgroup per row. The ids of the history are counted in an open-addressing table in LDS (`slots` entries,
// a power of two of at least twice the history length): every distinct id ends up in one slot with its number
// of occurrences, and the slot's owner applies the penalty once, from the unpenalised value.
template<int DT>
__global__ void __launch_bounds__(REP_THREADS)
frequency_kernel(typename Storage<DT>::T* __restrict__ logits, const float* __restrict__ presence,
                 const float* __restrict__ frequency, const int* __restrict__ output_ids, int batch_size,
                 int vocab_stride, const int* __restrict__ input_lengths, int max_input_length, int step, int slots)
{
    typedef Storage<DT>   S;
    extern __shared__ int table[];  // ids [slots], counts [slots]
    int*                  ids          = table;
    int*                  counts       = table + slots;
    const int             row          = blockIdx.x;
    const int             input_length = input_lengths != nullptr ? input_lengths[row] : max_input_length;
    typename S::T*        rowp         = logits + (size_t)row * vocab_stride;
    for (int i = threadIdx.x; i < slots; i += REP_THREADS) {
        ids[i]    = -1;
        counts[i] = 0;
    }
    __syncthreads();
    const int shift = __builtin_clz((unsigned)slots) + 1;  // the top log2(slots) bits of the product
    for (int t = threadIdx.x; t < step; t += REP_THREADS) {
        const bool pad = t >= input_length && t < max_input_length;
        const int  id  = output_ids[(size_t)t * batch_size + row];
        if (pad || id < 0 || id >= vocab_stride) {
            continue;
        }
        int h = (int)(((unsigned)id * 2654435761u) >> shift);
        for (;;) {  // (the table is at most half full: an empty slot is always found)
            const int old = atomicCAS(&ids[h], -1, id);
            if (old == -1 || old == id) {
                atomicAdd(&counts[h], 1);
                break;
            }
            h = (h + 1) & (slots - 1);
        }
    }
    __syncthreads();
    const float pres = presence[row], freq = frequency[row];
    for (int i = threadIdx.x; i < slots; i += REP_THREADS) {
        const int id = ids[i];
        if (id >= 0) {
            rowp[id] = S::st(frequency_value(S::ld(rowp[id]), pres, freq, counts[i]));
        }
    }
}

// ---- min length -----------------------------------------------------------------------------
template<int DT>
__global__ void min_length_kernel(typename Storage<DT>::T* __restrict__ logits, const int* __restrict__ min_lengths,
                                  const int* __restrict__ end_ids, const int* __restrict__ sequence_lengths,
                                  int max_input_length, int batch, int Vp)
{
    typedef Storage<DT> S;
    const int           b = blockIdx.x * blockDim.x + threadIdx.x;
    if (b >= batch) {
        return;
    }
    if (min_length_masks(sequence_lengths[b], max_input_length, min_lengths[b])) {
        logits[(size_t)b * Vp + end_ids[b]] = S::st(-S::max_t());
    }
}

// ---- end-id / padding mask (+ bias) ------------------------------------------------------------
template<int DT>
__global__ void __launch_bounds__(EW_THREADS)
end_mask_kernel(typename Storage<DT>::T* __restrict__ logits, const typename Storage<DT>::T* __restrict__ bias,
                const int* __restrict__ end_ids, const bool* __restrict__ finished, int V, int Vp)
{
    typedef Storage<DT> S;
    const int           row = blockIdx.y;
    const bool          fin = finished != nullptr ? finished[row] : false;
    typename S::T*      rowp = logits + (size_t)row * Vp;
    // unfinished rows without bias only need their pad columns written
    const int start = (fin || bias != nullptr) ? 0 : V;
    const int end_id = fin ? end_ids[row] : -1;
    for (int v = start + blockIdx.x * EW_THREADS + threadIdx.x; v < Vp; v += gridDim.x * EW_THREADS) {
        if (v >= V) {
            rowp[v] = S::st(-S::max_t());
        }
        else if (fin) {
            rowp[v] = S::st(v == end_id ? S::max_t() : -S::max_t());
        }
        else {
            rowp[v] = S::st(S::ld(rowp[v]) + S::ld(bias[v]));
        }
    }
}

}  // namespace ftk

using namespace ftk;

extern "C" {

int ftk_invoke_apply_temperature_penalty(int dtype, void* logits, const void* bias, float temperature, int batch_size,
                                         int vocab_size, int vocab_size_padd, ftk_stream_t stream)
{
    FTK_DISPATCH_DTYPE(dtype, return launch_temperature<DT>(logits, bias, nullptr, temperature, batch_size, vocab_size,
                                                            vocab_size_padd, true, (hipStream_t)stream));
    return 0;
}

int ftk_invoke_batch_apply_temperature_penalty(int dtype, void* logits, const void* bias, const float* temperatures,
                                               int batch_size, int vocab_size, int vocab_size_padd,
                                               ftk_stream_t stream)
{
    if (temperatures == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    FTK_DISPATCH_DTYPE(dtype, return launch_temperature<DT>(logits, bias, temperatures, 1.0f, batch_size, vocab_size,
                                                            vocab_size_padd, false, (hipStream_t)stream));
    return 0;
}

static int launch_repetition(int dtype, void* logits, const float* penalties, float scalar_penalty,
                             const int* output_ids, int batch_size, int local_batch_size, int vocab_stride,
                             int id_limit, const int* input_lengths, int max_input_length, int step, int type,
                             hipStream_t stream)
{
    if (type == FTK_PENALTY_NONE || local_batch_size <= 0 || step <= 0) {
        return dtype >= 0 && dtype <= 2 ? 0 : FTK_ERR_DTYPE;
    }
    if (type != FTK_PENALTY_ADDITIVE && type != FTK_PENALTY_MULTIPLICATIVE) {
        return FTK_ERR_ARGUMENT;
    }
    FTK_DISPATCH_DTYPE(dtype, repetition_kernel<DT><<<local_batch_size, REP_THREADS, 0, stream>>>(
                                  (Storage<DT>::T*)logits, penalties, scalar_penalty, output_ids, batch_size,
                                  vocab_stride, id_limit, input_lengths, max_input_length, step, type));
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_apply_repetition_penalty(int dtype, void* logits, float penalty, const int* start_ids,
                                        const int* output_ids, int batch_size, int local_batch_size, int vocab_size,
                                        int vocab_size_padd, const int* input_lengths, int max_input_len, int step,
                                        int penalty_type, ftk_stream_t stream)
{
    (void)start_ids;
    // this variant skips ids >= vocab_size and strides rows by vocab_size_padd
    return launch_repetition(dtype, logits, nullptr, penalty, output_ids, batch_size, local_batch_size,
                             vocab_size_padd, vocab_size, input_lengths, max_input_len, step, penalty_type,
                             (hipStream_t)stream);
}

int ftk_invoke_batch_apply_repetition_penalty(int dtype, void* logits, const float* penalties, const int* output_ids,
                                              int batch_size, int local_batch_size, int vocab_size,
                                              const int* input_lengths, int max_input_length, int step,
                                              int penalty_type, ftk_stream_t stream)
{
    if (penalties == nullptr && penalty_type != FTK_PENALTY_NONE) {
        return FTK_ERR_ARGUMENT;
    }
    return launch_repetition(dtype, logits, penalties, 0.0f, output_ids, batch_size, local_batch_size, vocab_size,
                             vocab_size, input_lengths, max_input_length, step, penalty_type, (hipStream_t)stream);
}

int ftk_invoke_batch_apply_frequency_penalty(int dtype, void* logits, const float* presence, const float* frequency,
                                             const int* output_ids, int batch_size, int local_batch_size,
                                             int vocab_size, const int* input_lengths, int max_input_length,
                                             int step, ftk_stream_t stream)
{
    if (presence == nullptr || frequency == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    if (local_batch_size <= 0 || step <= 0) {
        return 0;
    }
    // a table at most half full where that fits 128 KB of LDS, otherwise the smallest power of two above the
    // history length (distinct ids are fewer than slots, so the probing always ends)
    constexpr int MAX_SLOTS = 16384;
    int           slots     = 256;
    while (slots < 2 * step && slots < MAX_SLOTS) {
        slots <<= 1;
    }
    if (step >= slots) {
        return FTK_ERR_ARGUMENT;  // a history of 16384 tokens or more does not fit the counting table
    }
    const size_t smem = (size_t)slots * 2 * sizeof(int);
    FTK_DISPATCH_DTYPE(dtype, {
        if (smem > 64 * 1024) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&frequency_kernel<DT>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
            if (e != hipSuccess) {
                return (int)e;
            }
        }
        frequency_kernel<DT><<<local_batch_size, REP_THREADS, smem, (hipStream_t)stream>>>(
            (Storage<DT>::T*)logits, presence, frequency, output_ids, batch_size, vocab_size, input_lengths,
            max_input_length, step, slots);
    });
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_min_length_penalty(int dtype, void* logits, const int* min_lengths, const int* end_ids,
                                  const int* sequence_lengths, int max_input_length, int batch_size,
                                  int vocab_size_padded, ftk_stream_t stream)
{
    if (batch_size <= 0) {
        return 0;
    }
    const int block = 256, grid = (batch_size + block - 1) / block;
    FTK_DISPATCH_DTYPE(dtype, min_length_kernel<DT><<<grid, block, 0, (hipStream_t)stream>>>(
                                  (Storage<DT>::T*)logits, min_lengths, end_ids, sequence_lengths, max_input_length,
                                  batch_size, vocab_size_padded));
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_add_bias_end_mask(int dtype, void* logits, const void* bias, const int* end_ids, const bool* finished,
                                 int batch_size, int vocab_size, int vocab_size_padded, ftk_stream_t stream)
{
    if (batch_size <= 0) {
        return 0;
    }
    dim3 grid(max(1, min((vocab_size_padded + EW_THREADS - 1) / EW_THREADS, 64)), batch_size);
    FTK_DISPATCH_DTYPE(dtype, end_mask_kernel<DT><<<grid, EW_THREADS, 0, (hipStream_t)stream>>>(
                                  (Storage<DT>::T*)logits, (const Storage<DT>::T*)bias, end_ids, finished, vocab_size,
                                  vocab_size_padded));
    FTK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
