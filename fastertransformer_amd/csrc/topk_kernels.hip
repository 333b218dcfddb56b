// Stand-alone top-k sampling entry point (invokeBatchTopKSampling and friends,
// src/fastertransformer/kernels/sampling_topk_kernels.cu:345-544). The algorithm lives in
// ftk_topk.cuh; this file instantiates it for rows that are already final (logits or, when log-prob
// outputs are requested, probabilities).
#include "ftk_sampling.h"
#include "ftk_topk.cuh"

namespace ftk {

template<int DT>
struct PlainRowAt: PlainRow<DT> {
    __device__ __forceinline__ uint32_t key_at(int v) const
    {
        return order_key(Storage<DT>::ld(this->rowp[v]));
    }
    __device__ __forceinline__ void prepare_whole_row() {}
};

template<int DT>
__global__ void __launch_bounds__(TK_THREADS, 4)
topk_gather_kernel(const typename Storage<DT>::T* __restrict__ log_probs, const bool* __restrict__ finished,
                   const bool* __restrict__ skip_decode, const int* __restrict__ top_ks, int max_top_k, int vocab,
                   int splits, int nvt, int cap, size_t row_entries, TopkChunkHeader* __restrict__ headers,
                   TopkEntry* __restrict__ entries)
{
    const int row   = blockIdx.y;
    const int chunk = blockIdx.x;
    if (skip_decode != nullptr && skip_decode[row]) {
        return;
    }
    if (finished != nullptr && finished[row]) {
        return;
    }
    const int      k = top_ks != nullptr ? top_ks[row] : max_top_k;
    PlainRowAt<DT> r;
    r.rowp = log_probs + (size_t)row * vocab;
    topk_gather_chunk<DT>(r, vocab, k, chunk, splits, nvt, cap, headers + (size_t)row * splits + chunk,
                          entries + (size_t)row * row_entries + (size_t)chunk * cap);
}

template<int DT>
__global__ void __launch_bounds__(TK_THREADS)
topk_select_kernel(const typename Storage<DT>::T* __restrict__ log_probs, int* __restrict__ ids,
                   int* __restrict__ sequence_length, bool* __restrict__ finished, float* __restrict__ cum_log_probs,
                   float* __restrict__ output_log_probs, RngState* rng, const float* __restrict__ uniforms,
                   const bool* __restrict__ skip_decode, const int* __restrict__ top_ks, int max_top_k, float top_p,
                   const float* __restrict__ top_ps, int vocab, const int* __restrict__ end_ids, int splits, int cap,
                   size_t row_entries, const TopkChunkHeader* __restrict__ headers, TopkEntry* __restrict__ entries)
{
    __shared__ TopkSelectShared s;
    const int                   row = blockIdx.x;
    if (skip_decode != nullptr && skip_decode[row]) {
        return;
    }
    if (finished != nullptr && finished[row]) {
        if (threadIdx.x == 0) {
            ids[row] = end_ids[row];  // no draw, no length / log-prob update (:249-252)
        }
        return;
    }
    const int   k = top_ks != nullptr ? top_ks[row] : max_top_k;
    const float p = top_ps != nullptr ? top_ps[row] : top_p;
    if (threadIdx.x == 0) {
        s.misc[0] = __float_as_int(row_uniform(rng, uniforms, row));
    }
    __syncthreads();
    const float    u = __int_as_float(s.misc[0]);
    PlainRowAt<DT> r;
    r.rowp = log_probs + (size_t)row * vocab;
    const TopkOutputs out{ids, sequence_length, finished, cum_log_probs, output_log_probs};
    topk_select_row<DT>(r, s, row, vocab, k, p, max_top_k, splits, headers + (size_t)row * splits,
                        entries + (size_t)row * row_entries, cap,
                        cum_log_probs != nullptr || output_log_probs != nullptr, u, end_ids, out);
}

}  // namespace ftk

using namespace ftk;

extern "C" {

int ftk_invoke_batch_topk_sampling(int dtype, void* workspace, size_t* workspace_size, const void* log_probs, int* ids,
                                   int* sequence_length, bool* finished, float* cum_log_probs,
                                   float* output_log_probs, ftk_rng_state* rng_state, const float* uniform_draws,
                                   int max_top_k, const int* top_ks, float top_p, const float* top_ps,
                                   int vocab_size_padded, const int* end_ids, ftk_stream_t stream, int batch_size,
                                   const bool* skip_decode)
{
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (max_top_k < 1 || max_top_k > 1024) {
        return FTK_ERR_TOPK_DOMAIN;
    }
    const int      elem = dtype == FTK_DTYPE_F32 ? 4 : 2;
    const TopkPlan plan = topk_plan(vocab_size_padded, batch_size, max_top_k, elem);
    if (workspace == nullptr) {
        if (workspace_size == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        *workspace_size = plan.bytes;
        return 0;
    }
    if (workspace_size != nullptr && *workspace_size < plan.bytes) {
        return FTK_ERR_WORKSPACE;
    }
    if (batch_size <= 0) {
        return 0;
    }
    if (log_probs == nullptr || ids == nullptr || end_ids == nullptr
        || (rng_state == nullptr && uniform_draws == nullptr)) {
        return FTK_ERR_ARGUMENT;
    }
    TopkChunkHeader* headers = (TopkChunkHeader*)workspace;
    TopkEntry*       entries = (TopkEntry*)(headers + (size_t)batch_size * plan.splits);
    hipStream_t      st      = (hipStream_t)stream;
    dim3             grid(plan.splits, batch_size);
    FTK_DISPATCH_DTYPE(dtype, topk_gather_kernel<DT><<<grid, TK_THREADS, 0, st>>>(
                                  (const Storage<DT>::T*)log_probs, finished, skip_decode, top_ks, max_top_k,
                                  vocab_size_padded, plan.splits, plan.nvt, plan.cap, plan.row_entries, headers,
                                  entries));
    FTK_LAUNCH_CHECK();
    FTK_DISPATCH_DTYPE(dtype, topk_select_kernel<DT><<<batch_size, TK_THREADS, 0, st>>>(
                                  (const Storage<DT>::T*)log_probs, ids, sequence_length, finished, cum_log_probs,
                                  output_log_probs, (RngState*)rng_state, uniform_draws, skip_decode, top_ks,
                                  max_top_k, top_p, top_ps, vocab_size_padded, end_ids, plan.splits, plan.cap,
                                  plan.row_entries, headers, entries));
    FTK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
