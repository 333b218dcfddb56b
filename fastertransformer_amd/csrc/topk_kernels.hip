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

struct TopkKernelArgs {
    const void*  log_probs;
    int*         ids;
    int*         sequence_length;
    bool*        finished;
    float*       cum_log_probs;
    float*       output_log_probs;
    RngState*    rng;
    const float* uniforms;
    const bool*  skip_decode;
    const int*   top_ks;
    int          max_top_k;
    float        top_p;
    const float* top_ps;
    int          vocab;
    const int*   end_ids;
    int          splits;
    int          tiles_per_wg;
    size_t       row_entries;
    TopkChunkHeader* headers;
    TopkEntry*       entries;
};

// one draw per live row, broadcast to the workgroup
__device__ __forceinline__ float topk_row_draw(TopkShared& s, RngState* rng, const float* uniforms, int row)
{
    if (threadIdx.x == 0) {
        s.misc[0] = __float_as_int(row_uniform(rng, uniforms, row));
    }
    __syncthreads();
    return __int_as_float(s.misc[0]);
}

// rows owned by one workgroup: stream and select in a single launch
template<int DT, int MANY = 0>
__global__ void __launch_bounds__(TK_THREADS, MANY > 0 ? TK_MIN_WGS_MANY : TK_MIN_WGS) topk_row_kernel(TopkKernelArgs a)
{
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    if (a.skip_decode != nullptr && a.skip_decode[row]) {
        return;
    }
    if (a.finished != nullptr && a.finished[row]) {
        if (threadIdx.x == 0) {
            a.ids[row] = a.end_ids[row];  // no draw, no length / log-prob update (:249-252)
        }
        return;
    }
    const int      k = a.top_ks != nullptr ? a.top_ks[row] : a.max_top_k;
    const float    p = a.top_ps != nullptr ? a.top_ps[row] : a.top_p;
    const float    u = topk_row_draw(s, a.rng, a.uniforms, row);
    const TopkOutputs out = topk_outputs(a.ids, a.sequence_length, a.finished, a.cum_log_probs, a.output_log_probs, row, a.end_ids);
    PlainRowAt<DT> r;
    r.rowp = (const typename Storage<DT>::T*)a.log_probs + (size_t)row * a.vocab;
    uint32_t  thr = 0u;
    const int n   = topk_stream<DT, PlainRowAt<DT>, MANY>(r, s, a.vocab, k, 0, topk_row_tiles<DT>(r.rowp, a.vocab), &thr);
    topk_select_lds<DT>(r, s, n, thr, row, a.vocab, k, p, a.max_top_k, a.entries + (size_t)row * a.row_entries,
                        a.cum_log_probs != nullptr || a.output_log_probs != nullptr, u, a.end_ids, out);
}

// rows split over `splits` workgroups: each leaves its candidate list in the workspace
template<int DT, int MANY = 0>
__global__ void __launch_bounds__(TK_THREADS, MANY > 0 ? TK_MIN_WGS_MANY : TK_MIN_WGS) topk_gather_kernel(TopkKernelArgs a)
{
    __shared__ TopkShared s;
    const int             row   = blockIdx.y;
    const int             chunk = blockIdx.x;
    if (a.skip_decode != nullptr && a.skip_decode[row]) {
        return;
    }
    if (a.finished != nullptr && a.finished[row]) {
        return;
    }
    const int      k = a.top_ks != nullptr ? a.top_ks[row] : a.max_top_k;
    PlainRowAt<DT> r;
    r.rowp = (const typename Storage<DT>::T*)a.log_probs + (size_t)row * a.vocab;
    const int tiles = topk_row_tiles<DT>(r.rowp, a.vocab);
    const int t0    = min(tiles, chunk * a.tiles_per_wg);
    const int t1    = min(tiles, t0 + a.tiles_per_wg);
    uint32_t  thr   = 0u;
    const int n     = topk_stream<DT, PlainRowAt<DT>, MANY>(r, s, a.vocab, k, t0, t1, &thr);
    topk_dump_list(s, n, k, a.splits, thr, a.headers + (size_t)row * a.splits + chunk,
                   a.entries + (size_t)row * a.row_entries + (size_t)chunk * TK_CCAP);
}

template<int DT>
__global__ void __launch_bounds__(TK_THREADS) topk_select_kernel(TopkKernelArgs a)
{
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    // the chunk lists and the row's arguments are requested before the first decision
    TopkEntry*             row_entries = a.entries + (size_t)row * a.row_entries;
    const TopkListPrefetch pf          = topk_prefetch_lists(a.splits, row_entries);
    const bool     skip = a.skip_decode != nullptr && a.skip_decode[row];
    const bool     fin  = a.finished != nullptr && a.finished[row];
    const int      k    = a.top_ks != nullptr ? a.top_ks[row] : a.max_top_k;
    const float    p    = a.top_ps != nullptr ? a.top_ps[row] : a.top_p;
    if (skip) {
        return;
    }
    if (fin) {
        if (threadIdx.x == 0) {
            a.ids[row] = a.end_ids[row];
        }
        return;
    }
    const float    u = topk_row_draw(s, a.rng, a.uniforms, row);
    const TopkOutputs out = topk_outputs(a.ids, a.sequence_length, a.finished, a.cum_log_probs, a.output_log_probs, row, a.end_ids);
    PlainRowAt<DT> r;
    r.rowp = (const typename Storage<DT>::T*)a.log_probs + (size_t)row * a.vocab;
    uint32_t   thr = 0u;
    const int  n   = topk_merge_lists<DT>(s, k, a.splits, a.headers + (size_t)row * a.splits, row_entries, &thr, pf);
    topk_select_lds<DT, PlainRowAt<DT>, true>(r, s, n, thr, row, a.vocab, k, p, a.max_top_k, row_entries,
                        a.cum_log_probs != nullptr || a.output_log_probs != nullptr, u, a.end_ids, out);
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
    TopkKernelArgs a;
    a.log_probs        = log_probs;
    a.ids              = ids;
    a.sequence_length  = sequence_length;
    a.finished         = finished;
    a.cum_log_probs    = cum_log_probs;
    a.output_log_probs = output_log_probs;
    a.rng              = (RngState*)rng_state;
    a.uniforms         = uniform_draws;
    a.skip_decode      = skip_decode;
    a.top_ks           = top_ks;
    a.max_top_k        = max_top_k;
    a.top_p            = top_p;
    a.top_ps           = top_ps;
    a.vocab            = vocab_size_padded;
    a.end_ids          = end_ids;
    a.splits           = plan.splits;
    a.tiles_per_wg     = plan.tiles_per_wg;
    a.row_entries      = plan.row_entries;
    a.headers          = (TopkChunkHeader*)workspace;
    a.entries          = (TopkEntry*)(a.headers + (size_t)batch_size * plan.splits);
    hipStream_t st     = (hipStream_t)stream;
    const int many = topk_many_level(max_top_k);  // > 0: the large-k variants of the streaming kernels
    if (plan.splits == 1) {
        if (many == 2) {
            FTK_DISPATCH_DTYPE(dtype, topk_row_kernel<DT, 2><<<batch_size, TK_THREADS, 0, st>>>(a));
        }
        else if (many == 1) {
            FTK_DISPATCH_DTYPE(dtype, topk_row_kernel<DT, 1><<<batch_size, TK_THREADS, 0, st>>>(a));
        }
        else {
            FTK_DISPATCH_DTYPE(dtype, topk_row_kernel<DT><<<batch_size, TK_THREADS, 0, st>>>(a));
        }
        FTK_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid(plan.splits, batch_size);
    if (many == 2) {
        FTK_DISPATCH_DTYPE(dtype, topk_gather_kernel<DT, 2><<<grid, TK_THREADS, 0, st>>>(a));
    }
    else if (many == 1) {
        FTK_DISPATCH_DTYPE(dtype, topk_gather_kernel<DT, 1><<<grid, TK_THREADS, 0, st>>>(a));
    }
    else {
        FTK_DISPATCH_DTYPE(dtype, topk_gather_kernel<DT><<<grid, TK_THREADS, 0, st>>>(a));
    }
    FTK_LAUNCH_CHECK();
    FTK_DISPATCH_DTYPE(dtype, topk_select_kernel<DT><<<batch_size, TK_THREADS, 0, st>>>(a));
    FTK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
