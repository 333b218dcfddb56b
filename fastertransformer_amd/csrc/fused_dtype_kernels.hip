// The general-stream kernels of the fused decode step for one element type: this file is compiled once per
// type with -DFTK_FUSED_DT=0 (f32), 1 (f16), 2 (bf16), so that the three sets of kernels build side by side.
//   fused_row_kernel      - one workgroup per row: stream, transform, select, sample, bookkeeping
//   fused_gather_kernel / fused_select_kernel - the same in two launches for batches whose rows are split over
//                           several workgroups; fused_select_kernel also merges the lists of the lean gather
// (reference: src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.cc:302-352,
//  src/fastertransformer/layers/sampling_layers/TopKSamplingLayer.cu:220-266)
#include <hip/hip_ext.h>

#include "ftk_fused.cuh"

#ifndef FTK_FUSED_DT
#error "build with -DFTK_FUSED_DT=0|1|2"
#endif

namespace ftk {

template<int DT, int BMW, int MANY = 0>
__global__ void __launch_bounds__(TK_THREADS, MANY > 0 ? TK_MIN_WGS_MANY : BMW <= FUSED_BITMAP_WORDS_SMALL ? TK_MIN_WGS : (TK_MIN_WGS * 3 + 3) / 4)
fused_row_kernel(FusedParams p, FusedLaunch l)
{
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    if (p.skip_decode != nullptr && p.skip_decode[row]) {
        return;
    }
    if (l.finished != nullptr && l.finished[row]) {
        if (threadIdx.x == 0) {
            l.ids[row] = p.end_ids[row];  // a finished row emits its end id without looking at the logits
        }
        return;
    }
    const int    k  = p.top_ks != nullptr ? p.top_ks[row] : p.max_top_k;
    const float  tp = p.top_ps != nullptr ? p.top_ps[row] : 1.0f;
    const float  u  = fused_row_draw(s, l, row);
    const TopkOutputs out = topk_outputs(l.ids, l.sequence_length, l.finished, nullptr, nullptr, row, p.end_ids);
    FusedRow<DT, BMW> r(p, row);
    uint32_t     thr = 0u;
    const int    n   = topk_stream<DT, FusedRow<DT, BMW>, MANY>(r, s, p.Vp, k, 0, topk_row_tiles<DT>(r.rowp, p.Vp), &thr);
    topk_select_lds<DT>(r, s, n, thr, row, p.Vp, k, tp, p.max_top_k, l.entries + (size_t)row * l.row_entries, false, u,
                        p.end_ids, out);
}

template<int DT, int BMW, int MANY = 0>
__global__ void __launch_bounds__(TK_THREADS, MANY > 0 ? TK_MIN_WGS_MANY : BMW <= FUSED_BITMAP_WORDS_SMALL ? TK_MIN_WGS : (TK_MIN_WGS * 3 + 3) / 4)
fused_gather_kernel(FusedParams p, FusedLaunch l)
{
    __shared__ TopkShared s;
    const int             row   = blockIdx.y;
    const int             chunk = blockIdx.x;
    if (p.skip_decode != nullptr && p.skip_decode[row]) {
        return;
    }
    if (p.finished_in != nullptr && p.finished_in[row]) {
        return;
    }
    const int    k = p.top_ks != nullptr ? p.top_ks[row] : p.max_top_k;
    FusedRow<DT, BMW> r(p, row);
    const int    tiles = topk_row_tiles<DT>(r.rowp, p.Vp);
    const int    t0    = min(tiles, chunk * l.tiles_per_wg);
    const int    t1    = min(tiles, t0 + l.tiles_per_wg);
    uint32_t     thr   = 0u;
    const int    n     = topk_stream<DT, FusedRow<DT, BMW>, MANY>(r, s, p.Vp, k, t0, t1, &thr);
    topk_dump_list(s, n, k, l.splits, thr, l.headers + (size_t)row * l.splits + chunk,
                   l.entries + (size_t)row * l.row_entries + (size_t)chunk * TK_CCAP);
}

template<int DT>
__global__ void __launch_bounds__(TK_THREADS) fused_select_kernel(FusedParams p, FusedLaunch l)
{
    constexpr int BMW = 0;  // the literal replay reads whole-row bitmaps from global memory
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    // everything the row needs is requested before the first decision: the arguments (scalar loads), the
    // chunk lists (vector loads), the draw
    TopkEntry*             row_entries = l.entries + (size_t)row * l.row_entries;
    const TopkListPrefetch pf          = topk_prefetch_lists(l.splits, row_entries);
    const bool   skip = p.skip_decode != nullptr && p.skip_decode[row];
    const bool   fin  = l.finished != nullptr && l.finished[row];
    const int    k    = p.top_ks != nullptr ? p.top_ks[row] : p.max_top_k;
    const float  tp   = p.top_ps != nullptr ? p.top_ps[row] : 1.0f;
    FusedRow<DT, BMW> r(p, row);
    if (skip) {
        return;
    }
    if (fin) {
        if (threadIdx.x == 0) {
            l.ids[row] = p.end_ids[row];
        }
        return;
    }
    const float  u  = fused_row_draw(s, l, row);
    const TopkOutputs out = topk_outputs(l.ids, l.sequence_length, l.finished, nullptr, nullptr, row, p.end_ids);
    uint32_t     thr         = 0u;
    const int    n = topk_merge_lists<DT>(s, k, l.splits, l.headers + (size_t)row * l.splits, row_entries, &thr, pf);
    topk_select_lds<DT, FusedRow<DT, BMW>, true>(r, s, n, thr, row, p.Vp, k, tp, p.max_top_k, row_entries, false, u, p.end_ids, out);
}


template<typename K>
static int fused_launch_one(K kernel, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                            hipEvent_t start, hipEvent_t stop)
{
    if (start != nullptr) {
        hipExtLaunchKernelGGL(kernel, grid, dim3(TK_THREADS), 0, st, start, stop, 0, p, l);
    }
    else {
        hipLaunchKernelGGL(kernel, grid, dim3(TK_THREADS), 0, st, p, l);
    }
    return (int)hipGetLastError();
}

template<int MANY>
static int fused_launch_stream(bool row_kernel, int window, dim3 grid, hipStream_t st, const FusedParams& p,
                               const FusedLaunch& l, hipEvent_t start, hipEvent_t stop)
{
    constexpr int DT = FTK_FUSED_DT;
    // the large-k variants read whole-row bitmaps from global memory only
    if (MANY > 0 || window == 0) {
        return row_kernel ?
                   fused_launch_one(fused_row_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL, MANY>, grid, st, p, l, start, stop) :
                   fused_launch_one(fused_gather_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL, MANY>, grid, st, p, l, start,
                                    stop);
    }
    if (window == 2) {
        return row_kernel ?
                   fused_launch_one(fused_row_kernel<DT, FUSED_BITMAP_WORDS_LARGE, 0>, grid, st, p, l, start, stop) :
                   fused_launch_one(fused_gather_kernel<DT, FUSED_BITMAP_WORDS_LARGE, 0>, grid, st, p, l, start, stop);
    }
    return row_kernel ?
               fused_launch_one(fused_row_kernel<DT, FUSED_BITMAP_WORDS_SMALL, 0>, grid, st, p, l, start, stop) :
               fused_launch_one(fused_gather_kernel<DT, FUSED_BITMAP_WORDS_SMALL, 0>, grid, st, p, l, start, stop);
}

#if FTK_FUSED_DT == 0
int fused_launch_f32
#elif FTK_FUSED_DT == 1
int fused_launch_f16
#else
int fused_launch_bf16
#endif
    (int kind, int window, int many, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
     hipEvent_t start, hipEvent_t stop)
{
    if (kind == FUSED_KIND_SELECT) {
        return fused_launch_one(fused_select_kernel<FTK_FUSED_DT>, grid, st, p, l, start, stop);
    }
    const bool row_kernel = kind == FUSED_KIND_ROW;
    if (many == 2) {
        return fused_launch_stream<2>(row_kernel, window, grid, st, p, l, start, stop);
    }
    if (many == 1) {
        return fused_launch_stream<1>(row_kernel, window, grid, st, p, l, start, stop);
    }
    return fused_launch_stream<0>(row_kernel, window, grid, st, p, l, start, stop);
}

}  // namespace ftk
