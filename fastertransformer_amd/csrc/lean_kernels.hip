// Instances of the lean gather (ftk_lean.cuh) for one element type: this file is compiled once per type with
// -DFTK_LEAN_DT=0 (f32), 1 (f16), 2 (bf16), so that the three sets of kernels build side by side.
#include "ftk_lean.cuh"
#include "ftk_largek.cuh"
#include "ftk_rowwide.cuh"
#include "ftk_sampling.h"

#ifndef FTK_LEAN_DT
#error "build with -DFTK_LEAN_DT=0|1|2"
#endif

namespace ftk {

template<int BMW, int OCC, int R, int MODE, bool BIAS, bool ROWSEL>
static int lean_launch_one(dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start,
                           hipEvent_t stop)
{
    if (start != nullptr) {
        hipExtLaunchKernelGGL((lean_gather_kernel<FTK_LEAN_DT, BMW, OCC, R, MODE, BIAS, ROWSEL>), grid, dim3(LG_THREADS), 0, st, start,
                              stop, 0, p, l);
    }
    else {
        hipLaunchKernelGGL((lean_gather_kernel<FTK_LEAN_DT, BMW, OCC, R, MODE, BIAS, ROWSEL>), grid, dim3(LG_THREADS), 0, st, p, l);
    }
    return (int)hipGetLastError();
}

template<int OCC, int R, int MODE, bool BIAS, bool ROWSEL = false>
static int lean_launch_window(int window, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                              hipEvent_t start, hipEvent_t stop)
{
    if (window == 0) {
        return lean_launch_one<FUSED_BITMAP_WORDS_GLOBAL, OCC, R, MODE, BIAS, ROWSEL>(grid, st, p, l, start, stop);
    }
    if (window == 2) {
        // (the large window leaves room for three workgroups per compute unit: built for that register budget)
        return lean_launch_one<FUSED_BITMAP_WORDS_LARGE, 3, R, MODE, BIAS, ROWSEL>(grid, st, p, l, start, stop);
    }
    return lean_launch_one<FUSED_BITMAP_WORDS_SMALL, OCC, R, MODE, BIAS, ROWSEL>(grid, st, p, l, start, stop);
}

#if FTK_LEAN_DT == 0
int lean_gather_launch_f32
#elif FTK_LEAN_DT == 1
int lean_gather_launch_f16
#else
int lean_gather_launch_bf16
#endif
    (int mode, bool row_select, int window, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
     hipEvent_t start, hipEvent_t stop)
{
    const bool bias = p.bias != nullptr;
    if (row_select) {
        if (mode != LG_MODE_STREAM || bias || grid.x != 1) {
            return FTK_ERR_ARGUMENT;
        }
        return lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_STREAM, false, true>(window, grid, st, p, l, start, stop);
    }
    if (mode == LG_MODE_SLOTS) {
        return bias ? lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_SLOTS, true>(window, grid, st, p, l, start, stop) :
                      lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_SLOTS, false>(window, grid, st, p, l, start, stop);
    }
    if (mode == LG_MODE_PRESET) {
        return bias ? lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_PRESET, true>(window, grid, st, p, l, start, stop) :
                      lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_PRESET, false>(window, grid, st, p, l, start, stop);
    }
    return bias ? lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_STREAM, true>(window, grid, st, p, l, start, stop) :
                  lean_launch_window<LG_OCCUPANCY, LG_RING, LG_MODE_STREAM, false>(window, grid, st, p, l, start, stop);
}

#if FTK_LEAN_DT == 0
int lean_select_launch_f32
#elif FTK_LEAN_DT == 1
int lean_select_launch_f16
#else
int lean_select_launch_bf16
#endif
    (int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start, hipEvent_t stop)
{
    if (start != nullptr) {
        hipExtLaunchKernelGGL((lean_select_kernel<FTK_LEAN_DT>), dim3(rows), dim3(TK_THREADS), 0, st, start, stop, 0, p,
                              l);
    }
    else {
        hipLaunchKernelGGL((lean_select_kernel<FTK_LEAN_DT>), dim3(rows), dim3(TK_THREADS), 0, st, p, l);
    }
    return (int)hipGetLastError();
}

#if FTK_LEAN_DT == 0
int rowwide_launch_f32
#elif FTK_LEAN_DT == 1
int rowwide_launch_f16
#else
int rowwide_launch_bf16
#endif
    (int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start, hipEvent_t stop)
{
    RowwideArgs a;
    a.p = p;
    a.l = l;
    auto launch = [&](auto kernel) {
        if (start != nullptr) {
            hipExtLaunchKernelGGL(kernel, dim3(rows), dim3(RW_THREADS), 0, st, start, stop, 0, a);
        }
        else {
            hipLaunchKernelGGL(kernel, dim3(rows), dim3(RW_THREADS), 0, st, a);
        }
    };
    if (window == 2) {
        launch(rowwide_step_kernel<FTK_LEAN_DT, FUSED_BITMAP_WORDS_LARGE>);
    }
    else {
        launch(rowwide_step_kernel<FTK_LEAN_DT, FUSED_BITMAP_WORDS_SMALL>);
    }
    return (int)hipGetLastError();
}

#if FTK_LEAN_DT == 0
int largek_gather_launch_f32
#elif FTK_LEAN_DT == 1
int largek_gather_launch_f16
#else
int largek_gather_launch_bf16
#endif
    (int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start, hipEvent_t stop)
{
    auto launch = [&](auto kernel) {
        if (start != nullptr) {
            hipExtLaunchKernelGGL(kernel, dim3(rows), dim3(LK_THREADS), 0, st, start, stop, 0, p, l);
        }
        else {
            hipLaunchKernelGGL(kernel, dim3(rows), dim3(LK_THREADS), 0, st, p, l);
        }
    };
    if (window == 2) {
        launch(largek_gather_kernel<FTK_LEAN_DT, FUSED_BITMAP_WORDS_LARGE>);
    }
    else {
        launch(largek_gather_kernel<FTK_LEAN_DT, FUSED_BITMAP_WORDS_SMALL>);
    }
    return (int)hipGetLastError();
}

}  // namespace ftk
