// Instances of the two-read log-prob step (ftk_logprob.cuh) for one element type: this file is compiled once
// per type with -DFTK_LP_DT=0 (f32), 1 (f16), 2 (bf16).
#include <type_traits>

#include "ftk_logprob.cuh"

#ifndef FTK_LP_DT
#error "build with -DFTK_LP_DT=0|1|2"
#endif

namespace ftk {

#if FTK_LP_DT == 0
int lp_rowmax_launch_f32
#elif FTK_LP_DT == 1
int lp_rowmax_launch_f16
#else
int lp_rowmax_launch_bf16
#endif
    (int window, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l, const LogProbLaunch& lp)
{
    constexpr int DT = FTK_LP_DT;
    if (window == 0) {
        hipLaunchKernelGGL((lp_rowmax_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL>), grid, dim3(LG_THREADS), 0, st, p, l, lp);
    }
    else if (window == 2) {
        hipLaunchKernelGGL((lp_rowmax_kernel<DT, FUSED_BITMAP_WORDS_LARGE>), grid, dim3(LG_THREADS), 0, st, p, l, lp);
    }
    else {
        hipLaunchKernelGGL((lp_rowmax_kernel<DT, FUSED_BITMAP_WORDS_SMALL>), grid, dim3(LG_THREADS), 0, st, p, l, lp);
    }
    return (int)hipGetLastError();
}

#if FTK_LP_DT == 0
int lp_row_launch_f32
#elif FTK_LP_DT == 1
int lp_row_launch_f16
#else
int lp_row_launch_bf16
#endif
    (int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, const LogProbLaunch& lp)
{
    constexpr int DT = FTK_LP_DT;
    if (window == 0) {
        hipLaunchKernelGGL((lp_row_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL>), dim3(rows), dim3(LP_THREADS), 0, st, p, l,
                           lp);
    }
    else if (window == 2) {
        hipLaunchKernelGGL((lp_row_kernel<DT, FUSED_BITMAP_WORDS_LARGE>), dim3(rows), dim3(LP_THREADS), 0, st, p, l,
                           lp);
    }
    else {
        hipLaunchKernelGGL((lp_row_kernel<DT, FUSED_BITMAP_WORDS_SMALL>), dim3(rows), dim3(LP_THREADS), 0, st, p, l,
                           lp);
    }
    return (int)hipGetLastError();
}

#if FTK_LP_DT == 0
int lp_wide_launch_f32
#elif FTK_LP_DT == 1
int lp_wide_launch_f16
#else
int lp_wide_launch_bf16
#endif
    (int window, int threads, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
     const LogProbLaunch& lp)
{
    constexpr int DT = FTK_LP_DT;
    auto launch = [&](auto words) {
        constexpr int BMW = decltype(words)::value;
        if (threads == 1024) {
            hipLaunchKernelGGL((lp_wide_kernel<DT, BMW, 1024>), dim3(rows), dim3(1024), 0, st, p, l, lp);
        }
        else if (threads == 512) {
            hipLaunchKernelGGL((lp_wide_kernel<DT, BMW, 512>), dim3(rows), dim3(512), 0, st, p, l, lp);
        }
        else {
            hipLaunchKernelGGL((lp_wide_kernel<DT, BMW, 256>), dim3(rows), dim3(256), 0, st, p, l, lp);
        }
    };
    if (window == 0) {
        launch(std::integral_constant<int, FUSED_BITMAP_WORDS_GLOBAL>());
    }
    else if (window == 2) {
        launch(std::integral_constant<int, FUSED_BITMAP_WORDS_LARGE>());
    }
    else {
        launch(std::integral_constant<int, FUSED_BITMAP_WORDS_SMALL>());
    }
    return (int)hipGetLastError();
}

}  // namespace ftk
