// Per-element logit arithmetic of the sampling path, written once and used both by the stand-alone
// in-place kernels and by the fused streaming kernel, so the two cannot drift apart.
// Each helper restates one reference kernel's arithmetic (file:line cited); storage rounding is
// explicit: values are carried as the exact fp32 image of a `T` and rounded once per reference store.
#pragma once
#include "ftk_device.cuh"

namespace ftk {

// round an fp32 value through the storage type
template<int DT>
__device__ __forceinline__ float round_t(float f)
{
    if constexpr (DT == DT_F32) {
        return f;
    }
    else {
        return Storage<DT>::ld(Storage<DT>::st(f));
    }
}

// batchApplyTemperaturePenalty / _h2 and applyTemperaturePenalty
// (src/fastertransformer/kernels/sampling_penalty_kernels.cu:25-73, :117-179):
//   float : (x + bias) * inv,  inv = 1 / (temperature + 1e-6)
//   half  : hmul(hadd(x, bias), half(inv)); the half2 kernels (even V and Vp) leave pad columns alone
//   bf16  : extension, generic branch: T(float(T(x + bias)) * inv)
// pad columns (v >= V) otherwise become -MAX_T.
template<int DT>
struct TemperatureCtx {
    float inv;       // 1 / (t + 1e-6), rounded to half for DT_F16
    int   V, Vp;
    bool  keep_pads;  // half2 variant
    bool  add_zero;   // the scalar generic kernel adds a zero bias when none is given (:37-39)

    __device__ __forceinline__ TemperatureCtx(float temperature, int V_, int Vp_, bool scalar_variant): V(V_), Vp(Vp_)
    {
        const float i = 1.0f / (temperature + 1e-6f);
        inv           = (DT == DT_F16) ? round_t<DT>(i) : i;
        keep_pads     = (DT == DT_F16) && (V_ % 2 == 0) && (Vp_ % 2 == 0);
        add_zero      = scalar_variant && (DT != DT_BF16) && !keep_pads;
    }

    // fp32 image in, fp32 image (already rounded to T) out; v < V
    __device__ __forceinline__ float value(float x, bool has_bias, float bias_v) const
    {
        if (has_bias) {
            x = round_t<DT>(x + bias_v);
        }
        else if (add_zero) {
            x = round_t<DT>(x + 0.0f);
        }
        return round_t<DT>(x * inv);
    }

    __device__ __forceinline__ typename Storage<DT>::T apply(typename Storage<DT>::T raw,
                                                              const typename Storage<DT>::T* bias, int v) const
    {
        typedef Storage<DT> S;
        if (v >= V) {
            return keep_pads ? raw : S::st(-S::max_t());
        }
        const bool hb = bias != nullptr;
        return S::st(value(S::ld(raw), hb, hb ? S::ld(bias[v]) : 0.0f));
    }
};

// batchApplyRepetitionPenalty (sampling_penalty_kernels.cu:396-405): fp32 arithmetic on the
// pre-penalty value, the caller rounds to T on store.
__device__ __forceinline__ float repetition_value(float x, float penalty, int type)
{
    if (type == 0 /* additive */) {
        return x - penalty;
    }
    return x < 0.0f ? x * penalty : x / penalty;
}

// presence + frequency extension: x - presence - frequency * count, evaluated left to right
__device__ __forceinline__ float frequency_value(float x, float presence, float frequency, int count)
{
    float y = x - presence;
    y       = y - frequency * (float)count;
    return y;
}

// batchApplyMinLengthPenalty (sampling_penalty_kernels.cu:493-499)
__device__ __forceinline__ bool min_length_masks(int sequence_length, int max_input_length, int min_length)
{
    return sequence_length + 1 - max_input_length < min_length;
}

}  // namespace ftk
