// Scalar arithmetic shared by every kernel of the sampling engine.
//
// exp / log: a fixed sequence of IEEE-754 binary32 operations (fma, mul, add, round-to-nearest-even),
// so the same input gives the same bits on the GPU and on any IEEE host. They replace the
// `__expf` / `logf` calls of the reference kernels
// (src/fastertransformer/kernels/sampling_topk_kernels.cu:274,290,
//  src/fastertransformer/kernels/sampling_topp_kernels.cu:924,989,1332), whose bit patterns are
// specific to NVIDIA's special-function unit. Both are within ~1 ulp of the exact function.
//
// The file compiles as HIP device code and as plain host C++ (the host instance backs the
// ftk_host_* test hooks of the C ABI).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#include <hip/hip_runtime.h>
#define FTK_HD __host__ __device__ __forceinline__
#else
#include <cmath>
#include <cstring>
#define FTK_HD inline
#endif

namespace ftk {

FTK_HD uint32_t f2u(float f)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(f);
#else
    uint32_t u;
    __builtin_memcpy(&u, &f, 4);
    return u;
#endif
}
FTK_HD float u2f(uint32_t u)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(u);
#else
    float f;
    __builtin_memcpy(&f, &u, 4);
    return f;
#endif
}

FTK_HD float fma_rn(float a, float b, float c)
{
    return __builtin_fmaf(a, b, c);
}

// exp(x) = 2^n * exp(r): n = rint(x * log2 e), r = x - n ln2 (two-term Cody-Waite),
// exp(r) = 1 + r + r^2 P(r), P = degree-5 Cephes minimax polynomial.
FTK_HD float det_expf(float x)
{
    if (x != x) {
        return x;
    }
    if (x > 88.72283935546875f) {
        return __builtin_inff();
    }
    if (x < -103.97283172607421875f) {
        return 0.0f;
    }
    const float n = __builtin_rintf(x * 1.44269502162933349609375f);
    float       r = fma_rn(n, -0.693145751953125f, x);
    r             = fma_rn(n, -1.428606765330187045e-06f, r);
    float p       = 1.9875691500e-4f;
    p             = fma_rn(p, r, 1.3981999507e-3f);
    p             = fma_rn(p, r, 8.3334519073e-3f);
    p             = fma_rn(p, r, 4.1665795894e-2f);
    p             = fma_rn(p, r, 1.6666665459e-1f);
    p             = fma_rn(p, r, 5.0000001201e-1f);
    const float z = r * r;
    float       y = fma_rn(p, z, r) + 1.0f;
    const int   ni = (int)n;
#if defined(__HIP_DEVICE_COMPILE__)
    // one exact scaling by 2^ni (a single rounding when the result is subnormal): the same value as the two
    // multiplications of the host branch, in one instruction
    return __builtin_ldexpf(y, ni);
#else
    const int   n1 = ni / 2;
    const int   n2 = ni - n1;
    y              = y * u2f((uint32_t)(n1 + 127) << 23);
    y              = y * u2f((uint32_t)(n2 + 127) << 23);
    return y;
#endif
}

// det_expf for arguments that are never positive (x <= 0 or NaN), as in exp(y - max): the same value bit for
// bit, without the range checks. Below -104 the scaled result is under half of the smallest subnormal and rounds
// to zero like det_expf's cut-off at -103.97 (between the two, 2^-150 times a factor below one does too); the
// clamp keeps -inf out of the argument reduction; it would also turn a NaN into a number, hence the two forms.
FTK_HD float det_expf_nonpos_number(float x)  // x is not a NaN (a NaN would come out as a number)
{
#if defined(__HIP_DEVICE_COMPILE__)
    x = __builtin_amdgcn_fmed3f(x, -104.0f, 0.0f);  // the clamp in one instruction (x <= 0: the upper end is never taken)
#else
    x = __builtin_fmaxf(x, -104.0f);
#endif
    const float n = __builtin_rintf(x * 1.44269502162933349609375f);
    float       r = fma_rn(n, -0.693145751953125f, x);
    r             = fma_rn(n, -1.428606765330187045e-06f, r);
    float p       = 1.9875691500e-4f;
    p             = fma_rn(p, r, 1.3981999507e-3f);
    p             = fma_rn(p, r, 8.3334519073e-3f);
    p             = fma_rn(p, r, 4.1665795894e-2f);
    p             = fma_rn(p, r, 1.6666665459e-1f);
    p             = fma_rn(p, r, 5.0000001201e-1f);
    const float z = r * r;
    float       y = fma_rn(p, z, r) + 1.0f;
    const int   ni = (int)n;
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_ldexpf(y, ni);
#else
    const int n1 = ni / 2;
    const int n2 = ni - n1;
    y            = y * u2f((uint32_t)(n1 + 127) << 23);
    y            = y * u2f((uint32_t)(n2 + 127) << 23);
    return y;
#endif
}
FTK_HD float det_expf_nonpos(float x)
{
    const float y = det_expf_nonpos_number(x);  // the clamp inside drops a NaN: it is put back here
    return x != x ? x : y;
}

// Cephes logf: x = m 2^e, m in [sqrt(1/2), sqrt 2), f = m - 1, log x = f - f^2/2 + f^3 P(f) + e ln2.
FTK_HD float det_logf(float x)
{
    if (x != x) {
        return x;
    }
    if (x < 0.0f) {
        return __builtin_nanf("");
    }
    if (x == 0.0f) {
        return -__builtin_inff();
    }
    if (x == __builtin_inff()) {
        return x;
    }
    uint32_t u = f2u(x);
    int      e = 0;
    if (u < 0x00800000u) {
        x = x * 8388608.0f;
        u = f2u(x);
        e = -23;
    }
    e += (int)(u >> 23) - 126;
    float m = u2f((u & 0x007FFFFFu) | 0x3F000000u);
    if (m < 0.707106769084930419921875f) {
        e -= 1;
        m = m + m - 1.0f;
    }
    else {
        m = m - 1.0f;
    }
    const float z = m * m;
    float       p = 7.0376836292e-2f;
    p             = fma_rn(p, m, -1.1514610310e-1f);
    p             = fma_rn(p, m, 1.1676998740e-1f);
    p             = fma_rn(p, m, -1.2420140846e-1f);
    p             = fma_rn(p, m, 1.4249322787e-1f);
    p             = fma_rn(p, m, -1.6668057665e-1f);
    p             = fma_rn(p, m, 2.0000714765e-1f);
    p             = fma_rn(p, m, -2.4999993993e-1f);
    p             = fma_rn(p, m, 3.3333331174e-1f);
    float       y  = (m * z) * p;
    const float fe = (float)e;
    y              = fma_rn(fe, -2.12194440e-4f, y);
    y              = fma_rn(-0.5f, z, y);
    float res      = m + y;
    res            = fma_rn(fe, 0.693359375f, res);
    return res;
}

// ---- storage types -----------------------------------------------------------------------
// binary16 <-> binary32, round-to-nearest-even with gradual underflow
FTK_HD float half_bits_to_float(uint16_t h)
{
#if defined(__HIP_DEVICE_COMPILE__)
    _Float16 v;
    __builtin_memcpy(&v, &h, 2);
    return (float)v;
#else
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp  = (h >> 10) & 0x1Fu;
    const uint32_t man  = h & 0x3FFu;
    if (exp == 0x1Fu) {
        return u2f(sign | 0x7F800000u | (man << 13));
    }
    if (exp == 0) {
        const float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
#endif
}

FTK_HD uint16_t float_to_half_bits(float f)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const _Float16 v = (_Float16)f;  // v_cvt_f16_f32, round-to-nearest-even
    uint16_t       h;
    __builtin_memcpy(&h, &v, 2);
    return h;
#else
    const uint32_t u    = f2u(f);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t au   = u & 0x7FFFFFFFu;
    if (au > 0x7F800000u) {
        return (uint16_t)(sign | 0x7E00u);
    }
    if (au >= 0x477FF000u) {
        return (uint16_t)(sign | 0x7C00u);
    }
    if (au < 0x38800000u) {
        if (au < 0x33000000u) {
            return (uint16_t)sign;
        }
        const int      e     = (int)(au >> 23);
        const uint32_t m     = (au & 0x7FFFFFu) | 0x800000u;
        const int      shift = 126 - e;
        uint32_t       q     = m >> shift;
        const uint32_t rem   = m & ((1u << shift) - 1u);
        const uint32_t halfv = 1u << (shift - 1);
        if (rem > halfv || (rem == halfv && (q & 1u))) {
            q++;
        }
        return (uint16_t)(sign | q);
    }
    uint32_t       h   = ((au - 0x38000000u) >> 13);
    const uint32_t rem = au & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) {
        h++;
    }
    return (uint16_t)(sign | h);
#endif
}

FTK_HD float bf16_bits_to_float(uint16_t b)
{
    return u2f((uint32_t)b << 16);
}

FTK_HD uint16_t float_to_bf16_bits(float f)
{
#if defined(__HIP_DEVICE_COMPILE__)
    const __bf16 v = (__bf16)f;  // v_cvt_pk_bf16_f32, round-to-nearest-even
    uint16_t     h;
    __builtin_memcpy(&h, &v, 2);
    return h;
#else
    const uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);
    }
    const uint32_t r = u + 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(r >> 16);
#endif
}

// Logits element types. `T` is the storage type; all arithmetic is done on the exact fp32 image
// and rounded once per store, which equals native half arithmetic for + and * of two halves.
enum DType { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };

template<int DT>
struct Storage;

template<>
struct Storage<DT_F32> {
    typedef float  T;
    static FTK_HD float ld(T v) { return v; }
    static FTK_HD T     st(float f) { return f; }
    static FTK_HD float max_t() { return 3.402823466e+38f; }
};
template<>
struct Storage<DT_F16> {
    typedef uint16_t T;
    static FTK_HD float ld(T v) { return half_bits_to_float(v); }
    static FTK_HD T     st(float f) { return float_to_half_bits(f); }
    static FTK_HD float max_t() { return 65504.0f; }
};
template<>
struct Storage<DT_BF16> {
    typedef uint16_t T;
    static FTK_HD float ld(T v) { return bf16_bits_to_float(v); }
    static FTK_HD T     st(float f) { return float_to_bf16_bits(f); }
    // largest finite bfloat16; FLT_MAX itself rounds to +inf in bfloat16
    static FTK_HD float max_t() { return u2f(0x7F7F0000u); }
};

// Order-preserving 32-bit image of an fp32 value for selection: a > b  <=>  key(a) > key(b) for
// ordinary values; -0 and +0 share a key (they compare equal); NaN maps to 0, below every number,
// because the reference's strict `>` never selects a NaN.
FTK_HD uint32_t order_key(float f)
{
    uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return 0u;
    }
    if (u == 0x80000000u) {
        u = 0u;
    }
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
// order_key for a value known to be +0, positive or NaN
FTK_HD uint32_t order_key_nonneg(float f)
{
    const uint32_t u = f2u(f);
    return u <= 0x7F800000u ? (u | 0x80000000u) : 0u;
}
FTK_HD float key_to_float(uint32_t k)
{
    return u2f((k & 0x80000000u) ? (k & 0x7FFFFFFFu) : ~k);
}

}  // namespace ftk
