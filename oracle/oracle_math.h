// CPU ORACLE (test infrastructure only; never linked into the product).
//
// Scalar arithmetic helpers of the oracle: storage-type conversions (IEEE binary16,
// bfloat16) and the deterministic single-precision exp/log that stand in for the
// reference's `__expf` / `logf` device intrinsics
// (src/fastertransformer/kernels/sampling_topk_kernels.cu:274,290,
//  src/fastertransformer/kernels/sampling_topp_kernels.cu:924,989,1332).
//
// The intrinsics' bit patterns are not reproducible outside a CUDA device, so the oracle
// uses a fixed sequence of IEEE-754 binary32 operations (fma, mul, add, round-to-nearest-even)
// that gives the same bits on every IEEE machine. tests/test_oracle_math.py pins both
// functions against float64 libm (<= 2 ulp) so they are a faithful `exp` / `log`.
//
// Compile with -ffp-contract=off: every rounding below is intentional.
#pragma once
#include <cmath>
#include <cstdint>
#include <cstring>

namespace oracle {

static inline uint32_t f2u(float f)
{
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return u;
}
static inline float u2f(uint32_t u)
{
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// ---- binary16 ------------------------------------------------------------------------------
static inline float half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp  = (h >> 10) & 0x1Fu;
    const uint32_t man  = h & 0x3FFu;
    if (exp == 0x1Fu) {
        return u2f(sign | 0x7F800000u | (man << 13));
    }
    if (exp == 0) {
        // subnormal: man * 2^-24 exactly
        const float v = (float)man * 5.9604644775390625e-08f;
        return sign ? -v : v;
    }
    return u2f(sign | ((exp + 112u) << 23) | (man << 13));
}

// round-to-nearest-even, overflow to infinity, gradual underflow (what `__float2half_rn` does)
static inline uint16_t float_to_half(float f)
{
    const uint32_t u    = f2u(f);
    const uint32_t sign = (u >> 16) & 0x8000u;
    const uint32_t au   = u & 0x7FFFFFFFu;
    if (au > 0x7F800000u) {
        return (uint16_t)(sign | 0x7E00u);  // NaN
    }
    if (au >= 0x477FF000u) {
        // >= 65520 rounds to infinity (65504 + half an ulp)
        return (uint16_t)(sign | 0x7C00u);
    }
    if (au < 0x38800000u) {
        // result is subnormal (or zero): value * 2^24 rounded to nearest even integer
        if (au < 0x33000000u) {
            // < 2^-25 : rounds to zero (2^-25 itself is a tie -> even -> 0)
            return (uint16_t)sign;
        }
        const int      e     = (int)(au >> 23);            // biased exponent, 102..112
        const uint32_t m     = (au & 0x7FFFFFu) | 0x800000u;
        const int      shift = 126 - e;                    // 14..24
        uint32_t       q     = m >> shift;
        const uint32_t rem   = m & ((1u << shift) - 1u);
        const uint32_t halfv = 1u << (shift - 1);
        if (rem > halfv || (rem == halfv && (q & 1u))) {
            q++;
        }
        return (uint16_t)(sign | q);
    }
    // normal
    uint32_t       h   = ((au - 0x38000000u) >> 13);
    const uint32_t rem = au & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) {
        h++;
    }
    return (uint16_t)(sign | h);
}

// ---- bfloat16 ------------------------------------------------------------------------------
static inline float bf16_to_float(uint16_t b)
{
    return u2f((uint32_t)b << 16);
}
static inline uint16_t float_to_bf16(float f)
{
    const uint32_t u = f2u(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) {
        return (uint16_t)((u >> 16) | 0x0040u);  // quiet NaN
    }
    const uint32_t r = u + 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(r >> 16);
}

// ---- deterministic expf -------------------------------------------------------------------
// exp(x) = 2^n * exp(r), n = rint(x*log2(e)), r = x - n*ln2 (two-term Cody-Waite),
// exp(r) = 1 + r + r^2 * P(r) with the degree-5 Cephes `expf` minimax polynomial.
static inline float det_expf(float x)
{
    if (x != x) {
        return x;
    }
    if (x > 88.72283935546875f) {
        return INFINITY;
    }
    if (x < -103.97283172607421875f) {
        return 0.0f;
    }
    const float n = std::nearbyintf(x * 1.44269502162933349609375f);
    float       r = std::fmaf(n, -0.693145751953125f, x);
    r             = std::fmaf(n, -1.428606765330187045e-06f, r);
    float p       = 1.9875691500e-4f;
    p             = std::fmaf(p, r, 1.3981999507e-3f);
    p             = std::fmaf(p, r, 8.3334519073e-3f);
    p             = std::fmaf(p, r, 4.1665795894e-2f);
    p             = std::fmaf(p, r, 1.6666665459e-1f);
    p             = std::fmaf(p, r, 5.0000001201e-1f);
    const float z = r * r;
    float       y = std::fmaf(p, z, r) + 1.0f;
    // scale by 2^n in two exact-or-single-rounding steps (n in [-150, 128])
    const int ni = (int)n;
    const int n1 = ni / 2;
    const int n2 = ni - n1;
    y            = y * u2f((uint32_t)(n1 + 127) << 23);
    y            = y * u2f((uint32_t)(n2 + 127) << 23);
    return y;
}

// ---- deterministic logf -------------------------------------------------------------------
// Cephes `logf`: x = m * 2^e, m in [sqrt(1/2), sqrt(2)), f = m - 1,
// log(x) = f - f^2/2 + f^3 * P(f) + e*ln2 (ln2 split in two terms).
static inline float det_logf(float x)
{
    if (x != x) {
        return x;
    }
    if (x < 0.0f) {
        return NAN;
    }
    if (x == 0.0f) {
        return -INFINITY;
    }
    if (x == INFINITY) {
        return x;
    }
    uint32_t u = f2u(x);
    int      e = 0;
    if (u < 0x00800000u) {
        // subnormal: renormalise exactly
        x = x * 8388608.0f;  // 2^23
        u = f2u(x);
        e = -23;
    }
    e += (int)(u >> 23) - 126;                            // x = m * 2^e with m in [0.5, 1)
    float m = u2f((u & 0x007FFFFFu) | 0x3F000000u);       // [0.5, 1)
    if (m < 0.707106769084930419921875f) {
        e -= 1;
        m = m + m - 1.0f;
    }
    else {
        m = m - 1.0f;
    }
    const float z = m * m;
    float       p = 7.0376836292e-2f;
    p             = std::fmaf(p, m, -1.1514610310e-1f);
    p             = std::fmaf(p, m, 1.1676998740e-1f);
    p             = std::fmaf(p, m, -1.2420140846e-1f);
    p             = std::fmaf(p, m, 1.4249322787e-1f);
    p             = std::fmaf(p, m, -1.6668057665e-1f);
    p             = std::fmaf(p, m, 2.0000714765e-1f);
    p             = std::fmaf(p, m, -2.4999993993e-1f);
    p             = std::fmaf(p, m, 3.3333331174e-1f);
    float       y = (m * z) * p;
    const float fe = (float)e;
    y             = std::fmaf(fe, -2.12194440e-4f, y);
    y             = std::fmaf(-0.5f, z, y);
    float res     = m + y;
    res           = std::fmaf(fe, 0.693359375f, res);
    return res;
}

}  // namespace oracle
