// Device-side building blocks shared by the sampling kernels (gfx950, 64-lane wavefronts).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "ftk_math.h"

namespace ftk {

constexpr int WAVE = 64;

// Many numerators over one denominator, bit for bit the IEEE quotient. The compiler expands `n / d` into
// v_div_scale (both operands), v_rcp, one refinement of the reciprocal, two corrections of the quotient, v_div_fmas
// and v_div_fixup; for operands that need no scaling and no fix-up the scale and fix-up instructions pass their
// inputs through, and what remains is the sequence below with the reciprocal's part computed once. No scaling is
// needed when the denominator lies in [1, 2^30] and the numerator is 0 or in [2^-100, 1] (the quotient is then a
// normal number and every remainder exact); other numerators take the ordinary division.
struct RowDivisor {
    float d, r;
    bool  ok;  // the denominator allows the short sequence (same for every thread that shares it)

    __device__ __forceinline__ explicit RowDivisor(float denom)
    {
        d              = denom;
        ok             = denom >= 1.0f && denom <= 1073741824.0f;
        const float r0 = __builtin_amdgcn_rcpf(denom);
        const float e0 = __builtin_fmaf(-denom, r0, 1.0f);
        r              = __builtin_fmaf(e0, r0, r0);
    }
    // requires ok; n must be +0, in (0, 1], or NaN
    __device__ __forceinline__ float divide(float n) const
    {
        if (n >= 7.888609052210118e-31f || n == 0.0f) {
            const float q0 = n * r;
            const float m0 = __builtin_fmaf(-d, q0, n);
            const float q1 = __builtin_fmaf(m0, r, q0);
            const float m1 = __builtin_fmaf(-d, q1, n);
            return __builtin_fmaf(m1, r, q1);
        }
        return n / d;
    }
};

#define FTK_LAUNCH_CHECK()                                                                                             \
    do {                                                                                                               \
        hipError_t e_ = hipGetLastError();                                                                             \
        if (e_ != hipSuccess) {                                                                                        \
            return (int)e_;                                                                                            \
        }                                                                                                              \
    } while (0)

#define FTK_DISPATCH_DTYPE(dtype, ...)                                                                                 \
    switch (dtype) {                                                                                                   \
        case DT_F32: {                                                                                                 \
            constexpr int DT = DT_F32;                                                                                 \
            __VA_ARGS__;                                                                                               \
        } break;                                                                                                       \
        case DT_F16: {                                                                                                 \
            constexpr int DT = DT_F16;                                                                                 \
            __VA_ARGS__;                                                                                               \
        } break;                                                                                                       \
        case DT_BF16: {                                                                                                \
            constexpr int DT = DT_BF16;                                                                                \
            __VA_ARGS__;                                                                                               \
        } break;                                                                                                       \
        default:                                                                                                       \
            return -1;                                                                                                 \
    }

__device__ __forceinline__ int lane_id()
{
    return (int)(threadIdx.x & (WAVE - 1));
}
__device__ __forceinline__ int wave_id()
{
    return (int)(threadIdx.x >> 6);
}

// ---- wave / block reductions ----------------------------------------------------------------
// The value of another lane through DPP (no LDS round trip): CTRL is the dpp_ctrl encoding; every pattern used
// here has a valid source lane for every lane. Works on 32-bit and 64-bit trivially copyable types.
template<int CTRL, typename V>
__device__ __forceinline__ V dpp_from(V v)
{
    static_assert(sizeof(V) == 4 || sizeof(V) == 8, "32-bit or 64-bit values");
    if constexpr (sizeof(V) == 4) {
        const int r = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false);
        return __builtin_bit_cast(V, r);
    }
    else {
        const unsigned long long u  = __builtin_bit_cast(unsigned long long, v);
        const int                lo = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)u, CTRL, 0xF, 0xF, false);
        const int                hi = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(u >> 32), CTRL, 0xF, 0xF, false);
        return __builtin_bit_cast(V, ((unsigned long long)(uint32_t)hi << 32) | (uint32_t)lo);
    }
}
// Reductions whose result does not depend on the order of the operands (maximum, minimum, integer sum), result
// in every lane: neighbours inside a quad (quad_perm), quads inside a row of 16 lanes (row_ror:4, row_ror:8),
// then the four rows through two lane exchanges.
constexpr int DPP_QUAD_XOR1 = 0xB1;   // quad_perm [1, 0, 3, 2]
constexpr int DPP_QUAD_XOR2 = 0x4E;   // quad_perm [2, 3, 0, 1]
constexpr int DPP_ROW_ROR4  = 0x124;  // row_ror:4
constexpr int DPP_ROW_ROR8  = 0x128;  // row_ror:8

template<typename V, typename Op>
__device__ __forceinline__ V wave_reduce_unordered(V v, Op op)
{
    v = op(v, dpp_from<DPP_QUAD_XOR1>(v));
    v = op(v, dpp_from<DPP_QUAD_XOR2>(v));
    v = op(v, dpp_from<DPP_ROW_ROR4>(v));
    v = op(v, dpp_from<DPP_ROW_ROR8>(v));
    v = op(v, __shfl_xor(v, 16, WAVE));
    v = op(v, __shfl_xor(v, 32, WAVE));
    return v;
}
template<typename V>
__device__ __forceinline__ V wave_max(V v)
{
    return wave_reduce_unordered(v, [](V a, V b) { return b > a ? b : a; });
}
template<typename V>
__device__ __forceinline__ V wave_min(V v)
{
    return wave_reduce_unordered(v, [](V a, V b) { return b < a ? b : a; });
}
__device__ __forceinline__ int wave_sum_i(int v)
{
    return wave_reduce_unordered(v, [](int a, int b) { return a + b; });
}

// Block-wide reductions over the threads of the block (multiple of 64, <= 1024). `smem` holds >= 16
// elements of V. The result is returned to every thread. Two barriers. NW is the number of waves of
// the block when the caller knows it (0: read from the launch, which costs a trip to memory).
template<typename V, int NW = 0>
__device__ __forceinline__ V block_max(V v, V* smem, V identity)
{
    v = wave_max(v);
    if (lane_id() == 0) {
        smem[wave_id()] = v;
    }
    __syncthreads();
    const int nw = NW > 0 ? NW : (int)(blockDim.x >> 6);
    V         r  = (lane_id() < nw) ? smem[lane_id()] : identity;
    r            = wave_max(r);
    __syncthreads();
    return r;
}
template<typename V, int NW = 0>
__device__ __forceinline__ V block_min(V v, V* smem, V identity)
{
    v = wave_min(v);
    if (lane_id() == 0) {
        smem[wave_id()] = v;
    }
    __syncthreads();
    const int nw = NW > 0 ? NW : (int)(blockDim.x >> 6);
    V         r  = (lane_id() < nw) ? smem[lane_id()] : identity;
    r            = wave_min(r);
    __syncthreads();
    return r;
}
template<int NW = 0>
__device__ __forceinline__ int block_sum_i(int v, int* smem)
{
    v = wave_sum_i(v);
    if (lane_id() == 0) {
        smem[wave_id()] = v;
    }
    __syncthreads();
    const int nw = NW > 0 ? NW : (int)(blockDim.x >> 6);
    int       r  = (lane_id() < nw) ? smem[lane_id()] : 0;
    r            = wave_sum_i(r);
    __syncthreads();
    return r;
}

// Descending bitonic sort of one value per lane across the 64-lane wave: afterwards lane i holds
// the (i+1)-th largest value.
__device__ __forceinline__ uint32_t wave_sort_desc(uint32_t v)
{
    const int lane = lane_id();
#pragma unroll
    for (int k = 2; k <= WAVE; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            const uint32_t other = __shfl_xor(v, j, WAVE);
            // in a descending sort the lower lane of a pair keeps the larger value inside
            // "descending" blocks ((lane & k) == 0) and the smaller one otherwise
            const bool lower     = (lane & j) == 0;
            const bool desc      = (lane & k) == 0;
            const bool keep_max  = lower == desc;
            const uint32_t mx    = other > v ? other : v;
            const uint32_t mn    = other > v ? v : other;
            v                    = keep_max ? mx : mn;
        }
    }
    return v;
}

__device__ __forceinline__ int next_pow2(int n)
{
    int p = 1;
    while (p < n) {
        p <<= 1;
    }
    return p;
}

// In-LDS ascending sort of any number n of 64-bit keys by all threads of the block. The network is the
// bitonic sorter in its form with comparators of one direction only (each merge starts by comparing
// mirrored positions); with every comparator putting the smaller key first, the positions from n up
// to the next power of two behave as if they held the largest key and never take part, so they are
// neither stored nor visited. THREADS is the size of the block (a constant here: reading blockDim
// costs a trip to memory in every stage).
template<int THREADS>
__device__ __forceinline__ void block_sort_u64(unsigned long long* keys, int n)
{
    const int half = next_pow2(n) >> 1;
    for (int k = 2; (k >> 1) <= half && k > 0; k <<= 1) {
        const int hk = k >> 1;
        for (int i = (int)threadIdx.x; i < half; i += THREADS) {
            const int pos = i & (hk - 1);
            const int lo  = ((i - pos) << 1) | pos;
            const int hi  = ((i - pos) << 1) | (k - 1 - pos);
            if (hi < n) {
                const unsigned long long a = keys[lo];
                const unsigned long long b = keys[hi];
                if (a > b) {
                    keys[lo] = b;
                    keys[hi] = a;
                }
            }
        }
        __syncthreads();
        for (int j = hk >> 1; j > 0; j >>= 1) {
            for (int i = (int)threadIdx.x; i < half; i += THREADS) {
                const int lo = ((i & ~(j - 1)) << 1) | (i & (j - 1));
                const int hi = lo | j;
                if (hi < n) {
                    const unsigned long long a = keys[lo];
                    const unsigned long long b = keys[hi];
                    if (a > b) {
                        keys[lo] = b;
                        keys[hi] = a;
                    }
                }
            }
            __syncthreads();
        }
    }
}

// The same result as block_sort_u64 for n <= 256 * PER keys, by a block of 256 threads, with the keys in
// registers: thread t holds the PER keys of positions t * PER .. t * PER + PER - 1 of the network. Partners
// less than PER apart are in the thread's own registers, partners in the same wave come through lane
// exchanges, and only the stages that pair up different waves go through LDS (in `keys` itself, which must
// hold 256 * PER entries). The positions from n on count as the largest key.
template<int PER>
__device__ __forceinline__ void block_sort_u64_regs(unsigned long long* keys, int n)
{
    constexpr int THREADS = 256;
    constexpr int N       = THREADS * PER;
    static_assert(PER == 2 || PER == 4 || PER == 8, "keys per thread");
    const int          t = (int)threadIdx.x;
    unsigned long long k[PER];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        const int e = r * THREADS + t;  // any assignment will do for unsorted input: this one has no bank conflicts
        k[r]        = e < n ? keys[e] : ~0ull;
    }
    // compare-exchange with a key of another thread: `keep_min` says which of the two this thread keeps
    auto exchange = [&](unsigned long long mine, unsigned long long other, bool keep_min) -> unsigned long long {
        const bool other_smaller = other < mine;
        return other_smaller == keep_min ? other : mine;
    };
#pragma unroll 1
    for (int size = 2; size <= N; size <<= 1) {
        // ascending where the position has the `size` bit clear (the whole thread agrees once size >= 2 * PER)
#pragma unroll 1
        for (int j = size >> 1; j >= PER; j >>= 1) {
            const int  tj       = j / PER;  // distance of the partner thread
            const bool asc      = ((t * PER) & size) == 0;
            const bool keep_min = ((t & tj) == 0) == asc;
            if (tj < WAVE) {
                // every key of the partner lane is requested before the first one is used
                int lo[PER], hi[PER];
                if (tj == 1) {
#pragma unroll
                    for (int r = 0; r < PER; ++r) {  // quad_perm [1, 0, 3, 2]
                        lo[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)k[r], 0xB1, 0xF, 0xF, false);
                        hi[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(k[r] >> 32), 0xB1, 0xF, 0xF, false);
                    }
                }
                else if (tj == 2) {
#pragma unroll
                    for (int r = 0; r < PER; ++r) {  // quad_perm [2, 3, 0, 1]
                        lo[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)k[r], 0x4E, 0xF, 0xF, false);
                        hi[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(k[r] >> 32), 0x4E, 0xF, 0xF, false);
                    }
                }
                else {
                    const int from = (lane_id() ^ tj) << 2;
#pragma unroll
                    for (int r = 0; r < PER; ++r) {
                        lo[r] = __builtin_amdgcn_ds_bpermute(from, (int)(uint32_t)k[r]);
                        hi[r] = __builtin_amdgcn_ds_bpermute(from, (int)(uint32_t)(k[r] >> 32));
                    }
                }
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    const unsigned long long other = ((unsigned long long)(uint32_t)hi[r] << 32) | (uint32_t)lo[r];
                    k[r]                           = exchange(k[r], other, keep_min);
                }
            }
            else {
                __syncthreads();  // earlier reads of `keys` are done
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    keys[r * THREADS + t] = k[r];
                }
                __syncthreads();
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    k[r] = exchange(k[r], keys[r * THREADS + (t ^ tj)], keep_min);
                }
            }
        }
#pragma unroll
        for (int j = PER >> 1; j > 0; j >>= 1) {
            if (j < size) {
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    if ((r & j) == 0) {
                        const bool               asc = ((t * PER + r) & size) == 0;
                        const unsigned long long a = k[r], b = k[r | j];
                        const bool               swap = (b < a) == asc;
                        k[r]     = swap ? b : a;
                        k[r | j] = swap ? a : b;
                    }
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        const int e = t * PER + r;
        if (e < n) {
            keys[e] = k[r];
        }
    }
    __syncthreads();
}

// Ascending sort of 64 * PER keys held by one wave, PER per lane: afterwards lane l holds positions
// l * PER .. l * PER + PER - 1 of the sorted sequence. No LDS, no barrier.
template<int PER>
__device__ __forceinline__ void wave_sort_keys_u64(unsigned long long (&k)[PER])
{
    constexpr int N = WAVE * PER;
    const int     l = lane_id();
#pragma unroll 1
    for (int size = 2; size <= N; size <<= 1) {
#pragma unroll 1
        for (int j = size >> 1; j >= PER; j >>= 1) {
            const int  lj       = j / PER;
            const bool asc      = ((l * PER) & size) == 0;
            const bool keep_min = ((l & lj) == 0) == asc;
            int        lo[PER], hi[PER];
            if (lj == 1) {
#pragma unroll
                for (int r = 0; r < PER; ++r) {  // quad_perm [1, 0, 3, 2]
                    lo[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)k[r], 0xB1, 0xF, 0xF, false);
                    hi[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(k[r] >> 32), 0xB1, 0xF, 0xF, false);
                }
            }
            else if (lj == 2) {
#pragma unroll
                for (int r = 0; r < PER; ++r) {  // quad_perm [2, 3, 0, 1]
                    lo[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)k[r], 0x4E, 0xF, 0xF, false);
                    hi[r] = __builtin_amdgcn_update_dpp(0, (int)(uint32_t)(k[r] >> 32), 0x4E, 0xF, 0xF, false);
                }
            }
            else {
                const int from = (l ^ lj) << 2;
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    lo[r] = __builtin_amdgcn_ds_bpermute(from, (int)(uint32_t)k[r]);
                    hi[r] = __builtin_amdgcn_ds_bpermute(from, (int)(uint32_t)(k[r] >> 32));
                }
            }
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                const unsigned long long other = ((unsigned long long)(uint32_t)hi[r] << 32) | (uint32_t)lo[r];
                k[r]                           = ((other < k[r]) == keep_min) ? other : k[r];
            }
        }
#pragma unroll
        for (int j = PER >> 1; j > 0; j >>= 1) {
            if (j < size) {
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    if ((r & j) == 0) {
                        const bool               asc = ((l * PER + r) & size) == 0;
                        const unsigned long long a = k[r], b = k[r | j];
                        const bool               swap = (b < a) == asc;
                        k[r]     = swap ? b : a;
                        k[r | j] = swap ? a : b;
                    }
                }
            }
        }
    }
}

// Ascending sort of n <= 2048 keys in LDS (`keys` holds 2048 entries) by a block of 256 threads. One copy per
// kernel: the callers are not on the path of the common, small lists.
__device__ __noinline__ void block_sort_u64_2048(unsigned long long* keys, int n)
{
    if (n <= 1024) {
        block_sort_u64_regs<4>(keys, n);
    }
    else {
        block_sort_u64_regs<8>(keys, n);
    }
}

// ---- Philox-4x32-10 (counter-based generator; replaces cuRAND's XORWOW) ---------------------
FTK_HD void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1, uint32_t out[4])
{
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        const uint32_t n1 = (uint32_t)p1;
        const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        const uint32_t n3 = (uint32_t)p0;
        c0 = n0;
        c1 = n1;
        c2 = n2;
        c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0;
    out[1] = c1;
    out[2] = c2;
    out[3] = c3;
}

struct RngState {
    uint64_t seed;
    uint64_t offset;
};

// One uniform in (0, 1] (the range of curand_uniform), advancing the row's counter.
__device__ __forceinline__ float rng_next_uniform(RngState* st)
{
    uint32_t       o[4];
    const uint64_t off = st->offset;
    philox4x32_10((uint32_t)off, (uint32_t)(off >> 32), 0u, 0u, (uint32_t)st->seed, (uint32_t)(st->seed >> 32), o);
    st->offset = off + 1;
    return (float)o[0] * 2.3283064365386963e-10f + 1.16415321826934814453125e-10f;
}

// What a row's draw is made from, requested ahead of time without control flow (`safe`: any valid 4-byte aligned
// address, read when an array is absent): the injected draw, or the row's generator state.
struct RowDrawSource {
    float    injected;
    uint32_t seed_lo, seed_hi, off_lo, off_hi;
};
__device__ __forceinline__ RowDrawSource row_draw_source(const RngState* rng, const float* injected, int b,
                                                         const void* safe)
{
    const uint32_t* st   = rng != nullptr ? reinterpret_cast<const uint32_t*>(rng + b) : nullptr;
    const uint32_t* from = reinterpret_cast<const uint32_t*>(safe);
    RowDrawSource   d;
    d.injected = *(injected != nullptr ? injected + b : reinterpret_cast<const float*>(safe));
    d.seed_lo  = *(st != nullptr ? st + 0 : from);
    d.seed_hi  = *(st != nullptr ? st + 1 : from);
    d.off_lo   = *(st != nullptr ? st + 2 : from);
    d.off_hi   = *(st != nullptr ? st + 3 : from);
    return d;
}
// One thread per row: the generated draw (same values as rng_next_uniform) and the counter the row's state goes on
// with, which the caller stores.
__device__ __forceinline__ float row_draw_generate(const RowDrawSource& d, uint64_t* next_offset)
{
    uint32_t o[4];
    philox4x32_10(d.off_lo, d.off_hi, 0u, 0u, d.seed_lo, d.seed_hi, o);
    *next_offset = (((uint64_t)d.off_hi << 32) | d.off_lo) + 1;
    return (float)o[0] * 2.3283064365386963e-10f + 1.16415321826934814453125e-10f;
}

// The draw of row `b`: injected when the caller supplied one, generated otherwise.
__device__ __forceinline__ float row_uniform(RngState* rng, const float* injected, int b)
{
    if (injected != nullptr) {
        return injected[b];
    }
    return rng_next_uniform(rng + b);
}

}  // namespace ftk
