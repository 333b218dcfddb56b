// Streaming over the columns of one row with 16-byte accesses where the address allows.
#pragma once
#include "ftk_device.cuh"

namespace ftk {

// Calls visit(column, value) for the columns [lo, hi) of a row, 16-byte loads where the address
// allows, four of them in flight per thread. A thread sees its columns in ascending order.
template<int DT, int THREADS, typename F>
__device__ __forceinline__ void stream_columns(const typename Storage<DT>::T* __restrict__ rowp, int lo, int hi,
                                               F&& visit)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    const int             t   = threadIdx.x;
    if (hi <= lo) {
        return;
    }
    const int a     = (int)(((16u - ((uintptr_t)(rowp + lo) & 15u)) & 15u) / sizeof(T));
    const int head  = min(a, hi - lo);
    const int nvec  = (hi - lo - head) / EPV;
    const int body0 = lo + head;
    const int tail0 = body0 + nvec * EPV;
    if (t < head) {
        visit(lo + t, S::ld(rowp[lo + t]));
    }
    const uint4*  vec = reinterpret_cast<const uint4*>(rowp + body0);
    constexpr int U   = 4;
    for (int i0 = t; i0 < nvec; i0 += U * THREADS) {
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * THREADS;
            raw[u]      = i < nvec ? vec[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * THREADS;
            if (i < nvec) {
                const T* e = reinterpret_cast<const T*>(&raw[u]);
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    visit(body0 + i * EPV + j, S::ld(e[j]));
                }
            }
        }
    }
    if (tail0 + t < hi) {
        visit(tail0 + t, S::ld(rowp[tail0 + t]));
    }
}

// In-place variant: every column of [lo, hi) is replaced by f(column, value).
template<int DT, int THREADS, typename F>
__device__ __forceinline__ void transform_columns(typename Storage<DT>::T* __restrict__ rowp, int lo, int hi, F&& f)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    const int             t   = threadIdx.x;
    if (hi <= lo) {
        return;
    }
    const int a     = (int)(((16u - ((uintptr_t)(rowp + lo) & 15u)) & 15u) / sizeof(T));
    const int head  = min(a, hi - lo);
    const int nvec  = (hi - lo - head) / EPV;
    const int body0 = lo + head;
    const int tail0 = body0 + nvec * EPV;
    if (t < head) {
        rowp[lo + t] = S::st(f(lo + t, S::ld(rowp[lo + t])));
    }
    uint4*        vec = reinterpret_cast<uint4*>(rowp + body0);
    constexpr int U   = 4;
    for (int i0 = t; i0 < nvec; i0 += U * THREADS) {
        uint4 raw[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * THREADS;
            raw[u]      = i < nvec ? vec[i] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int i = i0 + u * THREADS;
            if (i < nvec) {
                T* e = reinterpret_cast<T*>(&raw[u]);
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    e[j] = S::st(f(body0 + i * EPV + j, S::ld(e[j])));
                }
                vec[i] = raw[u];
            }
        }
    }
    if (tail0 + t < hi) {
        rowp[tail0 + t] = S::st(f(tail0 + t, S::ld(rowp[tail0 + t])));
    }
}

}  // namespace ftk
