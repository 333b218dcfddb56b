// Masked softmax and top-p (nucleus) sampling.
//
// Reference behaviour restated (src/fastertransformer/kernels/sampling_topp_kernels.cu):
//   :1294-1345 addBiasSoftMax          - in-place masked softmax, result rounded to T
//   :801-860   topp_beam_topk_kernel   - arg-max shortcut when max prob >= top_p
//   :1106-1119 cub segmented sort      - stable descending sort of every row
//   :877-1004  topp_sampling           - inclusive prefix sum over 256-wide tiles, first crossing
//   :1381-1412 computeToppDecay
//
// The replacement orders only the part of a row in front of the draw (see the top-p section).
#include "ftk_device.cuh"
#include "ftk_sampling.h"
#ifdef FTK_TEST_HOOKS
#include "ftk_test_hooks.h"
#endif
#include "ftk_columns.cuh"
#include "ftk_transform.cuh"

namespace ftk {

// =============================================================================================
// softmax
// =============================================================================================
constexpr int SM_THREADS = 1024;

// The reference block has BLK = min(n, 1024) threads and thread t owns columns t, t+BLK, ...;
// summation order (reduce_kernel_utils.cuh:73-103) = sequential per thread, xor butterfly
// (16,8,4,2,1) inside each 32-lane group, lane-0 partials through shared memory, butterfly again.
// STATS_ONLY: stops after the sum and leaves (maximum, denominator) of the row in `stats`; the row itself is
// not written (softmax_finish_histogram_kernel divides).
template<int DT, bool STATS_ONLY>
__global__ void __launch_bounds__(SM_THREADS)
softmax_kernel(typename Storage<DT>::T* __restrict__ logits, const typename Storage<DT>::T* __restrict__ bias,
               const int* __restrict__ end_ids, const bool* __restrict__ finished, int n_padded, int n,
               float2* __restrict__ stats)
{
    typedef Storage<DT> S;
    __shared__ float    sh[32];
    __shared__ float    sh_bcast;
    const int           row    = blockIdx.x;
    const int           t      = threadIdx.x;
    const int           BLK    = min(n, SM_THREADS);
    const bool          active = t < BLK;
    const bool          fin    = finished != nullptr ? finished[row] : false;
    const int           end_id = fin ? end_ids[row] : -1;
    typename S::T*      rowp   = logits + (size_t)row * n_padded;
    const float         MAXT   = S::max_t();

    auto masked = [&](int v) -> float {
        if (v >= n) {
            return -MAXT;
        }
        if (fin) {
            return v == end_id ? MAXT : -MAXT;
        }
        const float b = bias != nullptr ? S::ld(bias[v]) : 0.0f;
        return round_t<DT>(S::ld(rowp[v]) + b);
    };

    if (!fin && bias == nullptr) {
        // Ordinary rows. The maximum and the final division do not depend on the order of the columns
        // and go through 16-byte accesses; the sum keeps the reference's order (thread t adds its
        // columns t, t + BLK, ... one after the other), eight or sixteen loads in flight.
        float mx = -3.402823466e+38f;
        stream_columns<DT, SM_THREADS>(rowp, 0, n, [&](int, float x) { mx = __builtin_fmaxf(mx, x + 0.0f); });
        if (n_padded > n) {
            mx = __builtin_fmaxf(mx, -MAXT);
        }
        mx = block_max<float, SM_THREADS / WAVE>(mx, sh, -3.402823466e+38f);
        if (BLK < 1024) {
            mx = __builtin_fmaxf(mx, -1e20f);
        }
        const float pad_e = round_t<DT>(det_expf_nonpos(-MAXT - mx));
        float       sum   = 0.0f;
        if (active) {
            constexpr int U = DT == DT_F32 ? 8 : 16;  // 2-byte loads move half as much per instruction
            int           v = t;
            for (; v + (U - 1) * BLK < n; v += U * BLK) {
                float x[U];
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    x[u] = S::ld(rowp[v + u * BLK]);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    sum += round_t<DT>(det_expf_nonpos((x[u] + 0.0f) - mx));
                }
            }
            for (; v < n; v += BLK) {
                sum += round_t<DT>(det_expf_nonpos((S::ld(rowp[v]) + 0.0f) - mx));
            }
            for (; v < n_padded; v += BLK) {
                sum += pad_e;
            }
        }
#pragma unroll
        for (int m = 16; m > 0; m >>= 1) {
            sum += __shfl_xor(sum, m, 32);
        }
        if ((t & 31) == 0) {
            sh[t >> 5] = sum;
        }
        __syncthreads();
        if (t < 32) {
            float v = ((float)t < (float)BLK / 32.0f) ? sh[t] : 0.0f;
#pragma unroll
            for (int m = 16; m > 0; m >>= 1) {
                v += __shfl_xor(v, m, 32);
            }
            if (t == 0) {
                sh_bcast = v;
            }
        }
        __syncthreads();
        const float denom = sh_bcast + 1e-6f;
        if constexpr (STATS_ONLY) {
            if (t == 0) {
                stats[row] = make_float2(mx, denom);
            }
            return;
        }
        const RowDivisor div(denom);
        if (div.ok) {
            transform_columns<DT, SM_THREADS>(rowp, 0, n, [&](int, float x) {
                return div.divide(round_t<DT>(det_expf_nonpos((x + 0.0f) - mx)));
            });
        }
        else {
            transform_columns<DT, SM_THREADS>(rowp, 0, n, [&](int, float x) {
                return round_t<DT>(det_expf_nonpos((x + 0.0f) - mx)) / denom;
            });
        }
        transform_columns<DT, SM_THREADS>(rowp, n, n_padded, [&](int, float) { return pad_e / denom; });
        return;
    }

    float mx = -3.402823466e+38f;
    if (active) {
        for (int v = t; v < n_padded; v += BLK) {
            mx = __builtin_fmaxf(mx, masked(v));
        }
    }
    mx = block_max<float, SM_THREADS / WAVE>(mx, sh, -3.402823466e+38f);
    if (BLK < 1024) {
        mx = __builtin_fmaxf(mx, -1e20f);  // blockReduceMax pads its second stage with -1e20f
    }

    float sum = 0.0f;
    if (active) {
        for (int v = t; v < n_padded; v += BLK) {
            sum += round_t<DT>(det_expf_nonpos(masked(v) - mx));
        }
    }
#pragma unroll
    for (int m = 16; m > 0; m >>= 1) {
        sum += __shfl_xor(sum, m, 32);
    }
    if ((t & 31) == 0) {
        sh[t >> 5] = sum;
    }
    __syncthreads();
    if (t < 32) {
        float v = ((float)t < (float)BLK / 32.0f) ? sh[t] : 0.0f;
#pragma unroll
        for (int m = 16; m > 0; m >>= 1) {
            v += __shfl_xor(v, m, 32);
        }
        if (t == 0) {
            sh_bcast = v;
        }
    }
    __syncthreads();
    const float denom = sh_bcast + 1e-6f;
    if constexpr (STATS_ONLY) {
        if (t == 0) {
            stats[row] = make_float2(mx, denom);
        }
        return;
    }
    if (active) {
        for (int v = t; v < n_padded; v += BLK) {
            const float e = round_t<DT>(det_expf_nonpos(masked(v) - mx));
            rowp[v]       = S::st(e / denom);
        }
    }
}

// =============================================================================================
// top-p
// =============================================================================================
//
// The reference sorts every row completely and then scans it. Only the part of the sorted order in
// front of the draw matters, so the rows are cut first and only the part above the cut is ordered:
//   histogram  - (chunks x rows) workgroups stream the probabilities once: entries per bucket (six
//                mantissa bits under the exponent, 32 octaves below 1.0), a fixed-point lower bound
//                of the mass per bucket, and the arg-max;
//   cut        - one workgroup per row: the lowest bucket whose suffix of mass certainly covers the
//                draw, where every bucket and every chunk writes inside the ordered prefix, and the
//                prefix divided into segments of whole buckets;
//   gather     - second stream: entries at or above the cut go to their bucket's range as
//                (~key, id) pairs;
//   sort       - segments are sorted independently, dealt out over the workgroups of one launch: the
//                keys of a segment are spread over bins, neighbouring bins joined into groups of a few
//                dozen entries, and every group sorted by one wave in registers (a long group of equal
//                keys by the whole workgroup in LDS, a segment that one bucket alone makes too long
//                by a radix sort in memory);
//   pick       - one workgroup per row replays the reference's scan on the ordered prefix with its
//                exact rounding order (32 raking lanes x 8 items, Kogge-Stone over the 32 partials,
//                sequential carry over tiles) and emits the token.
// A row whose draw is not crossed inside its prefix (it cannot be unless the bound above fails)
// falls back to a stable radix sort of all its positive entries.
// Callers that do not need the probabilities afterwards take a second form of the step (topp_row_kernel below):
// softmax statistics, histogram, cut and gather in one kernel that only reads the logits, then sort and pick.
constexpr int      TP_THREADS = 1024;
constexpr int      TP_TILE    = 256;          // the reference's scan tile
constexpr int      TP_ROUND   = 1024;         // tiles whose totals are held in LDS at a time
constexpr uint32_t ZERO_KEY   = 0x80000000u;  // order_key(+0.0f); entries at or below never join the scan

constexpr int TPH_THREADS = 256;
constexpr int TPC_THREADS = 1024;  // the cut kernel
constexpr int TPB_SHIFT   = 17;                        // key bits below a bucket (6 mantissa bits stay)
constexpr int TPB_ONE     = 0x3F800000 >> TPB_SHIFT;   // bucket of 1.0 before the shift of origin
constexpr int TPB_SPAN    = 32 * 64;                   // 32 octaves below 1.0 are resolved
constexpr int TPB_NB      = TPB_SPAN + 2;              // [0]: everything smaller, [NB-1]: above 1 + 1/64
constexpr int TPS_SEG     = 2048;                      // segment boundaries follow multiples of this
constexpr int TPS_CAP     = 5632;                      // longest segment sorted in LDS

constexpr int TOPP_SKIP     = 1;
constexpr int TOPP_SHORTCUT = 2;

struct ToppRowMeta {
    unsigned long long best;   // (key << 32) | ~id of the arg-max (lowest id among equals)
    int                cut;    // lowest gathered bucket
    int                n;      // entries at or above the cut
    int                n_pos;  // positive entries of the row (0x7FFFFFFF: not known, some may lie below the cut)
    int                nseg;
    int                flags;
    float              best_prob;  // the arg-max's probability (rows sampled straight from logits)
    float              mx, denom;  // the row's softmax statistics (rows sampled straight from logits)
};

// Workspace sections (all offsets multiples of 256 bytes). `sorted` keeps the reference's shape of
// two 64-bit arrays per row; the second one is only touched by the radix sorts.
struct ToppPlan {
    int    splits;  // chunks per row of the two streaming kernels
    int    chunk;   // columns per chunk
    int    sorters; // workgroups of the sort kernel
    size_t off_pcnt, off_pmass, off_pbest, off_start, off_boff, off_seg, off_meta, bytes;
};

static inline size_t align256(size_t x)
{
    return (x + 255) & ~(size_t)255;
}

static ToppPlan topp_plan(int batch, size_t vocab)
{
    ToppPlan p;
    const int rows = batch > 0 ? batch : 1;
    int       s    = (1024 + rows - 1) / rows;
    const int cap  = (int)(vocab / 8192) > 0 ? (int)(vocab / 8192) : 1;
    s              = s < cap ? s : cap;
    s              = s < 64 ? s : 64;
    p.splits       = s;
    p.chunk        = (int)(((vocab + s - 1) / s + 7) / 8 * 8);
    p.sorters      = 512;
    size_t off     = align256((size_t)rows * vocab * 2 * sizeof(unsigned long long));
    p.off_pcnt     = off;
    off += align256((size_t)rows * s * TPB_NB * sizeof(uint32_t));
    p.off_pmass = off;
    off += align256((size_t)rows * s * TPB_NB * sizeof(uint32_t));
    p.off_pbest = off;
    off += align256((size_t)rows * s * sizeof(unsigned long long));
    p.off_start = off;
    off += align256((size_t)rows * s * TPB_NB * sizeof(uint32_t));
    p.off_boff = off;
    off += align256((size_t)rows * TPB_NB * sizeof(uint32_t));
    p.off_seg = off;
    off += align256((size_t)rows * TPB_NB * sizeof(uint32_t));
    p.off_meta = off;
    off += align256((size_t)rows * sizeof(ToppRowMeta));
    p.bytes = off;
    return p;
}

__device__ __forceinline__ int topp_bucket(uint32_t key)
{
    const int raw = (int)((key & 0x7FFFFFFFu) >> TPB_SHIFT) - (TPB_ONE - TPB_SPAN);
    return min(max(raw, 0), TPB_NB - 1);
}

__device__ __forceinline__ float key64_prob(unsigned long long k)
{
    return key_to_float(~(uint32_t)(k >> 32));
}

template<int DT>
__global__ void __launch_bounds__(TPH_THREADS)
topp_histogram_kernel(const typename Storage<DT>::T* __restrict__ probs, int vocab, int chunk,
                      const bool* __restrict__ skip_decode, uint32_t* __restrict__ part_cnt,
                      uint32_t* __restrict__ part_mass, unsigned long long* __restrict__ part_best)
{
    __shared__ uint32_t           cnt[TPB_NB];
    __shared__ uint32_t           mass[TPB_NB];
    __shared__ unsigned long long red[16];
    const int                     row = blockIdx.y;
    const int                     j   = blockIdx.x;
    const int                     S   = gridDim.x;
    const int                     t   = threadIdx.x;
    if (skip_decode != nullptr && skip_decode[row]) {
        return;
    }
    for (int b = t; b < TPB_NB; b += TPH_THREADS) {
        cnt[b]  = 0u;
        mass[b] = 0u;
    }
    __syncthreads();
    const int lo   = (int)min((long long)vocab, (long long)j * chunk);
    const int hi   = (int)min((long long)vocab, (long long)lo + chunk);
    uint32_t  tmax = 0;
    int       tidx = 0x7FFFFFFF;
    stream_columns<DT, TPH_THREADS>(probs + (size_t)row * vocab, lo, hi, [&](int v, float x) {
        const uint32_t k = order_key(x);
        if (k > tmax) {
            tmax = k;
            tidx = v;
        }
        if (k > ZERO_KEY) {
            const int b = topp_bucket(k);
            atomicAdd(&cnt[b], 1u);
            // truncation keeps the sum a lower bound of the mass
            atomicAdd(&mass[b], (uint32_t)(__builtin_fminf(x, 1.0f) * 2147483648.0f));
        }
    });
    __syncthreads();
    const size_t base = ((size_t)row * S + j) * TPB_NB;
    for (int b = t; b < TPB_NB; b += TPH_THREADS) {
        part_cnt[base + b]  = cnt[b];
        part_mass[base + b] = mass[b];
    }
    unsigned long long best = ((unsigned long long)tmax << 32) | (uint32_t)(~(uint32_t)tidx);
    best                    = block_max<unsigned long long, TPH_THREADS / WAVE>(best, red, 0ull);
    if (t == 0) {
        part_best[(size_t)row * S + j] = best;
    }
}

// Second half of the softmax for the fused step, (chunks x rows) workgroups: divides every column by the
// row's denominator (same expression as softmax_kernel, so the stored probabilities are the same bits) and
// tallies what topp_histogram_kernel would read back from the row, in the same pass.
template<int DT>
__global__ void __launch_bounds__(TPH_THREADS)
softmax_finish_histogram_kernel(typename Storage<DT>::T* __restrict__ logits,
                                const typename Storage<DT>::T* __restrict__ bias, const int* __restrict__ end_ids,
                                const bool* __restrict__ finished, const float2* __restrict__ stats, int n_padded,
                                int n, int chunk, const bool* __restrict__ skip_decode,
                                uint32_t* __restrict__ part_cnt, uint32_t* __restrict__ part_mass,
                                unsigned long long* __restrict__ part_best)
{
    typedef Storage<DT>           S;
    __shared__ uint32_t           cnt[TPB_NB];
    __shared__ uint32_t           mass[TPB_NB];
    __shared__ unsigned long long red[16];
    const int                     row    = blockIdx.y;
    const int                     j      = blockIdx.x;
    const int                     NS     = gridDim.x;
    const int                     t      = threadIdx.x;
    const bool                    tally  = !(skip_decode != nullptr && skip_decode[row]);
    const bool                    fin    = finished != nullptr ? finished[row] : false;
    const int                     end_id = fin ? end_ids[row] : -1;
    const float                   MAXT   = S::max_t();
    const float2                  st     = stats[row];
    const float                   mx     = st.x;
    const float                   denom  = st.y;
    for (int b = t; b < TPB_NB; b += TPH_THREADS) {
        cnt[b]  = 0u;
        mass[b] = 0u;
    }
    __syncthreads();
    const int lo   = (int)min((long long)n_padded, (long long)j * chunk);
    const int hi   = (int)min((long long)n_padded, (long long)lo + chunk);
    uint32_t  tmax = 0;
    int       tidx = 0x7FFFFFFF;
    auto finish = [&](int v, float y) {
        // y <= mx (or NaN): the argument of the exponential is never positive
        const float p = round_t<DT>(det_expf_nonpos(y - mx)) / denom;
        if (tally) {
            const float    pr = round_t<DT>(p);
            const uint32_t k  = order_key(pr);
            if (k > tmax) {
                tmax = k;
                tidx = v;
            }
            if (k > ZERO_KEY) {
                const int b = topp_bucket(k);
                atomicAdd(&cnt[b], 1u);
                atomicAdd(&mass[b], (uint32_t)(__builtin_fminf(pr, 1.0f) * 2147483648.0f));
            }
        }
        return p;
    };
    typename S::T*   rowp = logits + (size_t)row * n_padded;
    const RowDivisor div(denom);
    if (!fin && bias == nullptr && div.ok) {
        // Ordinary rows: no per-column cases in front of the arithmetic, the division with the row's reciprocal,
        // and keys of values that cannot be negative (the exponential is in [0, 1] or NaN, the denominator at
        // least 1: probabilities in [0, 1]). `x + 0.0f` is left out: it only turns -0 into +0, and the
        // exponential of both differences is the same.
        auto quick = [&](int v, float y) {
            const float p = div.divide(round_t<DT>(det_expf_nonpos(y - mx)));
            if (tally) {
                const float    pr = round_t<DT>(p);
                const uint32_t k  = order_key_nonneg(pr);
                if (k > tmax) {
                    tmax = k;
                    tidx = v;
                }
                if (k > ZERO_KEY) {
                    const int b = topp_bucket(k);
                    atomicAdd(&cnt[b], 1u);
                    atomicAdd(&mass[b], (uint32_t)(pr * 2147483648.0f));
                }
            }
            return p;
        };
        const int mid = min(hi, max(lo, n));
        transform_columns<DT, TPH_THREADS>(rowp, lo, mid, [&](int v, float x) { return quick(v, x); });
        transform_columns<DT, TPH_THREADS>(rowp, mid, hi, [&](int v, float) { return quick(v, -MAXT); });
    }
    else {
        transform_columns<DT, TPH_THREADS>(rowp, lo, hi, [&](int v, float x) {
            float y;
            if (v >= n) {
                y = -MAXT;
            }
            else if (fin) {
                y = v == end_id ? MAXT : -MAXT;
            }
            else {
                y = round_t<DT>(x + S::ld(bias[v]));
            }
            return finish(v, y);
        });
    }
    if (!tally) {
        return;
    }
    __syncthreads();
    const size_t base = ((size_t)row * NS + j) * TPB_NB;
    for (int b = t; b < TPB_NB; b += TPH_THREADS) {
        part_cnt[base + b]  = cnt[b];
        part_mass[base + b] = mass[b];
    }
    unsigned long long best = ((unsigned long long)tmax << 32) | (uint32_t)(~(uint32_t)tidx);
    best                    = block_max<unsigned long long, TPH_THREADS / WAVE>(best, red, 0ull);
    if (t == 0) {
        part_best[(size_t)row * NS + j] = best;
    }
}

// The draw of row `b` without consuming it (the pick kernel consumes it).
__device__ __forceinline__ float row_uniform_peek(const RngState* rng, const float* injected, int b)
{
    if (injected != nullptr) {
        return injected[b];
    }
    RngState copy = rng[b];
    return rng_next_uniform(&copy);
}

__global__ void __launch_bounds__(TPC_THREADS)
topp_cut_kernel(int S, const uint32_t* __restrict__ part_cnt, const uint32_t* __restrict__ part_mass,
                const unsigned long long* __restrict__ part_best, uint32_t* __restrict__ start,
                uint32_t* __restrict__ bucket_off, uint32_t* __restrict__ seg_ends, ToppRowMeta* __restrict__ meta,
                const RngState* rng,
                const float* __restrict__ uniforms, float top_p, const float* __restrict__ top_ps,
                const bool* __restrict__ skip_decode)
{
    __shared__ uint32_t           cnt[TPB_NB];
    __shared__ uint32_t           off[TPB_NB];
    __shared__ unsigned long long mass[TPB_NB];
    __shared__ unsigned long long red64[16];
    __shared__ uint32_t           wcnt[TPC_THREADS / WAVE];
    __shared__ unsigned long long wmass[TPC_THREADS / WAVE];
    __shared__ uint32_t           red32[16];
    const int                     row = blockIdx.x;
    const int                     t   = threadIdx.x;
    ToppRowMeta                   m;
    m.best = 0ull;
    m.cut = TPB_NB;
    m.n = m.n_pos = m.nseg = 0;
    m.flags = 0;
    m.best_prob = 0.0f;
    m.mx = m.denom = 0.0f;
    if (skip_decode != nullptr && skip_decode[row]) {
        if (t == 0) {
            m.flags   = TOPP_SKIP;
            meta[row] = m;
        }
        return;
    }
    // sums over the chunks; what the chunks before chunk j hold of a bucket goes to `start` on the way.
    // All loads of one chunk are issued together: the chunks follow each other, not the buckets.
    constexpr int      K    = (TPB_NB + TPC_THREADS - 1) / TPC_THREADS;
    const size_t       base = (size_t)row * S * TPB_NB;
    uint32_t           c[K];
    unsigned long long ms[K];
#pragma unroll
    for (int i = 0; i < K; ++i) {
        c[i]  = 0u;
        ms[i] = 0ull;
    }
    constexpr int J = 8;  // chunks whose loads are in flight together
    for (int j0 = 0; j0 < S; j0 += J) {
        uint32_t pc[J][K], pm[J][K];
#pragma unroll
        for (int jj = 0; jj < J; ++jj) {
#pragma unroll
            for (int i = 0; i < K; ++i) {
                const int  b  = t + i * TPC_THREADS;
                const bool ok = j0 + jj < S && b < TPB_NB;
                pc[jj][i]     = ok ? part_cnt[base + (size_t)(j0 + jj) * TPB_NB + b] : 0u;
                pm[jj][i]     = ok ? part_mass[base + (size_t)(j0 + jj) * TPB_NB + b] : 0u;
            }
        }
#pragma unroll
        for (int jj = 0; jj < J; ++jj) {
#pragma unroll
            for (int i = 0; i < K; ++i) {
                const int b = t + i * TPC_THREADS;
                if (j0 + jj < S && b < TPB_NB) {
                    start[base + (size_t)(j0 + jj) * TPB_NB + b] = c[i];
                }
                c[i] += pc[jj][i];
                ms[i] += pm[jj][i];
            }
        }
    }
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const int b = t + i * TPC_THREADS;
        if (b < TPB_NB) {
            cnt[b]  = c[i];
            mass[b] = ms[i];
        }
    }
    unsigned long long best = 0ull;
    for (int j = t; j < S; j += TPC_THREADS) {
        const unsigned long long v = part_best[(size_t)row * S + j];
        best                       = v > best ? v : best;
    }
    best = block_max<unsigned long long, TPC_THREADS / WAVE>(best, red64, 0ull);  // (also orders the LDS writes above)
    m.best = best;

    const float p         = top_ps != nullptr ? top_ps[row] : top_p;
    const float best_prob = (uint32_t)(best >> 32) == 0u ? __builtin_nanf("") : key_to_float((uint32_t)(best >> 32));
    if (best_prob >= p) {
        // arg-max shortcut of the reference (:842-849): nothing else of the row is needed
        if (t == 0) {
            m.flags   = TOPP_SHORTCUT;
            meta[row] = m;
        }
        return;
    }
    const float              rand_num = row_uniform_peek(rng, uniforms, row) * p;
    // smallest fixed-point mass that certainly covers the draw under the scan's own rounding
    const unsigned long long target = (unsigned long long)((double)rand_num * (1.0 + 1.0 / 1024.0) * 2147483648.0) + 64ull;

    // descending scan over buckets: thread t owns the descending positions [K*t, K*t + K)
    uint32_t           lc = 0;
    unsigned long long lm = 0;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const int d = K * t + i;
        if (d < TPB_NB) {
            lc += cnt[TPB_NB - 1 - d];
            lm += mass[TPB_NB - 1 - d];
        }
    }
    uint32_t           ic = lc;
    unsigned long long im = lm;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const uint32_t           uc = __shfl_up(ic, o, WAVE);
        const unsigned long long um = __shfl_up(im, o, WAVE);
        if (lane_id() >= o) {
            ic += uc;
            im += um;
        }
    }
    if (lane_id() == WAVE - 1) {
        wcnt[wave_id()]  = ic;
        wmass[wave_id()] = im;
    }
    __syncthreads();
    uint32_t           ec = ic - lc;
    unsigned long long em = im - lm;
    uint32_t           total = 0;
    for (int w = 0; w < TPC_THREADS / WAVE; ++w) {
        if (w < wave_id()) {
            ec += wcnt[w];
            em += wmass[w];
        }
        total += wcnt[w];
    }
    uint32_t first = 0xFFFFFFFFu;  // first descending position where the suffix covers the target
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const int d = K * t + i;
        if (d < TPB_NB) {
            const int b = TPB_NB - 1 - d;
            off[b]      = ec;
            ec += cnt[b];
            em += mass[b];
            if (em >= target && first == 0xFFFFFFFFu) {
                first = (uint32_t)d;
            }
        }
    }
    first = block_min<uint32_t, TPC_THREADS / WAVE>(first, red32, 0xFFFFFFFFu);
    const int cut = first == 0xFFFFFFFFu ? 0 : TPB_NB - 1 - (int)first;
    m.cut         = cut;
    m.n_pos       = (int)total;
    m.n           = (int)(off[cut] + cnt[cut]);

    // where the bucket starts in the ordered prefix (the gather adds what earlier chunks hold)
    for (int b = cut + t; b < TPB_NB; b += TPC_THREADS) {
        bucket_off[(size_t)row * TPB_NB + b] = off[b];
    }
    // Segments of whole buckets, in descending order: a bucket closes a segment when a multiple of
    // TPS_SEG lies inside it or at its end, and the last gathered bucket closes the last one. A segment
    // is therefore shorter than TPS_SEG plus its closing bucket. Segment i is [ends[i-1], ends[i]).
    const uint32_t n_gathered = (uint32_t)m.n;
    uint32_t       closes[K];
    uint32_t       lclose = 0;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        const int d = K * t + i;
        closes[i]   = 0u;
        if (d < TPB_NB && TPB_NB - 1 - d >= cut) {
            const int      b = TPB_NB - 1 - d;
            const uint32_t o = off[b];
            const uint32_t e = o + cnt[b];
            if (cnt[b] != 0u && (e / TPS_SEG != o / TPS_SEG || e == n_gathered)) {
                closes[i] = e;
                lclose++;
            }
        }
    }
    uint32_t iclose = lclose;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const uint32_t up = __shfl_up(iclose, o, WAVE);
        if (lane_id() >= o) {
            iclose += up;
        }
    }
    __syncthreads();
    if (lane_id() == WAVE - 1) {
        wcnt[wave_id()] = iclose;
    }
    __syncthreads();
    uint32_t at   = iclose - lclose;
    uint32_t nseg = 0;
    for (int w = 0; w < TPC_THREADS / WAVE; ++w) {
        at += w < wave_id() ? wcnt[w] : 0u;
        nseg += wcnt[w];
    }
    uint32_t* ends = seg_ends + (size_t)row * TPB_NB;
#pragma unroll
    for (int i = 0; i < K; ++i) {
        if (closes[i] != 0u) {
            ends[at++] = closes[i];
        }
    }
    if (t == 0) {
        m.nseg    = (int)nseg;
        meta[row] = m;
    }
}

template<int DT>
__global__ void __launch_bounds__(TPH_THREADS)
topp_gather_kernel(const typename Storage<DT>::T* __restrict__ probs, int vocab, int chunk,
                   const ToppRowMeta* __restrict__ meta, const uint32_t* __restrict__ start,
                   const uint32_t* __restrict__ bucket_off, unsigned long long* __restrict__ sorted)
{
    __shared__ uint32_t cur[TPB_NB];
    const int           row = blockIdx.y;
    const int           j   = blockIdx.x;
    const int           S   = gridDim.x;
    const int           t   = threadIdx.x;
    const ToppRowMeta   m   = meta[row];
    if (m.flags != 0 || m.n == 0) {
        return;
    }
    const size_t base = ((size_t)row * S + j) * TPB_NB;
    for (int b = m.cut + t; b < TPB_NB; b += TPH_THREADS) {
        cur[b] = bucket_off[(size_t)row * TPB_NB + b] + start[base + b];
    }
    __syncthreads();
    const int           lo  = (int)min((long long)vocab, (long long)j * chunk);
    const int           hi  = (int)min((long long)vocab, (long long)lo + chunk);
    const int           cut = m.cut;
    unsigned long long* A   = sorted + (size_t)row * 2 * vocab;
    stream_columns<DT, TPH_THREADS>(probs + (size_t)row * vocab, lo, hi, [&](int v, float x) {
        const uint32_t k = order_key(x);
        if (k > ZERO_KEY) {
            const int b = topp_bucket(k);
            if (b >= cut) {
                const uint32_t slot = atomicAdd(&cur[b], 1u);
                A[slot]             = ((unsigned long long)(~k) << 32) | (uint32_t)v;
            }
        }
    });
}

// ---------------------------------------------------------------------------------------------------------------
// Sampling straight from logits (ftk_fused_topp_sample_step): the probabilities are never written. One 1024-thread
// workgroup per row does what softmax, histogram, cut and gather do above, in three passes over the row:
//   1. the maximum;
//   2. the sum of e = T(exp(y - max)) in the reference's order and, on the way, the histogram - of e, not of the
//      probability e / denominator, which is not known yet. The division is monotone, so buckets of e are ranges of
//      probabilities too; the mass per bucket is kept in units of 2^-31 of e;
//   3. once the denominator is there: the cut in the histogram (the draw scaled by the denominator), then the
//      gather of what lies at or above the cut bucket, each entry with its exact probability T(e / denominator) as
//      the key the segments are sorted by.
// Two things differ from buckets of probabilities. Entries of different buckets can share a probability (numerators
// a few units apart can round to one quotient): sorted segment by segment they may then stand in the wrong order of
// ids across a segment boundary, which the pick kernel puts right for the entry it emits (topp_settle_ties). And an
// e above zero can give a probability of zero: buckets that may hold such entries are never gathered (b0 below);
// a draw that is not crossed above them sends the row to the exact fallback of the pick kernel.
struct ToppRowValues {
    // what the softmax sees of a row: y(v) as softmax_kernel's `masked`, rows without a bias
    float MAXT;
    bool  fin;
    int   end_id, n;
    __device__ __forceinline__ float masked(int v, float x) const
    {
        if (v >= n) {
            return -MAXT;
        }
        if (fin) {
            return v == end_id ? MAXT : -MAXT;
        }
        return x + 0.0f;
    }
};

// the probability the softmax would store for an element with e = T(exp(y - max)), as a float
template<int DT>
__device__ __forceinline__ float topp_prob_of(float e, const RowDivisor& div, float denom)
{
    return round_t<DT>(div.ok ? div.divide(e) : e / denom);
}

constexpr int TPR_BAND = 16;  // numerators this many units of T below 1 may share the arg-max's probability

template<int DT>
__global__ void __launch_bounds__(SM_THREADS)
topp_row_kernel(const typename Storage<DT>::T* __restrict__ logits, const int* __restrict__ end_ids,
                const bool* __restrict__ finished, int n_padded, int n, const bool* __restrict__ skip_decode,
                const RngState* rng, const float* __restrict__ uniforms, float top_p, const float* __restrict__ top_ps,
                uint32_t* __restrict__ seg_ends, ToppRowMeta* __restrict__ meta, unsigned long long* __restrict__ sorted)
{
    typedef Storage<DT>           S;
    constexpr int                 K = (TPB_NB + SM_THREADS - 1) / SM_THREADS;
    __shared__ uint32_t           cnt[TPB_NB];
    __shared__ uint32_t           off[TPB_NB];
    __shared__ unsigned long long mass[TPB_NB];
    __shared__ int                band[TPR_BAND + 1];
    __shared__ float              sh[32];
    __shared__ float              sh_bcast;
    __shared__ uint32_t           wcnt[SM_THREADS / WAVE];
    __shared__ unsigned long long wmass[SM_THREADS / WAVE];
    __shared__ uint32_t           red32[16];
    const int                     row = blockIdx.x;
    const int                     t   = threadIdx.x;
    ToppRowMeta                   m;
    m.best      = 0ull;
    m.cut       = TPB_NB;
    m.n = m.n_pos = m.nseg = 0;
    m.flags     = 0;
    m.best_prob = 0.0f;
    m.mx = m.denom = 0.0f;
    if (skip_decode != nullptr && skip_decode[row]) {
        if (t == 0) {
            m.flags   = TOPP_SKIP;
            meta[row] = m;
        }
        return;
    }
    ToppRowValues vals;
    vals.MAXT   = S::max_t();
    vals.fin    = finished != nullptr ? finished[row] : false;
    vals.end_id = vals.fin ? end_ids[row] : -1;
    vals.n      = n;
    const typename S::T* rowp = logits + (size_t)row * n_padded;
    const float          MAXT = vals.MAXT;

    // ---- 1. the maximum (softmax_kernel's, in any order of the columns)
    float mx = -3.402823466e+38f;
    if (!vals.fin) {
        stream_columns<DT, SM_THREADS>(rowp, 0, n, [&](int, float x) { mx = __builtin_fmaxf(mx, x + 0.0f); });
        if (n_padded > n) {
            mx = __builtin_fmaxf(mx, -MAXT);
        }
    }
    else {
        for (int v = t; v < n_padded; v += SM_THREADS) {
            mx = __builtin_fmaxf(mx, vals.masked(v, 0.0f));
        }
    }
    for (int b = t; b < TPB_NB; b += SM_THREADS) {
        cnt[b] = 0u;
    }
    if (t <= TPR_BAND) {
        band[t] = 0x7FFFFFFF;
    }
    mx = block_max<float, SM_THREADS / WAVE>(mx, sh, -3.402823466e+38f);  // (two barriers: the histogram is clear)

    // ---- 2. the sum in the reference's order, the histogram of e on the way
    constexpr uint32_t ONE_BITS  = 0x3F800000u;
    constexpr int      UNIT_LOG2 = DT == DT_F32 ? 0 : DT == DT_F16 ? 13 : 16;  // a unit of T in fp32 mantissa bits
    // (Only the entries are counted: a bucket's mass is taken as at least its count times its lower edge, which is
    // within 1/64 of the truth and costs no second atomic per element.)
    constexpr uint32_t BAND_LOW = (ONE_BITS - ((uint32_t)TPR_BAND << UNIT_LOG2)) | 0x80000000u;
    auto tally = [&](int v, float e) {
        const uint32_t k = order_key_nonneg(e);
        if (k > ZERO_KEY) {
            atomicAdd(&cnt[topp_bucket(k)], 1u);
            if (k >= BAND_LOW) {  // within a few units of 1: rare
                const uint32_t bits = k & 0x7FFFFFFFu;
                if (bits <= ONE_BITS) {
                    atomicMin(&band[(ONE_BITS - bits) >> UNIT_LOG2], v);
                }
            }
        }
    };
    const float pad_e = round_t<DT>(det_expf_nonpos(-MAXT - mx));
    float       sum   = 0.0f;
    if (!vals.fin) {
        // batches of U columns per thread, the next batch's loads issued before the current one is used (every load is
        // issued whatever the batch, one past the last fetches the last again, unused: with the same number of loads
        // on every path the waits can name the older batch instead of everything in flight)
        constexpr int        U     = 8;
        const int            nfull = n / (U * SM_THREADS);  // batches that every thread holds in full
        typename S::T        buf[2][U];
        auto                 load  = [&](typename S::T* raw, int b) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                raw[u] = rowp[(b * U + u) * SM_THREADS + t];
            }
        };
        auto batch = [&](const typename S::T* raw, int b) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const float e = round_t<DT>(det_expf_nonpos((S::ld(raw[u]) + 0.0f) - mx));
                sum += e;
                tally((b * U + u) * SM_THREADS + t, e);
            }
        };
        if (nfull > 0) {
            load(buf[0], 0);
        }
        for (int b = 0; b < nfull; b += 2) {
            load(buf[1], min(b + 1, nfull - 1));
            batch(buf[0], b);
            load(buf[0], min(b + 2, nfull - 1));
            if (b + 1 < nfull) {
                batch(buf[1], b + 1);
            }
        }
        int v = nfull * U * SM_THREADS + t;
        for (; v < n; v += SM_THREADS) {
            const float e = round_t<DT>(det_expf_nonpos((S::ld(rowp[v]) + 0.0f) - mx));
            sum += e;
            tally(v, e);
        }
        for (; v < n_padded; v += SM_THREADS) {
            sum += pad_e;
            tally(v, pad_e);
        }
    }
    else {
        for (int v = t; v < n_padded; v += SM_THREADS) {
            const float e = round_t<DT>(det_expf_nonpos(vals.masked(v, 0.0f) - mx));
            sum += e;
            tally(v, e);
        }
    }
#pragma unroll
    for (int mm = 16; mm > 0; mm >>= 1) {
        sum += __shfl_xor(sum, mm, 32);
    }
    if ((t & 31) == 0) {
        sh[t >> 5] = sum;
    }
    __syncthreads();
    if (t < 32) {
        float v = sh[t];
#pragma unroll
        for (int mm = 16; mm > 0; mm >>= 1) {
            v += __shfl_xor(v, mm, 32);
        }
        if (t == 0) {
            sh_bcast = v;
        }
    }
    __syncthreads();
    const float      denom = sh_bcast + 1e-6f;
    const RowDivisor div(denom);
    m.mx    = mx;
    m.denom = denom;
    if (!(denom == denom)) {
        // a NaN among the logits: every probability is a NaN, none is positive, nothing is gathered
        if (t == 0) {
            meta[row] = m;
        }
        return;
    }

    // ---- the arg-max: the lowest id among the entries that share the largest probability. The largest e is 1
    // (the maximum's own); numerators a few units below 1 may round to the same quotient.
    {
        const float p_one = topp_prob_of<DT>(1.0f, div, denom);
        int         best  = 0x7FFFFFFF;
        for (int j = 0; j <= TPR_BAND; ++j) {
            const float e_j = u2f(ONE_BITS - ((uint32_t)j << UNIT_LOG2));
            if (topp_prob_of<DT>(e_j, div, denom) == p_one) {
                best = min(best, band[j]);
            }
        }
        if (best != 0x7FFFFFFF) {
            m.best      = ((unsigned long long)order_key(p_one) << 32) | (uint32_t)(~(uint32_t)best);
            m.best_prob = p_one;
        }
    }
    const float p = top_ps != nullptr ? top_ps[row] : top_p;
    if ((uint32_t)(m.best >> 32) != 0u && round_t<DT>(0.0f + m.best_prob) >= p) {
        // arg-max shortcut of the reference (:842-849): nothing else of the row is needed
        if (t == 0) {
            m.flags   = TOPP_SHORTCUT;
            meta[row] = m;
        }
        return;
    }
    const float rand_num = row_uniform_peek(rng, uniforms, row) * p;

    // ---- 3a. the cut. Buckets up to b0 may hold numerators whose probability rounds to zero: never gathered.
    uint32_t total = 0;
    {
        const float tiny   = DT == DT_F32 ? 1.0e-44f : DT == DT_F16 ? 1.2e-7f : 2.0e-40f;  // above two units of T at zero
        const float e_zero = tiny * denom * 1.001f;
        const int   b0     = topp_bucket(order_key_nonneg(__builtin_fminf(e_zero, 2.0f)));
        // smallest mass (units of 2^-31 of e) that certainly covers the draw: the scan's own rounding, the rounding
        // of every quotient to T (relative, and absolute where the probabilities are subnormal in T)
        uint32_t lc = 0;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const int d = K * t + i;
            if (d < TPB_NB) {
                lc += cnt[TPB_NB - 1 - d];
            }
        }
        // a bucket's mass in units of 2^-31 of e: at least its count times its lower edge (the lowest bucket holds
        // everything under 2^-32 and counts for nothing, the highest one only values above 1, of which there are none)
        auto mass_of = [&](int b) -> unsigned long long {
            if (b <= 0 || b >= TPB_NB - 1) {
                return 0ull;
            }
            const float edge_b = u2f((uint32_t)(b + (TPB_ONE - TPB_SPAN)) << TPB_SHIFT);
            return (unsigned long long)cnt[b] * (unsigned long long)(edge_b * 2147483648.0f);
        };
        unsigned long long lm = 0;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const int d = K * t + i;
            if (d < TPB_NB) {
                mass[TPB_NB - 1 - d] = mass_of(TPB_NB - 1 - d);
                lm += mass[TPB_NB - 1 - d];
            }
        }
        uint32_t           ic = lc;
        unsigned long long im = lm;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            const uint32_t           uc = __shfl_up(ic, o, WAVE);
            const unsigned long long um = __shfl_up(im, o, WAVE);
            if (lane_id() >= o) {
                ic += uc;
                im += um;
            }
        }
        if (lane_id() == WAVE - 1) {
            wcnt[wave_id()]  = ic;
            wmass[wave_id()] = im;
        }
        __syncthreads();
        uint32_t           ec = ic - lc;
        unsigned long long em = im - lm;
        for (int w = 0; w < SM_THREADS / WAVE; ++w) {
            if (w < wave_id()) {
                ec += wcnt[w];
                em += wmass[w];
            }
            total += wcnt[w];
        }
        const double half_unit = DT == DT_F32 ? 0.0 : DT == DT_F16 ? 2.98023223876953125e-08 : 4.6e-41;
        const double slack     = DT == DT_BF16 ? 1.0 / 100.0 : 1.0 / 512.0;  // (half a unit of bfloat16 is 2^-9)
        const double want      = ((double)rand_num * (1.0 + slack) + (double)total * half_unit) * (double)denom;
        const unsigned long long target = (unsigned long long)(want * 2147483648.0) + 64ull;
        uint32_t first = 0xFFFFFFFFu;  // first descending position where the suffix covers the target
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const int d = K * t + i;
            if (d < TPB_NB) {
                const int b = TPB_NB - 1 - d;
                off[b]      = ec;
                ec += cnt[b];
                em += mass[b];
                if (em >= target && first == 0xFFFFFFFFu) {
                    first = (uint32_t)d;
                }
            }
        }
        first = block_min<uint32_t, SM_THREADS / WAVE>(first, red32, 0xFFFFFFFFu);
        int cut = first == 0xFFFFFFFFu ? 0 : TPB_NB - 1 - (int)first;
        cut     = max(cut, b0 + 1);
        cut     = min(cut, TPB_NB - 1);
        // Entries that share a probability are ordered by id in the reference, whatever their e: the prefix must
        // hold all of them or none. The cut moves down while the two values of T either side of its lower edge give
        // the same probability (equal probabilities have numerators within a few units of T: a few buckets at most).
        bool splits = false;
        for (int guard = 0; guard < 64; ++guard) {
            if (cut >= TPB_NB - 1) {
                break;
            }
            const float edge_at = u2f((uint32_t)(cut + (TPB_ONE - TPB_SPAN)) << TPB_SHIFT);
            float       above, under;  // the smallest value of T at or above the edge, the largest below it
            if constexpr (DT == DT_F32) {
                above = edge_at;
                under = u2f(f2u(edge_at) - 1u);
            }
            else {
                const typename S::T r = S::st(edge_at);
                const bool          up = S::ld(r) >= edge_at;
                above                  = up ? S::ld(r) : S::ld((typename S::T)(r + 1));
                under                  = up ? S::ld((typename S::T)(r - 1)) : S::ld(r);
            }
            splits = topp_prob_of<DT>(above, div, denom) == topp_prob_of<DT>(under, div, denom);
            if (!splits || cut <= b0 + 1) {
                break;
            }
            cut--;
        }
        m.cut   = cut;
        m.n     = (int)(off[cut] + cnt[cut]);
        // every positive entry is in the prefix exactly when nothing lies below the cut (then none of them is one
        // of the numerators whose probability may be zero)
        m.n_pos = (uint32_t)m.n == total ? (int)total : 0x7FFFFFFF;
        if (splits && (uint32_t)m.n != total) {
            // (the lowest bucket that may be gathered still shares a probability with what lies below it: the
            // exact fallback of the pick kernel orders the whole row)
            m.n     = 0;
            m.n_pos = 0x7FFFFFFF;
        }
    }
    const int cut = m.cut;

    // segments of whole buckets, as topp_cut_kernel makes them
    {
        const uint32_t n_gathered = (uint32_t)m.n;
        uint32_t       closes[K];
        uint32_t       lclose = 0;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            const int d = K * t + i;
            closes[i]   = 0u;
            if (d < TPB_NB && TPB_NB - 1 - d >= cut) {
                const int      b = TPB_NB - 1 - d;
                const uint32_t o = off[b];
                const uint32_t e = o + cnt[b];
                if (cnt[b] != 0u && (e / TPS_SEG != o / TPS_SEG || e == n_gathered)) {
                    closes[i] = e;
                    lclose++;
                }
            }
        }
        uint32_t iclose = lclose;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            const uint32_t up = __shfl_up(iclose, o, WAVE);
            if (lane_id() >= o) {
                iclose += up;
            }
        }
        __syncthreads();
        if (lane_id() == WAVE - 1) {
            wcnt[wave_id()] = iclose;
        }
        __syncthreads();
        uint32_t at   = iclose - lclose;
        uint32_t nseg = 0;
        for (int w = 0; w < SM_THREADS / WAVE; ++w) {
            at += w < wave_id() ? wcnt[w] : 0u;
            nseg += wcnt[w];
        }
        uint32_t* ends = seg_ends + (size_t)row * TPB_NB;
#pragma unroll
        for (int i = 0; i < K; ++i) {
            if (closes[i] != 0u) {
                ends[at++] = closes[i];
            }
        }
        m.nseg = m.n == 0 ? 0 : (int)nseg;  // (a row sent to the fallback has nothing to sort here)
    }
    if (t == 0) {
        meta[row] = m;
    }
    if (m.n == 0) {
        return;
    }

    // ---- 3b. the gather: every bucket's cursor starts at the bucket's place in the prefix
    __syncthreads();
    for (int b = t; b < TPB_NB; b += SM_THREADS) {
        cnt[b] = off[b];
    }
    __syncthreads();
    unsigned long long* A = sorted + (size_t)row * 2 * n_padded;
    // Nothing whose y lies under this can reach the cut bucket: the y of half the bucket's lower edge, less a margin.
    // (An exponential under half the edge stays under the edge when it is rounded to T, also where T is subnormal:
    // the edge is at least two units of T there, see b0. The margin covers the errors of exponential and logarithm
    // many times over.)
    const float edge  = u2f((uint32_t)(cut + (TPB_ONE - TPB_SPAN)) << TPB_SHIFT);
    const float y_cut = cut >= TPB_NB - 1 ? -3.402823466e+38f :
                                            (mx + det_logf(edge)) - (0.75f + 1e-6f * __builtin_fabsf(mx));
    auto place = [&](int v, float y) {
        if (y < y_cut) {
            return;
        }
        const float    e = round_t<DT>(det_expf_nonpos(y - mx));
        const uint32_t k = order_key_nonneg(e);
        if (k > ZERO_KEY) {
            const int b = topp_bucket(k);
            if (b >= cut) {
                const uint32_t kp   = order_key(topp_prob_of<DT>(e, div, denom));
                const uint32_t slot = atomicAdd(&cnt[b], 1u);
                A[slot]             = ((unsigned long long)(~kp) << 32) | (uint32_t)v;
            }
        }
    };
    if (!vals.fin) {
        stream_columns<DT, SM_THREADS>(rowp, 0, n, [&](int v, float x) { place(v, x + 0.0f); });
        for (int v = n + t; v < n_padded; v += SM_THREADS) {
            place(v, -MAXT);
        }
    }
    else {
        for (int v = t; v < n_padded; v += SM_THREADS) {
            place(v, vals.masked(v, 0.0f));
        }
    }
}

// Scratch of the radix sort below.
struct RadixScratch {
    unsigned short*     cnt16;  // [16][TP_THREADS]
    int*                wtot;   // [256]
    unsigned long long* red64;  // [16]
};

// Stable LSD radix sort (4-bit digits over bits [lowbit, 64)) of n 64-bit entries in memory by a
// TP_THREADS workgroup; digits that are constant over the range are skipped. Thread t owns the
// contiguous slice [t*chunk, (t+1)*chunk), n <= 65535 * TP_THREADS. Returns where the result is
// (a or b).
__device__ unsigned long long* radix_sort_range(unsigned long long* a, unsigned long long* b, int n, int lowbit,
                                                RadixScratch rs)
{
    const int t     = threadIdx.x;
    const int chunk = (n + TP_THREADS - 1) / TP_THREADS;
    const int lo    = min(n, t * chunk);
    const int hi    = min(n, lo + chunk);
    unsigned long long vor = 0ull, vand = ~0ull;
    for (int i = lo; i < hi; ++i) {
        vor |= a[i];
        vand &= a[i];
    }
    for (int o = 32; o > 0; o >>= 1) {
        vor |= __shfl_xor(vor, o, WAVE);
        vand &= __shfl_xor(vand, o, WAVE);
    }
    __syncthreads();
    if (lane_id() == 0) {
        rs.red64[wave_id()] = vor;
    }
    __syncthreads();
    unsigned long long all_or = 0ull;
    for (int w = 0; w < TP_THREADS / WAVE; ++w) {
        all_or |= rs.red64[w];
    }
    __syncthreads();
    if (lane_id() == 0) {
        rs.red64[wave_id()] = vand;
    }
    __syncthreads();
    unsigned long long all_and = ~0ull;
    for (int w = 0; w < TP_THREADS / WAVE; ++w) {
        all_and &= rs.red64[w];
    }
    __syncthreads();
    const unsigned long long diff = all_or ^ all_and;

    unsigned long long* src = a;
    unsigned long long* dst = b;
    for (int shift = lowbit; shift < 64; shift += 4) {
        if (((diff >> shift) & 0xFull) == 0ull) {
            continue;
        }
        // 1. private digit counts
        for (int d = 0; d < 16; ++d) {
            rs.cnt16[d * TP_THREADS + t] = 0;
        }
        for (int i = lo; i < hi; ++i) {
            const int d = (int)((src[i] >> shift) & 0xFull);
            rs.cnt16[d * TP_THREADS + t]++;
        }
        // 2. exclusive prefix over (digit major, thread minor)
        int base_off[16];
#pragma unroll
        for (int d = 0; d < 16; ++d) {
            const int val = rs.cnt16[d * TP_THREADS + t];
            int       inc = val;
#pragma unroll
            for (int o = 1; o < WAVE; o <<= 1) {
                const int up = __shfl_up(inc, o, WAVE);
                if (lane_id() >= o) {
                    inc += up;
                }
            }
            base_off[d] = inc - val;
            if (lane_id() == WAVE - 1) {
                rs.wtot[d * 16 + wave_id()] = inc;
            }
        }
        __syncthreads();
        {
            int digit_base = 0;
#pragma unroll
            for (int d = 0; d < 16; ++d) {
                int pre = 0, tot = 0;
                for (int w = 0; w < TP_THREADS / WAVE; ++w) {
                    const int x = rs.wtot[d * 16 + w];
                    pre += w < wave_id() ? x : 0;
                    tot += x;
                }
                base_off[d] += digit_base + pre;
                digit_base += tot;
            }
        }
        __syncthreads();
        // 3. stable scatter
        for (int i = lo; i < hi; ++i) {
            const unsigned long long e = src[i];
            const int                d = (int)((e >> shift) & 0xFull);
            int                      pos = 0;
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                if (q == d) {
                    pos = base_off[q]++;
                }
            }
            dst[pos] = e;
        }
        __threadfence_block();
        __syncthreads();
        unsigned long long* tmp = src;
        src                     = dst;
        dst                     = tmp;
    }
    return src;
}

// Ascending bitonic sort of 64 * R 64-bit keys held R per lane by one wave; key r of lane l has the
// position r * 64 + l. Exchanges inside a register go through lane shuffles, the others stay in the
// lane.
template<int R>
__device__ __forceinline__ void wave_sort_u64(unsigned long long (&v)[R])
{
    const int lane = lane_id();
#pragma unroll
    for (int k = 2; k <= 64 * R; k <<= 1) {
#pragma unroll
        for (int j = k >> 1; j > 0; j >>= 1) {
            if (j < 64) {
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    const int                idx   = r * 64 + lane;
                    const unsigned long long other = __shfl_xor(v[r], j, WAVE);
                    const bool               up    = (idx & k) == 0;
                    const bool               lower = (idx & j) == 0;
                    const bool               less  = other < v[r];
                    // the lower position keeps the smaller key in ascending runs
                    v[r] = ((lower == up) == less) ? other : v[r];
                }
            }
            else {
                const int jj = j >> 6;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if ((r & jj) == 0) {
                        const bool               up = ((r * 64) & k) == 0;
                        const unsigned long long a  = v[r];
                        const unsigned long long b  = v[r | jj];
                        const bool               sw = (a > b) == up;
                        v[r]                        = sw ? b : a;
                        v[r | jj]                   = sw ? a : b;
                    }
                }
            }
        }
    }
}

// One wave sorts buf[s0, s0 + len), len <= 64 * R, and writes the result to out[s0, ...).
template<int R>
__device__ __forceinline__ void wave_sort_group(const unsigned long long* buf, unsigned long long* out, int s0, int len)
{
    const int          lane = lane_id();
    unsigned long long v[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int i = r * 64 + lane;
        v[r]        = i < len ? buf[s0 + i] : ~0ull;
    }
    wave_sort_u64<R>(v);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int i = r * 64 + lane;
        if (i < len) {
            out[s0 + i] = v[r];
        }
    }
}

constexpr int TPS_DIGITS = 1024;  // bins of the partition inside a segment
constexpr int TPS_GROUP  = 48;    // group boundaries follow multiples of this
constexpr int TPS_EPT    = (TPS_CAP + TP_THREADS - 1) / TP_THREADS;

// The radix path needs 32 KB of digit counters; its small arrays live behind them in the same buffer.
struct ToppSortShared {
    unsigned long long buf[TPS_CAP];
    uint32_t           hist[TPS_DIGITS];  // entries per bin, then the write cursors
    uint32_t           base[TPS_DIGITS];  // first position of a bin
    uint32_t           gend[TPS_DIGITS];  // end of every group of bins
    uint32_t           psum[TP_THREADS];  // running number of segments over a tile of rows
    uint32_t           wtot[TP_THREADS / WAVE];
    uint32_t           red32[16];
    int                big[64];           // groups left to the whole workgroup
    int                nbig;
};
static_assert(sizeof(ToppSortShared) <= 65536, "static LDS");

// Inclusive scan of one value per thread over the TP_THREADS threads; `total` gets the sum. Two barriers.
__device__ __forceinline__ uint32_t block_scan_incl(uint32_t v, uint32_t* wtot, uint32_t& total)
{
    uint32_t inc = v;
#pragma unroll
    for (int o = 1; o < WAVE; o <<= 1) {
        const uint32_t up = __shfl_up(inc, o, WAVE);
        if (lane_id() >= o) {
            inc += up;
        }
    }
    __syncthreads();
    if (lane_id() == WAVE - 1) {
        wtot[wave_id()] = inc;
    }
    __syncthreads();
    total = 0;
    for (int w = 0; w < TP_THREADS / WAVE; ++w) {
        const uint32_t x = wtot[w];
        inc += w < wave_id() ? x : 0u;
        total += x;
    }
    return inc;
}

// Sorts seg[0, n) ascending (descending probability, ascending id among equals), n <= TPS_CAP: the keys
// are spread over TPS_DIGITS bins of equal width between the smallest and the largest, neighbouring
// bins are joined into groups of about TPS_GROUP entries, and every group is sorted by one wave in
// registers. A group too long for that (equal keys land in one bin) is left to the whole workgroup.
__device__ void sort_segment(ToppSortShared& s, unsigned long long* __restrict__ seg, int n)
{
    const int          t = threadIdx.x;
    unsigned long long e[TPS_EPT];
    uint32_t           kmin = 0xFFFFFFFFu, kmax = 0u;
#pragma unroll
    for (int r = 0; r < TPS_EPT; ++r) {
        const int i = t + r * TP_THREADS;
        if (i < n) {
            e[r]             = seg[i];
            const uint32_t h = (uint32_t)(e[r] >> 32);
            kmin             = min(kmin, h);
            kmax             = max(kmax, h);
        }
    }
    s.hist[t] = 0u;  // TPS_DIGITS == TP_THREADS
    if (t == 0) {
        s.nbig = 0;
    }
    kmin = block_min<uint32_t, TP_THREADS / WAVE>(kmin, s.red32, 0xFFFFFFFFu);
    kmax = block_max<uint32_t, TP_THREADS / WAVE>(kmax, s.red32, 0u);
    const uint32_t range = kmax - kmin;
    const int      nbits = range == 0u ? 0 : 32 - __clz(range);
    const int      shift = nbits > 10 ? nbits - 10 : 0;
#pragma unroll
    for (int r = 0; r < TPS_EPT; ++r) {
        if (t + r * TP_THREADS < n) {
            atomicAdd(&s.hist[((uint32_t)(e[r] >> 32) - kmin) >> shift], 1u);
        }
    }
    __syncthreads();
    const uint32_t cnt = s.hist[t];
    uint32_t       total;
    const uint32_t en = block_scan_incl(cnt, s.wtot, total);
    const uint32_t o  = en - cnt;
    s.base[t]         = o;
    s.hist[t]         = 0u;
    const bool     closes = cnt != 0u && (en / TPS_GROUP != o / TPS_GROUP || en == (uint32_t)n);
    uint32_t       ngroups;
    const uint32_t gi = block_scan_incl(closes ? 1u : 0u, s.wtot, ngroups);
    if (closes) {
        s.gend[gi - 1] = en;
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < TPS_EPT; ++r) {
        if (t + r * TP_THREADS < n) {
            const uint32_t d   = ((uint32_t)(e[r] >> 32) - kmin) >> shift;
            const uint32_t pos = s.base[d] + atomicAdd(&s.hist[d], 1u);
            s.buf[pos]         = e[r];
        }
    }
    __syncthreads();
    for (int g = wave_id(); g < (int)ngroups; g += TP_THREADS / WAVE) {
        const int s0  = g > 0 ? (int)s.gend[g - 1] : 0;
        const int len = (int)s.gend[g] - s0;
        if (len <= 64) {
            wave_sort_group<1>(s.buf, seg, s0, len);
        }
        else if (len <= 128) {
            wave_sort_group<2>(s.buf, seg, s0, len);
        }
        else if (len <= 256) {
            wave_sort_group<4>(s.buf, seg, s0, len);
        }
        else if (lane_id() == 0) {
            const int slot = atomicAdd(&s.nbig, 1);
            if (slot < 64) {
                s.big[slot] = g;
            }
        }
    }
    __syncthreads();
    const int nbig = s.nbig;
    if (nbig > 64) {
        // cannot happen with more than 256 entries per long group and n <= TPS_CAP; sort everything
        block_sort_u64<TP_THREADS>(s.buf, n);
        for (int i = t; i < n; i += TP_THREADS) {
            seg[i] = s.buf[i];
        }
    }
    else {
        for (int q = 0; q < nbig; ++q) {
            const int g   = s.big[q];
            const int s0  = g > 0 ? (int)s.gend[g - 1] : 0;
            const int len = (int)s.gend[g] - s0;
            block_sort_u64<TP_THREADS>(s.buf + s0, len);
            for (int i = t; i < len; i += TP_THREADS) {
                seg[s0 + i] = s.buf[s0 + i];
            }
        }
    }
    __syncthreads();
}

// Every workgroup takes the segments whose running number over all rows is its own modulo the grid.
__global__ void __launch_bounds__(TP_THREADS)
topp_sort_kernel(unsigned long long* __restrict__ sorted, const uint32_t* __restrict__ seg_ends,
                 const ToppRowMeta* __restrict__ meta, int vocab, int rows)
{
    __shared__ ToppSortShared s;
    const int                 t     = threadIdx.x;
    const uint32_t            G     = gridDim.x;
    uint32_t                  first = 0;  // running number of the first segment of the tile
    for (int rb = 0; rb < rows; rb += TP_THREADS) {
        const int row = rb + t;
        uint32_t  my  = 0;
        if (row < rows && meta[row].flags == 0) {
            my = (uint32_t)meta[row].nseg;
        }
        uint32_t       tile_total;
        const uint32_t incl = block_scan_incl(my, s.wtot, tile_total);
        s.psum[t]           = incl;
        __syncthreads();
        uint32_t w = first + (blockIdx.x + G - first % G) % G;
        for (; w < first + tile_total; w += G) {
            const uint32_t local = w - first;
            int            lo = 0, hi = TP_THREADS - 1;
            while (lo < hi) {
                const int mid = (lo + hi) >> 1;
                if (s.psum[mid] > local) {
                    hi = mid;
                }
                else {
                    lo = mid + 1;
                }
            }
            const int       r    = rb + lo;
            const int       i    = (int)(local - (lo > 0 ? s.psum[lo - 1] : 0u));
            const uint32_t* ends = seg_ends + (size_t)r * TPB_NB;
            const uint32_t  s0   = i > 0 ? ends[i - 1] : 0u;
            const int       n    = (int)(ends[i] - s0);
            unsigned long long* A   = sorted + (size_t)r * 2 * vocab;
            unsigned long long* seg = A + s0;
            if (n < 2) {
                continue;
            }
            if (n <= 256) {
                // one wave, straight from memory (most rows only order a few dozen entries)
                if (wave_id() == 0) {
                    if (n <= 64) {
                        wave_sort_group<1>(seg, seg, 0, n);
                    }
                    else {
                        wave_sort_group<4>(seg, seg, 0, n);
                    }
                }
            }
            else if (n <= TPS_CAP) {
                sort_segment(s, seg, n);
            }
            else {
                RadixScratch        rs{reinterpret_cast<unsigned short*>(s.buf), reinterpret_cast<int*>(s.buf + 4096),
                                reinterpret_cast<unsigned long long*>(s.buf + 4096 + 128)};
                unsigned long long* res = radix_sort_range(seg, A + vocab + s0, n, 0, rs);
                if (res != seg) {
                    for (int q = t; q < n; q += TP_THREADS) {
                        seg[q] = res[q];
                    }
                }
                __threadfence_block();
                __syncthreads();
            }
        }
        first += tile_total;
        __syncthreads();
    }
}

struct TopPShared {
    unsigned long long buf[4096];  // digit counters of the fallback sort
    unsigned long long red64[16];
    uint32_t           red32[16];
    float              agg[TP_ROUND];
    float              carry[TP_ROUND + 1];
    uint32_t           tilemask[32][8];
    int                wtot[256];
    int                misc[8];
    float              fmisc[4];
};

// One 32-lane group loads the eight items of each of its lanes from tile `tile` of the ordered
// array (entries at or beyond n count as 0).
__device__ __forceinline__ void tile_load(const unsigned long long* __restrict__ src, int n, int tile, int l, float x[8])
{
    const int i0 = tile * TP_TILE + l * 8;
    if (i0 + 8 <= n && ((uintptr_t)src & 15u) == 0u) {
        const ulonglong2* v = reinterpret_cast<const ulonglong2*>(src + i0);  // i0 is a multiple of 8
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const ulonglong2 p = v[j];
            x[2 * j]           = key64_prob(p.x);
            x[2 * j + 1]       = key64_prob(p.y);
        }
    }
    else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            x[j] = i0 + j < n ? key64_prob(src[i0 + j]) : 0.0f;
        }
    }
}

// Inclusive raking scan of the lane totals of a tile.
__device__ __forceinline__ float tile_scan(const float x[8], int l)
{
    float seg = x[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) {
        seg = seg + x[j];
    }
    float incl = seg;
#pragma unroll
    for (int d = 1; d < 32; d <<= 1) {
        const float up = __shfl_up(incl, d, 32);
        if (l >= d) {
            incl = up + incl;
        }
    }
    return incl;
}

// Replays the reference scan over the ordered array `src[0, n)`. Returns the position the
// reference would pick (it can lie in the zero padding of the last tile, >= n) or -1 when the draw
// is never reached. All threads must call; the result is block-uniform.
__device__ int scan_sorted(TopPShared& s, const unsigned long long* __restrict__ src, int n, float rand_num)
{
    const int t     = threadIdx.x;
    const int group = t >> 5;
    const int l     = t & 31;
    const int nt    = (n + TP_TILE - 1) / TP_TILE;
    // a tile whose running total stays below this cannot hold the crossing: the prefixes inside a
    // tile and the tile's total differ by rounding only
    const float near = rand_num * (1.0f - 1.0f / 4096.0f);
    float       carry_in = 0.0f;
    for (int base = 0; base < nt; base += TP_ROUND) {
        const int ntr = min(TP_ROUND, nt - base);
        constexpr int NG = TP_THREADS / 32;
        constexpr int Q  = 8;  // tiles in flight per lane group
        for (int g = group; g < ntr; g += Q * NG) {
            float x[Q][8];
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                if (g + q * NG < ntr) {
                    tile_load(src, n, base + g + q * NG, l, x[q]);
                }
            }
#pragma unroll
            for (int q = 0; q < Q; ++q) {
                if (g + q * NG < ntr) {
                    const float incl = tile_scan(x[q], l);
                    if (l == 31) {
                        s.agg[g + q * NG] = incl;
                    }
                }
            }
        }
        __syncthreads();
        if (t == 0) {
            // the additions depend on each other, the loads do not: eight totals are fetched at a time
            float c  = carry_in;
            int   g0 = -1;
            for (int g = 0; g < ntr; g += 8) {
                float a[8];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    a[j] = s.agg[g + j];  // TP_ROUND is a multiple of 8; entries from ntr on are not used
                }
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    if (g + j < ntr) {
                        s.carry[g + j] = c;
                        c              = c + a[j];
                        if (g0 < 0 && c >= near) {
                            g0 = g + j;
                        }
                    }
                }
            }
            s.carry[ntr] = c;
            s.misc[1]    = g0;
        }
        __syncthreads();
        const int g0 = s.misc[1];
        if (g0 >= 0) {
            for (int gs = g0; gs < ntr; gs += TP_THREADS / 32) {
                const int g  = gs + group;
                uint32_t  m8 = 0;
                if (g < ntr) {
                    float x[8];
                    tile_load(src, n, base + g, l, x);
                    const float incl   = tile_scan(x, l);
                    const float excl   = __shfl_up(incl, 1, 32);
                    const float prefix = s.carry[g];
                    float       a      = l == 0 ? prefix : prefix + excl;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        a = a + x[j];
                        if (rand_num <= a) {
                            m8 |= 1u << j;
                        }
                    }
                }
                reinterpret_cast<unsigned char*>(&s.tilemask[group][0])[l] = (unsigned char)m8;
                __syncthreads();
                if (t == 0) {
                    int found = -1;
                    for (int q = 0; q < TP_THREADS / 32 && found < 0; ++q) {
                        for (int w = 0; w < 8; ++w) {
                            const uint32_t mk = s.tilemask[q][w];
                            if (mk != 0u) {
                                found = (base + gs + q) * TP_TILE + w * 32 + (32 - __popc(mk));
                                break;
                            }
                        }
                    }
                    s.misc[0] = found;
                }
                __syncthreads();
                const int found = s.misc[0];
                __syncthreads();
                if (found >= 0) {
                    return found;
                }
            }
        }
        carry_in = s.carry[ntr];
        __syncthreads();
    }
    return -1;
}

// id of the `nth` (0-based) entry with probability exactly zero, in ascending id order: what a
// stable descending sort leaves behind the positive entries. Single thread; reached only when a
// draw lands within rounding distance of the total mass.
// the id of the nth entry (in id order) whose probability is not positive; prob(v) gives the probability of column v
template<class P>
__device__ int nth_zero_entry(P&& prob, int vocab, int nth)
{
    int seen = 0, last = vocab - 1;
    for (int v = 0; v < vocab; ++v) {
        if (order_key(prob(v)) <= ZERO_KEY) {
            last = v;
            if (seen == nth) {
                return v;
            }
            seen++;
        }
    }
    return last;
}

// Rows sampled straight from logits: the segments of the ordered prefix are ranges of e, not of the probability,
// and entries of neighbouring segments can share a probability. Within a segment equal probabilities stand in
// ascending order of id, as in the reference's stable sort of the whole row; across a boundary they may not. The
// walk's sums do not depend on the order of equal values, only the emitted id does: the reference emits, of the
// entries that share the probability at position `found`, the one with as many smaller ids as there are entries of
// the run in front of `found`. Called by every thread of the workgroup; every thread gets the entry to emit.
__device__ unsigned long long topp_settle_ties(TopPShared& s, const unsigned long long* __restrict__ A, int n, int found,
                                               const uint32_t* __restrict__ ends, int nseg, int vocab)
{
    const int t = threadIdx.x;
    if (t == 0) {
        const unsigned long long here = A[found];
        const uint32_t           key  = (uint32_t)(here >> 32);
        // The prefix is in ascending order of this word as a whole (the division keeps the order of the segments).
        // Runs are short as a rule, and every probe is a dependent load: both ends are looked for outwards from
        // `found` in doubling steps, then by bisection inside the last step.
        auto high = [&](int i) { return (uint32_t)(A[i] >> 32); };
        int  hi = found, lo = 0;  // first position of the run: in [lo, hi], A[hi] belongs to it
        for (int step = 1;; step <<= 1) {
            const int probe = hi - step;
            if (probe < 0) {
                lo = 0;
                break;
            }
            if (high(probe) == key) {
                hi = probe;
            }
            else {
                lo = probe + 1;
                break;
            }
        }
        while (lo < hi) {
            const int mid = (lo + hi) >> 1;
            if (high(mid) < key) {
                lo = mid + 1;
            }
            else {
                hi = mid;
            }
        }
        const int a = lo;
        lo = found;
        hi = n - 1;  // last position of the run: in [lo, hi], A[lo] belongs to it
        for (int step = 1;; step <<= 1) {
            const int probe = lo + step;
            if (probe > n - 1) {
                hi = n - 1;
                break;
            }
            if (high(probe) == key) {
                lo = probe;
            }
            else {
                hi = probe - 1;
                break;
            }
        }
        while (lo < hi) {
            const int mid = (lo + hi + 1) >> 1;
            if (high(mid) > key) {
                hi = mid - 1;
            }
            else {
                lo = mid;
            }
        }
        const int b = lo;
        // does a segment end inside (a, b]?
        int slo = 0, shi = nseg - 1;
        while (slo < shi) {
            const int mid = (slo + shi) >> 1;
            if ((int)ends[mid] > a) {
                shi = mid;
            }
            else {
                slo = mid + 1;
            }
        }
        const bool crosses = (int)ends[slo] > a && (int)ends[slo] <= b;
        s.misc[4] = a;
        s.misc[5] = b;
        s.misc[6] = crosses ? 1 : 0;
    }
    __syncthreads();
    const int  a       = s.misc[4];
    const int  b       = s.misc[5];
    const bool crosses = s.misc[6] != 0;
    if (!crosses) {
        return A[found];  // the run lies inside one segment: already in the reference's order
    }
    // the id with exactly (found - a) smaller ids in the run: bisection over the ids, counting with all threads
    const int want = found - a;
    int       lo = 0, hi = vocab;  // the answer lies in [lo, hi)
    while (hi - lo > 1) {
        const int mid = lo + (hi - lo) / 2;
        if (t == 0) {
            s.misc[7] = 0;
        }
        __syncthreads();
        int mine = 0;
        for (int i = a + t; i <= b; i += TP_THREADS) {
            mine += (int)(uint32_t)A[i] < mid ? 1 : 0;
        }
        mine = wave_sum_i(mine);
        if (lane_id() == 0 && mine != 0) {
            atomicAdd(&s.misc[7], mine);
        }
        __syncthreads();
        const int below_mid = s.misc[7];
        __syncthreads();
        // ids are distinct: the answer is below mid exactly when more than `want` ids are
        if (below_mid > want) {
            hi = mid;
        }
        else {
            lo = mid;
        }
    }
    const uint32_t key = (uint32_t)(A[found] >> 32);
    return ((unsigned long long)key << 32) | (uint32_t)lo;
}

// LOGITS: `probs` holds the row's logits (n of its `vocab` columns are the vocabulary proper) and every probability
// that is needed is worked out from them with the row's statistics in `meta` (topp_row_kernel); `seg_ends` are the
// segments of the ordered prefix.
template<int DT, bool LOGITS>
__device__ __forceinline__ void
topp_pick_row(TopPShared& s, const typename Storage<DT>::T* __restrict__ probs, int* ids,
              int* __restrict__ sequence_length, bool* __restrict__ finished, float* __restrict__ cum_log_probs,
              float* __restrict__ output_log_probs, RngState* rng, const float* __restrict__ uniforms, int vocab,
              const int* __restrict__ end_ids, float top_p, const float* top_ps,
              const bool* __restrict__ skip_decode, unsigned long long* __restrict__ sorted,
              const ToppRowMeta* __restrict__ meta, int force_deep, int n, const uint32_t* __restrict__ seg_ends)
{
    typedef Storage<DT>   S;
    const int             row = blockIdx.x;
    const int             t   = threadIdx.x;
    if (skip_decode != nullptr && skip_decode[row]) {
        return;
    }
    const typename S::T* rowp = probs + (size_t)row * vocab;
    const float          p    = top_ps != nullptr ? top_ps[row] : top_p;
    const ToppRowMeta    m    = meta[row];
    int                  best_id = (int)(~(uint32_t)m.best);
    if ((uint32_t)(m.best >> 32) == 0u) {
        best_id = 0;  // nothing comparable in the row (all NaN): the reference keeps index 0
    }
    ToppRowValues vals;
    vals.MAXT   = S::max_t();
    vals.fin    = LOGITS && finished != nullptr ? finished[row] : false;  // (read before this kernel writes the flag)
    vals.end_id = vals.fin ? end_ids[row] : -1;
    vals.n      = n;
    const RowDivisor div(LOGITS ? m.denom : 1.0f);
    // the probability of column v as the sampler of the reference would read it from the softmax's output
    auto prob_at = [&](int v) -> float {
        if constexpr (LOGITS) {
            const float y = vals.masked(v, v < n ? S::ld(rowp[v]) : 0.0f);
            return topp_prob_of<DT>(round_t<DT>(det_expf_nonpos(y - m.mx)), div, m.denom);
        }
        else {
            return S::ld(rowp[v]);
        }
    };
    const float best_prob = LOGITS ? ((uint32_t)(m.best >> 32) == 0u ? prob_at(0) : m.best_prob) : S::ld(rowp[best_id]);

    if (t == 0) {
        const float u = row_uniform(rng, uniforms, row);  // drawn for every non-skipped row
        s.fmisc[0]    = u * p;
    }
    __syncthreads();
    const float rand_num = s.fmisc[0];

    auto emit = [&](int id, float prob) {
        // single thread
        ids[row] = id;
        if (cum_log_probs != nullptr || output_log_probs != nullptr) {
            const float lp = det_logf(prob);
            if (cum_log_probs != nullptr) {
                cum_log_probs[row] += lp;
            }
            if (output_log_probs != nullptr) {
                output_log_probs[row] = lp;
            }
        }
        if (sequence_length != nullptr && finished != nullptr) {
            sequence_length[row] = finished[row] ? sequence_length[row] : sequence_length[row] + 1;
            finished[row]        = id == end_ids[row];
        }
    };

    // ---- shortcut: sum_prob = T(0) + max prob, compared in fp32 (:842-849)
    if (round_t<DT>(0.0f + best_prob) >= p) {
        if (t == 0) {
            emit(best_id, best_prob);
        }
        return;
    }
    if (t == 0) {
        ids[row] = best_id;  // kept when no prefix sum ever reaches the draw (:954)
    }

    unsigned long long* A = sorted + (size_t)row * 2 * vocab;
    unsigned long long* B = A + vocab;
    if (!force_deep && m.flags == 0) {
        const bool all   = m.n == m.n_pos;
        const int  found = m.n > 0 ? scan_sorted(s, A, m.n, rand_num) : -1;
        if (found >= 0 && (found < m.n || all)) {
            unsigned long long e = 0ull;
            if (found < m.n) {
                if constexpr (LOGITS) {
                    e = topp_settle_ties(s, A, m.n, found, seg_ends + (size_t)row * TPB_NB, m.nseg, vocab);
                }
                else {
                    e = A[found];
                }
            }
            if (t == 0) {
                if (found < m.n) {
                    emit((int)(uint32_t)e, key64_prob(e));
                }
                else {
                    const int id = nth_zero_entry(prob_at, vocab, found - m.n);
                    emit(id, prob_at(id));
                }
            }
            return;
        }
        if (all) {
            return;  // every positive entry scanned, never crossed: ids keeps the arg-max
        }
    }

    // ---- fallback: every positive entry, compacted in id order, stable radix sort on the key bits
    if (t == 0) {
        s.misc[2] = 0;
    }
    __syncthreads();
    for (int base = 0; base < vocab; base += TP_THREADS) {
        const int                v    = base + t;
        const uint32_t           k    = v < vocab ? order_key(prob_at(v)) : 0u;
        const bool               keep = k > ZERO_KEY;
        const unsigned long long bal  = __ballot(keep);
        const int                below = __popcll(bal & ((1ull << lane_id()) - 1ull));
        if (lane_id() == 0) {
            s.red32[wave_id()] = (uint32_t)__popcll(bal);
        }
        __syncthreads();
        int off = s.misc[2];
        for (int w = 0; w < wave_id(); ++w) {
            off += (int)s.red32[w];
        }
        if (keep) {
            A[off + below] = ((unsigned long long)(~k) << 32) | (uint32_t)v;
        }
        __syncthreads();
        if (t == 0) {
            int tot = 0;
            for (int w = 0; w < TP_THREADS / WAVE; ++w) {
                tot += (int)s.red32[w];
            }
            s.misc[2] += tot;
        }
        __syncthreads();
    }
    const int n_all = s.misc[2];
    __threadfence_block();
    __syncthreads();
    RadixScratch              rs{reinterpret_cast<unsigned short*>(s.buf), s.wtot, s.red64};
    const unsigned long long* src   = radix_sort_range(A, B, n_all, 32, rs);
    const int                 found = n_all > 0 ? scan_sorted(s, src, n_all, rand_num) : -1;
    if (found >= 0 && t == 0) {
        if (found < n_all) {
            const unsigned long long e = src[found];
            emit((int)(uint32_t)e, key64_prob(e));
        }
        else {
            const int id = nth_zero_entry(prob_at, vocab, found - n_all);
            emit(id, prob_at(id));
        }
    }
}

// What computeToppDecay (:1381-1412) does to one row; the fused step runs it at the end of the row's pick.
struct ToppDecayArgs {
    float*         runtime_top_p;  // NULL: no decay
    const float*   initial_top_p;
    const float*   decay;
    const float*   top_p_min;
    const int32_t* reset_ids;
};

template<int DT, bool LOGITS>
__global__ void __launch_bounds__(TP_THREADS)
topp_pick_kernel(const typename Storage<DT>::T* __restrict__ probs, int* ids, int* __restrict__ sequence_length,
                 bool* __restrict__ finished, float* __restrict__ cum_log_probs, float* __restrict__ output_log_probs,
                 RngState* rng, const float* __restrict__ uniforms, int vocab, const int* __restrict__ end_ids,
                 float top_p, const float* top_ps, const bool* __restrict__ skip_decode,
                 unsigned long long* __restrict__ sorted, const ToppRowMeta* __restrict__ meta, int force_deep,
                 ToppDecayArgs dec, int n, const uint32_t* __restrict__ seg_ends)
{
    __shared__ TopPShared s;
    topp_pick_row<DT, LOGITS>(s, probs, ids, sequence_length, finished, cum_log_probs, output_log_probs, rng, uniforms,
                              vocab, end_ids, top_p, top_ps, skip_decode, sorted, meta, force_deep, n, seg_ends);
    // thread 0 wrote the row's id itself (a skipped row keeps what an earlier kernel left there) and every
    // thread read the row's top_p before the first barrier of the pick
    if (dec.runtime_top_p != nullptr && threadIdx.x == 0) {
        const int row = blockIdx.x;
        if (ids[row] == dec.reset_ids[row]) {
            dec.runtime_top_p[row] = dec.initial_top_p[row];
        }
        else {
            dec.runtime_top_p[row] = __builtin_fmaxf(dec.runtime_top_p[row] * dec.decay[row], dec.top_p_min[row]);
        }
    }
}

__global__ void topp_decay_kernel(float* __restrict__ runtime_top_p, const float* __restrict__ initial_top_p,
                                  const int* __restrict__ output_ids, const float* __restrict__ decay,
                                  const float* __restrict__ top_p_min, const int32_t* __restrict__ reset_ids, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) {
        return;
    }
    if (output_ids[i] == reset_ids[i]) {
        runtime_top_p[i] = initial_top_p[i];
    }
    else {
        runtime_top_p[i] = __builtin_fmaxf(runtime_top_p[i] * decay[i], top_p_min[i]);
    }
}

__global__ void topp_initialize_kernel(int* id_vals, int* offsets, int* begin_offsets, int batch, int n)
{
    const size_t tid = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
    if (blockIdx.x == 0 && offsets != nullptr) {
        for (int i = threadIdx.x; i < batch + 1; i += blockDim.x) {
            offsets[i] = i * n;
            if (begin_offsets != nullptr) {
                begin_offsets[i] = i * n;
            }
        }
    }
    if (id_vals != nullptr) {
        for (size_t i = tid; i < (size_t)batch * n; i += (size_t)gridDim.x * blockDim.x) {
            id_vals[i] = (int)(i % n);
        }
    }
}

}  // namespace ftk

using namespace ftk;

extern "C" {

int ftk_invoke_add_bias_softmax(int dtype, void* logits, const void* bias, const int* end_ids, const bool* finished,
                                int m, int n_padded, int n, ftk_stream_t stream)
{
    if (m <= 0 || n <= 0) {
        return 0;
    }
    FTK_DISPATCH_DTYPE(dtype, (softmax_kernel<DT, false><<<m, SM_THREADS, 0, (hipStream_t)stream>>>(
                                  (Storage<DT>::T*)logits, (const Storage<DT>::T*)bias, end_ids, finished, n_padded, n,
                                  nullptr)));
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_topp_initialize(int* topp_id_val_buf, int* topp_offset_buf, int* begin_topp_offset_buf,
                               size_t batch_size, int n, ftk_stream_t stream)
{
    if (batch_size == 0 || (topp_id_val_buf == nullptr && topp_offset_buf == nullptr)) {
        return 0;
    }
    topp_initialize_kernel<<<32, 512, 0, (hipStream_t)stream>>>(topp_id_val_buf, topp_offset_buf,
                                                                begin_topp_offset_buf, (int)batch_size, n);
    FTK_LAUNCH_CHECK();
    return 0;
}

#ifdef FTK_TEST_HOOKS
// Test hook (hooks build of the library only): a non-zero value routes every row through the radix-sort
// fallback, so that it can be exercised on small inputs.
static int g_topp_force_deep = 0;
void       ftk_test_set_topp_force_deep(int v)
{
    g_topp_force_deep = v;
}
#else
static constexpr int g_topp_force_deep = 0;
#endif

// Shared by the two entry points below. `softmax_first`: `log_probs` holds logits on entry; the softmax runs as
// two kernels, the second of which also tallies the histogram, and the decay runs at the end of the pick.
static int topp_sampling_launch(int dtype, void* workspace, size_t* workspace_size, size_t* cub_temp_storage_size,
                                int* output_ids, int* sequence_length, bool* finished, float* cum_log_probs,
                                float* output_log_probs, void* log_probs, ftk_rng_state* rng_state,
                                const float* uniform_draws, int batch_size, size_t vocab_size_padded,
                                const int* end_ids, float max_top_p, const float* top_ps, hipStream_t st,
                                const bool* skip_decode, bool softmax_first, const void* bias, int vocab_size,
                                ToppDecayArgs dec, bool from_logits = false)
{
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (batch_size < 0 || batch_size > 65535) {
        return FTK_ERR_ARGUMENT;
    }
    const ToppPlan plan      = topp_plan(batch_size, vocab_size_padded);
    const size_t   off_stats = plan.bytes;
    const size_t   need      = plan.bytes + (softmax_first ? align256((size_t)(batch_size > 0 ? batch_size : 1) * sizeof(float2)) : 0);
    if (workspace == nullptr) {
        if (workspace_size == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        *workspace_size = need;
        if (cub_temp_storage_size != nullptr) {
            *cub_temp_storage_size = 0;
        }
        return 0;
    }
    if (workspace_size != nullptr && *workspace_size < need) {
        return FTK_ERR_WORKSPACE;
    }
    if (batch_size <= 0) {
        return 0;
    }
    if (rng_state == nullptr && uniform_draws == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    if (log_probs == nullptr || output_ids == nullptr
        || (end_ids == nullptr && finished != nullptr && (sequence_length != nullptr || softmax_first))) {
        return FTK_ERR_ARGUMENT;  // (the kernels read and write these unconditionally)
    }
    if (vocab_size_padded > (size_t)65535 * TP_THREADS) {
        return FTK_ERR_ARGUMENT;
    }
    if (softmax_first && (vocab_size <= 0 || (size_t)vocab_size > vocab_size_padded)) {
        return FTK_ERR_ARGUMENT;
    }
    char*               ws      = (char*)workspace;
    unsigned long long* sorted  = (unsigned long long*)ws;
    uint32_t*           pcnt    = (uint32_t*)(ws + plan.off_pcnt);
    uint32_t*           pmass   = (uint32_t*)(ws + plan.off_pmass);
    unsigned long long* pbest   = (unsigned long long*)(ws + plan.off_pbest);
    uint32_t*           start   = (uint32_t*)(ws + plan.off_start);
    uint32_t*           boff    = (uint32_t*)(ws + plan.off_boff);
    uint32_t*           segs    = (uint32_t*)(ws + plan.off_seg);
    ToppRowMeta*        meta    = (ToppRowMeta*)(ws + plan.off_meta);
    const int           vocab   = (int)vocab_size_padded;
    const dim3          chunks(plan.splits, batch_size);
    if (from_logits) {
        // the probabilities are never written: three launches
        FTK_DISPATCH_DTYPE(dtype, topp_row_kernel<DT><<<batch_size, SM_THREADS, 0, st>>>(
                                      (const Storage<DT>::T*)log_probs, end_ids, finished, vocab, vocab_size,
                                      skip_decode, (const RngState*)rng_state, uniform_draws, max_top_p, top_ps, segs,
                                      meta, sorted));
        FTK_LAUNCH_CHECK();
        topp_sort_kernel<<<plan.sorters, TP_THREADS, 0, st>>>(sorted, segs, meta, vocab, batch_size);
        FTK_LAUNCH_CHECK();
        FTK_DISPATCH_DTYPE(dtype, (topp_pick_kernel<DT, true><<<batch_size, TP_THREADS, 0, st>>>(
                                      (const Storage<DT>::T*)log_probs, output_ids, sequence_length, finished,
                                      cum_log_probs, output_log_probs, (RngState*)rng_state, uniform_draws, vocab,
                                      end_ids, max_top_p, top_ps, skip_decode, sorted, meta, g_topp_force_deep, dec,
                                      vocab_size, segs)));
        FTK_LAUNCH_CHECK();
        return 0;
    }
    if (softmax_first) {
        float2* stats = (float2*)(ws + off_stats);
        FTK_DISPATCH_DTYPE(dtype, (softmax_kernel<DT, true><<<batch_size, SM_THREADS, 0, st>>>(
                                      (Storage<DT>::T*)log_probs, (const Storage<DT>::T*)bias, end_ids, finished, vocab,
                                      vocab_size, stats)));
        FTK_LAUNCH_CHECK();
        FTK_DISPATCH_DTYPE(dtype, softmax_finish_histogram_kernel<DT><<<chunks, TPH_THREADS, 0, st>>>(
                                      (Storage<DT>::T*)log_probs, (const Storage<DT>::T*)bias, end_ids, finished, stats,
                                      vocab, vocab_size, plan.chunk, skip_decode, pcnt, pmass, pbest));
        FTK_LAUNCH_CHECK();
    }
    else {
        FTK_DISPATCH_DTYPE(dtype, topp_histogram_kernel<DT><<<chunks, TPH_THREADS, 0, st>>>(
                                      (const Storage<DT>::T*)log_probs, vocab, plan.chunk, skip_decode, pcnt, pmass,
                                      pbest));
        FTK_LAUNCH_CHECK();
    }
    topp_cut_kernel<<<batch_size, TPC_THREADS, 0, st>>>(plan.splits, pcnt, pmass, pbest, start, boff, segs, meta,
                                                        (const RngState*)rng_state, uniform_draws, max_top_p, top_ps,
                                                        skip_decode);
    FTK_LAUNCH_CHECK();
    if (!g_topp_force_deep) {
        FTK_DISPATCH_DTYPE(dtype, topp_gather_kernel<DT><<<chunks, TPH_THREADS, 0, st>>>(
                                      (const Storage<DT>::T*)log_probs, vocab, plan.chunk, meta, start, boff, sorted));
        FTK_LAUNCH_CHECK();
        topp_sort_kernel<<<plan.sorters, TP_THREADS, 0, st>>>(sorted, segs, meta, vocab, batch_size);
        FTK_LAUNCH_CHECK();
    }
    FTK_DISPATCH_DTYPE(dtype, (topp_pick_kernel<DT, false><<<batch_size, TP_THREADS, 0, st>>>(
                                  (const Storage<DT>::T*)log_probs, output_ids, sequence_length, finished,
                                  cum_log_probs, output_log_probs, (RngState*)rng_state, uniform_draws, vocab,
                                  end_ids, max_top_p, top_ps, skip_decode, sorted, meta, g_topp_force_deep, dec, vocab,
                                  segs)));
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_batch_topp_sampling(int dtype, void* workspace, size_t* workspace_size, size_t* cub_temp_storage_size,
                                   int* output_ids, int* sequence_length, bool* finished, float* cum_log_probs,
                                   float* output_log_probs, const void* log_probs, const int* id_vals,
                                   int* offset_buf, int* begin_offset_buf, ftk_rng_state* rng_state,
                                   const float* uniform_draws, int batch_size, size_t vocab_size_padded,
                                   const int* end_ids, float max_top_p, const float* top_ps, ftk_stream_t stream,
                                   const bool* skip_decode)
{
    (void)id_vals;
    (void)offset_buf;
    (void)begin_offset_buf;
    const ToppDecayArgs none = {nullptr, nullptr, nullptr, nullptr, nullptr};
    return topp_sampling_launch(dtype, workspace, workspace_size, cub_temp_storage_size, output_ids, sequence_length,
                                finished, cum_log_probs, output_log_probs, const_cast<void*>(log_probs), rng_state,
                                uniform_draws, batch_size, vocab_size_padded, end_ids, max_top_p, top_ps,
                                (hipStream_t)stream, skip_decode, false, nullptr, 0, none);
}

int ftk_fused_topp_step(int dtype, void* workspace, size_t* workspace_size, void* logits, const void* bias,
                        int vocab_size, size_t vocab_size_padded, int batch_size, const int* end_ids, bool* finished,
                        int* sequence_length, int* output_ids, float* cum_log_probs, float* output_log_probs,
                        ftk_rng_state* rng_state, const float* uniform_draws, float max_top_p, float* runtime_top_p,
                        const float* initial_top_p, const float* top_p_decay, const float* top_p_min,
                        const int32_t* top_p_reset_ids, const bool* skip_decode, ftk_stream_t stream)
{
    ToppDecayArgs dec = {nullptr, nullptr, nullptr, nullptr, nullptr};
    if (top_p_decay != nullptr) {
        if (runtime_top_p == nullptr || initial_top_p == nullptr || top_p_min == nullptr || top_p_reset_ids == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        dec = ToppDecayArgs{runtime_top_p, initial_top_p, top_p_decay, top_p_min, top_p_reset_ids};
    }
    return topp_sampling_launch(dtype, workspace, workspace_size, nullptr, output_ids, sequence_length, finished,
                                cum_log_probs, output_log_probs, logits, rng_state, uniform_draws, batch_size,
                                vocab_size_padded, end_ids, max_top_p, runtime_top_p, (hipStream_t)stream,
                                skip_decode, true, bias, vocab_size, dec);
}

int ftk_fused_topp_sample_step(int dtype, void* workspace, size_t* workspace_size, const void* logits,
                               int vocab_size, size_t vocab_size_padded, int batch_size, const int* end_ids,
                               bool* finished, int* sequence_length, int* output_ids, float* cum_log_probs,
                               float* output_log_probs, ftk_rng_state* rng_state, const float* uniform_draws,
                               float max_top_p, float* runtime_top_p, const float* initial_top_p,
                               const float* top_p_decay, const float* top_p_min, const int32_t* top_p_reset_ids,
                               const bool* skip_decode, ftk_stream_t stream)
{
    if (vocab_size < SM_THREADS) {
        return FTK_ERR_UNSUPPORTED;  // (the sum's order follows the softmax's block of min(n, 1024) threads)
    }
    ToppDecayArgs dec = {nullptr, nullptr, nullptr, nullptr, nullptr};
    if (top_p_decay != nullptr) {
        if (runtime_top_p == nullptr || initial_top_p == nullptr || top_p_min == nullptr || top_p_reset_ids == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        dec = ToppDecayArgs{runtime_top_p, initial_top_p, top_p_decay, top_p_min, top_p_reset_ids};
    }
    return topp_sampling_launch(dtype, workspace, workspace_size, nullptr, output_ids, sequence_length, finished,
                                cum_log_probs, output_log_probs, const_cast<void*>(logits), rng_state, uniform_draws,
                                batch_size, vocab_size_padded, end_ids, max_top_p, runtime_top_p, (hipStream_t)stream,
                                skip_decode, true, nullptr, vocab_size, dec, true);
}

int ftk_invoke_compute_topp_decay(float* runtime_top_p, const float* runtime_initial_top_p, const int* output_ids,
                                  const float* top_p_decay, const float* top_p_min, const int32_t* top_p_reset_ids,
                                  int local_batch_size, ftk_stream_t stream)
{
    if (local_batch_size <= 0) {
        return 0;
    }
    topp_decay_kernel<<<(local_batch_size + 255) / 256, 256, 0, (hipStream_t)stream>>>(
        runtime_top_p, runtime_initial_top_p, output_ids, top_p_decay, top_p_min, top_p_reset_ids, local_batch_size);
    FTK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
