// One step of beam search over [batch * beam_width, vocab] logits: log-softmax, the 2K best tokens of every beam,
// the K best continuations of every batch entry, finished hypotheses moved to the BeamHypotheses arrays.
//
// Reference behaviour restated (src/fastertransformer/kernels/online_softmax_beamsearch_kernels.cu):
//   :366-514  beam_online_softmax_topk_stage1 / stage2 - per row (max, sum of exponentials) and the 2K best
//             elements under TopK<T, MAX_K>::insert (kernels/reduce_kernel_utils.cuh:275-322): value
//             descending, id ascending, which no merge order changes
//   :99-262   batch_topk_kernel - the 2 * MAX_K best of a batch entry's K * 2K candidates after length penalty
//             and diversity term, then one thread walks them: end tokens among the first K go to the
//             hypotheses (kernels/beam_search_topk_kernels.h:31-58), the others become the next beams
//   :549-701  launchers and the beam-width classes
//
// The reference finds the best elements by inserting into per-thread sorted arrays and merging them with cub. Here
// every selection is an exact radix select over 64-bit keys (order-preserving value bits, then the complement of
// the position, so that keys are distinct and ties need no rule of their own): byte by byte from the top, a
// 256-bin LDS histogram of the keys that match the bytes fixed so far; as soon as few enough match they are moved
// to LDS and the remaining bytes are settled there.
#include "ftk_columns.cuh"
#include "ftk_device.cuh"
#include "ftk_sampling.h"
#include "ftk_transform.cuh"
#ifdef FTK_TEST_HOOKS
#include "ftk_test_hooks.h"
#endif

namespace ftk {

constexpr int BM_THREADS = 256;
constexpr int BM_WAVES   = BM_THREADS / WAVE;
constexpr int BM_CAP     = 2048;  // keys settled in LDS
constexpr int BM_MAX_N   = 128;   // 2 * beam_width and 2 * MAX_K are at most this

struct BeamSelect {
    __attribute__((aligned(16))) unsigned long long list[BM_CAP];
    unsigned long long cand[BM_CAP];     // a section's elements at or above the bound from the thread maxima
    unsigned long long slots[BM_THREADS];
    unsigned long long out[BM_MAX_N];
    int                n_cand;
    uint32_t           hist[256];
    uint32_t           wave_total[BM_WAVES];
    int                n_list;
    int                n_out;
    int                found_bin;
    int                found_above;
};

// The `need`-th largest of `count` keys key(i), 1 <= need <= count, distinct at least down to that one (zero keys
// that pad a list may repeat below it): every thread of the workgroup gets it. key(i) is evaluated once per byte
// that is settled on the caller's data (until BM_CAP or fewer keys match).
template<class F>
__device__ __forceinline__ unsigned long long beam_nth_key(BeamSelect& s, F&& key, int count, int need)
{
    const int          t      = threadIdx.x;
    unsigned long long prefix = 0ull;
    bool               in_lds = false;
    int                n      = count;
    for (int shift = 56; shift >= 0; shift -= 8) {
        s.hist[t] = 0u;
        __syncthreads();
        for (int i = t; i < n; i += BM_THREADS) {
            const unsigned long long k = in_lds ? s.list[i] : key(i);
            if (shift == 56 || (k >> (shift + 8)) == prefix) {
                atomicAdd(&s.hist[(uint32_t)(k >> shift) & 255u], 1u);
            }
        }
        __syncthreads();
        // thread t looks at bin 255 - t: inclusive sums from the top bin down
        const uint32_t mine = s.hist[255 - t];
        uint32_t       inc  = mine;
#pragma unroll
        for (int o = 1; o < WAVE; o <<= 1) {
            const uint32_t up = __shfl_up(inc, o, WAVE);
            if (lane_id() >= o) {
                inc += up;
            }
        }
        if (lane_id() == WAVE - 1) {
            s.wave_total[wave_id()] = inc;
        }
        __syncthreads();
        for (int w = 0; w < wave_id(); ++w) {
            inc += s.wave_total[w];
        }
        if (inc >= (uint32_t)need && inc - mine < (uint32_t)need) {
            s.found_bin   = 255 - t;
            s.found_above = (int)(inc - mine);
        }
        __syncthreads();
        const int bin     = s.found_bin;
        const int matched = (int)s.hist[bin];
        need -= s.found_above;
        prefix = (prefix << 8) | (unsigned long long)bin;
        if (!in_lds && matched <= BM_CAP && shift > 0) {
            // few enough keys carry the bytes fixed so far: the rest is settled on a copy in LDS
            if (t == 0) {
                s.n_list = 0;
            }
            __syncthreads();
            for (int i = t; i < n; i += BM_THREADS) {
                const unsigned long long k = key(i);
                if ((k >> shift) == prefix) {
                    s.list[atomicAdd(&s.n_list, 1)] = k;
                }
            }
            __syncthreads();
            in_lds = true;
            n      = matched;
        }
        __syncthreads();
    }
    return prefix;
}

// Leaves the `need` largest of `count` distinct keys in s.out, largest first; need <= BM_MAX_N, need <= count.
template<class F>
__device__ __forceinline__ void beam_select(BeamSelect& s, F&& key, int count, int need)
{
    const int t = threadIdx.x;
    if (count <= BM_THREADS) {
        // one key per thread: its place is the number of larger keys
        const unsigned long long k = t < count ? key(t) : 0ull;
        __syncthreads();  // (the caller may still be reading what key() reads from, or s.list)
        s.list[t] = k;  // (zeros behind the last key: they are larger than nothing)
        __syncthreads();
        const ulonglong2* pairs = reinterpret_cast<const ulonglong2*>(s.list);
        int               r     = 0;
        for (int j = 0; j < (count + 3) / 4; ++j) {
            const ulonglong2 a = pairs[2 * j];
            const ulonglong2 b = pairs[2 * j + 1];
            r += (a.x > k ? 1 : 0) + (a.y > k ? 1 : 0) + (b.x > k ? 1 : 0) + (b.y > k ? 1 : 0);
        }
        if (t < count && r < need) {
            s.out[r] = k;
        }
        __syncthreads();
        return;
    }
    const unsigned long long bound = beam_nth_key(s, key, count, need);
    if (t == 0) {
        s.n_out = 0;
    }
    __syncthreads();
    for (int i = t; i < count; i += BM_THREADS) {
        const unsigned long long k = key(i);
        if (k >= bound) {
            s.list[atomicAdd(&s.n_out, 1)] = k;  // exactly `need` of them
        }
    }
    __syncthreads();
    if (t < need) {
        const unsigned long long k = s.list[t];
        int                      r = 0;
        for (int j = 0; j < need; ++j) {
            r += s.list[j] > k ? 1 : 0;
        }
        s.out[r] = k;
    }
    __syncthreads();
}

__device__ __forceinline__ unsigned long long beam_key(float value, uint32_t position)
{
    return ((unsigned long long)order_key(value) << 32) | (unsigned long long)(0xFFFFFFFFu - position);
}
__device__ __forceinline__ uint32_t beam_key_position(unsigned long long k)
{
    return 0xFFFFFFFFu - (uint32_t)k;
}
__device__ __forceinline__ float beam_key_value(unsigned long long k)
{
    return key_to_float((uint32_t)(k >> 32));
}

// element `v` of row `r` as the reference's kernels see it (:341-347, :410-416)
template<int DT>
__device__ __forceinline__ float beam_element(const typename Storage<DT>::T* __restrict__ x,
                                              const typename Storage<DT>::T* __restrict__ bias, size_t row_base, int v)
{
    typedef Storage<DT> S;
    const float         b = bias != nullptr ? S::ld(bias[v]) : 0.0f;
    return round_t<DT>(S::ld(x[row_base + v]) + b);
}

// the same from a value that is already loaded
template<int DT>
__device__ __forceinline__ float beam_element_of(float xv, const typename Storage<DT>::T* __restrict__ bias, int v)
{
    if (bias == nullptr) {
        return xv;  // adding T(0) changes -0 into +0 and nothing else: same key, same exponential
    }
    return round_t<DT>(xv + Storage<DT>::ld(bias[v]));
}

struct BeamPlan {
    int    parts;  // sections per row
    int    section;
    size_t off_pmax, off_psum, off_pkeys, off_cand_id, off_cand_val, bytes;
};

static inline size_t beam_align(size_t x)
{
    return (x + 255) & ~(size_t)255;
}

static BeamPlan beam_plan(int rows, int beam_width, int vocab)
{
    BeamPlan  p;
    const int N = 2 * beam_width;
    int       parts = (1024 + rows - 1) / (rows > 0 ? rows : 1);
    const int by_len = vocab / 4096 > 0 ? vocab / 4096 : 1;
    parts   = parts < by_len ? parts : by_len;
    parts   = parts < BM_CAP / N ? parts : BM_CAP / N;  // the lists of a row are merged in LDS
    parts   = parts < 1 ? 1 : parts;
    while (parts > 1 && (vocab + parts - 1) / parts < N) {
        parts--;  // every section holds at least 2K elements
    }
    p.parts   = parts;
    p.section = (vocab + parts - 1) / parts;
    const size_t r = (size_t)(rows > 0 ? rows : 1);
    size_t       off = 0;
    p.off_pmax = off;
    off += beam_align(r * parts * sizeof(float));
    p.off_psum = off;
    off += beam_align(r * parts * sizeof(double));
    p.off_pkeys = off;
    off += beam_align(r * parts * N * sizeof(unsigned long long));
    p.off_cand_id = off;
    off += beam_align(r * N * sizeof(int));
    p.off_cand_val = off;
    off += beam_align(r * N * sizeof(float));
    p.bytes = off;
    return p;
}

// (parts x rows) workgroups: the maximum of a section
template<int DT>
__global__ void __launch_bounds__(BM_THREADS)
beam_section_max_kernel(const typename Storage<DT>::T* __restrict__ x, const typename Storage<DT>::T* __restrict__ bias,
                        const bool* __restrict__ finished, int vocab, int section, float* __restrict__ pmax)
{
    __shared__ float red[BM_WAVES];
    const int        row = blockIdx.y;
    const int        t   = threadIdx.x;
    if (finished[row]) {
        return;
    }
    const int    lo = min(vocab, (int)blockIdx.x * section);
    const int    hi = min(vocab, lo + section);
    const size_t rb = (size_t)row * vocab;
    float        m  = -Storage<DT>::max_t();
    stream_columns<DT, BM_THREADS>(x + rb, lo, hi, [&](int v, float xv) {
        const float e = beam_element_of<DT>(xv, bias, v);
        m             = e > m ? e : m;
    });
    m = block_max<float, BM_WAVES>(m, red, -Storage<DT>::max_t());
    if (t == 0) {
        pmax[(size_t)row * gridDim.x + blockIdx.x] = m;
    }
}

// (parts x rows) workgroups: the sum of exponentials of a section against the row's maximum and its 2K best
template<int DT>
__global__ void __launch_bounds__(BM_THREADS)
beam_section_kernel(const typename Storage<DT>::T* __restrict__ x, const typename Storage<DT>::T* __restrict__ bias,
                    const bool* __restrict__ finished, int vocab, int section, int N, const float* __restrict__ pmax,
                    double* __restrict__ psum, unsigned long long* __restrict__ pkeys)
{
    __shared__ BeamSelect s;
    __shared__ double     red[BM_WAVES];
    const int             row   = blockIdx.y;
    const int             part  = blockIdx.x;
    const int             parts = gridDim.x;
    const int             t     = threadIdx.x;
    if (finished[row]) {
        return;
    }
    const int    lo = min(vocab, part * section);
    const int    hi = min(vocab, lo + section);
    const size_t rb = (size_t)row * vocab;
    float        m  = -Storage<DT>::max_t();
    for (int p = 0; p < parts; ++p) {
        const float pm = pmax[(size_t)row * parts + p];
        m              = pm > m ? pm : m;
    }
    // first pass: the sum, and every thread's largest element
    double d    = 0.0;
    float  fmax = -__builtin_inff();
    stream_columns<DT, BM_THREADS>(x + rb, lo, hi, [&](int v, float xv) {
        const float e = beam_element_of<DT>(xv, bias, v);
        d += (double)det_expf_nonpos(e - m);  // m is the row's maximum: the argument is never positive
        fmax = __builtin_fmaxf(fmax, e);      // (a NaN is never the maximum, as under order_key)
    });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        d += __shfl_xor(d, o, WAVE);
    }
    if (lane_id() == 0) {
        red[wave_id()] = d;
    }
    // N <= 32 needs no more than 64 maxima to choose the N-th largest from, N <= 64 no more than 128: neighbouring
    // threads join theirs, and the ranking below is that much shorter
    const int group = N <= 32 ? 4 : N <= 64 ? 2 : 1;
    if (group >= 2) {
        fmax = __builtin_fmaxf(fmax, __shfl_xor(fmax, 1, WAVE));
    }
    if (group == 4) {
        fmax = __builtin_fmaxf(fmax, __shfl_xor(fmax, 2, WAVE));
    }
    const int n_slots = BM_THREADS / group;
    if (t % group == 0) {
        s.slots[t / group] = ((unsigned long long)order_key(fmax) << 32) | (unsigned long long)(BM_THREADS - 1 - t);
    }
    if (t == 0) {
        s.n_cand = 0;
    }
    __syncthreads();
    if (t == 0) {
        double tot = 0.0;
        for (int w = 0; w < BM_WAVES; ++w) {
            tot += red[w];
        }
        psum[(size_t)row * parts + part] = tot;
    }
    // a short last section gives fewer than N keys; the rest of its list is 0, below every key of an element
    const int take = min(N, hi - lo);
    // The N-th largest of the thread maxima is an element with at least N elements at or above it (N threads hold
    // one each): nothing below it can be among the N best. Usually a few times N elements pass.
    // (a group that saw no element reports -inf, which lowers the bound at most to "every number")
    beam_select(s, [&](int i) { return s.slots[i]; }, n_slots, N);
    const uint32_t floor_key = (uint32_t)(s.out[N - 1] >> 32);
    const float    floor_val = key_to_float(floor_key);
    const bool     all_pass  = floor_key <= order_key(-__builtin_inff());  // then NaN columns are wanted too
    stream_columns<DT, BM_THREADS>(x + rb, lo, hi, [&](int v, float xv) {
        const float e = beam_element_of<DT>(xv, bias, v);
        if (e >= floor_val || all_pass) {
            const int at = atomicAdd(&s.n_cand, 1);
            if (at < BM_CAP) {
                s.cand[at] = beam_key(e, (uint32_t)v);
            }
        }
    });
    __syncthreads();
    const int passed = s.n_cand;
    if (take > 0) {
        if (passed <= BM_CAP) {
            beam_select(s, [&](int i) { return s.cand[i]; }, passed, take);
        }
        else {
            // (rows of many equal values) the selection runs over the section itself
            beam_select(s, [&](int i) { return beam_key(beam_element<DT>(x, bias, rb, lo + i), (uint32_t)(lo + i)); },
                        hi - lo, take);
        }
    }
    if (t < N) {
        pkeys[((size_t)row * parts + part) * N + t] = t < take ? s.out[t] : 0ull;
    }
}

// one workgroup per row: the row's 2K best from its sections' lists, val = u - m - log(d) + cum_log_probs as T
template<int DT>
__global__ void __launch_bounds__(BM_THREADS)
beam_row_kernel(const bool* __restrict__ finished, const int* __restrict__ end_ids,
                const float* __restrict__ cum_log_probs, int vocab, int K, int parts, const float* __restrict__ pmax,
                const double* __restrict__ psum, const unsigned long long* __restrict__ pkeys,
                int* __restrict__ cand_id, float* __restrict__ cand_val)
{
    typedef Storage<DT>   S;
    __shared__ BeamSelect s;
    const int             row  = blockIdx.x;
    const int             t    = threadIdx.x;
    const int             N    = 2 * K;
    const float           MAXT = S::max_t();
    const float           cum  = cum_log_probs[row];
    if (finished[row]) {
        // MAX_T at the end id, -MAX_T elsewhere (:328-336): the end id first, then the lowest ids
        const int  end_id = end_ids[row / K];
        const bool inside = end_id >= 0 && end_id < vocab;
        if (t < N) {
            int   id;
            float u;
            if (inside) {
                id = t == 0 ? end_id : (t - 1 < end_id ? t - 1 : t);
                u  = t == 0 ? MAXT : -MAXT;
            }
            else {
                id = t;
                u  = -MAXT;
            }
            // inside: m = MAX_T, every other exponential is 0, d = 1; otherwise m = -MAX_T and d = vocab
            const float m    = inside ? MAXT : -MAXT;
            const float logd = inside ? 0.0f : det_logf((float)vocab);
            cand_id[(size_t)row * N + t]  = id + row * vocab;
            cand_val[(size_t)row * N + t] = round_t<DT>((u - m - logd) + cum);
        }
        return;
    }
    float  m = -MAXT;
    double d = 0.0;
    for (int p = 0; p < parts; ++p) {
        const float pm = pmax[(size_t)row * parts + p];
        m              = pm > m ? pm : m;
        d += psum[(size_t)row * parts + p];
    }
    const float               logd = det_logf((float)d);
    const unsigned long long* keys = pkeys + (size_t)row * parts * N;
    if (parts == 1) {
        if (t < N) {
            s.out[t] = keys[t];
        }
        __syncthreads();
    }
    else {
        beam_select(s, [&](int i) { return keys[i]; }, parts * N, N);
    }
    if (t < N) {
        const unsigned long long k    = s.out[t];
        cand_id[(size_t)row * N + t]  = (int)beam_key_position(k) + row * vocab;
        cand_val[(size_t)row * N + t] = round_t<DT>((beam_key_value(k) - m - logd) + cum);
    }
}

// The three kernels above in one launch: one 1024-thread workgroup per row finds the row's maximum, the sum of exponentials and every thread's largest
// element, takes a bound from 256 (128, 64) joined thread maxima, collects what reaches it and leaves the row's 2K
// best with their values. The passes over the row are the section kernels' with the whole row as the one section
// (the second and third come from the caches); the bound is found by the first wave alone (a bisection with
// ballots over the top 24 key bits: a floor at or below the 2K-th largest maximum, which is all the argument
// needs) so that the other fifteen waves only wait at two barriers; after the last pass twelve waves leave and the
// first four select with the code of the 256-thread kernels (a barrier counts the waves that are left).
// With more rows than compute units the workgroups have 512 threads and two of them share a compute unit: one's reads
// run beside the other's exponentials (64 x 8 beams x 152064 fp16: 120 -> 116 us).
constexpr int BR_THREADS = 1024;

template<int DT, int THREADS>
__global__ void __launch_bounds__(THREADS)
beam_rowwide_kernel(const typename Storage<DT>::T* __restrict__ x, const typename Storage<DT>::T* __restrict__ bias,
                    const bool* __restrict__ finished, const int* __restrict__ end_ids,
                    const float* __restrict__ cum_log_probs, int vocab, int K, int* __restrict__ cand_id,
                    float* __restrict__ cand_val)
{
    typedef Storage<DT>   S;
    constexpr int         BR_WAVES = THREADS / WAVE;
    static_assert(THREADS == 1024 || THREADS == 512, "256, 128 or 64 joined maxima");
    __shared__ BeamSelect s;
    __shared__ double     red[BR_WAVES];
    __shared__ float      redf[BR_WAVES];
    __shared__ double     row_sum;
    __shared__ uint32_t   row_floor;
    const int             row  = blockIdx.x;
    const int             t    = threadIdx.x;
    const int             N    = 2 * K;
    const float           MAXT = S::max_t();
    const float           cum  = cum_log_probs[row];
    if (finished[row]) {
        // MAX_T at the end id, -MAX_T elsewhere (:328-336): the end id first, then the lowest ids
        const int  end_id = end_ids[row / K];
        const bool inside = end_id >= 0 && end_id < vocab;
        if (t < N) {
            int   id;
            float u;
            if (inside) {
                id = t == 0 ? end_id : (t - 1 < end_id ? t - 1 : t);
                u  = t == 0 ? MAXT : -MAXT;
            }
            else {
                id = t;
                u  = -MAXT;
            }
            const float m    = inside ? MAXT : -MAXT;
            const float logd = inside ? 0.0f : det_logf((float)vocab);
            cand_id[(size_t)row * N + t]  = id + row * vocab;
            cand_val[(size_t)row * N + t] = round_t<DT>((u - m - logd) + cum);
        }
        return;
    }
    const size_t rb = (size_t)row * vocab;
    // first pass: the row's maximum
    float m = -MAXT;
    stream_columns<DT, THREADS>(x + rb, 0, vocab, [&](int v, float xv) {
        const float e = beam_element_of<DT>(xv, bias, v);
        m             = e > m ? e : m;
    });
    m = block_max<float, BR_WAVES>(m, redf, -MAXT);
    // second pass: the sum, and every thread's largest element
    double d    = 0.0;
    float  fmax = -__builtin_inff();
    stream_columns<DT, THREADS>(x + rb, 0, vocab, [&](int v, float xv) {
        const float e = beam_element_of<DT>(xv, bias, v);
        d += (double)det_expf_nonpos(e - m);
        fmax = __builtin_fmaxf(fmax, e);
    });
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        d += __shfl_xor(d, o, WAVE);
    }
    if (lane_id() == 0) {
        red[wave_id()] = d;
    }
    // 2K <= 32 needs no more than 64 maxima to choose the 2K-th largest from, 2K <= 64 no more than 128
    const int n_slots = N <= 32 ? 64 : N <= 64 ? 128 : 256;
    const int join    = THREADS / n_slots;  // neighbouring threads that join their maxima: 2 to 16
    fmax              = __builtin_fmaxf(fmax, __shfl_xor(fmax, 1, WAVE));
    if (join >= 4) {
        fmax = __builtin_fmaxf(fmax, __shfl_xor(fmax, 2, WAVE));
    }
    if (join >= 8) {
        fmax = __builtin_fmaxf(fmax, __shfl_xor(fmax, 4, WAVE));
    }
    if (join == 16) {
        fmax = __builtin_fmaxf(fmax, __shfl_xor(fmax, 8, WAVE));
    }
    uint32_t* slot_key = reinterpret_cast<uint32_t*>(s.slots);
    if (t % join == 0) {
        slot_key[t / join] = order_key(fmax);
    }
    if (t == 0) {
        s.n_cand = 0;
    }
    __syncthreads();
    if (wave_id() == 0) {
        uint32_t kk[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int i = lane_id() + g * WAVE;
            kk[g]       = i < n_slots ? slot_key[i] : 0u;
        }
        // The 2K-th largest of the maxima is an element with at least 2K elements at or above it: nothing below it
        // can be among the 2K best; so is any value below that one. (A group that saw no element reports -inf.)
        uint32_t P = 0u;
        for (int bit = 31; bit >= 8; --bit) {
            const uint32_t cand = P | (1u << bit);
            int            c    = 0;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                c += (int)__builtin_popcountll(__ballot(kk[g] >= cand));
            }
            P = c >= N ? cand : P;
        }
        if (lane_id() == 0) {
            double tot = 0.0;
            for (int w = 0; w < BR_WAVES; ++w) {
                tot += red[w];
            }
            row_sum   = tot;
            row_floor = P;
        }
    }
    __syncthreads();
    const uint32_t floor_key = row_floor;
    const float    floor_val = key_to_float(floor_key);
    const bool     all_pass  = floor_key <= order_key(-__builtin_inff());  // then NaN columns are wanted too
    stream_columns<DT, THREADS>(x + rb, 0, vocab, [&](int v, float xv) {
        const float e = beam_element_of<DT>(xv, bias, v);
        if (e >= floor_val || all_pass) {
            const int at = atomicAdd(&s.n_cand, 1);
            if (at < BM_CAP) {
                s.cand[at] = beam_key(e, (uint32_t)v);
            }
        }
    });
    __syncthreads();
    if (wave_id() >= BM_WAVES) {
        return;  // the first four waves select
    }
    const int passed = s.n_cand;
    const int take   = min(N, vocab);
    if (passed <= BM_CAP) {
        beam_select(s, [&](int i) { return s.cand[i]; }, passed, take);
    }
    else {
        // (rows of many equal values) the selection runs over the row itself
        beam_select(s, [&](int i) { return beam_key(beam_element<DT>(x, bias, rb, i), (uint32_t)i); }, vocab, take);
    }
    const float logd = det_logf((float)row_sum);
    if (t < N) {
        const unsigned long long k    = t < take ? s.out[t] : 0ull;
        cand_id[(size_t)row * N + t]  = (int)beam_key_position(k) + row * vocab;
        cand_val[(size_t)row * N + t] = round_t<DT>((beam_key_value(k) - m - logd) + cum);
    }
}

struct BeamHypsDevice {
    int*         output_ids_tgt;
    int*         sequence_lengths_tgt;
    float*       cum_log_probs;
    float*       normed_scores;
    float*       log_probs;
    float*       min_normed_scores;
    int*         num_beams;
    bool*        is_done;
    const int*   output_ids_src;
    const int*   parent_ids_src;
    const int*   end_ids;
    const float* log_probs_src;
    int          step;
    int          ite;
    int          batch_size;
    int          local_batch_size;
    int          max_seq_len;
    int          early_stopping;
};

// one workgroup per batch entry (:99-262)
template<int DT>
__global__ void __launch_bounds__(BM_THREADS)
beam_batch_kernel(const int* __restrict__ cand_id, const float* __restrict__ cand_val, int* __restrict__ ids,
                  float* cum_log_probs, float* __restrict__ output_log_probs, const bool* __restrict__ finished,
                  const int* __restrict__ sequence_lengths, BeamHypsDevice h, int K, int max_k2, int vocab,
                  float length_penalty, float diversity_rate)
{
    __shared__ BeamSelect s;
    __shared__ float      old_cum[64];
    __shared__ float      score_of[BM_MAX_N];
    const int             b = blockIdx.x;
    const int             t = threadIdx.x;
    const int             C = K * 2 * K;
    const int*            x = cand_id + (size_t)b * C;
    const float*          y = cand_val + (size_t)b * C;
    if (t < K) {
        old_cum[t] = cum_log_probs[b * K + t];
    }
    const bool with_hyps = h.num_beams != nullptr;
    const int  g         = h.ite * h.local_batch_size + b;
    if (with_hyps) {
        const int nb = h.num_beams[g];
        if (nb == 0 && t == 0) {
            h.min_normed_scores[g] = 3.402823466e+38f;
        }
        else if (nb == K) {
            return;
        }
    }
    // (:146-156) the batch entry's own flag and length are used for all of its beams, as in the reference
    float denom = 1.0f;
    if (length_penalty != 0.0f) {
        const int length = finished[b] ? sequence_lengths[b] : sequence_lengths[b] + 1;
        if (length != 1) {
            denom = round_t<DT>(det_expf(length_penalty * det_logf((float)length)));
        }
        else {
            length_penalty = 0.0f;
        }
    }
    const float div_t = round_t<DT>(diversity_rate);
    auto        score = [&](int c) {
        float elem = y[c];
        if (length_penalty != 0.0f) {
            elem = round_t<DT>(elem / denom);
        }
        return round_t<DT>(elem + round_t<DT>(div_t * round_t<DT>((float)(c % K))));
    };
    const int take = max_k2 < C ? max_k2 : C;
    beam_select(s, [&](int c) { return beam_key(score(c), (uint32_t)c); }, C, take);
    // what the walk reads about its candidates, fetched by one thread each
    __shared__ int   cand_x[BM_MAX_N];
    __shared__ float cand_y[BM_MAX_N];
    if (t < take) {
        const int p = (int)beam_key_position(s.out[t]);
        score_of[t] = score(p);
        cand_x[t]   = x[p];
        cand_y[t]   = y[p];
    }
    __syncthreads();
    if (t != 0) {
        return;
    }
    int*   z        = ids + (size_t)b * K;
    float* v        = cum_log_probs + (size_t)b * K;
    int    selected = 0;
    const int end_id = with_hyps ? h.end_ids[b] : -1;
    for (int i = 0; i < take; ++i) {
        const int   xp = cand_x[i];
        const float yp = cand_y[i];
        if (with_hyps && xp % vocab == end_id) {
            if (i < K) {
                const float normed_score = score_of[i];
                const int   num_beam     = h.num_beams[g];
                int         beam_idx     = num_beam;
                if (num_beam == K) {
                    if (normed_score < h.min_normed_scores[g]) {
                        selected = K;
                        break;
                    }
                    for (int j = 0; j < K; ++j) {
                        if (h.normed_scores[g * (K * 2) + j] == h.min_normed_scores[g]) {
                            beam_idx = j;
                            h.num_beams[g]--;
                            h.min_normed_scores[g]           = 3.402823466e+38f;
                            h.normed_scores[g * (K * 2) + j] = normed_score;
                            for (int l = 0; l < K; ++l) {
                                h.min_normed_scores[g] =
                                    __builtin_fminf(h.min_normed_scores[g], h.normed_scores[g * (K * 2) + l]);
                            }
                            break;
                        }
                    }
                }
                const size_t tgt = ((size_t)(b + h.ite * h.local_batch_size) * (K * 2) + beam_idx) * h.max_seq_len;
                h.output_ids_tgt[tgt + h.step] = end_id;
                if (h.log_probs != nullptr) {
                    h.log_probs[tgt + h.step] = yp - old_cum[(xp / vocab) % K];
                }
                int prev_id = (xp / vocab) % K;
                for (int j = h.step - 1; j >= 0; --j) {
                    const size_t src =
                        (size_t)j * h.batch_size * K + (size_t)h.ite * h.local_batch_size * K + (size_t)b * K + prev_id;
                    h.output_ids_tgt[tgt + j] = h.output_ids_src[src];
                    if (h.log_probs != nullptr && h.log_probs_src != nullptr) {
                        h.log_probs[tgt + j] = h.log_probs_src[src];
                    }
                    prev_id = h.parent_ids_src[src];
                }
                const int tgt_beam              = g * (K * 2) + beam_idx;
                h.sequence_lengths_tgt[tgt_beam] = h.step;
                h.normed_scores[tgt_beam]        = normed_score;
                h.min_normed_scores[g] = __builtin_fminf(h.min_normed_scores[g], h.normed_scores[tgt_beam]);
                h.num_beams[g]++;
                h.cum_log_probs[tgt_beam] = yp;
            }
        }
        else if ((with_hyps && i < 2 * K) || (!with_hyps && i < K)) {
            z[selected] = xp;
            if (output_log_probs != nullptr) {
                output_log_probs[b * K + selected] = yp - old_cum[(z[selected] / vocab) % K];
            }
            v[selected] = yp;
            selected++;
        }
        if (selected >= K) {
            break;
        }
    }
    if (with_hyps) {
        if (h.num_beams[b] < K) {
            h.is_done[b] = false;
        }
        else if (h.early_stopping) {
            h.is_done[b] = true;
        }
    }
}

// ---- the kernels around the step -----------------------------------------------------------------------------
// kernels/beam_search_penalty_kernels.cu:24-86 (add_bias_temperature, generic and half2 forms): one workgroup per
// (chunk, row); pad columns are masked in both forms here (the sampling layers' half2 form leaves them alone).
template<int DT>
__global__ void __launch_bounds__(BM_THREADS)
beam_bias_temperature_kernel(typename Storage<DT>::T* __restrict__ logits,
                             const typename Storage<DT>::T* __restrict__ bias, int V, int Vp, int chunk,
                             float temperature)
{
    typedef Storage<DT>   S;
    const int             row   = blockIdx.y;
    const float           inv   = 1.0f / (temperature + 1e-6f);
    const float           inv_t = round_t<DT>(inv);
    const bool            pairs = DT == DT_F16 && V % 2 == 0 && Vp % 2 == 0;
    const int             lo    = min(Vp, (int)blockIdx.x * chunk);
    const int             hi    = min(Vp, lo + chunk);
    typename S::T*        rowp  = logits + (size_t)row * Vp;
    transform_columns<DT, BM_THREADS>(rowp, lo, hi, [&](int v, float x) {
        if (v >= V) {
            return -S::max_t();
        }
        if (pairs) {
            const float y = bias != nullptr ? round_t<DT>(x + S::ld(bias[v])) : x;
            return y * inv_t;
        }
        const float b = bias != nullptr ? S::ld(bias[v]) : 0.0f;
        return round_t<DT>(x + b) * (DT == DT_F32 ? inv : inv_t);
    });
}

// :88-154 (apply_repetition_penalty): one workgroup per beam; thread 0 follows the beam back through parent_ids and
// computes every penalised value from the row as it is, then all threads store. Dynamic LDS: step values and ids.
template<int DT>
__global__ void __launch_bounds__(BM_THREADS)
beam_repetition_kernel(typename Storage<DT>::T* __restrict__ logits, int batch_size, int K, int Vp, int step,
                       const int* __restrict__ current_ids, const int* __restrict__ previous_ids,
                       const int* __restrict__ parent_ids, const int* __restrict__ input_lengths,
                       int max_input_length, float repetition_penalty, int additive)
{
    typedef Storage<DT>   S;
    extern __shared__ int beam_hist[];  // [step] ids, then [step] values
    int*                  idx  = beam_hist;
    float*                val  = reinterpret_cast<float*>(beam_hist + step);
    const int             t    = threadIdx.x;
    const int             r    = blockIdx.x;
    const int             b    = r / K;
    typename S::T*        row  = logits + (size_t)r * Vp;
    const int             len  = input_lengths != nullptr ? input_lengths[r] : max_input_length;
    if (t == 0) {
        const int   bbsize = batch_size * K;
        const float pen    = round_t<DT>(repetition_penalty);
        auto        penalised = [&](float x) {
            if (additive) {
                return round_t<DT>(x - pen);
            }
            return x > 0.0f ? round_t<DT>(x / pen) : round_t<DT>(x * pen);
        };
        int prev_id   = current_ids[r];
        idx[step - 1] = prev_id;
        val[step - 1] = penalised(S::ld(row[prev_id]));
        int beam      = r % K;
        for (int i = step - 2; i >= 0; --i) {
            if (i >= len && i < max_input_length) {
                continue;
            }
            beam    = parent_ids[(size_t)i * bbsize + b * K + beam];
            prev_id = previous_ids[(size_t)i * bbsize + b * K + beam];
            idx[i]  = prev_id;
            val[i]  = penalised(S::ld(row[prev_id]));
        }
    }
    __syncthreads();
    for (int i = t; i < step; i += BM_THREADS) {
        if (i >= len && i < max_input_length) {
            continue;
        }
        row[idx[i]] = S::st(val[i]);
    }
}

// :156-173 (apply_min_length_penalty)
template<int DT>
__global__ void beam_min_length_kernel(typename Storage<DT>::T* __restrict__ logits, int min_length,
                                       const int* __restrict__ end_ids, const int* __restrict__ sequence_lengths,
                                       int max_input_length, int K, int Vp, int rows)
{
    const int r = threadIdx.x + blockIdx.x * blockDim.x;
    if (r < rows && sequence_lengths[r] + 1 - max_input_length < min_length) {
        logits[(size_t)r * Vp + end_ids[r / K]] = Storage<DT>::st(-Storage<DT>::max_t());
    }
}

// layers/beam_search_layers/OnlineBeamSearchLayer.cu:24-61 (update_kernel): one wave per batch entry, so that what
// the reference leaves to the order of its threads is fixed: every row counts its token, then takes the length of
// the beam it continues; an entry with beam_width hypotheses is finished.
__global__ void __launch_bounds__(WAVE)
beam_update_kernel(bool* __restrict__ finished, int* __restrict__ parent_ids, int* __restrict__ sequence_length,
                   int* word_ids, int* output_ids, const int* __restrict__ num_beams, int ite, int hyps_local_batch,
                   int K, int Vp, const int* __restrict__ end_ids)
{
    __shared__ int counted[WAVE];
    const int      b = blockIdx.x;
    const int      k = threadIdx.x;
    const int      i = b * K + k;
    int            word = 0;
    if (k < K) {
        counted[k] = finished[i] ? sequence_length[i] : sequence_length[i] + 1;
        word       = word_ids[i];
    }
    __syncthreads();
    if (k < K) {
        // A slot the step left untouched (an entry that is complete, or one with fewer than K continuations) holds
        // whatever the caller's buffer held: a negative value counts as "this beam, its end token", so that no index
        // below leaves its range (the reference reads other rows' memory there; ids are absolute over the batch,
        // (entry * K + beam) * Vp + token, and any non-negative one is brought into range by the modulo).
        const bool valid   = word >= 0;
        const int  beam_id = valid ? (word / Vp) % K : k;
        const int  word_id = valid ? word % Vp : end_ids[b];
        const bool done    = num_beams != nullptr && num_beams[ite * hyps_local_batch + b] == K;
        sequence_length[i] = counted[beam_id];
        finished[i]        = done || word_id == end_ids[b];
        parent_ids[i]      = beam_id;
        word_ids[i]        = word_id;
        output_ids[i]      = word_id;
    }
}

// layers/beam_search_layers/BaseBeamSearchLayer.cu:22-49 (update_indir_cache_kernel)
__global__ void beam_indir_cache_kernel(int* __restrict__ tgt, const int* __restrict__ src,
                                        const int* __restrict__ beam_ids, const bool* __restrict__ finished,
                                        int start_step, int local_batch_size, int K, int max_seq_len, int step)
{
    int       time_step = threadIdx.x + blockIdx.x * blockDim.x;
    const int bb        = blockIdx.y;
    const int b         = bb / K;
    const int beam      = bb % K;
    if (bb >= K * local_batch_size || time_step >= min(step + 1, max_seq_len) || finished[bb]) {
        return;
    }
    time_step += start_step;
    const int    circ     = time_step % max_seq_len;
    const int    src_beam = beam_ids[b * K + beam];
    const size_t t_off    = (size_t)b * K * max_seq_len + (size_t)beam * max_seq_len + circ;
    const size_t s_off    = (size_t)b * K * max_seq_len + (size_t)src_beam * max_seq_len + circ;
    tgt[t_off]            = time_step == step ? beam : src[s_off];
}

}  // namespace ftk

using namespace ftk;

constexpr int BR_SHORT_ROW = 65536;
constexpr int BR_MANY_ROWS = 192;
#ifdef FTK_TEST_HOOKS
// Test hook (hooks build of the library only): 1 = sections of rows and three launches everywhere, 2 = one
// 1024-thread workgroup per row everywhere, 3 = one 512-thread workgroup per row everywhere, 0 = by the shape.
static int g_beam_path = 0;
extern "C" void ftk_test_set_beam_path(int v)
{
    g_beam_path = v;
}
#endif

extern "C" {

int ftk_invoke_topk_softmax(int dtype, const void* log_probs, const void* bias, const bool* finished,
                            const int* sequence_lengths, float* cum_log_probs, float* output_log_probs, int* ids,
                            void* temp_storage, size_t* temp_storage_size, const ftk_beam_hypotheses* beam_hyps,
                            int batch_size, int beam_width, int vocab_size, const int* end_ids, float diversity_rate,
                            float length_penalty, ftk_stream_t stream)
{
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (beam_width < 2 || beam_width > 64) {
        return FTK_ERR_ARGUMENT;  // the reference's launcher covers 1..64 (:650-688) and rejects 1 (:625)
    }
    if (batch_size < 0 || vocab_size < 2 * beam_width || (long long)batch_size * beam_width > 65535
        || (long long)batch_size * beam_width * vocab_size > 0x7FFFFFFFll) {
        return FTK_ERR_ARGUMENT;  // candidate ids are row * vocab + token in an int, as in the reference
    }
    const int      rows = batch_size * beam_width;
    const BeamPlan plan = beam_plan(rows, beam_width, vocab_size);
    if (temp_storage == nullptr) {
        if (temp_storage_size == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        *temp_storage_size = plan.bytes;
        return 0;
    }
    if (temp_storage_size != nullptr && *temp_storage_size < plan.bytes) {
        return FTK_ERR_WORKSPACE;
    }
    if (batch_size == 0) {
        return 0;
    }
    if (length_penalty != 0.0f && sequence_lengths == nullptr) {
        return FTK_ERR_ARGUMENT;  // (:572)
    }
    if (log_probs == nullptr || finished == nullptr || cum_log_probs == nullptr || ids == nullptr
        || end_ids == nullptr) {
        return FTK_ERR_ARGUMENT;  // the reference's kernels read and write all of these
    }
    if (beam_hyps != nullptr && beam_hyps->num_beams != nullptr
        && (beam_hyps->output_ids_tgt == nullptr || beam_hyps->sequence_lengths_tgt == nullptr
            || beam_hyps->cum_log_probs == nullptr || beam_hyps->normed_scores == nullptr
            || beam_hyps->min_normed_scores == nullptr || beam_hyps->is_done == nullptr
            || beam_hyps->end_ids == nullptr
            || (beam_hyps->step > 0 && (beam_hyps->output_ids_src == nullptr || beam_hyps->parent_ids_src == nullptr))
            || beam_hyps->step < 0 || beam_hyps->step >= beam_hyps->max_seq_len)) {
        return FTK_ERR_ARGUMENT;  // a hypothesis is written at position `step` of a max_seq_len-long row
    }
    char*               ws       = (char*)temp_storage;
    float*              pmax     = (float*)(ws + plan.off_pmax);
    double*             psum     = (double*)(ws + plan.off_psum);
    unsigned long long* pkeys    = (unsigned long long*)(ws + plan.off_pkeys);
    int*                cand_id  = (int*)(ws + plan.off_cand_id);
    float*              cand_val = (float*)(ws + plan.off_cand_val);
    hipStream_t         st       = (hipStream_t)stream;
    const int           N        = 2 * beam_width;
    const int           max_k    = beam_width <= 4 ? 4 : beam_width <= 8 ? 8 : beam_width <= 16 ? 16 : beam_width <= 32 ? 32 : 64;
    BeamHypsDevice      h        = {};
    if (beam_hyps != nullptr) {
        h.output_ids_tgt       = beam_hyps->output_ids_tgt;
        h.sequence_lengths_tgt = beam_hyps->sequence_lengths_tgt;
        h.cum_log_probs        = beam_hyps->cum_log_probs;
        h.normed_scores        = beam_hyps->normed_scores;
        h.log_probs            = beam_hyps->log_probs;
        h.min_normed_scores    = beam_hyps->min_normed_scores;
        h.num_beams            = beam_hyps->num_beams;
        h.is_done              = beam_hyps->is_done;
        h.output_ids_src       = beam_hyps->output_ids_src;
        h.parent_ids_src       = beam_hyps->parent_ids_src;
        h.end_ids              = beam_hyps->end_ids;
        h.log_probs_src        = beam_hyps->log_probs_src;
        h.step                 = beam_hyps->step;
        h.ite                  = beam_hyps->ite;
        h.batch_size           = beam_hyps->batch_size;
        h.local_batch_size     = beam_hyps->local_batch_size;
        h.max_seq_len          = beam_hyps->max_seq_len;
        h.early_stopping       = beam_hyps->early_stopping ? 1 : 0;
    }
    const dim3 sections(plan.parts, rows);
    // One 1024-thread workgroup per row does the work of the first three launches, except where a few long rows
    // would leave most compute units idle (measured on MI355X, f16: 32 rows of 128256 take 40 us that way and 34 us
    // in sections; 64 rows of 50257 27 against 30 us, 256 rows 29 against 36 us, 512 rows of 152064 112 against
    // 115 us).
    bool one_per_row = vocab_size <= BR_SHORT_ROW || rows >= BR_MANY_ROWS;
    bool half_size   = rows > 256;  // two 512-thread workgroups per compute unit
#ifdef FTK_TEST_HOOKS
    one_per_row = g_beam_path == 0 ? one_per_row : g_beam_path >= 2;
    half_size   = g_beam_path <= 1 ? half_size : g_beam_path == 3;
#endif
    FTK_DISPATCH_DTYPE(dtype, {
        typedef Storage<DT>::T T;
        if (one_per_row && half_size) {
            beam_rowwide_kernel<DT, BR_THREADS / 2><<<rows, BR_THREADS / 2, 0, st>>>(
                (const T*)log_probs, (const T*)bias, finished, end_ids, cum_log_probs, vocab_size, beam_width, cand_id,
                cand_val);
            FTK_LAUNCH_CHECK();
        }
        else if (one_per_row) {
            beam_rowwide_kernel<DT, BR_THREADS><<<rows, BR_THREADS, 0, st>>>(
                (const T*)log_probs, (const T*)bias, finished, end_ids, cum_log_probs, vocab_size, beam_width, cand_id,
                cand_val);
            FTK_LAUNCH_CHECK();
        }
        else {
            beam_section_max_kernel<DT><<<sections, BM_THREADS, 0, st>>>((const T*)log_probs, (const T*)bias, finished,
                                                                         vocab_size, plan.section, pmax);
            FTK_LAUNCH_CHECK();
            beam_section_kernel<DT><<<sections, BM_THREADS, 0, st>>>((const T*)log_probs, (const T*)bias, finished,
                                                                     vocab_size, plan.section, N, pmax, psum, pkeys);
            FTK_LAUNCH_CHECK();
            beam_row_kernel<DT><<<rows, BM_THREADS, 0, st>>>(finished, end_ids, cum_log_probs, vocab_size, beam_width,
                                                             plan.parts, pmax, psum, pkeys, cand_id, cand_val);
            FTK_LAUNCH_CHECK();
        }
        beam_batch_kernel<DT><<<batch_size, BM_THREADS, 0, st>>>(cand_id, cand_val, ids, cum_log_probs,
                                                                 output_log_probs, finished, sequence_lengths, h,
                                                                 beam_width, 2 * max_k, vocab_size, length_penalty,
                                                                 diversity_rate);
        FTK_LAUNCH_CHECK();
    });
    return 0;
}


int ftk_invoke_add_bias_apply_penalties(int dtype, int step, void* logits, const int* current_ids,
                                        const int* previous_ids, const int* parent_ids, const int* input_lengths,
                                        const int* sequence_lengths, const void* bias, int ite, int max_input_length,
                                        int local_batch_size, int batch_size, int beam_width, int vocab_size,
                                        int vocab_size_padded, const int* end_ids, float temperature,
                                        float repetition_penalty, int repetition_penalty_type, int min_length,
                                        ftk_stream_t stream)
{
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (local_batch_size < 0 || beam_width < 1 || vocab_size < 1 || vocab_size_padded < vocab_size || step < 0
        || (long long)local_batch_size * beam_width > 65535) {
        return FTK_ERR_ARGUMENT;
    }
    const int rows = local_batch_size * beam_width;
    if (rows == 0) {
        return 0;
    }
    if (logits == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    hipStream_t st = (hipStream_t)stream;
    if (bias != nullptr || temperature != 1.0f || vocab_size != vocab_size_padded) {
        int chunks = (1024 + rows - 1) / rows;
        chunks     = chunks < (vocab_size_padded + 8191) / 8192 ? chunks : (vocab_size_padded + 8191) / 8192;
        const int  chunk = ((vocab_size_padded + chunks - 1) / chunks + 7) / 8 * 8;
        const dim3 grid((vocab_size_padded + chunk - 1) / chunk, rows);
        FTK_DISPATCH_DTYPE(dtype, beam_bias_temperature_kernel<DT><<<grid, BM_THREADS, 0, st>>>(
                                      (Storage<DT>::T*)logits, (const Storage<DT>::T*)bias, vocab_size,
                                      vocab_size_padded, chunk, temperature));
        FTK_LAUNCH_CHECK();
    }
    const bool  additive = repetition_penalty_type == FTK_PENALTY_ADDITIVE;
    const float neutral  = repetition_penalty_type == FTK_PENALTY_MULTIPLICATIVE ? 1.0f : 0.0f;
    if (repetition_penalty_type != FTK_PENALTY_NONE && step > 0 && repetition_penalty != neutral) {
        if (current_ids == nullptr || (step > 1 && (previous_ids == nullptr || parent_ids == nullptr))) {
            return FTK_ERR_ARGUMENT;
        }
        const size_t smem = (size_t)step * 2 * sizeof(int);
        if (smem > 64 * 1024) {
            return FTK_ERR_ARGUMENT;  // a history of more than 8192 steps does not fit the kernel's table
        }
        FTK_DISPATCH_DTYPE(dtype, beam_repetition_kernel<DT><<<rows, BM_THREADS, smem, st>>>(
                                      (Storage<DT>::T*)logits, batch_size, beam_width, vocab_size_padded, step,
                                      current_ids, previous_ids,
                                      parent_ids != nullptr ? parent_ids + (size_t)ite * beam_width * local_batch_size :
                                                              nullptr,
                                      input_lengths, max_input_length, repetition_penalty, additive ? 1 : 0));
        FTK_LAUNCH_CHECK();
    }
    if (step - max_input_length < min_length) {
        if (sequence_lengths == nullptr || end_ids == nullptr) {
            return FTK_ERR_ARGUMENT;  // the reference checks the same two
        }
        FTK_DISPATCH_DTYPE(dtype, beam_min_length_kernel<DT><<<(rows + 255) / 256, 256, 0, st>>>(
                                      (Storage<DT>::T*)logits, min_length, end_ids, sequence_lengths, max_input_length,
                                      beam_width, vocab_size_padded, rows));
        FTK_LAUNCH_CHECK();
    }
    return 0;
}

int ftk_invoke_beam_update(bool* finished, int* parent_ids, int* sequence_length, int* word_ids, int* output_ids,
                           const ftk_beam_hypotheses* beam_hyps, int local_batch_size, int beam_width,
                           int vocab_size_padded, const int* end_ids, ftk_stream_t stream)
{
    if (local_batch_size < 0 || beam_width < 1 || beam_width > WAVE || vocab_size_padded < 1) {
        return FTK_ERR_ARGUMENT;
    }
    if (local_batch_size == 0) {
        return 0;
    }
    if (finished == nullptr || parent_ids == nullptr || sequence_length == nullptr || word_ids == nullptr
        || output_ids == nullptr || end_ids == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    const int* num_beams = beam_hyps != nullptr ? beam_hyps->num_beams : nullptr;
    beam_update_kernel<<<local_batch_size, WAVE, 0, (hipStream_t)stream>>>(
        finished, parent_ids, sequence_length, word_ids, output_ids, num_beams, beam_hyps != nullptr ? beam_hyps->ite : 0,
        beam_hyps != nullptr ? beam_hyps->local_batch_size : 0, beam_width, vocab_size_padded, end_ids);
    FTK_LAUNCH_CHECK();
    return 0;
}

int ftk_invoke_update_indir_cache(int* tgt_indir_cache, const int* src_indir_cache, const int* beam_ids,
                                  const bool* finished, int batch_dim, int local_batch_size, int beam_width,
                                  int max_seq_len, int step, ftk_stream_t stream)
{
    (void)batch_dim;
    if (local_batch_size < 0 || beam_width < 1 || max_seq_len < 1 || step < 0
        || (long long)local_batch_size * beam_width > 65535) {
        return FTK_ERR_ARGUMENT;
    }
    if (local_batch_size == 0) {
        return 0;
    }
    if (tgt_indir_cache == nullptr || src_indir_cache == nullptr || beam_ids == nullptr || finished == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    const int  start_step = step + 1 - max_seq_len > 0 ? step + 1 - max_seq_len : 0;
    const int  num_steps  = step + 1 < max_seq_len ? step + 1 : max_seq_len;
    const dim3 grid((num_steps + 63) / 64, local_batch_size * beam_width);
    beam_indir_cache_kernel<<<grid, 64, 0, (hipStream_t)stream>>>(tgt_indir_cache, src_indir_cache, beam_ids, finished,
                                                                  start_step, local_batch_size, beam_width, max_seq_len,
                                                                  step);
    FTK_LAUNCH_CHECK();
    return 0;
}

}  // extern "C"
