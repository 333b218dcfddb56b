// Top-k selection and sampling, shared by the stand-alone entry point and the fused decode step.
//
// Reference behaviour restated (src/fastertransformer/kernels/sampling_topk_kernels.cu:130-396):
// stage 1 splits a row into 8 interleaved slices (BS1-wide stripes) and extracts each slice's k
// largest values by k arg-max passes; stage 2 extracts the k largest of the 8k candidates the same
// way, then thread 0 samples by inverse CDF. With cub::BlockReduce and `a.u > b.u ? a : b`, equal
// values resolve to the highest thread id, so the picks follow two total orders:
//   stage 1, inside a slice : value desc, (i mod BS1) desc, i asc
//   stage 2, over positions : value desc, (pos mod BS2) desc, pos asc,  pos = slice*k + rank
// The reference reads the row k+2 times. Here the row is read once:
//   gather kernel  - grid (splits, rows), 256 threads, <= 64 elements per thread held in registers
//                    as order-preserving keys. A lower bound on the k-th largest value comes from
//                    the order statistics of the per-thread maxima; everything at or above it
//                    (typically ~100 elements per chunk) is written to a per-chunk candidate list.
//   select kernel  - one workgroup per row merges the lists, replays both tie orders on the
//                    candidates with two LDS bitonic sorts of 64-bit composite keys and samples.
// Rows whose candidates cannot be bounded (thousands of identical values around the k-th) take a
// literal, slow replay of the reference's passes.
#pragma once
#include "ftk_device.cuh"
#include "ftk_transform.cuh"

namespace ftk {

constexpr int TK_THREADS = 256;
constexpr int TK_ELEMS   = 64;    // elements per thread
constexpr int TK_MAXCAP  = 2048;  // candidates per chunk, upper limit
constexpr int TK_SELCAP  = 4096;  // candidates per row the select kernel sorts in LDS
constexpr int TK_MAXSPLIT = 64;

struct TopkChunkHeader {
    uint32_t count;       // entries written
    uint32_t threshold;   // every element of the chunk with key >= threshold is in the list
    uint32_t threshold8;  // 0, or a key with >= ceil(k/splits) elements of the chunk at or above it
    uint32_t flags;       // bit 0: count >= k, `threshold` bounds the row's k-th largest key from below
                          // bit 1: the chunk could not bound its candidates (row takes the literal replay)
};

struct TopkEntry {
    uint32_t key;
    uint32_t idx;
};

struct TopkPlan {
    int    splits;       // chunks per row
    int    nvt;          // 16-byte vectors per thread
    int    cap;          // candidate capacity per chunk
    size_t row_entries;  // TopkEntry slots per row
    size_t bytes;        // whole workspace
};

inline TopkPlan topk_plan(int vocab_padded, int batch, int max_top_k, int elem_bytes)
{
    TopkPlan  p;
    const int epv      = 16 / elem_bytes;
    const int nvt_max  = TK_ELEMS / epv;
    const int nvec     = vocab_padded / epv + 2;  // worst case over row misalignments
    const int s_min    = (nvec + TK_THREADS * nvt_max - 1) / (TK_THREADS * nvt_max);
    const int s_fill   = (2048 + batch - 1) / (batch > 0 ? batch : 1);  // aim at >= 2048 workgroups
    const int s_max    = (nvec + TK_THREADS - 1) / TK_THREADS;          // at least one vector per thread
    int       s        = s_min > s_fill ? s_min : s_fill;
    if (s > s_max) {
        s = s_max;
    }
    if (s > TK_MAXSPLIT) {
        s = TK_MAXSPLIT;
    }
    if (s < s_min) {
        s = s_min;  // very large vocabularies: more than TK_MAXSPLIT chunks
    }
    p.splits = s;
    p.nvt    = (nvec + s * TK_THREADS - 1) / (s * TK_THREADS);
    int cap  = 256;
    while (cap < 2 * max_top_k && cap < TK_MAXCAP) {
        cap <<= 1;
    }
    p.cap           = cap;
    size_t entries  = (size_t)s * cap;
    const size_t lit = (size_t)8 * (max_top_k > 0 ? max_top_k : 1);  // literal replay keeps 8k picks
    if (entries < lit) {
        entries = lit;
    }
    p.row_entries = entries;
    p.bytes       = (size_t)batch * (s * sizeof(TopkChunkHeader) + entries * sizeof(TopkEntry));
    return p;
}

// -------------------------------------------------------------------------------------------
// Row accessors: turn (column, raw storage value) into the value the reference would hand to top-k
// (an fp32 image of a `T`). PlainRow is the identity (stand-alone entry point); the fused decode
// step supplies one that applies masks and penalties on the fly.
//   prepare(lo, hi)        - once per workgroup, before streaming columns [lo, hi)
//   vector_bits(first, n)  - per 16-byte vector: one bit per column that needs the slow path
//   plain_vector(first, n) - true when every column of the vector takes fast()
//   fast(x)                - index-independent transform of an interior column
//   slow(v, x, bit)        - the full chain for column v
//   never_selected(v)      - column v is masked to -MAX_T whatever it holds (pad columns)
// -------------------------------------------------------------------------------------------
template<int DT>
struct PlainRow {
    typedef typename Storage<DT>::T T;
    const T*                        rowp;
    __device__ __forceinline__ void prepare(int lo, int hi) const
    {
        (void)lo;
        (void)hi;
    }
    __device__ __forceinline__ uint32_t vector_bits(int first, int n) const
    {
        (void)first;
        (void)n;
        return 0u;
    }
    __device__ __forceinline__ bool plain_vector(int first, int n) const
    {
        (void)first;
        (void)n;
        return true;
    }
    __device__ __forceinline__ bool has_vector_bits() const
    {
        return false;
    }
    // columns whose value is -MAX_T by construction need not be looked at
    __device__ __forceinline__ bool never_selected(int v) const
    {
        (void)v;
        return false;
    }
    __device__ __forceinline__ float fast(float x) const
    {
        return x;
    }
    __device__ __forceinline__ float slow(int v, float x, uint32_t bit) const
    {
        (void)v;
        (void)bit;
        return x;
    }
    __device__ __forceinline__ const T* data() const
    {
        return rowp;
    }
};

template<int DT>
__device__ __forceinline__ uint32_t min_valid_key()
{
    return order_key(-Storage<DT>::max_t()) + 1u;  // strict `>` against -MAX_T in TopK_2::insert
}

// -------------------------------------------------------------------------------------------
// gather: one chunk of one row.
// The chunk lives in registers as fp32 values; float comparisons already have the reference's
// semantics (-0 == +0, NaN never greater), so the streaming part costs a handful of VALU operations
// per element: transform, running maximum, one compare against the threshold. Order-preserving keys
// are only built for the ~100 elements that survive.
// Columns that need individual treatment (row edges, the vocabulary / padding boundary, the masked end
// id, columns with a history penalty) are evaluated once by a small rolled loop and parked in an LDS
// list; the unrolled register pass stays branch-free and small. Chunks the fast path cannot bound
// (fewer than k survivors, thousands of ties, an overfull list) go to topk_gather_rare, which works
// from memory with rolled loops.
// -------------------------------------------------------------------------------------------
constexpr int TK_SLOWCAP = 2048;  // columns per chunk that may take the per-column path

struct TopkGatherShared {
    uint32_t red[16];
    int      cnt;
    int      n_slow;
    int      slow_v[TK_SLOWCAP];
    float    slow_x[TK_SLOWCAP];
};

// value of column v as top-k sees it, re-read from memory
template<int DT, class Row>
__device__ __forceinline__ float topk_value_at(const Row& rowctx, int v)
{
    return rowctx.slow(v, Storage<DT>::ld(rowctx.data()[v]), rowctx.vector_bits(v, 1));
}

// Threshold search by bisection on the key over columns [lo_col, hi_col), then compaction; everything is
// recomputed from memory (the chunk sits in L2), nothing depends on the caller's registers.
template<int DT, class Row>
__device__ __noinline__ void topk_gather_rare(const Row& rowctx, TopkGatherShared& s, int k, int lo_col, int hi_col,
                                              int cap, uint32_t thr, uint32_t thr8, TopkChunkHeader* header,
                                              TopkEntry* entries)
{
    const int      t    = threadIdx.x;
    const uint32_t KMIN = min_valid_key<DT>();
    auto count_ge = [&](uint32_t thr_key) -> int {
        const float thr_f = key_to_float(thr_key);
        int         c     = 0;
        for (int v = lo_col + t; v < hi_col; v += TK_THREADS) {
            c += topk_value_at<DT>(rowctx, v) >= thr_f ? 1 : 0;
        }
        return block_sum_i(c, (int*)s.red);
    };
    uint32_t cmax = 0u;
    for (int v = lo_col + t; v < hi_col; v += TK_THREADS) {
        const uint32_t kk = order_key(topk_value_at<DT>(rowctx, v));
        cmax              = kk > cmax ? kk : cmax;
    }
    cmax              = block_max<uint32_t>(cmax, s.red, 0u);
    const int n_valid = count_ge(KMIN);
    const int kneed   = k < n_valid ? k : n_valid;
    int       cnt     = count_ge(thr);
    bool      ok      = cnt >= kneed && cnt <= cap;
    if (!ok) {
        uint32_t lo, hi;  // count(lo) > cap (or lo == KMIN); count(hi) < kneed
        if (cnt > cap) {
            lo = thr;
            hi = cmax + 1u;
        }
        else {
            lo = KMIN;
            hi = thr;
            if (n_valid <= cap) {
                thr = KMIN;
                ok  = true;
            }
        }
        while (!ok && hi - lo > 1u) {
            const uint32_t mid = lo + (hi - lo) / 2u;
            const int      c   = count_ge(mid);
            if (c > cap) {
                lo = mid;
            }
            else if (c < kneed) {
                hi = mid;
            }
            else {
                thr = mid;
                ok  = true;
            }
        }
    }
    cnt = 0;
    if (ok) {
        const float thr_f = key_to_float(thr);
        if (t == 0) {
            s.cnt = 0;
        }
        __syncthreads();
        for (int v = lo_col + t; v < hi_col; v += TK_THREADS) {
            const float xv = topk_value_at<DT>(rowctx, v);
            if (xv >= thr_f) {
                const int slot = atomicAdd(&s.cnt, 1);
                if (slot < cap) {
                    entries[slot] = TopkEntry{order_key(xv), (uint32_t)v};
                }
            }
        }
        __syncthreads();
        cnt = s.cnt;
    }
    if (t == 0) {
        TopkChunkHeader h;
        h.count      = ok ? (uint32_t)cnt : 0u;
        h.threshold  = thr;
        h.threshold8 = thr8;
        h.flags      = ((ok && cnt >= k) ? 1u : 0u) | (ok ? 0u : 2u);
        *header      = h;
    }
}

template<int DT, class Row>
__device__ __forceinline__ void topk_gather_chunk(Row& rowctx, int vocab, int k, int chunk, int splits, int nvt,
                                                  int cap, TopkChunkHeader* header, TopkEntry* entries)
{
    typedef Storage<DT>         S;
    typedef typename S::T       T;
    constexpr int               EPV = (int)(16 / sizeof(T));
    constexpr int               NVT = TK_ELEMS / EPV;
    __shared__ TopkGatherShared s;
    const int                   t = threadIdx.x;

    const T*       rowp     = rowctx.data();
    const int      a        = (int)(((uintptr_t)rowp & 15u) / sizeof(T));  // columns between the aligned base and column 0
    const uint4*   base     = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(rowp) - a * sizeof(T));
    const int      nvec     = (a + vocab + EPV - 1) / EPV;
    const int      vfull_lo = (a + EPV - 1) / EPV;  // vectors [vfull_lo, vfull_hi) lie entirely inside the row
    const int      vfull_hi = (a + vocab) / EPV;
    const bool     any_full = vfull_hi > vfull_lo;
    const int      vec0     = chunk * nvt * TK_THREADS;
    const uint32_t KMIN     = min_valid_key<DT>();
    const float    NEG_INF  = -__builtin_inff();
    const int      lo_col   = max(0, vec0 * EPV - a);
    const int      hi_col   = max(lo_col, min(vocab, (vec0 + nvt * TK_THREADS) * EPV - a));

    // A chunk is "plain" when every one of its vectors lies inside the row and no column needs an
    // index-dependent rule (pads, masked end id, bias): true for all but a handful of chunks per row.
    // Plain chunks run a loop without per-vector index checks.
    const bool chunk_plain = any_full && nvt == NVT && vec0 >= vfull_lo && vec0 + NVT * TK_THREADS <= vfull_hi
                             && rowctx.plain_vector(lo_col, hi_col - lo_col);

    // ---- load: every vector load is issued before the first use. Lanes whose vector is not entirely
    // inside the row read a harmless in-row vector instead and visit their columns one by one.
    uint4 raw[NVT];
    if (chunk_plain) {
        const uint4* p0 = base + vec0 + t;
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            raw[it] = p0[it * TK_THREADS];
        }
    }
    else if (any_full) {
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            const int  vi   = vec0 + it * TK_THREADS + t;
            const bool full = it < nvt && vi >= vfull_lo && vi < vfull_hi;
            raw[it]         = base[full ? vi : vfull_lo];
        }
    }
    else {
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            raw[it] = make_uint4(0, 0, 0, 0);
        }
    }
    // per-workgroup side data of the row (e.g. the history bitmap) while the loads are in flight
    if (t == 0) {
        s.n_slow = 0;
    }
    rowctx.prepare(lo_col, hi_col);
    __syncthreads();

    float    x[TK_ELEMS];
    float    tmax     = NEG_INF;
    uint32_t slowmask = 0u;  // bit `it`: vector `it` of this thread takes the per-column path
    if (chunk_plain && !rowctx.has_vector_bits()) {
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            const T* e = reinterpret_cast<const T*>(&raw[it]);
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                x[it * EPV + j] = rowctx.fast(S::ld(e[j]));
                tmax            = __builtin_fmaxf(tmax, x[it * EPV + j]);  // NaN never becomes the maximum
            }
        }
    }
    else if (chunk_plain) {
        const int first0 = (vec0 + t) * EPV - a;
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            const T*   e     = reinterpret_cast<const T*>(&raw[it]);
            const bool fastv = rowctx.vector_bits(first0 + it * TK_THREADS * EPV, EPV) == 0u;
            slowmask |= fastv ? 0u : (1u << it);
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                const float v   = rowctx.fast(S::ld(e[j]));
                x[it * EPV + j] = fastv ? v : NEG_INF;
                tmax            = __builtin_fmaxf(tmax, x[it * EPV + j]);
            }
        }
    }
    else {
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            const int  vi    = vec0 + it * TK_THREADS + t;
            const int  first = vi * EPV - a;
            const T*   e     = reinterpret_cast<const T*>(&raw[it]);
            const bool live  = it < nvt && vi < nvec;
            const bool fastv = live && any_full && vi >= vfull_lo && vi < vfull_hi && rowctx.plain_vector(first, EPV)
                               && rowctx.vector_bits(first, EPV) == 0u;
            slowmask |= (live && !fastv) ? (1u << it) : 0u;
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                const float v   = rowctx.fast(S::ld(e[j]));
                x[it * EPV + j] = fastv ? v : NEG_INF;
                tmax            = __builtin_fmaxf(tmax, x[it * EPV + j]);
            }
        }
    }
    // per-column path: evaluate once, park in LDS
    bool slow_overflow = false;
    for (uint32_t m = slowmask; m != 0u; m &= m - 1u) {
        const int it    = __builtin_ctz(m);
        const int first = (vec0 + it * TK_THREADS + t) * EPV - a;
        for (int j = 0; j < EPV; ++j) {
            const int v = first + j;
            if (v >= 0 && v < vocab && !rowctx.never_selected(v)) {
                const float xv   = topk_value_at<DT>(rowctx, v);
                tmax             = __builtin_fmaxf(tmax, xv);
                const int   slot = atomicAdd(&s.n_slow, 1);
                if (slot < TK_SLOWCAP) {
                    s.slow_v[slot] = v;
                    s.slow_x[slot] = xv;
                }
                else {
                    slow_overflow = true;
                }
            }
        }
    }

    // ---- lower bounds from thread maxima. Each wave sorts its 64 maxima; the q-th largest of each wave,
    // minimised over the 4 waves, has >= 4q elements of the chunk at or above it.
    //   thr  (q  = ceil(k/4))          : >= k elements        -> everything >= thr goes to the candidate list
    //   thr8 (qs = ceil(k/(4*splits))) : >= k/splits elements -> the smallest one over the row's chunks has
    //                                    >= k elements above it; lets the select kernel tighten its bound
    const uint32_t sorted = wave_sort_desc(order_key(tmax));
    const int      q      = k <= 4 * WAVE ? (k + 3) / 4 : WAVE;
    int            qs     = (k + 4 * splits - 1) / (4 * splits);
    qs                    = qs < 1 ? 1 : qs;
    uint32_t thr  = block_min<uint32_t>(__shfl(sorted, q - 1, WAVE), s.red, 0xFFFFFFFFu);
    uint32_t thr8 = block_min<uint32_t>(__shfl(sorted, (qs <= WAVE ? qs : WAVE) - 1, WAVE), s.red, 0xFFFFFFFFu);
    if (thr < KMIN) {
        thr = KMIN;
    }
    if (thr8 < KMIN || qs > WAVE) {
        thr8 = 0u;  // no guarantee
    }

    // ---- compaction. x >= key_to_float(thr)  <=>  order_key(x) >= thr (NaN fails both)
    const float thr_f = key_to_float(thr);
    if (t == 0) {
        s.cnt = 0;
    }
    __syncthreads();  // also publishes the slow list
    auto push = [&](int v, float xv) {
        const int slot = atomicAdd(&s.cnt, 1);
        if (slot < cap) {
            entries[slot] = TopkEntry{order_key(xv), (uint32_t)v};
        }
    };
    // survivors of the register pass: one bit per vector whose maximum reaches the threshold, then a
    // rolled loop that re-reads those few vectors column by column
    uint32_t hits = 0u;
#pragma unroll
    for (int it = 0; it < NVT; ++it) {
        float vmax = x[it * EPV];
#pragma unroll
        for (int j = 1; j < EPV; ++j) {
            vmax = __builtin_fmaxf(vmax, x[it * EPV + j]);
        }
        hits |= vmax >= thr_f ? (1u << it) : 0u;
    }
    for (; hits != 0u; hits &= hits - 1u) {
        const int it    = __builtin_ctz(hits);
        const int first = (vec0 + it * TK_THREADS + t) * EPV - a;
        for (int j = 0; j < EPV; ++j) {
            const float xv = rowctx.fast(S::ld(rowp[first + j]));
            if (xv >= thr_f) {
                push(first + j, xv);
            }
        }
    }
    const int n_slow = s.n_slow < TK_SLOWCAP ? s.n_slow : TK_SLOWCAP;
    for (int i = t; i < n_slow; i += TK_THREADS) {
        if (s.slow_x[i] >= thr_f) {
            push(s.slow_v[i], s.slow_x[i]);
        }
    }
    const int any_overflow = __syncthreads_or(slow_overflow ? 1 : 0);
    const int cnt          = s.cnt;
    if (cnt >= k && cnt <= cap && !any_overflow) {
        if (t == 0) {
            TopkChunkHeader h;
            h.count      = (uint32_t)cnt;
            h.threshold  = thr;
            h.threshold8 = thr8;
            h.flags      = 1u;
            *header      = h;
        }
        return;
    }
    __syncthreads();
    topk_gather_rare<DT, Row>(rowctx, s, k, lo_col, hi_col, cap, thr, thr8, header, entries);
}

// -------------------------------------------------------------------------------------------
// select: merge, replay the reference's two tie orders, sample
// -------------------------------------------------------------------------------------------
struct TopkSelectShared {
    unsigned long long keys[TK_SELCAP];  // 32 KB
    int                idx[TK_SELCAP];   // 16 KB
    __attribute__((aligned(16))) float w[1024];
    unsigned long long red64[16];
    uint32_t           red32[16];
    int                slice_count[8];
    int                counter;
    int                misc[4];
};

struct TopkOutputs {
    int*   ids;
    int*   sequence_length;
    bool*  finished;
    float* cum_log_probs;
    float* output_log_probs;
};

// thread 0 only: weights w[0..n) in selection order -> sampled position (sampling_topk_kernels.cu:282-311).
// `w` is 16-byte aligned LDS, zero padded to a multiple of 4 (adding +0 to a non-negative sum is exact),
// so the strictly sequential sum runs from registers loaded four at a time.
__device__ __forceinline__ int topk_sample_walk(const float* w, int n, float u, float p, float* s_sum_out)
{
    const float4* w4    = reinterpret_cast<const float4*>(w);
    const int     n4    = (n + 3) >> 2;
    float         s_sum = 0.0f;
#pragma unroll 4
    for (int i = 0; i < n4; ++i) {
        const float4 v = w4[i];
        s_sum          = s_sum + v.x;
        s_sum          = s_sum + v.y;
        s_sum          = s_sum + v.z;
        s_sum          = s_sum + v.w;
    }
    float rand_num = u * p * s_sum;
    int   pick     = n - 1;
    for (int i = 0; i < n; ++i) {
        rand_num = rand_num - w[i];
        if (rand_num <= 0.0f || i == n - 1) {
            pick = i;
            break;
        }
    }
    *s_sum_out = s_sum;
    return pick;
}

__device__ __forceinline__ void topk_emit(const TopkOutputs& o, int row, int id, bool probs_in, float w, float s_sum,
                                          const int* end_ids, bool any_valid)
{
    o.ids[row] = id;
    if (probs_in && any_valid) {
        const float lp = det_logf(w);
        if (o.cum_log_probs != nullptr) {
            o.cum_log_probs[row] += lp;
        }
        if (o.output_log_probs != nullptr) {
            o.output_log_probs[row] = lp - det_logf(s_sum);
        }
    }
    if (o.sequence_length != nullptr && o.finished != nullptr) {
        o.sequence_length[row] = o.finished[row] ? o.sequence_length[row] : o.sequence_length[row] + 1;
        o.finished[row]        = id == end_ids[row];
    }
}

// Literal replay for rows the gather could not bound. `Row::key_at(v)` re-reads the row.
// Every pick is the smallest composite key strictly greater than the previous pick, where the
// composite encodes the reference's order; picks of stage 1 go to `picks` (8k entries, global).
template<int DT, class Row>
__device__ void topk_literal(Row& rowctx, TopkSelectShared& s, int vocab, int k, int BS1, int BS2,
                             TopkEntry* picks, int* n_list_out)
{
    const int      t    = threadIdx.x;
    const uint32_t KMIN = min_valid_key<DT>();
    rowctx.prepare_whole_row();
    // stage 1
    for (int slice = 0; slice < 8; ++slice) {
        unsigned long long last = 0ull;
        bool               have_last = false;
        for (int ite = 0; ite < k; ++ite) {
            unsigned long long best = ~0ull;
            // elements of this slice: i = (j*8 + slice)*BS1 + tt
            for (int blk = slice; blk * BS1 < vocab; blk += 8) {
                for (int tt = t; tt < BS1; tt += TK_THREADS) {
                    const int i = blk * BS1 + tt;
                    if (i < vocab) {
                        const uint32_t kk = rowctx.key_at(i);
                        if (kk >= KMIN) {
                            const unsigned long long c = ((unsigned long long)(~kk) << 29)
                                                         | ((unsigned long long)(BS1 - 1 - tt) << 21)
                                                         | (unsigned long long)(blk / 8);
                            if ((!have_last || c > last) && c < best) {
                                best = c;
                            }
                        }
                    }
                }
            }
            best = ~block_max<unsigned long long>(~best, s.red64, 0ull);
            if (t == 0) {
                TopkEntry e{0u, 0xFFFFFFFFu};
                if (best != ~0ull) {
                    const uint32_t kk = ~(uint32_t)(best >> 29);
                    const int      tt = BS1 - 1 - (int)((best >> 21) & 0xFFull);
                    const int      j  = (int)(best & 0x1FFFFFull);
                    e.key             = kk;
                    e.idx             = (uint32_t)((j * 8 + slice) * BS1 + tt);
                }
                picks[slice * k + ite] = e;
            }
            if (best == ~0ull) {
                // slice exhausted: remaining picks are empty
                for (int r = ite + 1 + t; r < k; r += TK_THREADS) {
                    picks[slice * k + r] = TopkEntry{0u, 0xFFFFFFFFu};
                }
                break;
            }
            last      = best;
            have_last = true;
        }
    }
    __threadfence_block();
    __syncthreads();
    // stage 2: first k of the 8k positions under (key desc, pos % BS2 desc, pos asc)
    unsigned long long last = 0ull;
    bool               have_last = false;
    int                n_list = 0;
    for (int ite = 0; ite < k; ++ite) {
        unsigned long long best = ~0ull;
        for (int pos = t; pos < 8 * k; pos += TK_THREADS) {
            const TopkEntry e = picks[pos];
            if (e.idx != 0xFFFFFFFFu) {
                const unsigned long long c = ((unsigned long long)(~e.key) << 32)
                                             | ((unsigned long long)(BS2 - 1 - pos % BS2) << 24)
                                             | (unsigned long long)pos;
                if ((!have_last || c > last) && c < best) {
                    best = c;
                }
            }
        }
        best = ~block_max<unsigned long long>(~best, s.red64, 0ull);
        if (best == ~0ull) {
            break;
        }
        if (t == 0) {
            const int pos = (int)(best & 0xFFFFFFull);
            s.keys[ite]   = (unsigned long long)(~picks[pos].key) << 32;
            s.idx[ite]    = (int)picks[pos].idx;
        }
        last      = best;
        have_last = true;
        n_list++;
    }
    __syncthreads();
    *n_list_out = n_list;
}

template<int DT, class Row>
__device__ __forceinline__ void topk_select_row(Row& rowctx, TopkSelectShared& s, int row, int vocab, int k,
                                                float p, int max_top_k, int splits, const TopkChunkHeader* headers,
                                                TopkEntry* entries, int cap, bool probs_in, float u,
                                                const int* end_ids, const TopkOutputs& out)
{
    const int t   = threadIdx.x;
    const int BS1 = max_top_k <= 16 ? 128 : 256;
    const int BS2 = max_top_k <= 32 ? 128 : 256;

    // ---- merge chunk headers
    // Row-wide lower bound T0 of the k-th largest key. Two valid bounds, take the larger:
    //   any chunk's `threshold` with >= k elements above it;
    //   the smallest `threshold8` when every chunk has one (splits x ceil(k/splits) >= k elements).
    // A list is complete above its own `threshold` (lists of chunks with fewer than k valid elements
    // hold all of them), and T0 is never below the threshold of a list that was cut.
    uint32_t T0       = min_valid_key<DT>();
    uint32_t min8     = 0xFFFFFFFFu;
    bool     overflow = false;
    for (int c = 0; c < splits; ++c) {
        const TopkChunkHeader h = headers[c];
        overflow                = overflow || (h.flags & 2u) != 0u;
        min8                    = h.threshold8 < min8 ? h.threshold8 : min8;
        if ((h.flags & 1u) && h.threshold > T0) {
            T0 = h.threshold;
        }
    }
    if (min8 > T0) {
        T0 = min8;  // min8 == 0 when some chunk has no threshold8
    }
    int  n_list  = 0;  // length of the final ordered list: values in s.w (as fp32), ids in s.idx
    bool literal = overflow;
    int  n       = 0;

    // candidates at or above a threshold over all chunk lists -> LDS with the stage-1 composite key
    //   slice(3) | ~key(32) | BS1-1-t (8) | j (21),   i = (j*8 + slice)*BS1 + t
    auto gather = [&](uint32_t thr) -> int {
        if (t < 8) {
            s.slice_count[t] = 0;
        }
        if (t == 0) {
            s.counter = 0;
        }
        __syncthreads();
        for (int ch = 0; ch < splits; ++ch) {
            const int        cnt = (int)headers[ch].count;
            const TopkEntry* e   = entries + (size_t)ch * cap;
            for (int i = t; i < cnt; i += TK_THREADS) {
                const TopkEntry en = e[i];
                if (en.key >= thr) {
                    const int idx   = (int)en.idx;
                    const int blk   = idx / BS1;
                    const int tt    = idx - blk * BS1;
                    const int slice = blk & 7;
                    const int slot  = atomicAdd(&s.counter, 1);
                    if (slot < TK_SELCAP) {
                        atomicAdd(&s.slice_count[slice], 1);
                        s.keys[slot] = ((unsigned long long)slice << 61) | ((unsigned long long)(~en.key) << 29)
                                       | ((unsigned long long)(BS1 - 1 - tt) << 21) | (unsigned long long)(blk >> 3);
                    }
                }
            }
        }
        __syncthreads();
        const int total = s.counter;
        __syncthreads();
        return total;
    };

    if (!literal) {
        n = gather(T0);
        if (n > TK_SELCAP) {
            // every chunk had to keep >= k candidates (k in the hundreds): find the exact k-th largest
            // key by bisection over the lists, then gather again
            auto count_ge = [&](uint32_t thr) -> int {
                int c = 0;
                for (int ch = 0; ch < splits; ++ch) {
                    const int        cnt = (int)headers[ch].count;
                    const TopkEntry* e   = entries + (size_t)ch * cap;
                    for (int i = t; i < cnt; i += TK_THREADS) {
                        c += e[i].key >= thr ? 1 : 0;
                    }
                }
                return block_sum_i(c, (int*)s.red32);
            };
            uint32_t lo = T0, hi = 0xFFFFFFFFu;  // count(lo) >= k always holds
            while (hi - lo > 1u) {
                const uint32_t mid = lo + (hi - lo) / 2u;
                if (count_ge(mid) >= k) {
                    lo = mid;
                }
                else {
                    hi = mid;
                }
            }
            T0 = lo;
            n  = gather(T0);
        }
        if (n > TK_SELCAP) {
            literal = true;  // thousands of identical values around the k-th
        }
    }

    if (!literal) {
        int slice_start[8];
        {
            int acc = 0;
#pragma unroll
            for (int sl = 0; sl < 8; ++sl) {
                slice_start[sl] = acc;
                acc += s.slice_count[sl];
            }
        }
        // decode a stage-1 composite at sorted position q into (vocabulary index, stage-2 composite)
        //   stage 2: ~key(32) | BS2-1-pos%BS2 (8) | pos/BS2 (12) | payload (12),  pos = slice*k + rank
        auto stage2_key = [&](unsigned long long c, int q, int payload, int* idx_out) -> unsigned long long {
            const int      slice = (int)(c >> 61);
            const uint32_t ikey  = (uint32_t)(c >> 29);
            const int      tt    = BS1 - 1 - (int)((c >> 21) & 0xFFull);
            const int      j     = (int)(c & 0x1FFFFFull);
            int            start = 0;
#pragma unroll
            for (int sl = 0; sl < 8; ++sl) {
                start = sl == slice ? slice_start[sl] : start;
            }
            const int r = q - start;
            *idx_out    = (j * 8 + slice) * BS1 + tt;
            if (r >= k) {
                return ~0ull;
            }
            const int pos = slice * k + r;
            return ((unsigned long long)ikey << 32) | ((unsigned long long)(BS2 - 1 - pos % BS2) << 24)
                   | ((unsigned long long)(pos / BS2) << 12) | (unsigned long long)payload;
        };

        if (n <= TK_THREADS) {
            // ---- small candidate sets (the usual case): rank by counting, one candidate per thread.
            // Composite keys are unique, so "number of smaller keys" is the sorted position.
            const unsigned long long mine = t < n ? s.keys[t] : ~0ull;
            int                      q    = 0;
            for (int j = 0; j < n; ++j) {
                q += s.keys[j] < mine ? 1 : 0;
            }
            int                      my_idx = 0;
            const unsigned long long k2     = t < n ? stage2_key(mine, q, 0, &my_idx) : ~0ull;
            __syncthreads();
            s.keys[t] = k2;
            __syncthreads();
            int q2 = 0;
            for (int j = 0; j < n; ++j) {
                q2 += s.keys[j] < k2 ? 1 : 0;
            }
            const bool kept = k2 != ~0ull;
            n_list          = block_sum_i(kept ? 1 : 0, (int*)s.red32);
            n_list          = n_list < k ? n_list : k;
            if (kept && q2 < n_list) {
                s.w[q2]   = key_to_float(~(uint32_t)(k2 >> 32));
                s.idx[q2] = my_idx;
            }
            __syncthreads();
        }
        else {
            // ---- large candidate sets: two bitonic sorts
            const int np2 = max(2, next_pow2(n));
            for (int i = n + t; i < np2; i += TK_THREADS) {
                s.keys[i] = ~0ull;
            }
            __syncthreads();
            block_bitonic_sort_u64(s.keys, np2);
            for (int qi = t; qi < np2; qi += TK_THREADS) {
                unsigned long long nk = ~0ull;
                if (qi < n) {
                    int idx;
                    nk        = stage2_key(s.keys[qi], qi, qi, &idx);
                    s.idx[qi] = idx;
                }
                s.keys[qi] = nk;
            }
            __syncthreads();
            block_bitonic_sort_u64(s.keys, np2);
            {
                int cnt = 0;
                for (int i = t; i < min(k, n); i += TK_THREADS) {
                    cnt += s.keys[i] != ~0ull ? 1 : 0;
                }
                n_list = block_sum_i(cnt, (int*)s.red32);
            }
            // resolve the payload (position in the first sort) into the vocabulary index
            int   my_idx[4];
            float my_val[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = t + r * TK_THREADS;
                my_idx[r]   = i < n_list ? s.idx[(int)(s.keys[i] & 0xFFFull)] : 0;
                my_val[r]   = i < n_list ? key_to_float(~(uint32_t)(s.keys[i] >> 32)) : 0.0f;
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = t + r * TK_THREADS;
                if (i < n_list) {
                    s.idx[i] = my_idx[r];
                    s.w[i]   = my_val[r];
                }
            }
            __syncthreads();
        }
    }
    else {
        topk_literal<DT, Row>(rowctx, s, vocab, k, BS1, BS2, entries, &n_list);
        for (int i = t; i < n_list; i += TK_THREADS) {
            s.w[i] = key_to_float(~(uint32_t)(s.keys[i] >> 32));
        }
        __syncthreads();
    }

    // ---- weights (sampling_topk_kernels.cu:264-279): exp(x - max) on logits, the value itself on
    // probabilities; the list is padded with zero weights to a multiple of 4 for the vectorised walk
    const float x0 = n_list > 0 ? s.w[0] : 0.0f;
    __syncthreads();
    for (int i = t; i < ((n_list + 3) & ~3); i += TK_THREADS) {
        const float x = i < n_list ? s.w[i] : 0.0f;
        s.w[i]        = i < n_list ? (probs_in ? x : det_expf(x - x0)) : 0.0f;
    }
    __syncthreads();
    if (t == 0) {
        if (n_list == 0) {
            topk_emit(out, row, 0, probs_in, 0.0f, 0.0f, end_ids, false);
        }
        else {
            float     s_sum;
            const int pick = topk_sample_walk(s.w, n_list, u, p, &s_sum);
            topk_emit(out, row, s.idx[pick] % vocab, probs_in, s.w[pick], s_sum, end_ids, true);
        }
    }
}

}  // namespace ftk
