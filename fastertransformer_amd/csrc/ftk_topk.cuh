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
    uint32_t count;      // entries written
    uint32_t threshold;  // every element of the chunk with key >= threshold is in the list
    uint32_t bound_ok;   // count >= k: `threshold` is a lower bound of the row's k-th largest key
    uint32_t overflow;   // the chunk could not bound its candidates
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
// Row accessors: map (column, raw storage value) to the order-preserving key of the value the
// reference would hand to top-k. PlainRow is the identity (stand-alone entry point); the fused
// decode step supplies one that applies masks and penalties on the fly.
// -------------------------------------------------------------------------------------------
template<int DT>
struct PlainRow {
    typedef typename Storage<DT>::T T;
    const T*                        rowp;
    // per-vector side information (none for a plain row)
    __device__ __forceinline__ uint32_t vector_bits(int first, int n) const
    {
        (void)first;
        (void)n;
        return 0u;
    }
    __device__ __forceinline__ uint32_t key(int v, T raw, uint32_t bit) const
    {
        (void)v;
        (void)bit;
        return order_key(Storage<DT>::ld(raw));
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
// gather: one chunk of one row
// -------------------------------------------------------------------------------------------
template<int DT, class Row>
__device__ __forceinline__ void topk_gather_chunk(const Row& rowctx, int vocab, int k, int chunk, int nvt, int cap,
                                                  TopkChunkHeader* header, TopkEntry* entries)
{
    typedef typename Storage<DT>::T T;
    constexpr int                   EPV = (int)(16 / sizeof(T));
    constexpr int                   NVT = TK_ELEMS / EPV;
    __shared__ uint32_t             s_red[16];
    __shared__ int                  s_cnt;
    const int                       t = threadIdx.x;

    const T*        rowp   = rowctx.data();
    const uintptr_t addr   = (uintptr_t)rowp;
    const int       a      = (int)((addr & 15u) / sizeof(T));  // elements between the aligned base and column 0
    const uint4*    base   = reinterpret_cast<const uint4*>(addr & ~(uintptr_t)15u);
    const int       nvec   = (a + vocab + EPV - 1) / EPV;
    const int       vec0   = chunk * nvt * TK_THREADS;
    const uint32_t  KMIN   = min_valid_key<DT>();

    // ---- load: all vector loads are issued before the first use
    uint4 raw[NVT];
#pragma unroll
    for (int it = 0; it < NVT; ++it) {
        const int vi = vec0 + it * TK_THREADS + t;
        raw[it]      = make_uint4(0, 0, 0, 0);
        if (it < nvt && vi < nvec) {
            const int first = vi * EPV - a;
            if (first >= 0 && first + EPV <= vocab) {
                raw[it] = base[vi];
            }
            else {
                T* e = reinterpret_cast<T*>(&raw[it]);
                for (int j = 0; j < EPV; ++j) {
                    const int v = first + j;
                    if (v >= 0 && v < vocab) {
                        e[j] = rowp[v];
                    }
                }
            }
        }
    }
    uint32_t keys[TK_ELEMS];
    uint32_t tmax = 0;
#pragma unroll
    for (int it = 0; it < NVT; ++it) {
        const int vi    = vec0 + it * TK_THREADS + t;
        const int first = vi * EPV - a;
        const T*  e     = reinterpret_cast<const T*>(&raw[it]);
        const uint32_t vb = (it < nvt && vi < nvec) ? rowctx.vector_bits(first, EPV) : 0u;
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
            const int  v  = first + j;
            const bool in = it < nvt && v >= 0 && v < vocab;
            uint32_t   kk = in ? rowctx.key(v, e[j], (vb >> j) & 1u) : 0u;
            kk            = kk >= KMIN ? kk : 0u;  // never selectable
            keys[it * EPV + j] = kk;
            tmax               = kk > tmax ? kk : tmax;
        }
    }

    auto count_ge = [&](uint32_t thr) -> int {
        int c = 0;
#pragma unroll
        for (int e = 0; e < TK_ELEMS; ++e) {
            c += keys[e] >= thr ? 1 : 0;
        }
        return block_sum_i(c, (int*)s_red);
    };

    // ---- lower bound from thread maxima: the q-th largest maximum of each of the 4 waves,
    // minimised over the waves, has >= 4q elements at or above it.
    const uint32_t sorted = wave_sort_desc(tmax);
    const int      q      = k <= 4 * WAVE ? (k + 3) / 4 : WAVE;
    uint32_t       thr    = block_min<uint32_t>(__shfl(sorted, q - 1, WAVE), s_red, 0xFFFFFFFFu);
    const uint32_t cmax   = block_max<uint32_t>(tmax, s_red, 0u);
    if (thr < KMIN) {
        thr = KMIN;
    }
    const int n_valid = count_ge(KMIN);
    const int kneed   = k < n_valid ? k : n_valid;
    int       cnt     = count_ge(thr);
    bool      ok      = cnt >= kneed && cnt <= cap;
    if (!ok) {
        // bisection on the key for a threshold with kneed <= count <= cap
        uint32_t lo, hi;  // count(lo) > cap or lo == KMIN; count(hi) < kneed
        if (cnt > cap) {
            lo = thr;
            hi = cmax + 1u;
        }
        else {
            lo = KMIN;
            hi = thr;
            if (n_valid <= cap) {
                thr = KMIN;
                cnt = n_valid;
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
                cnt = c;
                ok  = true;
            }
        }
    }
    if (t == 0) {
        s_cnt = 0;
    }
    __syncthreads();
    if (ok) {
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            const int vi    = vec0 + it * TK_THREADS + t;
            const int first = vi * EPV - a;
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                const uint32_t kk = keys[it * EPV + j];
                if (kk >= thr) {
                    const int slot = atomicAdd(&s_cnt, 1);
                    if (slot < cap) {
                        entries[slot] = TopkEntry{kk, (uint32_t)(first + j)};
                    }
                }
            }
        }
    }
    if (t == 0) {
        TopkChunkHeader h;
        h.count     = ok ? (uint32_t)cnt : 0u;
        h.threshold = thr;
        h.bound_ok  = (ok && cnt >= k) ? 1u : 0u;
        h.overflow  = ok ? 0u : 1u;
        *header     = h;
    }
}

// -------------------------------------------------------------------------------------------
// select: merge, replay the reference's two tie orders, sample
// -------------------------------------------------------------------------------------------
struct TopkSelectShared {
    unsigned long long keys[TK_SELCAP];  // 32 KB
    int                idx[TK_SELCAP];   // 16 KB
    float              w[1024];
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

// thread 0 only: weights w[0..n) in selection order -> sampled position (sampling_topk_kernels.cu:282-311)
__device__ __forceinline__ int topk_sample_walk(const float* w, int n, float u, float p, float* s_sum_out)
{
    float s_sum = 0.0f;
    for (int i = 0; i < n; ++i) {
        s_sum += w[i];
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
__device__ void topk_literal(const Row& rowctx, TopkSelectShared& s, int vocab, int k, int BS1, int BS2,
                             TopkEntry* picks, int* n_list_out)
{
    const int      t    = threadIdx.x;
    const uint32_t KMIN = min_valid_key<DT>();
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
__device__ __forceinline__ void topk_select_row(const Row& rowctx, TopkSelectShared& s, int row, int vocab, int k,
                                                float p, int max_top_k, int splits, const TopkChunkHeader* headers,
                                                TopkEntry* entries, int cap, bool probs_in, float u,
                                                const int* end_ids, const TopkOutputs& out)
{
    const int t   = threadIdx.x;
    const int BS1 = max_top_k <= 16 ? 128 : 256;
    const int BS2 = max_top_k <= 32 ? 128 : 256;

    // ---- merge chunk headers
    uint32_t T0       = min_valid_key<DT>();
    bool     overflow = false;
    for (int c = 0; c < splits; ++c) {
        const TopkChunkHeader h = headers[c];
        overflow                = overflow || h.overflow != 0u;
        if (h.bound_ok && h.threshold > T0) {
            T0 = h.threshold;
        }
    }
    int n_list = 0;  // entries of the final ordered list, in s.keys (high word = ~key) / s.idx
    bool literal = overflow;

    if (!literal) {
        // candidates at or above T0 over all chunks
        auto count_ge = [&](uint32_t thr) -> int {
            int c = 0;
            for (int ch = 0; ch < splits; ++ch) {
                const int        n = (int)headers[ch].count;
                const TopkEntry* e = entries + (size_t)ch * cap;
                for (int i = t; i < n; i += TK_THREADS) {
                    c += e[i].key >= thr ? 1 : 0;
                }
            }
            return block_sum_i(c, (int*)s.red32);
        };
        int total = count_ge(T0);
        if (total > TK_SELCAP) {
            // exact k-th largest key by bisection on the key (only for k in the hundreds, where
            // every chunk had to keep >= k candidates)
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
            T0    = lo;
            total = count_ge(T0);
        }
        if (total > TK_SELCAP) {
            literal = true;  // thousands of identical values around the k-th
        }
    }

    if (!literal) {
        // ---- gather into LDS with the stage-1 composite key:
        // slice(3) | ~key(32) | BS1-1-t (8) | j (21)
        if (t < 8) {
            s.slice_count[t] = 0;
        }
        if (t == 0) {
            s.counter = 0;
        }
        __syncthreads();
        for (int ch = 0; ch < splits; ++ch) {
            const int        n = (int)headers[ch].count;
            const TopkEntry* e = entries + (size_t)ch * cap;
            for (int i = t; i < n; i += TK_THREADS) {
                const TopkEntry en = e[i];
                if (en.key >= T0) {
                    const int idx   = (int)en.idx;
                    const int blk   = idx / BS1;
                    const int tt    = idx - blk * BS1;
                    const int slice = blk & 7;
                    const int j     = blk >> 3;
                    const int slot  = atomicAdd(&s.counter, 1);
                    atomicAdd(&s.slice_count[slice], 1);
                    s.keys[slot] = ((unsigned long long)slice << 61) | ((unsigned long long)(~en.key) << 29)
                                   | ((unsigned long long)(BS1 - 1 - tt) << 21) | (unsigned long long)j;
                }
            }
        }
        __syncthreads();
        const int n   = s.counter;
        const int np2 = max(2, next_pow2(n));
        for (int i = n + t; i < np2; i += TK_THREADS) {
            s.keys[i] = ~0ull;
        }
        __syncthreads();
        block_bitonic_sort_u64(s.keys, np2);
        // ---- rank inside the slice -> stage-2 composite key: ~key(32) | BS2-1-pos%BS2 (8) | pos/BS2 (6) | q (12)
        int slice_start[8];
        {
            int acc = 0;
#pragma unroll
            for (int sl = 0; sl < 8; ++sl) {
                slice_start[sl] = acc;
                acc += s.slice_count[sl];
            }
        }
        for (int qi = t; qi < np2; qi += TK_THREADS) {
            unsigned long long nk = ~0ull;
            if (qi < n) {
                const unsigned long long c     = s.keys[qi];
                const int                slice = (int)(c >> 61);
                const uint32_t           ikey  = (uint32_t)(c >> 29);
                const int                tt    = BS1 - 1 - (int)((c >> 21) & 0xFFull);
                const int                j     = (int)(c & 0x1FFFFFull);
                int                      start = 0;
#pragma unroll
                for (int sl = 0; sl < 8; ++sl) {
                    start = sl == slice ? slice_start[sl] : start;
                }
                const int r = qi - start;
                s.idx[qi]   = (j * 8 + slice) * BS1 + tt;
                if (r < k) {
                    const int pos = slice * k + r;
                    nk = ((unsigned long long)ikey << 32) | ((unsigned long long)(BS2 - 1 - pos % BS2) << 24)
                         | ((unsigned long long)(pos / BS2) << 12) | (unsigned long long)qi;
                }
            }
            s.keys[qi] = nk;
        }
        __syncthreads();
        block_bitonic_sort_u64(s.keys, np2);
        // resolve the payload (position in the first sort) into the vocabulary index
        n_list = 0;
        {
            int cnt = 0;
            for (int i = t; i < min(k, n); i += TK_THREADS) {
                cnt += s.keys[i] != ~0ull ? 1 : 0;
            }
            n_list = block_sum_i(cnt, (int*)s.red32);
        }
        int my_idx[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = t + r * TK_THREADS;
            my_idx[r]   = i < n_list ? s.idx[(int)(s.keys[i] & 0xFFFull)] : 0;
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = t + r * TK_THREADS;
            if (i < n_list) {
                s.idx[i] = my_idx[r];
            }
        }
        __syncthreads();
    }
    else {
        topk_literal<DT, Row>(rowctx, s, vocab, k, BS1, BS2, entries, &n_list);
    }

    // ---- weights (sampling_topk_kernels.cu:264-279): exp(x - max) on logits, the value itself on probabilities
    const float x0 = n_list > 0 ? key_to_float(~(uint32_t)(s.keys[0] >> 32)) : 0.0f;
    for (int i = t; i < n_list; i += TK_THREADS) {
        const float x = key_to_float(~(uint32_t)(s.keys[i] >> 32));
        s.w[i]        = probs_in ? x : det_expf(x - x0);
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
