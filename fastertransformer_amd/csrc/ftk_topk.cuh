// Top-k selection and sampling, shared by the stand-alone entry point and the fused decode step.
//
// Reference behaviour restated (src/fastertransformer/kernels/sampling_topk_kernels.cu:130-396):
// stage 1 splits a row into 8 interleaved slices (BS1-wide stripes) and extracts each slice's k
// largest values by k arg-max passes; stage 2 extracts the k largest of the 8k candidates the same
// way, then thread 0 samples by inverse CDF. With cub::BlockReduce and `a.u > b.u ? a : b`, equal
// values resolve to the highest thread id, so the picks follow two total orders:
//   stage 1, inside a slice : value desc, (i mod BS1) desc, i asc
//   stage 2, over positions : value desc, (pos mod BS2) desc, pos asc,  pos = slice*k + rank
// The reference reads the row k+2 times. Here the row is read once, as a stream:
//   stream  - a 256-thread workgroup walks its share of the row tile by tile (16 vectors of 16 bytes per
//             thread, 64 KB per tile, the next tile requested before the bookkeeping of the current one).
//             It keeps a lower bound of the row's k-th largest value and an LDS list of everything
//             at or above it. The bound starts from the order statistics of per-thread maxima of
//             the first tile and is tightened to the exact k-th largest of the list whenever the
//             list grows long, so that after the first tile an element costs one multiply, one
//             maximum and a fraction of a compare.
//   select  - replays both tie orders on the candidates (ranking by counting for <= 256
//             candidates, two LDS bitonic sorts of 64-bit composite keys otherwise) and samples.
// When the batch has at least four rows per compute unit, one workgroup owns a whole row and runs both
// phases (no workspace traffic, one launch). Smaller batches split each row over several workgroups
// that leave their lists in the workspace, and a second launch merges them.
// Rows whose candidates cannot be bounded (thousands of identical values around the k-th) take a
// literal, slow replay of the reference's passes.
#pragma once
#include "ftk_device.cuh"
#include "ftk_transform.cuh"

namespace ftk {

#ifndef FTK_TK_THREADS
#define FTK_TK_THREADS 256
#endif
constexpr int TK_THREADS  = FTK_TK_THREADS;
constexpr int TK_WAVES    = TK_THREADS / 64;
constexpr int TK_MIN_WGS  = 1024 / TK_THREADS;  // workgroups per compute unit the kernels are built for
// The variants for a large k hold a whole tile and two transformed copies of a vector in registers beside the
// bookkeeping of the general tile loop: they are built for half as many workgroups, with twice the registers.
constexpr int TK_MIN_WGS_MANY = TK_MIN_WGS / 2;
constexpr int TK_NVT      = 16;    // 16-byte vectors per thread and tile: 64 KB per workgroup in flight
constexpr int TK_CCAP     = 2048;  // candidates a workgroup can hold
constexpr int TK_SLICE_CAP = TK_CCAP / 8;  // ... of one stage-1 slice, for the per-slice sort of the select
constexpr int TK_MAXSPLIT = 64;
constexpr int TK_FILL_WGS = 256 * TK_MIN_WGS;  // workgroups wanted in flight: every compute unit full
constexpr int TK_STAGE    = 512 / TK_WAVES;    // vectors a wave can park per tile

struct TopkChunkHeader {
    uint32_t count;      // entries written
    uint32_t threshold;  // every element of the chunk with key >= threshold is in the list
    uint32_t flags;      // bit 0: count >= k, `threshold` bounds the row's k-th largest key from below
                         // bit 1: the chunk could not bound its candidates (row takes the literal replay)
    uint32_t share;      // 0, or the chunk's ceil(k/splits)-th largest key: the smallest `share` of a row
                         // has >= k elements at or above it
};

struct TopkEntry {
    uint32_t key;
    uint32_t idx;
};

// which variant of the streaming kernels a launch takes (see topk_stream)
__host__ __device__ inline int topk_many_level(int max_top_k)
{
    return max_top_k > TK_CCAP / 4 ? 2 : (max_top_k > TK_STAGE ? 1 : 0);
}

struct TopkPlan {
    int    splits;         // workgroups per row
    int    tiles_per_wg;   // tiles each of them streams
    size_t row_entries;    // TopkEntry slots per row in the workspace
    size_t bytes;          // whole workspace
};

inline TopkPlan topk_plan(int vocab_padded, int batch, int max_top_k, int elem_bytes)
{
    TopkPlan  p;
    const int epv       = 16 / elem_bytes;
    const int tile_vecs = TK_THREADS * TK_NVT;
    const int nvec      = vocab_padded / epv + 2;  // worst case over row misalignments
    const int tiles     = (nvec + tile_vecs - 1) / tile_vecs;
    // as many workgroups as the chip holds at once (the large-k variants are built for fewer per compute unit)
    auto split = [&](int fill, int* tiles_per_wg) -> int {
        int s         = (fill + batch - 1) / (batch > 0 ? batch : 1);
        s             = s > tiles ? tiles : s;
        s             = s > TK_MAXSPLIT ? TK_MAXSPLIT : s;
        s             = s < 1 ? 1 : s;
        *tiles_per_wg = (tiles + s - 1) / s;
        return (tiles + *tiles_per_wg - 1) / *tiles_per_wg;
    };
    int       unused;
    const int splits_most = split(TK_FILL_WGS, &unused);
    p.splits = split(topk_many_level(max_top_k) > 0 ? 256 * TK_MIN_WGS_MANY : TK_FILL_WGS, &p.tiles_per_wg);
    size_t entries   = p.splits > 1 ? (size_t)p.splits * TK_CCAP : 0;
    const size_t lit = (size_t)8 * (max_top_k > 0 ? max_top_k : 1);  // the literal replay keeps 8k picks
    if (entries < lit) {
        entries = lit;
    }
    p.row_entries = entries;
    // the size asked for never shrinks with a larger k: it covers the split of the small-k variants too
    const size_t entries_most = splits_most > 1 ? (size_t)splits_most * TK_CCAP : 0;
    p.bytes = (size_t)batch
              * ((size_t)(splits_most > p.splits ? splits_most : p.splits) * sizeof(TopkChunkHeader)
                 + (entries_most > entries ? entries_most : entries) * sizeof(TopkEntry));
    return p;
}

// Workgroup barrier for code that only communicates through LDS: global loads issued earlier stay
// in flight across it.
__device__ __forceinline__ void lds_barrier()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

// -------------------------------------------------------------------------------------------
// Row accessors: turn (column, raw storage value) into the value the reference would hand to top-k
// (an fp32 image of a `T`). PlainRow is the identity (stand-alone entry point); the fused decode
// step supplies one that applies masks and penalties on the fly.
//   prepare(lo, hi)        - once per workgroup, before streaming columns [lo, hi)
//   has_vector_bits()      - some columns carry a flag (history membership)
//   vector_bits(first, n)  - one bit per flagged column of a 16-byte vector
//   plain_vector(first, n) - true when no column of the span needs an index-dependent rule
//   fast(x)                - index-independent transform of an interior column
//   flagged(xf, v)         - fast(x) -> value of the flagged interior column v
//   flagged_upper(xf)      - a cheap value that is never below flagged(xf): decides which vectors are
//                            looked at again, the exact value is computed for those only
//   tile_bits(...)         - the flags of a whole tile of an aligned row, EPV bits per vector, packed
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
    __device__ __forceinline__ bool never_selected(int v) const
    {
        (void)v;
        return false;
    }
    __device__ __forceinline__ float fast(float x) const
    {
        return x;
    }
    __device__ __forceinline__ float flagged(float xf, int) const
    {
        return xf;
    }
    __device__ __forceinline__ float flagged_upper(float xf) const
    {
        return xf;
    }
    template<int EPV, int NVT>
    __device__ __forceinline__ void tile_bits(int first0, int stride, uint32_t* packed) const
    {
        (void)first0;
        (void)stride;
        (void)packed;
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

// tiles of a row, given where it starts relative to 16-byte alignment
template<int DT>
__device__ __forceinline__ int topk_row_tiles(const void* rowp, int vocab)
{
    typedef typename Storage<DT>::T T;
    constexpr int                   EPV       = (int)(16 / sizeof(T));
    constexpr int                   TILE_VECS = TK_NVT * TK_THREADS;
    const int                       a         = (int)(((uintptr_t)rowp & 15u) / sizeof(T));
    const int                       nvec      = (a + vocab + EPV - 1) / EPV;
    return (nvec + TILE_VECS - 1) / TILE_VECS;
}

struct TopkShared {
    union {
        struct {
            uint32_t key[TK_CCAP];
            uint32_t idx[TK_CCAP];
        } cand;                            // stream: candidates (order-preserving key, column)
        unsigned long long keys[TK_CCAP];  // select: composite sort keys
    };
    union {
        struct {
            uint4 raw[TK_THREADS / WAVE][TK_STAGE];    // stream: vectors with an element at or above the bound,
            int   first[TK_THREADS / WAVE][TK_STAGE];  // one private list per wave
        } stage;
        struct {
            int                                idx[TK_CCAP];
            __attribute__((aligned(16))) float w[1024];
        } sel;  // select: the ordered list
    };
    unsigned long long red64[16];
    uint32_t           red32[16];
    int                slice_count[8];
    int                n_cand;
    uint32_t           thr_new;
    int                misc[4];
};

// element j of a 16-byte vector as fp32, extracted with 32-bit operations on the register that holds it
template<int DT>
__device__ __forceinline__ float vector_element(const uint4& v, int j)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    if constexpr (DT == DT_F32) {
        return __uint_as_float(w[j]);
    }
    else if constexpr (DT == DT_F16) {
        return Storage<DT>::ld((uint16_t)(j & 1 ? w[j >> 1] >> 16 : w[j >> 1] & 0xFFFFu));
    }
    else {
        return __uint_as_float(j & 1 ? (w[j >> 1] & 0xFFFF0000u) : (w[j >> 1] << 16));
    }
}

// value of column v as top-k sees it, re-read from memory
template<int DT, class Row>
__device__ __forceinline__ float topk_value_at(const Row& rowctx, int v)
{
    return rowctx.slow(v, Storage<DT>::ld(rowctx.data()[v]), rowctx.vector_bits(v, 1));
}

// keep the candidates with key >= thr (in place, order not preserved); returns how many
__device__ __forceinline__ int topk_prune(TopkShared& s, int n, uint32_t thr)
{
    const int t = threadIdx.x;
    uint32_t  ck[TK_CCAP / TK_THREADS], ci[TK_CCAP / TK_THREADS];
#pragma unroll
    for (int r = 0; r < TK_CCAP / TK_THREADS; ++r) {
        const int i = t + r * TK_THREADS;
        ck[r]       = i < n ? s.cand.key[i] : 0u;
        ci[r]       = i < n ? s.cand.idx[i] : 0u;
    }
    if (t == 0) {
        s.n_cand = 0;
    }
    lds_barrier();
    // one slot reservation per wave and batch of 64 entries (a ballot and a prefix count place the lanes)
#pragma unroll
    for (int r = 0; r < TK_CCAP / TK_THREADS; ++r) {
        if (r * TK_THREADS < n) {
            const bool               keep = t + r * TK_THREADS < n && ck[r] >= thr;
            const unsigned long long m    = __ballot(keep);
            int                      base = 0;
            if (lane_id() == 0 && m != 0ull) {
                base = atomicAdd(&s.n_cand, (int)__builtin_popcountll(m));
            }
            base = __builtin_amdgcn_readfirstlane(base);
            if (keep) {
                const int slot =
                    base + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                s.cand.key[slot] = ck[r];
                s.cand.idx[slot] = ci[r];
            }
        }
    }
    lds_barrier();
    const int m = s.n_cand;
    lds_barrier();
    return m;
}

// The exact k-th largest key of the list (n >= k, every entry >= lower). Uses the staging area of the
// stream (idle between tiles) as scratch.
template<bool DEEP = false>
__device__ __forceinline__ uint32_t topk_kth_key(TopkShared& s, int n, int k, uint32_t lower)
{
    const int t = threadIdx.x;
    uint32_t  nt;
    if (n <= TK_THREADS) {
        // Rank by counting; ties are ordered by position so exactly one entry has rank k-1.
        // Entry j precedes entry i when key_j > key_i, or the keys are equal and j < i:
        //   key_j >= key_i for j < i,  key_j > key_i for j > i   <=>   key_j + (j < i) > key_i
        // (keys stay below 0xFFFFFFFF, so the increment cannot wrap).
        // The work is cut the other way round from "one entry per thread": every wave compares a
        // quarter of the list (read four entries at a time) against all entries, four per lane, so a
        // thread waits for a quarter of the LDS reads and does sixteen compares per read; the partial
        // ranks meet in LDS.
        static_assert(TK_WAVES * WAVE == TK_THREADS && TK_STAGE * sizeof(uint4) >= TK_THREADS * sizeof(int),
                      "partial ranks live in the idle staging area");
        int (*part)[TK_THREADS] = reinterpret_cast<int(*)[TK_THREADS]>(&s.stage.raw[0][0]);
        const int l = lane_id(), w = wave_id();
        uint32_t  mk[TK_WAVES];
        int       mr[TK_WAVES];
#pragma unroll
        for (int q = 0; q < TK_WAVES; ++q) {
            const int i = l + q * WAVE;
            mk[q]       = i < n ? s.cand.key[i] : 0xFFFFFFFFu;
            mr[q]       = 0;
        }
        const int n4  = (n + 3) & ~3;
        const int per = ((n4 / 4 + TK_WAVES - 1) / TK_WAVES) * 4;  // entries per wave, a multiple of four
        const int jlo = w * per;
        const int jhi = min(n4, jlo + per);
#pragma unroll 2
        for (int j = jlo; j < jhi; j += 4) {
            const uint4    kk    = *reinterpret_cast<const uint4*>(&s.cand.key[j]);
            const uint32_t kj[4] = {kk.x, kk.y, kk.z, kk.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int      jj = j + e;
                const uint32_t kv = jj < n ? kj[e] : 0u;
#pragma unroll
                for (int q = 0; q < TK_WAVES; ++q) {
                    mr[q] += (kv + (jj < l + q * WAVE ? 1u : 0u)) > mk[q] ? 1 : 0;
                }
            }
        }
#pragma unroll
        for (int q = 0; q < TK_WAVES; ++q) {
            part[w][l + q * WAVE] = mr[q];
        }
        lds_barrier();
        if (t < n) {
            int r0 = 0;
#pragma unroll
            for (int q = 0; q < TK_WAVES; ++q) {
                r0 += part[q][t];
            }
            if (r0 == k - 1) {
                s.thr_new = s.cand.key[t];
            }
        }
        lds_barrier();
        nt = s.thr_new;
    }
    else {
        // Radix select on the key, most significant byte first: a 256-bin histogram of the entries that
        // still match the bytes found so far, a suffix sum over the bins (one bin per thread), and the
        // bin that holds the k-th largest gives the next byte. Four rounds of four barriers.
        static_assert(TK_THREADS == 256, "one histogram bin per thread");
        constexpr int PER  = TK_CCAP / TK_THREADS;
        int*          hist = reinterpret_cast<int*>(&s.stage.raw[0][0]);
        uint32_t      ck[PER];
#pragma unroll
        for (int r = 0; r < PER; ++r) {
            const int i = t + r * TK_THREADS;
            ck[r]       = i < n ? s.cand.key[i] : 0u;
        }
        (void)lower;
        uint32_t prefix = 0u, mask = 0u;
        int      kk     = k;  // rank wanted among the entries that match `prefix` on `mask`
#pragma unroll 1
        for (int shift = 24; shift >= 0; shift -= 8) {
            hist[t] = 0;
            lds_barrier();
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                if (r * TK_THREADS < n && t + r * TK_THREADS < n && (ck[r] & mask) == prefix) {
                    atomicAdd(&hist[(ck[r] >> shift) & 255u], 1);
                }
            }
            lds_barrier();
            // entries in bins >= t: suffix sum inside the wave, then the totals of the higher waves
            const int mine = hist[t];
            int       suf  = mine;
#pragma unroll
            for (int o = 1; o < WAVE; o <<= 1) {
                const int dn = __shfl_down(suf, o, WAVE);
                if (lane_id() + o < WAVE) {
                    suf += dn;
                }
            }
            if (lane_id() == 0) {
                s.red32[wave_id()] = (uint32_t)suf;
            }
            lds_barrier();
#pragma unroll
            for (int w = 0; w < TK_WAVES; ++w) {
                suf += w > wave_id() ? (int)s.red32[w] : 0;
            }
            if (suf >= kk && suf - mine < kk) {  // exactly one bin
                s.misc[1] = t;
                s.misc[2] = kk - (suf - mine);
            }
            lds_barrier();
            prefix |= (uint32_t)s.misc[1] << shift;
            mask |= 255u << shift;
            kk = s.misc[2];
        }
        const uint32_t lo = prefix;
        nt = lo;
    }
    lds_barrier();  // s.thr_new and the counters may be reused right away
    return nt;
}

// Raise the bound to the exact k-th largest key of the list (n >= k, every entry >= *thr) and drop
// what falls below it: k entries plus ties with the k-th remain.
template<bool DEEP = false>
__device__ __forceinline__ int topk_tighten(TopkShared& s, int n, int k, uint32_t* thr)
{
    *thr = topk_kth_key<DEEP>(s, n, k, *thr);
    return topk_prune(s, n, *thr);
}

// Keep the candidates that at most k-1 others beat (the k largest keys and every tie with the k-th); in place,
// order not preserved; returns how many remain. n <= 4 * TK_THREADS. An entry is dropped exactly when k or more
// keys are strictly greater, so nothing the reference could pick is lost. Every thread counts, for up to four
// entries of its own, the keys above them: the list is read four keys at a time (all lanes read the same
// address), several reads in flight.
__device__ __forceinline__ int topk_cut_to_k(TopkShared& s, int n, int k)
{
    constexpr int PER = 4;
    const int     t   = threadIdx.x;
    const int     per = (n + TK_THREADS - 1) / TK_THREADS;  // entries per thread that exist at all (uniform)
    uint32_t      ck[PER], ci[PER];
    int           above[PER];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        const int i = t + r * TK_THREADS;
        ck[r]       = (r < per && i < n) ? s.cand.key[i] : 0xFFFFFFFFu;
        ci[r]       = (r < per && i < n) ? s.cand.idx[i] : 0u;
        above[r]    = 0;
    }
    const int n16 = (n + 15) & ~15;
    if (t < n16 - n) {
        s.cand.key[n + t] = 0u;  // padding that is above nothing
    }
    if (t == 0) {
        s.n_cand = 0;
    }
    lds_barrier();
    for (int j0 = 0; j0 < n16; j0 += 16) {
        uint4 kk[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            kk[b] = *reinterpret_cast<const uint4*>(&s.cand.key[j0 + 4 * b]);
        }
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t kj[4] = {kk[b].x, kk[b].y, kk[b].z, kk[b].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    if (r < per) {
                        above[r] += kj[e] > ck[r] ? 1 : 0;
                    }
                }
            }
        }
    }
    lds_barrier();  // every thread has read the list: it can be rewritten
#pragma unroll
    for (int r = 0; r < PER; ++r) {
        if (r < per) {
            const bool               keep = t + r * TK_THREADS < n && above[r] < k;
            const unsigned long long m    = __ballot(keep);
            int                      base = 0;
            if (lane_id() == 0 && m != 0ull) {
                base = atomicAdd(&s.n_cand, (int)__builtin_popcountll(m));
            }
            base = __builtin_amdgcn_readfirstlane(base);
            if (keep) {
                const int slot =
                    base + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                s.cand.key[slot] = ck[r];
                s.cand.idx[slot] = ci[r];
            }
        }
    }
    lds_barrier();
    const int m = s.n_cand;
    lds_barrier();
    return m;
}

// -------------------------------------------------------------------------------------------
// stream: tiles [tile_begin, tile_end) of one row -> candidate list in LDS
// -------------------------------------------------------------------------------------------
// The recovery path of a tile that overfills the list: everything is recomputed from memory (the tile
// sits in L2) with rolled loops, nothing depends on the caller's registers. On entry the list holds
// n_before entries, all >= thr, from earlier tiles. Looks for a higher bound that leaves between k and
// TK_CCAP candidates; returns the new list length (bound in s.thr_new) or -1 when no bound does.
template<int DT, class Row>
__device__ __noinline__ int topk_stream_rare(Row rowctx, TopkShared& s, int k, int n_before, int lo_col, int hi_col,
                                             uint32_t thr)
{
    const int t        = threadIdx.x;
    auto      count_ge = [&](uint32_t key) -> int {
        const float f = key_to_float(key);
        int         c = 0;
        for (int i = t; i < n_before; i += TK_THREADS) {
            c += s.cand.key[i] >= key ? 1 : 0;
        }
        for (int v = lo_col + t; v < hi_col; v += TK_THREADS) {
            c += topk_value_at<DT>(rowctx, v) >= f ? 1 : 0;
        }
        return block_sum_i<TK_WAVES>(c, (int*)s.red32);
    };
    uint32_t lo = thr, hi = 0xFFFFFFFFu;  // count(lo) > TK_CCAP, count(hi) == 0
    bool     ok = count_ge(thr) <= TK_CCAP;  // (a wave ran out of parking space, the list itself fits)
    while (!ok && hi - lo > 1u) {
        const uint32_t mid = lo + (hi - lo) / 2u;
        const int      c   = count_ge(mid);
        if (c > TK_CCAP) {
            lo = mid;
        }
        else if (c < k) {
            hi = mid;
        }
        else {
            thr = mid;
            ok  = true;
        }
    }
    if (!ok) {
        return -1;
    }
    (void)topk_prune(s, n_before, thr);
    const float thr_f = key_to_float(thr);
    for (int v = lo_col + t; v < hi_col; v += TK_THREADS) {
        const float xv = topk_value_at<DT>(rowctx, v);
        if (xv >= thr_f) {
            const int slot   = atomicAdd(&s.n_cand, 1);
            s.cand.key[slot] = order_key(xv);
            s.cand.idx[slot] = (uint32_t)v;
        }
    }
    if (t == 0) {
        s.thr_new = thr;
    }
    lds_barrier();
    const int n = s.n_cand;
    lds_barrier();
    return n;
}

// Returns the number of candidates left in s.cand (all elements of the tiles with key >= *thr_out), or
// -1 when the range could not be bounded. When the result is >= k, *thr_out bounds the k-th largest key
// of the range from below; otherwise the list holds every selectable element of the range.
// MANY > 0: the variant for launches whose largest k exceeds what a wave can park per tile (TK_STAGE): the
// bound of the first tile is refined on the registers that hold it, and every tile takes the general loop,
// which then writes its candidates to the list directly. MANY == 2 (largest k beyond a quarter of the
// list's capacity) also cuts the list back in the middle of a tile. Rows of such a launch with a small k
// keep the parking loop.
template<int DT, class Row, int MANY = 0>
__device__ __forceinline__ int topk_stream(Row& rowctx, TopkShared& s, int vocab, int k, int tile_begin, int tile_end,
                                           uint32_t* thr_out)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV       = (int)(16 / sizeof(T));
    constexpr int         NVT       = TK_NVT;
    constexpr int         TILE_VECS = NVT * TK_THREADS;
    const int             t         = threadIdx.x;

    const T*       rowp     = rowctx.data();
    const int      a        = (int)(((uintptr_t)rowp & 15u) / sizeof(T));  // columns between the aligned base and column 0
    const uint4*   base     = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(rowp) - a * sizeof(T));
    const int      nvec     = (a + vocab + EPV - 1) / EPV;
    const int      vfull_lo = (a + EPV - 1) / EPV;  // vectors [vfull_lo, vfull_hi) lie entirely inside the row
    const int      vfull_hi = (a + vocab) / EPV;
    const bool     any_full = vfull_hi > vfull_lo;
    const uint32_t KMIN     = min_valid_key<DT>();
    const float    NEG_INF  = -__builtin_inff();
    const int      lo_col   = max(0, tile_begin * TILE_VECS * EPV - a);
    const int      hi_col   = max(lo_col, min(vocab, tile_end * TILE_VECS * EPV - a));

    // A tile is "plain" when every one of its vectors lies inside the row and no column needs an
    // index-dependent rule (pads, masked end id, bias): true for all but a handful of tiles per row.
    auto tile_plain = [&](int tile) -> bool {
        const int vec0 = tile * TILE_VECS;
        return any_full && vec0 >= vfull_lo && vec0 + TILE_VECS <= vfull_hi
               && rowctx.plain_vector(vec0 * EPV - a, TILE_VECS * EPV);
    };
    // Every vector load of a tile is issued back to back. Lanes whose vector is not entirely inside the
    // row read a harmless in-row vector instead and visit their columns one by one.
    uint4 raw[NVT];
    auto  load_tile = [&](int tile) {
        const int vec0 = tile * TILE_VECS;
        if (tile_plain(tile)) {
            const uint4* p0 = base + vec0 + t;
#pragma unroll
            for (int it = 0; it < NVT; ++it) {
                raw[it] = p0[it * TK_THREADS];
            }
        }
        else if (any_full) {
#pragma unroll
            for (int it = 0; it < NVT; ++it) {
                const int vi = vec0 + it * TK_THREADS + t;
                raw[it]      = base[(vi >= vfull_lo && vi < vfull_hi) ? vi : vfull_lo];
            }
        }
        else {
#pragma unroll
            for (int it = 0; it < NVT; ++it) {
                raw[it] = make_uint4(0, 0, 0, 0);
            }
        }
    };

    if (t == 0) {
        s.n_cand = 0;
    }
    load_tile(tile_begin);
    // per-workgroup side data of the row (e.g. the history bitmap) while the loads are in flight
    rowctx.prepare(lo_col, hi_col);
    lds_barrier();
    const bool bitsv = rowctx.has_vector_bits();
    // flags of the tile being examined, EPV bits per vector of this thread, fetched in one go for plain
    // tiles of rows that start on a 16-byte boundary (no vector straddles a word of the bitmap then)
    constexpr int PW = NVT * EPV / 32;
    uint32_t      packed[PW];
    const bool    packed_ok = bitsv && a == 0;
    auto          flags_of  = [&](int it, int first) -> uint32_t {
        if (packed_ok) {
            return (packed[(it * EPV) >> 5] >> ((it * EPV) & 31)) & ((1u << EPV) - 1u);
        }
        return rowctx.vector_bits(first, EPV);
    };

    // ---- initial bound from the first tile: maxima over the vectors that take the fast transform
    // (leaving the others out only lowers the bound).
    uint32_t thr;
    {
        const int  vec0        = tile_begin * TILE_VECS;
        const bool first_plain = tile_plain(tile_begin);
        if (first_plain && packed_ok) {
            rowctx.template tile_bits<EPV, NVT>((vec0 + t) * EPV - a, TK_THREADS * EPV, packed);
        }
        auto vec_max = [&](int it) -> float {
            const int  vi    = vec0 + it * TK_THREADS + t;
            const int  first = vi * EPV - a;
            const bool fastv = first_plain ?
                                   (!bitsv || flags_of(it, first) == 0u) :
                                   (any_full && vi >= vfull_lo && vi < vfull_hi && rowctx.plain_vector(first, EPV)
                                    && (!bitsv || rowctx.vector_bits(first, EPV) == 0u));
            float vmax = NEG_INF;
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                vmax = __builtin_fmaxf(vmax, rowctx.fast(vector_element<DT>(raw[it], j)));  // NaN never wins
            }
            return fastv ? vmax : NEG_INF;
        };
        // maxima of four groups of this thread's vectors: four distinct elements per thread
        float gm[4] = {NEG_INF, NEG_INF, NEG_INF, NEG_INF};
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            gm[it / (NVT / 4)] = __builtin_fmaxf(gm[it / (NVT / 4)], vec_max(it));
        }
        if (k <= TK_WAVES * WAVE) {
            // each wave sorts its 64 thread maxima; the q-th largest of each wave, minimised over the
            // waves, has >= waves * q >= k elements of the tile at or above it
            const float    tmax   = __builtin_fmaxf(__builtin_fmaxf(gm[0], gm[1]), __builtin_fmaxf(gm[2], gm[3]));
            const uint32_t sorted = wave_sort_desc(order_key(tmax));
            const int      q      = (k + TK_WAVES - 1) / TK_WAVES;
            thr = block_min<uint32_t, TK_WAVES>(__shfl(sorted, q - 1, WAVE), s.red32, 0xFFFFFFFFu);
        }
        else {
            // the same with the group maxima: four sorted sequences per wave
            const int q = (k + 4 * TK_WAVES - 1) / (4 * TK_WAVES);
            uint32_t  m = 0xFFFFFFFFu;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const uint32_t sorted = wave_sort_desc(order_key(gm[g]));
                const uint32_t qth    = __shfl(sorted, q - 1, WAVE);
                m                     = qth < m ? qth : m;
            }
            thr = block_min<uint32_t, TK_WAVES>(m, s.red32, 0xFFFFFFFFu);
        }
        if (thr < KMIN) {
            thr = KMIN;  // fewer than k usable maxima: take every selectable element
        }
        if constexpr (MANY > 0) {
            // The maxima bound is loose for a large k (for k = 1024 a third of the tile lies above it).
            // Raise it by bisection on the key, counting the tile's elements in the registers that hold
            // them (vectors on the fast transform only: leaving the others out keeps the count a lower
            // bound), until between k and 1.25 k of them remain.
            if (k > TK_STAGE) {
                uint32_t fastmask = 0u;
#pragma unroll
                for (int it = 0; it < NVT; ++it) {
                    fastmask |= vec_max(it) > NEG_INF ? (1u << it) : 0u;
                }
                float tmax = NEG_INF;
#pragma unroll
                for (int g = 0; g < 4; ++g) {
                    tmax = __builtin_fmaxf(tmax, gm[g]);
                }
                uint32_t lo = thr;
                uint32_t hi = block_max<uint32_t, TK_WAVES>(order_key(tmax), s.red32, 0u) + 1u;  // no element reaches it
                for (int round = 0; round < 24 && hi - lo > 1u; ++round) {
                    const uint32_t mid  = lo + (hi - lo) / 2u;
                    const float    midf = key_to_float(mid);
                    int            c    = 0;
#pragma unroll
                    for (int it = 0; it < NVT; ++it) {
                        if ((fastmask >> it) & 1u) {
#pragma unroll
                            for (int j = 0; j < EPV; ++j) {
                                c += rowctx.fast(vector_element<DT>(raw[it], j)) >= midf ? 1 : 0;
                            }
                        }
                    }
                    c = block_sum_i<TK_WAVES>(c, (int*)s.red32);
                    if (c >= k) {
                        lo = mid;
                        if (c <= k + k / 4) {
                            break;
                        }
                    }
                    else {
                        hi = mid;
                    }
                }
                thr = lo;
            }
        }
    }
    thr         = (uint32_t)__builtin_amdgcn_readfirstlane((int)thr);  // uniform: keep it in a scalar register
    float thr_f = key_to_float(thr);  // x >= thr_f  <=>  order_key(x) >= thr (NaN fails both)
    // The first tile is examined a second time below. Keep the compiler from carrying the converted
    // values of the first pass along in registers: make the tile opaque here (no instructions).
#pragma unroll
    for (int it = 0; it < NVT; ++it) {
        asm volatile("" : "+v"(raw[it].x), "+v"(raw[it].y), "+v"(raw[it].z), "+v"(raw[it].w));
    }

    auto push = [&](int v, float xv) {
        const int slot = atomicAdd(&s.n_cand, 1);
        if (slot < TK_CCAP) {
            s.cand.key[slot] = order_key(xv);
            s.cand.idx[slot] = (uint32_t)v;
        }
    };
    // the elements of one vector at or above the bound: one slot allocation for all of them
    auto push_vector = [&](int first, const float* x) {
        uint32_t m = 0u;
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
            m |= x[j] >= thr_f ? (1u << j) : 0u;
        }
        int slot = atomicAdd(&s.n_cand, __builtin_popcount(m));
#pragma unroll
        for (int j = 0; j < EPV; ++j) {
            if ((m >> j) & 1u) {
                if (slot < TK_CCAP) {
                    s.cand.key[slot] = order_key(x[j]);
                    s.cand.idx[slot] = (uint32_t)(first + j);
                }
                ++slot;
            }
        }
    };
    // Vectors with an element at or above the bound are parked in the wave's private LDS list (slot from
    // a ballot, no atomics, nothing to wait for) and expanded into candidates after the tile's last vector.
    const int wv     = wave_id();
    int       wcount = 0;  // wave-uniform
    auto      park   = [&](bool hit, const uint4& v, int first) {
        const unsigned long long m = __ballot(hit);
        if (m != 0ull) {
            if (hit) {
                const int slot =
                    wcount + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                if (slot < TK_STAGE) {
                    s.stage.raw[wv][slot]   = v;
                    s.stage.first[wv][slot] = first;
                }
            }
            wcount += __builtin_popcountll(m);
        }
    };
    auto drain = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
        const int staged = wcount < TK_STAGE ? wcount : TK_STAGE;
        for (int e = lane_id(); e < staged; e += WAVE) {
            const uint4 v     = s.stage.raw[wv][e];
            const int   first = s.stage.first[wv][e];
            float       x[EPV];
#pragma unroll
            for (int j = 0; j < EPV; ++j) {
                x[j] = rowctx.fast(vector_element<DT>(v, j));
            }
            if (bitsv) {
                const uint32_t bits = rowctx.vector_bits(first, EPV);
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    if ((bits >> j) & 1u) {
                        x[j] = rowctx.flagged(x[j], first + j);
                    }
                }
            }
            push_vector(first, x);
        }
        if (wcount > TK_STAGE && lane_id() == 0) {
            atomicAdd(&s.n_cand, TK_CCAP + 1);  // out of parking space: the tile takes the recovery path
        }
        wcount = 0;
    };
    // the list is cut back to its k largest between tiles when it has grown past this; with a large k
    // after every tile (another tile's worth at the old bound would not fit)
    const int tighten_at = (MANY > 0 && k > TK_STAGE) ? k : min(max(256, 2 * k), 3 * TK_CCAP / 4);
    int       n          = 0;
    // With a large k a tile holds more candidates than a wave can park before the tile's drain (k alone
    // can exceed the space): such rows take the general tile loop, which then writes its candidates to the
    // list directly.
    const bool     many    = MANY > 0 && k > TK_STAGE;  // rows with a small k of such a launch keep the fast loop
    constexpr bool cut_mid = MANY > 1;

    for (int tile = tile_begin; tile < tile_end; ++tile) {
        bool      cut_early = false;  // large k: the list was cut back in the middle of this tile
        const int vec0      = tile * TILE_VECS;
        const int first0   = (vec0 + t) * EPV - a;
        uint32_t  slowmask = 0u;  // bit `it`: vector `it` of this thread takes the per-column path
        if (tile_plain(tile) && !many) {
            if (packed_ok && tile != tile_begin) {
                rowctx.template tile_bits<EPV, NVT>(first0, TK_THREADS * EPV, packed);
            }
#pragma unroll
            for (int it = 0; it < NVT; ++it) {
                const int first = first0 + it * TK_THREADS * EPV;
                float     x[EPV];
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    x[j] = rowctx.fast(vector_element<DT>(raw[it], j));
                }
                if (bitsv) {
                    const uint32_t bits = flags_of(it, first);
                    if (bits != 0u) {
#pragma unroll
                        for (int j = 0; j < EPV; ++j) {
                            x[j] = ((bits >> j) & 1u) ? rowctx.flagged_upper(x[j]) : x[j];
                        }
                    }
                }
                float vmax = x[0];
#pragma unroll
                for (int j = 1; j < EPV; ++j) {
                    vmax = __builtin_fmaxf(vmax, x[j]);
                }
                park(vmax >= thr_f, raw[it], first);
            }
        }
        else {
            // a plain tile of a row with a large k: the flags of all its vectors are requested in one go
            const bool flags_packed = MANY > 0 && packed_ok && tile_plain(tile);
            if (flags_packed && tile != tile_begin) {
                rowctx.template tile_bits<EPV, NVT>(first0, TK_THREADS * EPV, packed);
            }
            auto general_vector = [&](int it) {
                const int  vi    = vec0 + it * TK_THREADS + t;
                const int  first = first0 + it * TK_THREADS * EPV;
                // vectors inside the row with no index-dependent column stay on the register path
                const bool fastv = any_full && vi >= vfull_lo && vi < vfull_hi && rowctx.plain_vector(first, EPV);
                slowmask |= (vi < nvec && !fastv) ? (1u << it) : 0u;
                float x[EPV];
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    x[j] = rowctx.fast(vector_element<DT>(raw[it], j));
                }
                if constexpr (MANY == 0) {
                    if (bitsv && fastv) {
                        const uint32_t bits = rowctx.vector_bits(first, EPV);
                        if (bits != 0u) {
#pragma unroll
                            for (int j = 0; j < EPV; ++j) {
                                x[j] = ((bits >> j) & 1u) ? rowctx.flagged_upper(x[j]) : x[j];
                            }
                        }
                    }
                    float vmax = x[0];
#pragma unroll
                    for (int j = 1; j < EPV; ++j) {
                        vmax = __builtin_fmaxf(vmax, x[j]);
                    }
                    park(fastv && vmax >= thr_f, raw[it], first);
                    return;
                }
                float xu[EPV];  // the same with upper bounds in the history's columns
#pragma unroll
                for (int j = 0; j < EPV; ++j) {
                    xu[j] = x[j];
                }
                const uint32_t bits =
                    (bitsv && fastv) ? (flags_packed ? flags_of(it, first) : rowctx.vector_bits(first, EPV)) : 0u;
                if (bits != 0u) {
#pragma unroll
                    for (int j = 0; j < EPV; ++j) {
                        xu[j] = ((bits >> j) & 1u) ? rowctx.flagged_upper(x[j]) : x[j];
                    }
                }
                float vmax = xu[0];
#pragma unroll
                for (int j = 1; j < EPV; ++j) {
                    vmax = __builtin_fmaxf(vmax, xu[j]);
                }
                if (!many) {
                    park(fastv && vmax >= thr_f, raw[it], first);
                }
                else if (fastv && vmax >= thr_f) {
                    // With a large k a quarter or more of the vectors hold a candidate: they go to the list
                    // directly, with the exact values of the history's columns.
                    if (bits != 0u) {
#pragma unroll
                        for (int j = 0; j < EPV; ++j) {
                            if ((bits >> j) & 1u) {
                                x[j] = rowctx.flagged(x[j], first + j);
                            }
                        }
                    }
                    push_vector(first, x);
                }
            };
#pragma unroll
            for (int it = 0; it < (MANY > 0 ? NVT / 2 : NVT); ++it) {
                general_vector(it);
            }
            if (cut_mid && many && k > TK_CCAP / 4) {
                // Half a tile at the bound of the tiles before it can add more than half of k: with
                // k beyond a quarter of the list's capacity the list is cut back in mid-tile too.
                lds_barrier();
                const int n_mid = s.n_cand;
                lds_barrier();
                if (n_mid > k && n_mid <= TK_CCAP) {
                    n         = topk_tighten(s, n_mid, k, &thr);
                    thr_f     = key_to_float(thr);
                    cut_early = true;
                }
            }
#pragma unroll
            for (int it = (MANY > 0 ? NVT / 2 : NVT); it < NVT; ++it) {
                general_vector(it);
            }
            for (; slowmask != 0u; slowmask &= slowmask - 1u) {
                const int first = first0 + __builtin_ctz(slowmask) * TK_THREADS * EPV;
                for (int j = 0; j < EPV; ++j) {
                    const int v = first + j;
                    if (v >= 0 && v < vocab && !rowctx.never_selected(v)) {
                        const float xv = topk_value_at<DT>(rowctx, v);
                        if (xv >= thr_f) {
                            push(v, xv);
                        }
                    }
                }
            }
        }
        drain();
        // the next tile is requested before the bookkeeping of this one
        if (tile + 1 < tile_end) {
            load_tile(tile + 1);
        }
        lds_barrier();
        const int n_now = s.n_cand;
        lds_barrier();
        if (n_now > TK_CCAP && cut_early) {
            return -1;  // the list already holds part of this tile: the recovery path cannot redo the tile
        }
        if (n_now > TK_CCAP) {
            const int tlo = max(0, vec0 * EPV - a);
            const int thi = max(tlo, min(vocab, (vec0 + TILE_VECS) * EPV - a));
            n             = topk_stream_rare<DT, Row>(rowctx, s, k, n, tlo, thi, thr);
            if (n < 0) {
                return -1;
            }
            thr   = s.thr_new;
            thr_f = key_to_float(thr);
            if (tile + 1 < tile_end) {
                load_tile(tile + 1);  // again, so that no tile data has to survive the call
            }
        }
        else if (n_now > tighten_at && n_now > k && tile + 1 < tile_end) {
            n     = topk_tighten(s, n_now, k, &thr);
            thr_f = key_to_float(thr);
        }
        else {
            n = n_now;
        }
    }
    *thr_out = thr;
    return n;
}

// A workgroup's list -> workspace, for rows that are split over several workgroups. A short list goes
// out as it is, with the bound it was gathered under: cutting it to its k largest here would keep every
// workgroup of the launch busy for several microseconds at the end of its stream, while the merging
// kernel cuts the union once per row. A long list is cut to the chunk's k largest first, and the chunk
// also reports its ceil(k/splits)-th largest key (`share`), which gives the merge a bound that keeps the
// union inside its list.
constexpr int TK_RAW_DUMP = 448;

__device__ __forceinline__ void topk_dump_list(TopkShared& s, int n, int k, int splits, uint32_t thr,
                                               TopkChunkHeader* header, TopkEntry* entries)
{
    const int t = threadIdx.x;
    uint32_t share = 0u;
    if (n > k && (n > TK_RAW_DUMP || n * splits > TK_CCAP)) {  // the union of raw lists fits the merge's list
        n                = topk_tighten(s, n, k, &thr);
        const int kshare = (k + splits - 1) / splits;
        if (n >= kshare) {
            share = topk_kth_key(s, n, kshare, thr);
        }
    }
    for (int i = t; i < n; i += TK_THREADS) {
        entries[i] = TopkEntry{s.cand.key[i], s.cand.idx[i]};
    }
    if (t == 0) {
        TopkChunkHeader h;
        h.count     = n < 0 ? 0u : (uint32_t)n;
        h.threshold = thr;
        h.flags     = n < 0 ? 2u : (n >= k ? 1u : 0u);
        h.share     = share;
        *header     = h;
    }
}

// -------------------------------------------------------------------------------------------
// sampling and the literal replay
// -------------------------------------------------------------------------------------------
struct TopkOutputs {
    int*   ids;
    int*   sequence_length;
    bool*  finished;
    float* cum_log_probs;
    float* output_log_probs;
    // values of the row read when the kernel starts, so that the last thread standing does not wait for
    // memory again; rows that are already finished never get here
    int   sequence_length_in;
    float cum_log_prob_in;
    int   end_id_in;  // -1 when the caller passed no end ids to topk_outputs
};

__device__ __forceinline__ TopkOutputs topk_outputs(int* ids, int* sequence_length, bool* finished,
                                                    float* cum_log_probs, float* output_log_probs, int row,
                                                    const int* end_ids = nullptr)
{
    TopkOutputs o;
    o.ids                = ids;
    o.sequence_length    = sequence_length;
    o.finished           = finished;
    o.cum_log_probs      = cum_log_probs;
    o.output_log_probs   = output_log_probs;
    o.sequence_length_in = sequence_length != nullptr ? sequence_length[row] : 0;
    o.cum_log_prob_in    = cum_log_probs != nullptr ? cum_log_probs[row] : 0.0f;
    o.end_id_in          = end_ids != nullptr ? end_ids[row] : -1;
    return o;
}

// thread 0 only: weights w[0..n) in selection order -> sampled position (sampling_topk_kernels.cu:282-311).
// `w` is 16-byte aligned LDS, zero padded to a multiple of 32 (adding +0 to a non-negative sum is exact).
// Both passes are strictly sequential in fp32, as in the reference; 32 weights are fetched at a time so that
// the chain of additions never waits for LDS.
__device__ __forceinline__ int topk_sample_walk(const float* w, int n, float u, float p, float* s_sum_out)
{
    const float4* w4    = reinterpret_cast<const float4*>(w);
    const int     n4    = (n + 3) >> 2;
    float         s_sum = 0.0f;
    for (int i0 = 0; i0 < n4; i0 += 8) {
        float4 v[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            v[b] = w4[i0 + b];
        }
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            s_sum = s_sum + v[b].x;
            s_sum = s_sum + v[b].y;
            s_sum = s_sum + v[b].z;
            s_sum = s_sum + v[b].w;
        }
    }
    // The running difference never rises again (the weights are non-negative), so the first position where it
    // is <= 0 is the number of positions in front of it, where it is still > 0 (or not a number, as in the
    // reference, whose `<= 0` test a NaN never passes). A batch of 32 whose last difference is still positive has
    // no such position: only the subtractions, one dependent chain, are paid for it. The batch where the walk
    // ends is looked at position by position.
    float rand_num = u * p * s_sum;
    int   ahead    = 0;
    bool  walking  = true;
    for (int i0 = 0; i0 < n4 && walking; i0 += 8) {
        float4 v[8];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            v[b] = w4[i0 + b];
        }
        float r[32];
#pragma unroll
        for (int b = 0; b < 8; ++b) {
            r[4 * b + 0] = rand_num = rand_num - v[b].x;
            r[4 * b + 1] = rand_num = rand_num - v[b].y;
            r[4 * b + 2] = rand_num = rand_num - v[b].z;
            r[4 * b + 3] = rand_num = rand_num - v[b].w;
        }
        if (r[31] > 0.0f) {
            ahead += 32;
        }
        else {
#pragma unroll
            for (int e = 0; e < 32; ++e) {
                walking = walking && !(r[e] <= 0.0f);
                ahead += walking ? 1 : 0;
            }
        }
    }
    const int pick = ahead < n - 1 ? ahead : n - 1;
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
            o.cum_log_probs[row] = o.cum_log_prob_in + lp;
        }
        if (o.output_log_probs != nullptr) {
            o.output_log_probs[row] = lp - det_logf(s_sum);
        }
    }
    if (o.sequence_length != nullptr && o.finished != nullptr) {
        o.sequence_length[row] = o.sequence_length_in + 1;  // the row was not finished (:317-320)
        o.finished[row]        = id == (o.end_id_in >= 0 ? o.end_id_in : end_ids[row]);
    }
}

// The end of the selection, by the TK_THREADS threads that are left of a workgroup: the ordered list (values in
// s.sel.w, columns in s.sel.idx, n_list entries) -> weights (sampling_topk_kernels.cu:264-279: exp(x - max) on
// logits, the value itself on probabilities), the sequential sum and walk of the reference by thread 0, the row's
// outputs. The list is padded with zero weights to a multiple of 32 for the walk, which reads 32 at a time.
template<int DT>
__device__ __forceinline__ void topk_finish_list(TopkShared& s, int n_list, int row, int vocab, float p, bool probs_in,
                                                 float u, const int* end_ids, const TopkOutputs& out)
{
    const int   t  = threadIdx.x;
    const float x0 = n_list > 0 ? s.sel.w[0] : 0.0f;
    __syncthreads();
    for (int i = t; i < ((n_list + 31) & ~31); i += TK_THREADS) {
        const float x = i < n_list ? s.sel.w[i] : 0.0f;
        s.sel.w[i]    = i < n_list ? (probs_in ? x : det_expf(x - x0)) : 0.0f;
    }
    __syncthreads();
    if (t == 0) {
        if (n_list == 0) {
            topk_emit(out, row, 0, probs_in, 0.0f, 0.0f, end_ids, false);
        }
        else {
            float     s_sum;
            const int pick = topk_sample_walk(s.sel.w, n_list, u, p, &s_sum);
            topk_emit(out, row, s.sel.idx[pick] % vocab, probs_in, s.sel.w[pick], s_sum, end_ids, true);
        }
    }
}

// Literal replay for rows the gather could not bound. `Row::key_at(v)` re-reads the row.
// Every pick is the smallest composite key strictly greater than the previous pick, where the
// composite encodes the reference's order; picks of stage 1 go to `picks` (8k entries, global).
template<int DT, class Row>
__device__ void topk_literal(Row& rowctx, TopkShared& s, int vocab, int k, int BS1, int BS2,
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
            best = ~block_max<unsigned long long, TK_WAVES>(~best, s.red64, 0ull);
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
        best = ~block_max<unsigned long long, TK_WAVES>(~best, s.red64, 0ull);
        if (best == ~0ull) {
            break;
        }
        if (t == 0) {
            const int pos = (int)(best & 0xFFFFFFull);
            s.keys[ite]   = (unsigned long long)(~picks[pos].key) << 32;
            s.sel.idx[ite]    = (int)picks[pos].idx;
        }
        last      = best;
        have_last = true;
        n_list++;
    }
    __syncthreads();
    *n_list_out = n_list;
}

// -------------------------------------------------------------------------------------------
// select: replay the reference's two tie orders on the candidates in s.cand, sample, emit.
// `n` < 0 asks for the literal replay.
// -------------------------------------------------------------------------------------------
// DEEP: see topk_kth_key.
template<int DT, class Row, bool DEEP = false>
__device__ __forceinline__ void topk_select_lds(Row& rowctx, TopkShared& s, int n, uint32_t thr, int row, int vocab,
                                                int k, float p, int max_top_k, TopkEntry* picks, bool probs_in,
                                                float u, const int* end_ids, const TopkOutputs& out)
{
    const int t       = threadIdx.x;
    const int bs1_log = max_top_k <= 16 ? 7 : 8;
    const int BS1     = 1 << bs1_log;
    const int BS2     = max_top_k <= 32 ? 128 : 256;
    int       n_list  = 0;  // length of the final ordered list: values in s.w (as fp32), ids in s.idx

    if (n >= 0) {
        if (n > TK_THREADS && n > k && k <= TK_THREADS) {
            n = topk_tighten<DEEP>(s, n, k, &thr);  // (a larger k goes to the sorts below, which take any n)
        }
        if (n <= TK_THREADS) {
            // ---- small candidate sets (the usual case): both tie orders by counting, no sort.
            //   stage 1: slice(3) | ~key(32) | BS1-1-t (8) | j (21),   i = (j*8 + slice)*BS1 + t
            //   stage 2: ~key(32) | BS2-1-pos%BS2 (8) | pos/BS2 (12) | 0,   pos = slice*k + rank in slice
            // Composite keys are unique, so "number of smaller keys" is the sorted position, and the rank inside
            // a slice is that minus the number of keys of lower slices. The all-pairs counting is spread over
            // all threads: with CP = n rounded up to a power of two, thread t counts for candidate t % CP over
            // part t / CP of the list, and the partial counts meet in LDS.
            const uint32_t my_key = t < n ? s.cand.key[t] : 0u;
            const uint32_t my_idx = t < n ? s.cand.idx[t] : 0u;
            unsigned long long* A   = s.keys;                        // stage-1 keys  [0, 256)
            unsigned long long* B   = s.keys + TK_THREADS;           // stage-2 keys  [256, 512)
            int*                cnt = reinterpret_cast<int*>(s.keys + 2 * TK_THREADS);  // 3 x 256 partial counts
            const int           n2  = (n + 1) & ~1;
            int                 CP  = 2;
            while (CP < n) {
                CP <<= 1;
            }
            const int parts = TK_THREADS / CP;  // CP <= 256
            const int c     = t & (CP - 1);
            const int part  = t / CP;
            // pairs of list entries [jlo, jhi) belong to this thread's part
            const int pairs = n2 >> 1;
            const int per   = (pairs + parts - 1) / parts;
            const int jlo   = min(pairs, part * per) * 2;
            const int jhi   = min(pairs, part * per + per) * 2;
            lds_barrier();  // every candidate is in registers: the list's memory can be reused
            unsigned long long mine = ~0ull;
            if (t < n) {
                const int blk   = (int)(my_idx >> bs1_log);
                const int tt    = (int)(my_idx & (uint32_t)(BS1 - 1));
                const int slice = blk & 7;
                mine = ((unsigned long long)slice << 61) | ((unsigned long long)(~my_key) << 29)
                       | ((unsigned long long)(BS1 - 1 - tt) << 21) | (unsigned long long)(blk >> 3);
            }
            if (t < n2) {
                A[t] = mine;  // (an odd list is padded with a key that never counts)
            }
            cnt[t]                  = 0;
            cnt[TK_THREADS + t]     = 0;
            cnt[2 * TK_THREADS + t] = 0;
            if (t == 0) {
                s.misc[1] = 0;
            }
            lds_barrier();
            {
                const unsigned long long key  = c < n ? A[c] : ~0ull;
                const unsigned long long base = key & (7ull << 61);  // below it: the keys of lower slices
                int                      q = 0, qs = 0;
#pragma unroll 4
                for (int j = jlo; j < jhi; j += 2) {
                    const ulonglong2 kk = *reinterpret_cast<const ulonglong2*>(&A[j]);
                    q += kk.x < key ? 1 : 0;
                    q += kk.y < key ? 1 : 0;
                    qs += kk.x < base ? 1 : 0;
                    qs += kk.y < base ? 1 : 0;
                }
                if (c < n && jhi > jlo) {
                    atomicAdd(&cnt[c], q);
                    atomicAdd(&cnt[TK_THREADS + c], qs);
                }
            }
            lds_barrier();
            unsigned long long k2 = ~0ull;
            if (t < n) {
                const int slice = (int)(mine >> 61);
                const int r     = cnt[t] - cnt[TK_THREADS + t];  // rank inside the slice
                if (r < k) {
                    const int pos = slice * k + r;
                    k2 = ((unsigned long long)(uint32_t)(mine >> 29) << 32)
                         | ((unsigned long long)(BS2 - 1 - pos % BS2) << 24) | ((unsigned long long)(pos / BS2) << 12);
                }
            }
            if (t < n2) {
                B[t] = k2;
            }
            lds_barrier();
            {
                const unsigned long long key = c < n ? B[c] : ~0ull;
                int                      q = 0, kept = 0;
#pragma unroll 4
                for (int j = jlo; j < jhi; j += 2) {
                    const ulonglong2 kk = *reinterpret_cast<const ulonglong2*>(&B[j]);
                    q += kk.x < key ? 1 : 0;
                    q += kk.y < key ? 1 : 0;
                    kept += kk.x != ~0ull ? 1 : 0;
                    kept += kk.y != ~0ull ? 1 : 0;
                }
                if (c < n && jhi > jlo) {
                    atomicAdd(&cnt[2 * TK_THREADS + c], q);
                }
                if (c == 0 && jhi > jlo) {
                    atomicAdd(&s.misc[1], kept);  // entries that stage 1 kept, over all parts
                }
            }
            lds_barrier();
            n_list = min(k, s.misc[1]);
            if (t < n && k2 != ~0ull) {
                const int q2 = cnt[2 * TK_THREADS + t];
                if (q2 < n_list) {
                    s.sel.w[q2]   = key_to_float(~(uint32_t)(k2 >> 32));
                    s.sel.idx[q2] = (int)my_idx;
                }
            }
            __syncthreads();
        }
        else {
            // candidates -> stage-1 composite keys, in place
            //   slice(3) | ~key(32) | BS1-1-t (8) | j (21),   i = (j*8 + slice)*BS1 + t
            constexpr int PER = TK_CCAP / TK_THREADS;
            uint32_t      ck[PER], ci[PER];
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                const int i = t + r * TK_THREADS;
                ck[r]       = i < n ? s.cand.key[i] : 0u;
                ci[r]       = i < n ? s.cand.idx[i] : 0u;
            }
            if (t < 8) {
                s.slice_count[t] = 0;
            }
            lds_barrier();
            unsigned long long comp[PER];  // stage-1 keys of this thread's candidates
            int                cs[PER];    // ... and their slots among the candidates of their slice
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                const int i = t + r * TK_THREADS;
                comp[r]     = ~0ull;
                cs[r]       = 0;
                if (i < n) {
                    const int blk   = (int)(ci[r] >> bs1_log);
                    const int tt    = (int)(ci[r] & (uint32_t)(BS1 - 1));
                    const int slice = blk & 7;
                    cs[r]           = atomicAdd(&s.slice_count[slice], 1);
                    comp[r] = ((unsigned long long)slice << 61) | ((unsigned long long)(~ck[r]) << 29)
                              | ((unsigned long long)(BS1 - 1 - tt) << 21) | (unsigned long long)(blk >> 3);
                }
            }
            lds_barrier();
            int slice_start[8];
            int most = 0;
            {
                int acc = 0;
#pragma unroll
                for (int sl = 0; sl < 8; ++sl) {
                    slice_start[sl] = acc;
                    acc += s.slice_count[sl];
                    most = max(most, s.slice_count[sl]);
                }
            }
            if (most <= TK_SLICE_CAP) {
                // ---- the usual case: no slice holds more than 256 candidates. Stage 1 is a sort per slice, two
                // slices per wave, in registers, which leaves eight sorted runs; stage 2 (below) merges them.
                unsigned long long* bucket = s.keys;  // [8][TK_SLICE_CAP], unused slots hold the largest key
#pragma unroll
                for (int r = 0; r < PER; ++r) {
                    const int i = t + r * TK_THREADS;  // (TK_CCAP slots: slice r, slot t)
                    if (t >= s.slice_count[r]) {
                        bucket[i] = ~0ull;
                    }
                    if (i < n) {
                        bucket[(int)(comp[r] >> 61) * TK_SLICE_CAP + cs[r]] = comp[r];
                    }
                }
                lds_barrier();
                static_assert(TK_SLICE_CAP == 4 * WAVE && TK_WAVES == 4, "a wave sorts two slices, four keys per lane");
#pragma unroll 1
                for (int h = 0; h < 2; ++h) {
                    unsigned long long* b = bucket + (wave_id() * 2 + h) * TK_SLICE_CAP;
                    unsigned long long  kk[4];
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        kk[r] = b[r * WAVE + lane_id()];
                    }
                    wave_sort_keys_u64<4>(kk);
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        b[lane_id() * 4 + r] = kk[r];
                    }
                }
                lds_barrier();
                int kept[8];  // entries of a run that stage 1 keeps
                int total_kept = 0;
#pragma unroll
                for (int sl = 0; sl < 8; ++sl) {
                    kept[sl] = min(s.slice_count[sl], k);
                    total_kept += kept[sl];
                }
                n_list = min(k, total_kept);
                // the second tie rule as a number: smaller comes first
                const int bs2_log = max_top_k <= 32 ? 7 : 8;  // BS2 is a power of two
                auto      tie2    = [&](int slice, int r) -> int {
                    const int pos = slice * k + r;
                    return ((BS2 - 1 - (pos & (BS2 - 1))) << 12) | (pos >> bs2_log);
                };
                // ---- stage 2. Each run is first put into the order of its stage-2 keys, which moves entries
                // among the entries of equal value of their run only; thread t handles entry t of every run. Then
                // the eight runs are merged in three rounds of pairwise merges.
                //   stage-2 key: ~key(32) | BS2-1-pos%BS2 (8) | pos/BS2 (12) | slot of the entry in its run (12)
                unsigned long long c2[8];
                int                newpos[8];
                {
                    uint32_t ikey[8];
                    int      mine[8], before[8], smaller[8];
#pragma unroll
                    for (int o = 0; o < 8; ++o) {
                        const unsigned long long c = bucket[o * TK_SLICE_CAP + t];
                        ikey[o]                    = (uint32_t)(c >> 29);
                        mine[o]                    = tie2(o, t);
                        before[o]                  = 0;
                        smaller[o]                 = 0;
                        const int tt               = BS1 - 1 - (int)((c >> 21) & 0xFFull);
                        const int j                = (int)(c & 0x1FFFFFull);
                        if (t < kept[o]) {
                            s.sel.idx[o * TK_SLICE_CAP + t] = (j * 8 + o) * BS1 + tt;
                        }
                    }
                    // neighbours of equal value at distance d, to the left and to the right, all runs together
                    uint32_t open_left = 0xFFu, open_right = 0xFFu;
                    for (int d = 1; (open_left | open_right) != 0u; ++d) {
                        unsigned long long vl[8], vr[8];
#pragma unroll
                        for (int o = 0; o < 8; ++o) {
                            vl[o] = bucket[o * TK_SLICE_CAP + max(t - d, 0)];
                            vr[o] = bucket[o * TK_SLICE_CAP + min(t + d, TK_SLICE_CAP - 1)];
                        }
#pragma unroll
                        for (int o = 0; o < 8; ++o) {
                            const bool l = ((open_left >> o) & 1u) != 0u && t < kept[o] && t - d >= 0
                                           && (uint32_t)(vl[o] >> 29) == ikey[o];
                            const bool r = ((open_right >> o) & 1u) != 0u && t + d < kept[o]
                                           && (uint32_t)(vr[o] >> 29) == ikey[o];
                            before[o] += l ? 1 : 0;
                            smaller[o] += (l && tie2(o, t - d) < mine[o] ? 1 : 0) + (r && tie2(o, t + d) < mine[o] ? 1 : 0);
                            open_left  = l ? open_left : (open_left & ~(1u << o));
                            open_right = r ? open_right : (open_right & ~(1u << o));
                        }
                    }
#pragma unroll
                    for (int o = 0; o < 8; ++o) {
                        newpos[o] = t - before[o] + smaller[o];
                        c2[o]     = ((unsigned long long)ikey[o] << 32) | ((unsigned long long)mine[o] << 12)
                                | (unsigned long long)(o * TK_SLICE_CAP + t);
                    }
                }
                lds_barrier();  // every entry of the runs has been read
#pragma unroll
                for (int o = 0; o < 8; ++o) {
                    if (t < kept[o]) {
                        bucket[o * TK_SLICE_CAP + newpos[o]] = c2[o];
                    }
                }
                if (t < 8) {
                    s.slice_count[t] = min(s.slice_count[t], k);  // run lengths for the merges
                }
                lds_barrier();
                // Pairwise merges in place: a thread finds where its eight outputs start in the two runs
                // (one binary search along the diagonal), merges them into registers, and writes them once
                // everybody has read. Run lengths alternate between two small arrays.
                int* len_a = s.slice_count;
                int* len_b = reinterpret_cast<int*>(s.red32);
#pragma unroll 1
                for (int round = 0; round < 3; ++round) {
                    const int cap  = (2 * TK_SLICE_CAP) << round;  // slots of a pair of runs
                    const int tpp  = cap / 8;                      // threads per pair
                    const int pair = t / tpp;
                    const int d    = (t % tpp) * 8;                // first output of this thread
                    const int nx = len_a[2 * pair], ny = len_a[2 * pair + 1];
                    const unsigned long long* X = bucket + pair * cap;
                    const unsigned long long* Y = X + cap / 2;
                    int lo = max(0, d - ny), hi = min(d, nx);
#pragma unroll 1
                    for (int step = 0; step < 11; ++step) {  // at most 1024 entries on either side
                        const int                mid = (lo + hi) >> 1;
                        const unsigned long long xv  = X[min(mid, cap / 2 - 1)];
                        const unsigned long long yv  = Y[min(max(d - 1 - mid, 0), cap / 2 - 1)];
                        const bool               go  = lo < hi;
                        const bool               up  = xv < yv;  // X[mid] comes before Y[d - 1 - mid]: take more of X
                        lo                           = go && up ? mid + 1 : lo;
                        hi                           = go && !up ? mid : hi;
                    }
                    int                xi = lo, yj = d - lo;
                    unsigned long long out[8];
                    unsigned long long xa = xi < nx ? X[xi] : ~0ull;
                    unsigned long long yb = yj < ny ? Y[yj] : ~0ull;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const bool take_x = xa < yb;
                        out[e]            = take_x ? xa : yb;
                        xi += take_x ? 1 : 0;
                        yj += take_x ? 0 : 1;
                        const unsigned long long nxt =
                            take_x ? (xi < nx ? X[min(xi, cap / 2 - 1)] : ~0ull) : (yj < ny ? Y[min(yj, cap / 2 - 1)] : ~0ull);
                        xa = take_x ? nxt : xa;
                        yb = take_x ? yb : nxt;
                    }
                    lds_barrier();
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        if (d + e < nx + ny) {
                            bucket[pair * cap + d + e] = out[e];
                        }
                    }
                    if (t % tpp == 0) {
                        len_b[pair] = nx + ny;
                    }
                    lds_barrier();
                    int* swap = len_a;
                    len_a     = len_b;
                    len_b     = swap;
                }
                // the first n_list entries, resolved into vocabulary index and value
                {
                    constexpr int LPT = 1024 / TK_THREADS;  // list entries per thread (k <= 1024)
                    int           my_idx[LPT];
                    float         my_val[LPT];
#pragma unroll
                    for (int r = 0; r < LPT; ++r) {
                        const int i = t + r * TK_THREADS;
                        my_idx[r]   = i < n_list ? s.sel.idx[(int)(bucket[i] & 0xFFFull)] : 0;
                        my_val[r]   = i < n_list ? key_to_float(~(uint32_t)(bucket[i] >> 32)) : 0.0f;
                    }
                    __syncthreads();
#pragma unroll
                    for (int r = 0; r < LPT; ++r) {
                        const int i = t + r * TK_THREADS;
                        if (i < n_list) {
                            s.sel.idx[i] = my_idx[r];
                            s.sel.w[i]   = my_val[r];
                        }
                    }
                }
                __syncthreads();
            }
            else {
#pragma unroll
            for (int r = 0; r < PER; ++r) {
                const int i = t + r * TK_THREADS;
                if (i < n) {
                    s.keys[i] = comp[r];
                }
            }
            __syncthreads();
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

            // ---- large candidate sets: two bitonic sorts (of exactly n keys: no padding to a power of two)
            block_sort_u64_2048(s.keys, n);
            for (int qi = t; qi < n; qi += TK_THREADS) {
                int                      idx;
                const unsigned long long nk = stage2_key(s.keys[qi], qi, qi, &idx);
                s.sel.idx[qi]               = idx;
                s.keys[qi]                  = nk;
            }
            __syncthreads();
            block_sort_u64_2048(s.keys, n);
            {
                int cnt = 0;
                for (int i = t; i < min(k, n); i += TK_THREADS) {
                    cnt += s.keys[i] != ~0ull ? 1 : 0;
                }
                n_list = block_sum_i<TK_WAVES>(cnt, (int*)s.red32);
            }
            // resolve the payload (position in the first sort) into the vocabulary index
            constexpr int LPT = 1024 / TK_THREADS;  // list entries per thread (k <= 1024)
            int           my_idx[LPT];
            float         my_val[LPT];
#pragma unroll
            for (int r = 0; r < LPT; ++r) {
                const int i = t + r * TK_THREADS;
                my_idx[r]   = i < n_list ? s.sel.idx[(int)(s.keys[i] & 0xFFFull)] : 0;
                my_val[r]   = i < n_list ? key_to_float(~(uint32_t)(s.keys[i] >> 32)) : 0.0f;
            }
            __syncthreads();
#pragma unroll
            for (int r = 0; r < LPT; ++r) {
                const int i = t + r * TK_THREADS;
                if (i < n_list) {
                    s.sel.idx[i] = my_idx[r];
                    s.sel.w[i]   = my_val[r];
                }
            }
            __syncthreads();
            }
        }
    }
    else {
        topk_literal<DT, Row>(rowctx, s, vocab, k, BS1, BS2, picks, &n_list);
        for (int i = t; i < n_list; i += TK_THREADS) {
            s.sel.w[i] = key_to_float(~(uint32_t)(s.keys[i] >> 32));
        }
        __syncthreads();
    }

    topk_finish_list<DT>(s, n_list, row, vocab, p, probs_in, u, end_ids, out);
}

// What a select workgroup asks for before it knows anything about its row: wave w takes the first
// 4 * 64 entries of chunk list w (most lists are shorter). Issued at the top of the kernel, the
// loads are in flight while the row's arguments arrive; topk_merge_lists consumes them.
constexpr int TK_PREFETCH = 4;
struct TopkListPrefetch {
    TopkEntry first[TK_PREFETCH];
};

__device__ __forceinline__ TopkListPrefetch topk_prefetch_lists(int splits, const TopkEntry* entries)
{
    TopkListPrefetch pf;
    const int        ch = wave_id();
    const TopkEntry* e  = entries + (size_t)(ch < splits ? ch : 0) * TK_CCAP;  // always inside the row's slots
#pragma unroll
    for (int r = 0; r < TK_PREFETCH; ++r) {
        pf.first[r] = e[r * WAVE + lane_id()];
    }
    return pf;
}

// Rows split over several workgroups: merge their lists from the workspace into s.cand.
// Returns the candidate count, or -1 for the literal replay; *thr_out is a valid bound when the result
// is >= k. `pf`: what topk_prefetch_lists returned at the top of the kernel (have_pf false: nothing was requested).
template<int DT>
__device__ __forceinline__ int topk_merge_lists(TopkShared& s, int k, int splits, const TopkChunkHeader* headers,
                                                const TopkEntry* entries, uint32_t* thr_out,
                                                const TopkListPrefetch& pf, bool have_pf = true)
{
    const int t = threadIdx.x;
    // Row-wide lower bound T0 of the k-th largest key, the larger of two valid ones: the largest
    // `threshold` of a chunk that holds >= k elements, and the smallest `share` when every chunk has one.
    // A list is complete above its own threshold (lists of chunks with fewer than k selectable elements
    // hold all of them), and T0 is never below the threshold of a list that was cut.
    uint32_t T0        = min_valid_key<DT>();
    uint32_t min_share = 0xFFFFFFFFu;
    bool     overflow  = false;
    for (int c = 0; c < splits; ++c) {
        const TopkChunkHeader h = headers[c];
        overflow                = overflow || (h.flags & 2u) != 0u;
        min_share               = h.share < min_share ? h.share : min_share;
        if ((h.flags & 1u) && h.threshold > T0) {
            T0 = h.threshold;
        }
    }
    if (overflow) {
        return -1;
    }
    if (min_share > T0) {
        T0 = min_share;  // 0 when some chunk has no share bound
    }
    // one wave per chunk list
    auto gather = [&](uint32_t thr) -> int {
        if (t == 0) {
            s.n_cand = 0;
        }
        __syncthreads();
        for (int ch = wave_id(); ch < splits; ch += TK_THREADS / WAVE) {
            const int        cnt = (int)headers[ch].count;
            const TopkEntry* e   = entries + (size_t)ch * TK_CCAP;
            for (int i0 = 0; i0 < cnt; i0 += WAVE) {
                const int i = i0 + lane_id();
                // the first rounds of a wave's first list were requested at the top of the kernel
                TopkEntry en = TopkEntry{0u, 0u};
                if (i < cnt) {
                    if (have_pf && ch == wave_id() && i0 < TK_PREFETCH * WAVE) {
                        en = pf.first[0];
#pragma unroll
                        for (int r = 1; r < TK_PREFETCH; ++r) {
                            en = i0 == r * WAVE ? pf.first[r] : en;
                        }
                    }
                    else {
                        en = e[i];
                    }
                }
                // one slot reservation per wave and round
                const bool               keep = i < cnt && en.key >= thr;
                const unsigned long long m    = __ballot(keep);
                int                      base = 0;
                if (lane_id() == 0 && m != 0ull) {
                    base = atomicAdd(&s.n_cand, (int)__builtin_popcountll(m));
                }
                base = __shfl(base, 0, WAVE);
                if (keep) {
                    const int slot = base + (int)__builtin_popcountll(m & ((1ull << lane_id()) - 1ull));
                    if (slot < TK_CCAP) {
                        s.cand.key[slot] = en.key;
                        s.cand.idx[slot] = en.idx;
                    }
                }
            }
        }
        __syncthreads();
        const int total = s.n_cand;
        __syncthreads();
        return total;
    };
    int n = gather(T0);
    if (n > TK_CCAP) {
        // large k over many chunks: find the exact k-th largest key by bisection over the lists
        auto count_ge = [&](uint32_t thr) -> int {
            int c = 0;
            for (int ch = 0; ch < splits; ++ch) {
                const int        cnt = (int)headers[ch].count;
                const TopkEntry* e   = entries + (size_t)ch * TK_CCAP;
                for (int i = t; i < cnt; i += TK_THREADS) {
                    c += e[i].key >= thr ? 1 : 0;
                }
            }
            return block_sum_i<TK_WAVES>(c, (int*)s.red32);
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
    if (n > TK_CCAP) {
        return -1;  // thousands of identical values around the k-th
    }
    if (n > k + k / 4 && n <= 4 * TK_THREADS) {
        // Cut the union to its k largest keys (and their ties) before the tie orders are replayed: the replay
        // ranks every candidate against every other one with 64-bit keys, twice.
        n = topk_cut_to_k(s, n, k);
    }
    *thr_out = T0;
    return n;
}

}  // namespace ftk
