// Fused decode step for rows of the top-k layer when cum_log_probs / output_log_probs are requested.
//
// The reference then turns the penalised logits into probabilities over the whole row before it samples
// (src/fastertransformer/layers/sampling_layers/TopKSamplingLayer.cu:220-266: invokeAddBiasSoftMax, then the
// top-k kernels on probabilities, whose log-prob outputs are log p and log p - log S). Its kernel sequence
// moves the row nine times (temperature R+W, penalties, softmax 3R+3W, top-k k+2 R). Here the row is read
// twice and never written. Both reads apply temperature, history penalty and the min-length mask in registers:
//   1. the exact maximum of the row;
//   2. e_v = T(exp(y_v - max)) summed in the order of the reference's softmax
//      (sampling_topp_kernels.cu:1308-1344: thread t of 1024 adds columns t, t + 1024, ... one after the other;
//      reduce_kernel_utils.cuh:73-103: xor butterflies 16..1 inside 32-lane groups, then over the 32 group sums),
//      so the sum has the reference's bits; on the way the candidates of the top-k selection are gathered by e_v,
//      with a bound lowered by what the division and rounding to T can merge, so that every column whose
//      probability ties with the k-th largest is among them. The candidates' e_v then become probabilities
//      T(e_v / (sum + 1e-6)), the reference's tie orders are replayed on them and the row is sampled
//      (topk_select_lds with probabilities in). Rows it cannot bound take the literal replay on probabilities
//      computed on the fly.
// Two forms:
//   lp_wide_kernel - the product's: one launch, one workgroup of 1024, 512 or 256 threads per row does both reads
//                    (the second one comes from the caches), a thread owning 1, 2 or 4 whole summation chains;
//   lp_rowmax_kernel + lp_row_kernel - two launches: the first streams the row in the launch shape of the lean
//                    gather and leaves the maximum of every workgroup's share in the workspace, the second gives
//                    a row to one 256-thread workgroup whose threads own four neighbouring chains each and walk
//                    them with 16-byte (fp32) or 8-byte (16-bit types) loads that are 1024 columns apart. The test
//                    build of the library can select it; the forms must agree bit for bit.
// Preconditions (checked by the host, which otherwise reports FTK_ERR_UNSUPPORTED and the layer runs the kernel
// sequence): no embedding bias, largest k <= 128, vocabulary >= 1024 (the reference's block is min(V, 1024)
// threads). Rows may have any pitch and start on any element boundary: vector loads are the aligned vectors of the
// memory, and the few columns of the first one that lie in front of the row are masked or looked at one by one.
#pragma once
#include <type_traits>

#include "ftk_lean.cuh"

namespace ftk {

constexpr int LP_THREADS = 256;
constexpr int LP_CHAINS  = 4;     // neighbouring summation chains per thread
constexpr int LP_BLOCK   = 1024;  // chains per row: the reference's block size
constexpr int LP_RING    = 8;     // loads in flight per thread
constexpr int LP_HEAD    = 4;     // rounds examined before the first bound exists
static_assert(LP_THREADS * LP_CHAINS == LP_BLOCK, "a workgroup owns all chains of its row");

struct LogProbLaunch {
    float* cum_log_probs;     // [rows] or null
    float* output_log_probs;  // [rows] or null
    float* partial_max;       // [rows][splits]
    int    splits;            // workgroups per row of lp_rowmax_kernel
};

// The exact value of the largest element of a 16-byte vector whose first element is column `first` (`a` columns of
// the row's first vector lie in front of the row): plain vectors through their raw maximum (rounding to T and a
// positive multiplier keep the order), the others element by element.
template<int DT, int BMW>
__device__ __forceinline__ float lp_vector_max(const FusedRow<DT, BMW>& rowctx, const uint4& v, int first, int a,
                                               bool bitsv, bool ordered)
{
    typedef Storage<DT> S;
    constexpr int       EPV  = (int)(16 / sizeof(typename S::T));
    uint32_t            bits = 0u;
    if (bitsv) {
        if (BMW > 0 && a == 0) {  // the flags of a vector never straddle a word of the bitmap
            const int rel = first - rowctx.bm_origin;
            bits          = (rowctx.bm_word(rel >> 5) >> (rel & 31)) & ((1u << EPV) - 1u);
        }
        else {
            bits = rowctx.vector_bits(first, EPV);
        }
    }
    const uint32_t rel_end = (uint32_t)(rowctx.masked_end_id - first);
    if (bits == 0u && rel_end >= (uint32_t)EPV && ordered) {
        return rowctx.fast(lean_raw_max<DT>(v));
    }
    float vm = -__builtin_inff();
#pragma unroll
    for (int c = 0; c < EPV; ++c) {
        float x = rowctx.fast(vector_element<DT>(v, c));
        if ((bits >> c) & 1u) {
            x = rowctx.flagged(x, first + c);
        }
        if ((uint32_t)c == rel_end) {
            x = -S::max_t();
        }
        vm = __builtin_fmaxf(vm, x);
    }
    return vm;
}

// ---- pass 1 --------------------------------------------------------------------------------------------
template<int DT, int BMW>
__global__ void __launch_bounds__(LG_THREADS, LG_OCCUPANCY) lp_rowmax_kernel(FusedParams p, FusedLaunch l, LogProbLaunch lp)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    constexpr int         R   = LG_RING;
    __shared__ float      red[LG_WAVES];
    const int             t     = threadIdx.x;
    const int             row   = blockIdx.y;
    const int             chunk = blockIdx.x;
    // Rows may start anywhere: the 16-byte vectors are those of the memory, `a` columns of the first one lie in
    // front of the row. Vectors [vlo, vhi) lie inside columns [0, V); the first and the last workgroup of a row
    // look at the few columns in front of and behind them one by one.
    const T*              rowp  = (const T*)p.logits + (size_t)row * p.Vp;
    const int             a     = (int)(((uintptr_t)rowp & 15u) / sizeof(T));
    const uint4*          base  = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(rowp) - a * sizeof(T));
    const int             vlo   = (a + EPV - 1) / EPV;
    const int             vhi   = max(vlo, (a + p.V) / EPV);
    const int             vb    = min(vhi, vlo + chunk * l.subs_per_wg * LG_SUB_VECS);
    const int             ve    = min(vhi, vb + l.subs_per_wg * LG_SUB_VECS);
    const int             nvec  = ve - vb;
    const int             nsub  = (nvec + LG_SUB_VECS - 1) / LG_SUB_VECS;

    const bool hist = BMW > 0 && p.bitmaps != nullptr && p.penalties != nullptr;
    int        hist_ids[LG_HIST_U];
    if (hist) {
#pragma unroll
        for (int u = 0; u < LG_HIST_U; ++u) {
            const int pos = t + u * LG_THREADS;
            hist_ids[u]   = pos < p.step ? p.output_ids[(size_t)pos * p.batch_size + row] : -1;
        }
    }
    uint4 raw[R][LG_NV];
    auto  load = [&](int slot, int q) {
#pragma unroll
        for (int j = 0; j < LG_NV; ++j) {
            const int vi = min(vb + q * LG_SUB_VECS + j * LG_THREADS + t, ve - 1);
            raw[slot][j] = lean_stream_load(base + vi);
        }
    };
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r < nsub) {
            load(r, r);
        }
    }
    const bool        skip = row_flag_or(p.skip_decode, row, p.end_ids + row, false);
    const bool        fin  = row_flag_or(p.finished_in, row, p.end_ids + row, false);
    FusedRow<DT, BMW> rowctx(p, row);
    if (skip || fin) {
        return;
    }
    const bool first_wg = chunk == 0;
    const bool last_wg  = chunk == (int)gridDim.x - 1;
    const int  lo_col   = first_wg ? 0 : vb * EPV - a;
    const int  hi_col   = last_wg ? p.V : ve * EPV - a;
    if (hist) {
        uint32_t* window = fused_lds_bitmap<FusedRow<DT, BMW>::LDS_WORDS>();
        const int origin = lo_col & ~31;
        const int words  = min(FusedRow<DT, BMW>::LDS_WORDS, (hi_col - origin + 31) / 32 + 1);
        for (int i = t; i < words; i += LG_THREADS) {
            window[i] = 0u;
        }
        lds_barrier();
        auto mark = [&](int pos, int id) {
            if (id >= lo_col && id < hi_col && rowctx.history_position_counts(pos)) {
                atomicOr(&window[(id - origin) >> 5], 1u << ((id - origin) & 31));
            }
        };
#pragma unroll
        for (int u = 0; u < LG_HIST_U; ++u) {
            mark(t + u * LG_THREADS, hist_ids[u]);
        }
        for (int pos = t + LG_HIST_U * LG_THREADS; pos < p.step; pos += LG_THREADS) {
            mark(pos, p.output_ids[(size_t)pos * p.batch_size + row]);
        }
        rowctx.bm_mode   = 1;
        rowctx.bm_origin = origin;
    }
    lds_barrier();
    const bool  bitsv   = rowctx.has_vector_bits();
    const float mul     = rowctx.fast_mul;
    const bool  ordered = mul > 0.0f && mul < __builtin_inff();  // the plain transform keeps the order
    const float NEG_INF = -__builtin_inff();
    float       m       = NEG_INF;
    auto vector_max = [&](const uint4& v, int first) -> float {
        return lp_vector_max<DT, BMW>(rowctx, v, first, a, bitsv, ordered);
    };
    for (int q0 = 0; q0 < nsub; q0 += R) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int q = q0 + r;
            if (q < nsub) {
#pragma unroll
                for (int j = 0; j < LG_NV; ++j) {
                    const int   rel = q * LG_SUB_VECS + j * LG_THREADS + t;
                    const float vm  = vector_max(raw[r][j], (vb + min(rel, nvec - 1)) * EPV - a);
                    m               = __builtin_fmaxf(m, rel < nvec ? vm : NEG_INF);
                }
                if (q + R < nsub) {
                    load(r, q + R);
                }
            }
        }
    }
    if (first_wg) {
        // the columns in front of the first whole vector
        for (int v = t; v < min(p.V, vlo * EPV - a); v += LG_THREADS) {
            m = __builtin_fmaxf(m, topk_value_at<DT>(rowctx, v));
        }
    }
    if (last_wg) {
        // the columns behind the last whole vector
        for (int v = vhi * EPV - a + t; v < p.V; v += LG_THREADS) {
            m = __builtin_fmaxf(m, topk_value_at<DT>(rowctx, v));
        }
    }
    m = wave_max(m);
    if (lane_id() == 0) {
        red[wave_id()] = m;
    }
    lds_barrier();
    if (t == 0) {
        float r = red[0];
#pragma unroll
        for (int w = 1; w < LG_WAVES; ++w) {
            r = __builtin_fmaxf(r, red[w]);
        }
        lp.partial_max[(size_t)row * lp.splits + chunk] = r;
    }
}

// ---- pass 2 --------------------------------------------------------------------------------------------
// Row accessor of the recovery paths: the key of column v is that of its probability.
template<int DT>
struct ProbRow {
    typedef Storage<DT>       S;
    typedef typename S::T     T;
    FusedRow<DT, 0>*          base;
    float                     row_max;
    float                     denom;  // sum + 1e-6
    __device__ __forceinline__ void prepare_whole_row()
    {
        base->prepare_whole_row();
    }
    __device__ __forceinline__ float prob_of(float y) const
    {
        const float e = round_t<DT>(det_expf(y - row_max));
        return round_t<DT>(e / denom);
    }
    __device__ __forceinline__ uint32_t key_at(int v) const
    {
        const uint32_t bit = base->bm_mode != 0 ? base->vector_bits(v, 1) : 0u;
        return order_key(prob_of(base->slow(v, S::ld(base->rowp[v]), bit)));
    }
};

// element c of a thread's chunk (four neighbouring columns) as fp32
template<int DT>
__device__ __forceinline__ float lp_chunk_element(const uint4& v, int c)
{
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
    return __uint_as_float(w[c]);
}
template<int DT>
__device__ __forceinline__ float lp_chunk_element(const uint2& v, int c)
{
    const uint32_t w[2] = {v.x, v.y};
    return Storage<DT>::ld((uint16_t)(c & 1 ? w[c >> 1] >> 16 : w[c >> 1] & 0xFFFFu));
}

// Ties after the division: two e values give the same probability T(e / denom) only if they differ by less than
// a unit in the last place of that probability times denom. While the k-th largest probability is a normal
// number of T that is at most 2^-(mantissa bits - 1) of e (four half-units, to be safe): candidates are gathered
// down to e_bound * (1 - LP_TIE_REL). When it is subnormal the unit no longer shrinks with the value, ties reach
// arbitrarily far down, and the row takes the literal replay (lp_ties_bounded tells).
template<int DT>
__device__ __forceinline__ float lp_tie_rel()
{
    return DT == DT_F32 ? 2.384185791015625e-07f : (DT == DT_F16 ? 0.001953125f : 0.015625f);
}
template<int DT>
__device__ __forceinline__ bool lp_ties_bounded(float e_bound, float denom)
{
    const float smallest_normal = DT == DT_F16 ? 6.103515625e-05f : 1.17549435e-38f;
    return e_bound >= 2.0f * smallest_normal * denom;
}

// The end of a row, by TK_THREADS threads: the candidates in s.cand carry e = T(exp(y - max)) as their keys; they
// become probabilities T(e / denom), the list is cut to little more than k entries and the reference's tie orders
// are replayed on probabilities (topk_select_lds), which also samples and writes the row's outputs. `slot` is scratch
// for TK_THREADS keys. Rows whose candidates cannot be trusted take the literal replay.
template<int DT>
__device__ __forceinline__ void lp_finish(TopkShared& s, uint32_t* slot, int n, bool valid, uint32_t thr, float denom,
                                          float row_max, int k, float tp, float u, const FusedParams& p,
                                          const FusedLaunch& l, int row, const TopkOutputs& out)
{
    const int      t    = threadIdx.x;
    const uint32_t KMIN = min_valid_key<DT>();
    // ---- candidates: e -> probability
    if (n > TK_CCAP || !valid || !lp_ties_bounded<DT>(key_to_float(thr), denom)) {
        // The list is incomplete, or fewer than k columns have a non-zero e (then columns of probability zero
        // are picked too, by the reference's tie rules), or the k-th largest probability may be subnormal
        // (ties without bound): the literal replay, on probabilities.
        n = -1;
    }
    else {
        int positive = 0;
        for (int i = t; i < n; i += TK_THREADS) {
            const uint32_t key = order_key(round_t<DT>(key_to_float(s.cand.key[i]) / denom));
            s.cand.key[i]      = key;
            positive += key > order_key(0.0f) ? 1 : 0;
        }
        positive = block_sum_i<TK_WAVES>(positive, (int*)s.red32);
        if (positive < k) {
            // probabilities that round to zero reach into the top k: they tie with every other zero of the row
            n = -1;
        }
        else if (n > k + k / 2 && n <= 4 * TK_THREADS) {
            // keep what reaches the k-th largest of 256 slot maxima (at least k candidates do, and everything
            // that ties with the k-th largest probability does)
            uint32_t mx = 0u;
            for (int i = t; i < n; i += TK_THREADS) {
                const uint32_t key = s.cand.key[i];
                mx                 = key > mx ? key : mx;
            }
            slot[t] = mx;
            lds_barrier();
            const uint32_t P = lean_kth_of_slots(slot, k);
            lds_barrier();
            if (P > KMIN) {
                n = topk_prune(s, n, P);
            }
        }
    }
    FusedRow<DT, 0> r0(p, row);
    r0.team = TK_THREADS;  // (the workgroup may have had more threads: those have left)
    ProbRow<DT>     prow{&r0, row_max, denom};
    topk_select_lds<DT, ProbRow<DT>, true>(prow, s, n, KMIN, row, p.Vp, k, tp, p.max_top_k,
                                           l.entries + (size_t)row * l.row_entries, true, u, p.end_ids, out);
}

template<int DT, int BMW>
__global__ void __launch_bounds__(LP_THREADS) lp_row_kernel(FusedParams p, FusedLaunch l, LogProbLaunch lp)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    // a thread's load: LP_CHAINS neighbouring columns
    typedef typename std::conditional<sizeof(T) == 4, uint4, uint2>::type Chunk;
    // The row's history bitmap lives in LDS that nothing else uses while the row streams: the ordered-list area
    // of the select phase holds its first words, an array behind the select state the rest (four workgroups then
    // fit a compute unit even with the window of the largest vocabularies). Both are addressed as words of one
    // object, so that the choice between them is a choice between two uniform offsets.
    constexpr int LP_BM_OVERLAY = (int)(sizeof(TopkShared::sel) / sizeof(uint32_t));
    constexpr int LP_BM_TAIL    = BMW > LP_BM_OVERLAY ? BMW - LP_BM_OVERLAY : 1;
    struct LpShared {
        TopkShared s;
        uint32_t   bitmap_tail[LP_BM_TAIL];
    };
    static_assert(sizeof(TopkShared) % sizeof(uint32_t) == 0 && offsetof(LpShared, bitmap_tail) == sizeof(TopkShared),
                  "the tail follows the select state word for word");
    static_assert(LP_BM_OVERLAY % (LP_BLOCK / 32) == 0, "a round's bitmap words lie on one side of the seam");
    constexpr int LP_BM_HEAD_AT = (int)(offsetof(TopkShared, sel) / sizeof(uint32_t));
    constexpr int LP_BM_TAIL_AT = (int)(sizeof(TopkShared) / sizeof(uint32_t)) - LP_BM_OVERLAY;
    __shared__ LpShared   sh;
    TopkShared&           s = sh.s;
    __shared__ uint32_t   slot_key[2][LP_THREADS];
    __shared__ float      warp_sum[32];
    const int             t   = threadIdx.x;
    const int             row = blockIdx.x;
    // Rows may start anywhere: the chunks are those of the memory, `a` columns of the first one lie in front of
    // the row. Slot c of thread t then holds column n * LP_BLOCK + 4 t + c - a in round n, always of the same
    // summation chain (4 t + c - a modulo LP_BLOCK) and in ascending order; the chains are put back in their
    // places before they are added up.
    const T*              rowp = (const T*)p.logits + (size_t)row * p.Vp;
    const int             a    = (int)(((uintptr_t)rowp % sizeof(Chunk)) / sizeof(T));
    const Chunk*          base = reinterpret_cast<const Chunk*>(reinterpret_cast<const char*>(rowp) - a * sizeof(T));
    const int             rounds = (p.V + a + LP_BLOCK - 1) / LP_BLOCK;  // columns outside [0, V) are masked: e = 0 exactly

    // history first, then the first loads of the row, then the arguments
    const bool hist = BMW > 0 && p.bitmaps != nullptr && p.penalties != nullptr;
    int        hist_ids[LG_HIST_U];
    if (hist) {
#pragma unroll
        for (int u = 0; u < LG_HIST_U; ++u) {
            const int pos = t + u * LP_THREADS;
            hist_ids[u]   = pos < p.step ? p.output_ids[(size_t)pos * p.batch_size + row] : -1;
        }
    }
    Chunk        raw[LP_RING];
    const int    tcol  = t * LP_CHAINS;  // the thread's first column within a round
    const Chunk* tbase = base + t;
    // the last round may reach past the row: such a thread reads its chunk of the round before (never used).
    // A chunk of the memory that starts in front of the padded row's end holds at least one of its elements.
    const bool last_inside = (rounds - 1) * LP_BLOCK + tcol < a + p.Vp;
    // Every load is issued whatever the round (one past the row's end fetches the last round's chunk again, unused):
    // with the same number of loads on every path the waits can name the oldest load instead of all of them.
    auto load = [&](int slot, int n) {
        const int m = min(n, rounds - 1);
        raw[slot]   = tbase[(size_t)((m + 1 < rounds || last_inside) ? m : m - 1) * LP_THREADS];
    };
#pragma unroll
    for (int r = 0; r < LP_RING; ++r) {
        load(r, r);
    }
    const bool        skip = row_flag_or(p.skip_decode, row, p.end_ids + row, false);
    const bool        fin  = row_flag_or(l.finished, row, p.end_ids + row, false);
    const int         k    = row_arg_or(p.top_ks, row, p.end_ids + row, p.max_top_k);
    const float       tp   = row_arg_or(p.top_ps, row, p.end_ids + row, 1.0f);
    FusedRow<DT, BMW> rowctx(p, row);
    if (skip) {
        return;
    }
    if (fin) {
        if (t == 0) {
            l.ids[row] = p.end_ids[row];  // a finished row emits its end id: no draw, no log-prob, no length update
        }
        return;
    }
    int draw_bits = 0;
    if (t == 0) {
        draw_bits = __float_as_int(row_uniform(l.rng, l.uniforms, row));
    }
    const TopkOutputs out =
        topk_outputs(l.ids, l.sequence_length, l.finished, lp.cum_log_probs, lp.output_log_probs, row, p.end_ids);
    // the row's maximum: pass 1 left one per workgroup; pad columns count as -MAX_T
    float row_max = -3.402823466e+38f;
    for (int c = 0; c < lp.splits; ++c) {
        row_max = __builtin_fmaxf(row_max, lp.partial_max[(size_t)row * lp.splits + c]);
    }
    if (p.V < p.Vp) {
        row_max = __builtin_fmaxf(row_max, -S::max_t());
    }
    row_max = uniform_f(row_max);
    if (t == 0) {
        s.n_cand  = 0;
        s.misc[0] = draw_bits;
    }
    uint32_t* const lds_words = reinterpret_cast<uint32_t*>(&sh);
    auto            bitmap_at = [&](int w) { return (w < LP_BM_OVERLAY ? LP_BM_HEAD_AT : LP_BM_TAIL_AT) + w; };
    if (hist) {
        const int words = min(BMW, (p.V + 31) / 32 + 1);
        for (int i = t; i < words; i += LP_THREADS) {
            lds_words[bitmap_at(i)] = 0u;
        }
        lds_barrier();
        auto mark = [&](int pos, int id) {
            if (id >= 0 && id < p.V && rowctx.history_position_counts(pos)) {
                const int w = id >> 5;
                atomicOr(&lds_words[bitmap_at(w)], 1u << (id & 31));
            }
        };
#pragma unroll
        for (int u = 0; u < LG_HIST_U; ++u) {
            mark(t + u * LP_THREADS, hist_ids[u]);
        }
        for (int pos = t + LG_HIST_U * LP_THREADS; pos < p.step; pos += LP_THREADS) {
            mark(pos, p.output_ids[(size_t)pos * p.batch_size + row]);
        }
    }
    lds_barrier();
    const float u     = __int_as_float(s.misc[0]);
    const bool  bitsv = hist || rowctx.has_vector_bits();
    const uint32_t KMIN = min_valid_key<DT>();

    // e values of the LP_CHAINS columns of round n that a chunk holds; columns >= V give 0. What depends on the
    // round alone (the side of the bitmap seam, whether the round holds the masked end id or the end of the
    // vocabulary) is decided in scalar registers.
    auto e_values = [&](const Chunk& v, int n, float* e) {
        const int col  = n * LP_BLOCK + tcol - a;
        uint32_t  bits = 0u;
        if (bitsv) {
            if constexpr (BMW > 0) {
                if (a == 0) {
                    const int at = (n < LP_BM_OVERLAY / (LP_BLOCK / 32) ? LP_BM_HEAD_AT : LP_BM_TAIL_AT) + n * (LP_BLOCK / 32);
                    bits         = (lds_words[at + (tcol >> 5)] >> (tcol & 31)) & ((1u << LP_CHAINS) - 1u);
                }
                else if (col >= 0) {
                    // the four flags may straddle two words (the bitmap carries one word of slack)
                    const int sh = col & 31;
                    bits         = lds_words[bitmap_at(col >> 5)] >> sh;
                    if (sh + LP_CHAINS > 32) {
                        bits |= lds_words[bitmap_at((col >> 5) + 1)] << (32 - sh);
                    }
                    bits &= (1u << LP_CHAINS) - 1u;
                }
                else {
                    bits = (lds_words[bitmap_at(0)] << (-col)) & ((1u << LP_CHAINS) - 1u);  // columns 0 .. at slots -col ..
                }
            }
            else {
                bits = rowctx.vector_bits(col, LP_CHAINS);
            }
        }
        float y[LP_CHAINS];
#pragma unroll
        for (int c = 0; c < LP_CHAINS; ++c) {
            y[c] = rowctx.fast(lp_chunk_element<DT>(v, c));
        }
        // rare: a column of the history, the masked end id, the end of the vocabulary
        const bool     edge_round = (n + 1) * LP_BLOCK - a > p.V || (a != 0 && n == 0);
        const bool     end_round  = (uint32_t)(rowctx.masked_end_id - (n * LP_BLOCK - a)) < (uint32_t)LP_BLOCK;
        const uint32_t rel_end    = (uint32_t)(rowctx.masked_end_id - col);
        bool           rare       = bits != 0u;
        if (edge_round || end_round) {
            rare = rare || rel_end < (uint32_t)LP_CHAINS || col + LP_CHAINS > p.V || col < 0;
        }
        if (rare) {
#pragma unroll
            for (int c = 0; c < LP_CHAINS; ++c) {
                if ((bits >> c) & 1u) {
                    y[c] = rowctx.flagged(y[c], col + c);
                }
                if ((uint32_t)c == rel_end || (uint32_t)(col + c) >= (uint32_t)p.V) {
                    y[c] = -S::max_t();
                }
            }
        }
        float d[LP_CHAINS];
#pragma unroll
        for (int c = 0; c < LP_CHAINS; ++c) {
            d[c] = y[c] - row_max;
        }
        // one look for a NaN per chunk instead of one per column
        if (__builtin_isunordered(d[0], d[1]) || __builtin_isunordered(d[2], d[3])) {
#pragma unroll
            for (int c = 0; c < LP_CHAINS; ++c) {
                e[c] = round_t<DT>(det_expf_nonpos(d[c]));
            }
        }
        else {
#pragma unroll
            for (int c = 0; c < LP_CHAINS; ++c) {
                e[c] = round_t<DT>(det_expf_nonpos_number(d[c]));
            }
        }
        if (edge_round && (col + LP_CHAINS > p.V || col < 0)) {
#pragma unroll
            for (int c = 0; c < LP_CHAINS; ++c) {
                e[c] = (uint32_t)(col + c) < (uint32_t)p.V ? e[c] : 0.0f;  // (what lies outside the row adds nothing)
            }
        }
    };

    float    acc[LP_CHAINS] = {0.0f, 0.0f, 0.0f, 0.0f};  // the chains' running sums
    uint32_t thr            = KMIN;                      // candidates: e with key >= thr_low
    float    thr_low        = key_to_float(KMIN);
    uint32_t dmax           = 0u;  // largest key this thread has put on the list
    bool     valid          = false;
    int      par            = 0;
    auto     set_threshold  = [&](uint32_t key) {
        thr           = key;
        const float e = key_to_float(key);
        thr_low       = uniform_f(e - e * lp_tie_rel<DT>());
    };
    auto push = [&](float e, int col) {
        const uint32_t key  = order_key(e);
        const int      slot = atomicAdd(&s.n_cand, 1);
        if (slot < TK_CCAP) {
            s.cand.key[slot] = key;
            s.cand.idx[slot] = (uint32_t)col;
        }
        dmax = key > dmax ? key : dmax;
    };
    auto rebound = [&](uint32_t mine) {
        slot_key[par][t] = mine;
        lds_barrier();
        const uint32_t P = lean_kth_of_slots(slot_key[par], k);
        par ^= 1;
        if (P > thr && P > order_key(0.0f)) {  // at least k columns with e > 0 at or above it
            set_threshold(P);
            valid = true;
        }
    };

    // ---- head: the first rounds are summed and kept; their largest e per thread gives the first bound
    float head_e[LP_HEAD][LP_CHAINS];
    const int head = min(rounds, LP_HEAD);
    {
        float tmax = 0.0f;
#pragma unroll
        for (int n = 0; n < LP_HEAD; ++n) {
            if (n < head) {
                e_values(raw[n], n, head_e[n]);
#pragma unroll
                for (int c = 0; c < LP_CHAINS; ++c) {
                    acc[c] = acc[c] + head_e[n][c];
                    tmax   = __builtin_fmaxf(tmax, head_e[n][c]);
                }
            }
            load(n, n + LP_RING);
        }
        rebound(order_key(tmax));
#pragma unroll
        for (int n = 0; n < LP_HEAD; ++n) {
            if (n < head) {
#pragma unroll
                for (int c = 0; c < LP_CHAINS; ++c) {
                    const int col = n * LP_BLOCK + tcol + c - a;
                    if (head_e[n][c] >= thr_low && (uint32_t)col < (uint32_t)p.V) {
                        push(head_e[n][c], col);
                    }
                }
            }
        }
    }
    // ---- the rest of the row; the bound is raised again after 8, 16, 32, ... rounds
    static_assert(LP_RING % LP_HEAD == 0 && LP_RING > LP_HEAD, "the ring continues where the head stopped");
    int  next_tighten = 2 * LP_HEAD;
    auto one_round    = [&](int slot, int n) {
        float     e[LP_CHAINS];
        const int col0 = n * LP_BLOCK + tcol - a;
        e_values(raw[slot], n, e);
#pragma unroll
        for (int c = 0; c < LP_CHAINS; ++c) {
            acc[c] = acc[c] + e[c];
        }
        // one look per chunk for a candidate (a NaN is none, with or without the maximum)
        if (__builtin_fmaxf(__builtin_fmaxf(e[0], e[1]), __builtin_fmaxf(e[2], e[3])) >= thr_low) {
#pragma unroll
            for (int c = 0; c < LP_CHAINS; ++c) {
                if (e[c] >= thr_low && (uint32_t)(col0 + c) < (uint32_t)p.V) {
                    push(e[c], col0 + c);
                }
            }
        }
    };
    auto tighten = [&](int n) {
        if (n + 1 == next_tighten && n + 1 < rounds) {
            next_tighten *= 2;
            rebound(dmax);
        }
    };
    int n0 = LP_HEAD;
    // whole groups of LP_RING rounds: no guards, every slot is loaded again
    for (; n0 + LP_RING <= rounds; n0 += LP_RING) {
#pragma unroll
        for (int r = 0; r < LP_RING; ++r) {
            const int slot = (LP_HEAD + r) % LP_RING;
            one_round(slot, n0 + r);
            load(slot, n0 + r + LP_RING);
            tighten(n0 + r);
        }
    }
    // the last rounds (fewer than LP_RING): their chunks are on their way or here
#pragma unroll
    for (int r = 0; r < LP_RING - 1; ++r) {
        if (n0 + r < rounds) {
            one_round((LP_HEAD + r) % LP_RING, n0 + r);
            tighten(n0 + r);
        }
    }
    if (a != 0) {
        // chain 4 t + c - a (modulo LP_BLOCK) back to slot c of thread t; the bitmap's first words are done with
        float* chain = reinterpret_cast<float*>(lds_words + LP_BM_HEAD_AT);
        static_assert(sizeof(TopkShared::sel) >= LP_BLOCK * sizeof(float), "one float per chain");
        __syncthreads();
#pragma unroll
        for (int c = 0; c < LP_CHAINS; ++c) {
            chain[(tcol + c - a) & (LP_BLOCK - 1)] = acc[c];
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < LP_CHAINS; ++c) {
            acc[c] = chain[tcol + c];
        }
    }
    // ---- the sum, in the reference's order: chain t = 4 * thread + c; butterflies with masks 16, 8, 4 run
    // between the eight threads of a 32-chain group, masks 2 and 1 inside a thread
#pragma unroll
    for (int o = 4; o >= 1; o >>= 1) {
#pragma unroll
        for (int c = 0; c < LP_CHAINS; ++c) {
            acc[c] = acc[c] + __shfl_xor(acc[c], o, WAVE);
        }
    }
    acc[0] = acc[0] + acc[2];
    acc[1] = acc[1] + acc[3];
    acc[0] = acc[0] + acc[1];
    if ((t & 7) == 0) {
        warp_sum[t >> 3] = acc[0];
    }
    __syncthreads();
    float total = t < 32 ? warp_sum[t] : 0.0f;
    if (t < WAVE) {
#pragma unroll
        for (int o = 16; o >= 1; o >>= 1) {
            total = total + __shfl_xor(total, o, WAVE);
        }
        if (t == 0) {
            warp_sum[0] = total;
        }
    }
    __syncthreads();
    const float denom = uniform_f(warp_sum[0] + 1e-6f);
    const int   n     = s.n_cand;
    __syncthreads();
    lp_finish<DT>(s, slot_key[par], n, valid, thr, denom, row_max, k, tp, u, p, l, row, out);
}

// ---- one launch: a workgroup per row reads it twice ---------------------------------------------------------------
// With few rows lp_row_kernel's four waves per row are what bounds the step (about a microsecond per 1024 columns),
// and most compute units idle. Here THREADS threads share a row, thread t owning summation chains t, t + THREADS, ...
// of the reference's 1024, so the sum has the reference's order without any regrouping. First pass: the row's maximum
// after temperature, penalties and masks, and every thread's own largest value, from which the bound of the candidates
// follows (the k-th largest of 256 joined thread maxima, each of them a column of its own). Second pass (the row
// comes from the caches this time): e = T(exp(y - max)) summed chain by chain, candidates collected on the way. Then
// all waves but four leave and those finish like lp_row_kernel (lp_finish).
// THREADS = 1024 for launches of at most one row per compute unit; with more rows, workgroups of fewer threads share a
// compute unit and one's first pass (memory) runs beside another's second (arithmetic).
constexpr int LPW_THREADS = 1024;

#ifdef FTK_LP_STAMPS  // development builds: wall-clock stamps of a row's phases in its candidate list area
#define LPW_STAMP(i) if (threadIdx.x == 0) { reinterpret_cast<unsigned long long*>(l.entries + (size_t)blockIdx.x * l.row_entries)[i] = wall_clock64(); }
#else
#define LPW_STAMP(i)
#endif

template<int DT, int BMW, int THREADS>
__global__ void __launch_bounds__(THREADS) lp_wide_kernel(FusedParams p, FusedLaunch l, LogProbLaunch lp)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         CH = LP_BLOCK / THREADS;  // chains of a thread
    constexpr int         U  = 8 / CH;              // rounds (1024 columns each) of a thread's batch: 8 columns
    constexpr int         N  = U * CH;
    static_assert(THREADS * CH == LP_BLOCK && U * CH == 8 && THREADS % 32 == 0 && THREADS >= TK_THREADS,
                  "a workgroup owns all chains of its row");
    __shared__ TopkShared s;
    __shared__ uint32_t   wide_key[THREADS];
    __shared__ uint32_t   slot_key[TK_THREADS];
    __shared__ float      warp_sum[32];
    __shared__ float      redf[THREADS / WAVE];
    const int             t    = threadIdx.x;
    // The last rows first: whatever produced the logits wrote them shortly before this launch, and of a batch that is
    // larger than the last-level cache the rows written last are the ones still in it.
    const int             row  = (int)gridDim.x - 1 - (int)blockIdx.x;
    const T*              rowp = (const T*)p.logits + (size_t)row * p.Vp;
    // A workgroup that shares its compute unit with others is served first while it waits for memory more than it
    // computes (set-up, first pass, selection): its few instructions then do not queue behind the arithmetic of a
    // neighbour's second pass, and its loads stay in flight.
    if constexpr (THREADS < LPW_THREADS) {
        __builtin_amdgcn_s_setprio(3);
    }
    // slot j of a batch: round j / CH of the batch, chain (j % CH) * THREADS + t
    auto offset_of = [](int j) { return (j / CH) * LP_BLOCK + (j % CH) * THREADS; };
    // First pass, for the maximum only: the order of the columns does not matter, so the row comes in as the 16-byte
    // vectors of the memory, thread t taking vectors vlo + t, vlo + t + THREADS, ... (`a` columns of the row's first
    // vector lie in front of the row; what lies in front of vector vlo and behind vector vhi is looked at column by
    // column). The first vectors are on their way before anything else is read.
    constexpr int EPV   = (int)(16 / sizeof(T));
    constexpr int R1    = 8;  // vectors a thread keeps in flight
    const int     a     = (int)(((uintptr_t)rowp & 15u) / sizeof(T));
    const uint4*  base  = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(rowp) - a * sizeof(T));
    const int     vlo   = (a + EPV - 1) / EPV;
    const int     vhi   = max(vlo + 1, (a + p.V) / EPV);  // (a row has at least 1024 columns)
    const int     nvec  = vhi - vlo;
    const int     turns = (nvec + THREADS - 1) / THREADS;
    // (the history before them: its ids are scattered reads that nothing should queue behind)
    constexpr int HU   = 2048 / THREADS;
    const bool    hist = BMW > 0 && p.bitmaps != nullptr && p.penalties != nullptr;
    int           hist_ids[HU];
    if (hist) {
#pragma unroll
        for (int i = 0; i < HU; ++i) {
            const int pos = t + i * THREADS;
            hist_ids[i]   = pos < p.step ? p.output_ids[(size_t)pos * p.batch_size + row] : -1;
        }
    }
    uint4         ring[R1];
    // (every load is issued whatever the turn, one past the last fetches the last again, unused: with the same number
    // of loads on every path the waits can name the oldest load instead of everything in flight)
    auto vload = [&](int slot, int q) { ring[slot] = base[vlo + min(min(q, turns - 1) * THREADS + t, nvec - 1)]; };
#pragma unroll
    for (int r = 0; r < R1; ++r) {
        vload(r, r);
    }
    // Second pass: thread t takes columns of its own chains, batches of N
    const int nfull = p.V / (U * LP_BLOCK);  // batches that every thread holds in full
    T         buf[2][N];
    auto      load = [&](T* raw, int b) {
#pragma unroll
        for (int j = 0; j < N; ++j) {
            raw[j] = rowp[b * U * LP_BLOCK + offset_of(j) + t];
        }
    };
    const bool            skip = row_flag_or(p.skip_decode, row, p.end_ids + row, false);
    const bool            fin  = row_flag_or(l.finished, row, p.end_ids + row, false);
    const int             k    = row_arg_or(p.top_ks, row, p.end_ids + row, p.max_top_k);
    const float           tp   = row_arg_or(p.top_ps, row, p.end_ids + row, 1.0f);
    FusedRow<DT, BMW>     rowctx(p, row);
    LPW_STAMP(0)
    if (skip) {
        return;
    }
    if (fin) {
        if (t == 0) {
            l.ids[row] = p.end_ids[row];  // a finished row emits its end id: no draw, no log-prob, no length update
        }
        return;
    }
    if (t == 0) {
        s.n_cand = 0;
    }
    const TopkOutputs out =
        topk_outputs(l.ids, l.sequence_length, l.finished, lp.cum_log_probs, lp.output_log_probs, row, p.end_ids);
    if (hist) {
        // the row's history bitmap in LDS (launches with a window and a history penalty)
        uint32_t* window = fused_lds_bitmap<FusedRow<DT, BMW>::LDS_WORDS>();
        const int words  = min(FusedRow<DT, BMW>::LDS_WORDS, (p.V + 31) / 32 + 1);
        for (int i = t; i < words; i += THREADS) {
            window[i] = 0u;
        }
        __syncthreads();
        auto mark = [&](int pos, int id) {
            id -= p.col_offset;
            if (id >= 0 && id < p.V && rowctx.history_position_counts(pos)) {
                atomicOr(&window[id >> 5], 1u << (id & 31));
            }
        };
#pragma unroll
        for (int i = 0; i < HU; ++i) {
            if (hist_ids[i] >= 0) {
                mark(t + i * THREADS, hist_ids[i]);
            }
        }
        for (int pos = t + HU * THREADS; pos < p.step; pos += THREADS) {
            mark(pos, p.output_ids[(size_t)pos * p.batch_size + row]);
        }
        rowctx.bm_mode   = 1;
        rowctx.bm_origin = 0;
    }
    __syncthreads();
    LPW_STAMP(1)
    const uint32_t KMIN    = min_valid_key<DT>();
    const float    NEG_INF = -__builtin_inff();
    // The values of a batch's columns (v0 = the first one's, t included) after temperature, history penalty and the
    // min-length mask. A column's history flag is bit t % 32 of word v / 32 of the bitmap. The words of a batch are
    // read together, and one look tells whether any of its columns needs more than the multiplication.
    const bool bitsv = rowctx.has_vector_bits();
    const int  bsh   = t & 31;
    auto values = [&](int v0, const T* raw, float* y) {
        uint32_t w[N];
        uint32_t any = 0u;
        if (bitsv) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                w[j] = rowctx.bm_word((v0 + offset_of(j)) >> 5);
            }
#pragma unroll
            for (int j = 0; j < N; ++j) {
                any |= w[j];
            }
            any = (any >> bsh) & 1u;
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            y[j] = rowctx.fast(S::ld(raw[j]));
        }
        const uint32_t to_end = (uint32_t)(rowctx.masked_end_id - v0);  // offset_of(j) for the masked end id at slot j
        if (any != 0u || (to_end < (uint32_t)(U * LP_BLOCK) && (to_end & (THREADS - 1)) == 0u)) {  // rare
#pragma unroll
            for (int j = 0; j < N; ++j) {
                if (bitsv && ((w[j] >> bsh) & 1u)) {
                    y[j] = rowctx.flagged(y[j], v0 + offset_of(j));
                }
                if (to_end == (uint32_t)offset_of(j)) {
                    y[j] = -S::max_t();
                }
            }
        }
    };
    // the same for one column
    auto value = [&](int v, T raw) -> float {
        float y = rowctx.fast(S::ld(raw));
        if (bitsv && ((rowctx.bm_word(v >> 5) >> (v & 31)) & 1u)) {
            y = rowctx.flagged(y, v);
        }
        return v == rowctx.masked_end_id ? -S::max_t() : y;
    };
    // The second pass over the row: whole batches with the next one's loads issued before the current one is used,
    // then the columns behind them one by one, loaded together.
    // use_batch(v0, y) takes a batch's values, use_one(j, v, y) the value of column v at slot j.
    auto stream = [&](auto&& use_batch, auto&& use_one) {
        if (nfull > 0) {
            load(buf[0], 0);
        }
        auto batch = [&](const T* raw, int b) {
            float     y[N];
            const int v0 = b * U * LP_BLOCK + t;
            values(v0, raw, y);
            use_batch(v0, y);
        };
        // (every load is issued whatever the batch, one past the last fetches the last again, unused: with the same
        // number of loads on every path the waits can name the older batch instead of everything in flight)
        for (int b = 0; b < nfull; b += 2) {
            load(buf[1], min(b + 1, nfull - 1));
            batch(buf[0], b);
            load(buf[0], min(b + 2, nfull - 1));
            if (b + 1 < nfull) {
                batch(buf[1], b + 1);
            }
        }
        const int v0 = nfull * U * LP_BLOCK + t;
        if (v0 < p.V) {
            T raw[N];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                raw[j] = rowp[min(v0 + offset_of(j), p.V - 1)];
            }
#pragma unroll
            for (int j = 0; j < N; ++j) {
                if (v0 + offset_of(j) < p.V) {
                    use_one(j, v0 + offset_of(j), value(v0 + offset_of(j), raw[j]));
                }
            }
        }
    };

    // ---- first pass: the maximum (pad columns count as -MAX_T), and the thread's own
    float m = NEG_INF;
    {
        const float mul     = rowctx.fast_mul;
        const bool  ordered = mul > 0.0f && mul < __builtin_inff();  // the plain transform keeps the order
        for (int q0 = 0; q0 < turns; q0 += R1) {
#pragma unroll
            for (int r = 0; r < R1; ++r) {
                const int q = q0 + r;
                if (q < turns) {
                    const int   rel = q * THREADS + t;
                    const float vm  = lp_vector_max<DT, BMW>(rowctx, ring[r], (vlo + min(rel, nvec - 1)) * EPV - a, a,
                                                            bitsv, ordered);
                    m               = __builtin_fmaxf(m, rel < nvec ? vm : NEG_INF);
                }
                vload(r, q + R1);
            }
        }
        // the columns in front of the first whole vector and behind the last
        for (int v = t; v < min(p.V, vlo * EPV - a); v += THREADS) {
            m = __builtin_fmaxf(m, value(v, rowp[v]));
        }
        for (int v = vhi * EPV - a + t; v < p.V; v += THREADS) {
            m = __builtin_fmaxf(m, value(v, rowp[v]));
        }
    }
    LPW_STAMP(2)
    if (t == 0) {
        s.misc[0] = __float_as_int(row_uniform(l.rng, l.uniforms, row));  // (read behind the barriers of the sum)
    }
    float row_max = block_max<float, THREADS / WAVE>(m, redf, NEG_INF);
    LPW_STAMP(3)
    row_max       = __builtin_fmaxf(-3.402823466e+38f, row_max);
    if (p.V < p.Vp) {
        row_max = __builtin_fmaxf(row_max, -S::max_t());
    }
    row_max = uniform_f(row_max);
    // the bound: every thread's largest e belongs to a column of its own
    wide_key[t] = order_key(round_t<DT>(det_expf_nonpos(m - row_max)));
    __syncthreads();
    if (t < TK_THREADS) {
        uint32_t key = wide_key[t];
#pragma unroll
        for (int g = 1; g < THREADS / TK_THREADS; ++g) {
            key = max(key, wide_key[t + g * TK_THREADS]);
        }
        slot_key[t] = key;
    }
    __syncthreads();
    uint32_t       thr     = KMIN;
    float          thr_low = key_to_float(KMIN);
    bool           valid   = false;
    const uint32_t P       = lean_kth_of_slots(slot_key, k);
    if (P > order_key(0.0f)) {  // at least k columns with e > 0 at or above it
        thr           = P;
        const float e = key_to_float(P);
        thr_low       = uniform_f(e - e * lp_tie_rel<DT>());
        valid         = true;
    }

    LPW_STAMP(4)
    if constexpr (THREADS < LPW_THREADS) {
        __builtin_amdgcn_s_setprio(0);
    }
    // ---- second pass: the sum chain by chain, candidates on the way
    float acc[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        acc[c] = 0.0f;
    }
    auto push = [&](int v, float e) {
        const int slot = atomicAdd(&s.n_cand, 1);
        if (slot < TK_CCAP) {
            s.cand.key[slot] = order_key(e);
            s.cand.idx[slot] = (uint32_t)v;
        }
    };
    stream(
        [&](int v0, const float* y) {
            float d[N], e[N];
            bool  number = true;  // one look for a NaN per pair of columns instead of one per column
#pragma unroll
            for (int j = 0; j < N; ++j) {
                d[j] = y[j] - row_max;
            }
#pragma unroll
            for (int j = 0; j < N; j += 2) {
                number = number && !__builtin_isunordered(d[j], d[j + 1]);
            }
            if (number) {
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    e[j] = round_t<DT>(det_expf_nonpos_number(d[j]));
                }
            }
            else {
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    e[j] = round_t<DT>(det_expf_nonpos(d[j]));
                }
            }
            float top = e[0];
#pragma unroll
            for (int j = 0; j < N; ++j) {
                acc[j % CH] = acc[j % CH] + e[j];  // (slots of a chain in ascending order of their columns)
                top         = __builtin_fmaxf(top, e[j]);
            }
            if (top >= thr_low) {  // (a NaN is no candidate, with or without the maximum)
#pragma unroll
                for (int j = 0; j < N; ++j) {
                    if (e[j] >= thr_low) {
                        push(v0 + offset_of(j), e[j]);
                    }
                }
            }
        },
        [&](int j, int v, float y) {
            const float e = round_t<DT>(det_expf_nonpos(y - row_max));
            acc[j % CH]   = acc[j % CH] + e;
            if (e >= thr_low) {
                push(v, e);
            }
        });
    LPW_STAMP(5)
    if constexpr (THREADS < LPW_THREADS) {
        __builtin_amdgcn_s_setprio(3);
    }
    // the reference's order: xor butterflies inside 32-chain groups, then over the 32 group sums
#pragma unroll
    for (int c = 0; c < CH; ++c) {
#pragma unroll
        for (int o = 16; o >= 1; o >>= 1) {
            acc[c] = acc[c] + __shfl_xor(acc[c], o, 32);
        }
        if ((t & 31) == 0) {
            warp_sum[(c * THREADS + t) >> 5] = acc[c];
        }
    }
    __syncthreads();
    if (t < 32) {
        float total = warp_sum[t];
#pragma unroll
        for (int o = 16; o >= 1; o >>= 1) {
            total = total + __shfl_xor(total, o, 32);
        }
        if (t == 0) {
            warp_sum[0] = total;
        }
    }
    __syncthreads();
    if (wave_id() >= TK_WAVES) {
        return;  // the first four waves select
    }
    const float denom = uniform_f(warp_sum[0] + 1e-6f);
    const int   n     = s.n_cand;
    const float u     = __int_as_float(s.misc[0]);
    __syncthreads();
    LPW_STAMP(6)
    lp_finish<DT>(s, slot_key, n, valid, thr, denom, row_max, k, tp, u, p, l, row, out);
    LPW_STAMP(7)
}

// Launchers, one translation unit per element type (logprob_kernels.hip built with FTK_LP_DT = 0, 1, 2).
// window: 0 = history bitmaps in global memory, 1 = small LDS window, 2 = large.
int lp_rowmax_launch_f32(int window, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                         const LogProbLaunch& lp);
int lp_rowmax_launch_f16(int window, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                         const LogProbLaunch& lp);
int lp_rowmax_launch_bf16(int window, dim3 grid, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                          const LogProbLaunch& lp);
int lp_row_launch_f32(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                      const LogProbLaunch& lp);
int lp_row_launch_f16(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                      const LogProbLaunch& lp);
int lp_row_launch_bf16(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                       const LogProbLaunch& lp);
// threads: 1024, 512 or 256 per row
int lp_wide_launch_f32(int window, int threads, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                       const LogProbLaunch& lp);
int lp_wide_launch_f16(int window, int threads, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                       const LogProbLaunch& lp);
int lp_wide_launch_bf16(int window, int threads, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                        const LogProbLaunch& lp);

}  // namespace ftk
