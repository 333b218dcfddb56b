// Fused decode step for rows owned by the top-k layer when no log-prob output is requested.
//
// The reference issues, per step, invokeBatchApplyTemperaturePenalty, invokeBatchApplyRepetitionPenalty,
// invokeMinLengthPenalty, invokeAddBiasEndMask and the two top-k kernels
// (src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.cc:302-352,
//  src/fastertransformer/layers/sampling_layers/TopKSamplingLayer.cu:220-266): each is a pass over
// the [batch, vocab_padded] logits, k+5 reads and 3 writes of every row in total. Here the row is read
// once and never written: the element arithmetic of those kernels (ftk_transform.cuh) is applied in
// registers while the chunk streams in, and the result feeds the candidate gather of ftk_topk.cuh.
//   fused_row_kernel      - one workgroup per row: stream, transform, select, sample, bookkeeping
//   fused_gather_kernel / fused_select_kernel - the same in two launches for small batches, whose rows
//                           are split over several workgroups
//   history_bitmap_kernel - very large vocabularies only: turns the time-major token history into a
//                           bitmap over the vocabulary (who gets the repetition / presence penalty)
#include <hip/hip_ext.h>

#include <vector>

#include "ftk_sampling.h"
#include "ftk_topk.cuh"

namespace ftk {

struct FusedParams {
    const void*  logits;
    const void*  bias;
    int          V, Vp, batch_size, step, max_input_length;
    const float* temperatures;
    const float* penalties;
    int          penalty_type;
    const int*   min_lengths;
    const int*   end_ids;
    const int*   input_lengths;
    const int*   output_ids;
    const int*   sequence_length_in;
    const int*   top_ks;
    const float* top_ps;
    int          max_top_k;
    const bool*  skip_decode;
    const bool*  finished_in;
    uint32_t*    bitmaps;        // [rows][bitmap_words] scratch, or null when no history penalty applies
    int          bitmap_words;
    int          bitmaps_ready;  // history_bitmap_kernel filled `bitmaps`
    int          lds_window;        // 0: none, 1: small LDS bitmap window, 2: large
};

// History bitmaps: bit v set <=> token v occurs in the row's (non-padding) history, i.e. column v gets
// the repetition / presence penalty. A streaming workgroup builds the window of the bitmap that covers
// its own columns in LDS (strided 4-byte reads of the history that overlap the logits loads already in
// flight). When the window does not fit, or many workgroups per row would each scan a long history,
// history_bitmap_kernel builds whole-row bitmaps in the workspace first.
constexpr int FUSED_BITMAP_WORDS_SMALL     = 2048 + 4;  // LDS window of 64 Ki columns: four workgroups per compute unit
constexpr int FUSED_BITMAP_WORDS_LARGE     = 5120 + 4;  // 160 Ki columns: three
constexpr int FUSED_BITMAP_WORDS_GLOBAL    = 0;         // no window: bitmaps in global memory
constexpr int FUSED_SPLIT_BITMAP_MAX_STEP  = 8192;

// the LDS window of the history bitmap (one per workgroup)
template<int BMW>
__device__ __forceinline__ uint32_t* fused_lds_bitmap()
{
    __shared__ uint32_t words[BMW];
    return words;
}

// BMW > 0: the history bitmap is a window of BMW words in LDS, built by prepare().
// BMW == 0: whole-row bitmaps in global memory (built by history_bitmap_kernel, or by
//           prepare_whole_row() for the literal replay).
__device__ __forceinline__ float uniform_f(float x)
{
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(x)));
}

template<int DT, int BMW>
struct FusedRow {
    static constexpr int  LDS_WORDS = BMW > 0 ? BMW : 1;
    typedef Storage<DT>   S;
    typedef typename S::T T;
    const T*              rowp;
    const T*              bias;
    int                   V, Vp;
    bool                  temp_active, keep_pads;
    float                 inv;
    float                 fast_mul;  // inv, or 1 when no temperature applies
    int                   penalty_type;  // 2 = none
    float                 penalty;
    float                 up_mul_neg, up_mul_pos, up_add;  // see flagged_upper
    bool                  up_ok;
    int                   masked_end_id;  // end id when the min-length mask applies, else -1
    // history bitmap
    int             bm_mode;    // 0: no history penalty, otherwise the bitmap is in place
    int             bm_origin;  // column of bit 0 of word 0
    uint32_t*       global_bm;  // this row's slice of the scratch bitmaps
    bool            global_ready;
    const int*      history;  // output_ids + row, stride batch_size
    int             batch_size, step, input_length, max_input_length;

    __device__ __forceinline__ FusedRow(const FusedParams& p, int row)
    {
        rowp        = (const T*)p.logits + (size_t)row * p.Vp;
        bias        = (const T*)p.bias;
        V           = p.V;
        Vp          = p.Vp;
        temp_active = p.temperatures != nullptr;
        const TemperatureCtx<DT> tc(temp_active ? p.temperatures[row] : 1.0f, V, Vp, false);
        inv           = tc.inv;
        fast_mul      = temp_active ? tc.inv : 1.0f;
        keep_pads     = tc.keep_pads;
        penalty_type  = p.penalties != nullptr ? p.penalty_type : 2;
        penalty       = p.penalties != nullptr ? p.penalties[row] : 0.0f;
        if (penalty_type == 0) {  // additive
            up_mul_neg = 1.0f;
            up_mul_pos = 1.0f;
            up_add     = -penalty;
            up_ok      = true;
        }
        else {
            up_ok      = penalty > 1e-30f && penalty < 1e30f;  // positive, finite, reciprocal not subnormal
            up_mul_neg = penalty;
            up_mul_pos = up_ok ? (1.0f / penalty) * 1.00000095367431640625f : 0.0f;
            up_add     = 0.0f;
        }
        global_bm     = (p.bitmaps != nullptr && penalty_type != 2) ? p.bitmaps + (size_t)row * p.bitmap_words : nullptr;
        global_ready  = p.bitmaps_ready != 0;
        bm_mode       = (BMW == 0 && global_bm != nullptr && global_ready) ? 1 : 0;
        bm_origin     = 0;
        history       = p.output_ids != nullptr ? p.output_ids + row : nullptr;
        batch_size    = p.batch_size;
        step          = p.step;
        max_input_length = p.max_input_length;
        input_length  = p.input_lengths != nullptr ? p.input_lengths[row] : p.max_input_length;
        // values that are the same for every lane of the workgroup but come out of floating-point
        // arithmetic: move them to scalar registers, they stay live for the whole kernel
        inv        = uniform_f(inv);
        fast_mul   = uniform_f(fast_mul);
        penalty    = uniform_f(penalty);
        up_mul_neg = uniform_f(up_mul_neg);
        up_mul_pos = uniform_f(up_mul_pos);
        up_add     = uniform_f(up_add);
        masked_end_id = -1;
        if (p.min_lengths != nullptr
            && min_length_masks(p.sequence_length_in[row], p.max_input_length, p.min_lengths[row])) {
            masked_end_id = p.end_ids[row];
        }
    }
    __device__ __forceinline__ const T* data() const
    {
        return rowp;
    }
    __device__ __forceinline__ bool history_position_counts(int t) const
    {
        return !(t >= input_length && t < max_input_length);  // skip the padding of short prompts
    }
    // called by every thread of the gather workgroup before it touches columns [lo, hi)
    __device__ __forceinline__ void prepare(int lo, int hi)
    {
        if (BMW == 0 || global_bm == nullptr) {
            return;
        }
        uint32_t* window = fused_lds_bitmap<LDS_WORDS>();
        const int origin = lo & ~31;
        const int words  = min(LDS_WORDS, (hi - origin + 31) / 32 + 1);
        for (int i = threadIdx.x; i < words; i += blockDim.x) {
            window[i] = 0u;
        }
        __syncthreads();
        // the history is time-major: every id is a cache line of its own, so the reads are issued eight
        // deep before the first one is used
        constexpr int U = 8;
        for (int t0 = threadIdx.x; t0 < step; t0 += U * blockDim.x) {
            int ids[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int t = t0 + u * blockDim.x;
                ids[u]      = (t < step && history_position_counts(t)) ? history[(size_t)t * batch_size] : -1;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (ids[u] >= lo && ids[u] < hi) {
                    atomicOr(&window[(ids[u] - origin) >> 5], 1u << ((ids[u] - origin) & 31));
                }
            }
        }
        __syncthreads();
        bm_mode   = 1;
        bm_origin = origin;
    }
    __device__ __forceinline__ uint32_t bm_word(int w) const
    {
        if (BMW > 0) {
            return fused_lds_bitmap<LDS_WORDS>()[w];
        }
        return global_bm[w];
    }
    // whole-row bitmap in global scratch, for the literal replay of rows the gather could not bound
    __device__ __forceinline__ void build_global_bitmap()
    {
        if (BMW > 0 || global_bm == nullptr || global_ready) {
            return;  // (a workgroup with an LDS window owns the whole row: the window already covers it)
        }
        const int words = (Vp + 31) / 32 + 1;
        for (int i = threadIdx.x; i < words; i += blockDim.x) {
            global_bm[i] = 0u;
        }
        __threadfence_block();
        __syncthreads();
        for (int t = threadIdx.x; t < step; t += blockDim.x) {
            if (history_position_counts(t)) {
                const int id = history[(size_t)t * batch_size];
                if (id >= 0 && id < Vp) {
                    atomicOr(&global_bm[id >> 5], 1u << (id & 31));
                }
            }
        }
        __threadfence_block();
        __syncthreads();
        bm_mode      = 1;
        bm_origin    = 0;
        global_ready = true;
    }
    // history-membership bits of columns first .. first+n-1 (n <= 8)
    __device__ __forceinline__ uint32_t vector_bits(int first, int n) const
    {
        if (bm_mode == 0) {
            return 0u;
        }
        uint32_t bits = 0u;
        if (first >= bm_origin) {
            const int rel = first - bm_origin;
            const int w   = rel >> 5;
            const int sh  = rel & 31;
            bits          = bm_word(w) >> sh;
            if (sh + n > 32) {
                bits |= bm_word(w + 1) << (32 - sh);  // both bitmaps carry one word of slack
            }
            bits &= (1u << n) - 1u;
        }
        else {
            for (int j = 0; j < n; ++j) {
                const int v = first + j;
                if (v >= bm_origin && v < Vp) {
                    bits |= ((bm_word((v - bm_origin) >> 5) >> ((v - bm_origin) & 31)) & 1u) << j;
                }
            }
        }
        return bits;
    }
    __device__ __forceinline__ bool plain_vector(int first, int n) const
    {
        return bias == nullptr && first + n <= V && !(masked_end_id >= first && masked_end_id < first + n);
    }
    __device__ __forceinline__ bool has_vector_bits() const
    {
        return bm_mode != 0;
    }
    // pad columns and the masked end id are -MAX_T whatever the logits hold
    __device__ __forceinline__ bool never_selected(int v) const
    {
        return v >= V || v == masked_end_id;
    }
    // interior column, no bias, not in the history, not the masked end id
    __device__ __forceinline__ float fast(float x) const
    {
        return round_t<DT>(x * fast_mul);  // fast_mul is 1 without a temperature: exact, and x is a T already
    }
    // the same column when it is in the history
    __device__ __forceinline__ float flagged(float xf) const
    {
        return round_t<DT>(repetition_value(xf, penalty, penalty_type));
    }
    // Never below flagged(xf), without the division and without branches: for the multiplicative rule
    // x * RN(1/p) * (1 + 2^-20) >= x / p for x >= 0 and a positive finite p (as real numbers, so also after
    // the monotone roundings); x < 0 and the additive rule are the exact operation. Rows whose penalty has
    // no usable reciprocal report +inf, which sends every flagged column to the exact evaluation.
    __device__ __forceinline__ float flagged_upper(float xf) const
    {
        const float y = round_t<DT>(xf * (xf < 0.0f ? up_mul_neg : up_mul_pos) + up_add);
        return up_ok ? y : __builtin_inff();
    }
    // flags of the NVT vectors a thread owns in one tile (first column first0, `stride` columns apart),
    // EPV bits each; requires (first0 - bm_origin) to be a multiple of EPV
    template<int EPV, int NVT>
    __device__ __forceinline__ void tile_bits(int first0, int stride, uint32_t* packed) const
    {
        constexpr int PW = NVT * EPV / 32;
#pragma unroll
        for (int i = 0; i < PW; ++i) {
            packed[i] = 0u;
        }
#pragma unroll
        for (int it = 0; it < NVT; ++it) {
            const int      rel = first0 + it * stride - bm_origin;
            const uint32_t b   = (bm_word(rel >> 5) >> (rel & 31)) & ((1u << EPV) - 1u);
            packed[(it * EPV) >> 5] |= b << ((it * EPV) & 31);
        }
    }
    // the value top-k would see for column v: temperature(+bias) -> history penalty -> min-length mask
    // -> pad mask, each rounded to T where the reference stores T
    __device__ __forceinline__ float slow(int v, float x, uint32_t in_history) const
    {
        if (temp_active) {
            if (v < V) {
                if (bias != nullptr) {
                    x = round_t<DT>(x + S::ld(bias[v]));
                }
                x = round_t<DT>(x * inv);
            }
            else if (!keep_pads) {
                x = -S::max_t();
            }
        }
        if (in_history) {
            x = round_t<DT>(repetition_value(x, penalty, penalty_type));
        }
        if (v == masked_end_id) {
            x = -S::max_t();
        }
        if (v >= V) {
            x = -S::max_t();  // addBiasEndMask: pad columns
        }
        return x;
    }
    __device__ __forceinline__ uint32_t key_at(int v) const
    {
        const uint32_t bit = bm_mode != 0 ? (bm_word((v - bm_origin) >> 5) >> ((v - bm_origin) & 31)) & 1u : 0u;
        return order_key(slow(v, S::ld(rowp[v]), bit));
    }
    // before key_at() may be used over the whole row
    __device__ __forceinline__ void prepare_whole_row()
    {
        build_global_bitmap();
    }
};

// Row -> bitmap of the token ids in its history window (skipping prompt padding), built in LDS and
// written out coalesced. Ids outside [0, Vp) are ignored.
constexpr int HB_THREADS = 256;
constexpr int HB_WORDS   = 8192;  // 262144 ids per LDS window

__global__ void __launch_bounds__(HB_THREADS)
history_bitmap_kernel(uint32_t* __restrict__ bitmaps, int bitmap_words, const int* __restrict__ output_ids,
                      int batch_size, int Vp, const int* __restrict__ input_lengths, int max_input_length, int step,
                      const bool* __restrict__ skip_decode, const bool* __restrict__ finished)
{
    __shared__ uint32_t bm[HB_WORDS];
    const int           row = blockIdx.x;
    if ((skip_decode != nullptr && skip_decode[row]) || (finished != nullptr && finished[row])) {
        return;
    }
    const int input_length = input_lengths != nullptr ? input_lengths[row] : max_input_length;
    uint32_t* out          = bitmaps + (size_t)row * bitmap_words;
    for (int base = 0; base < Vp; base += HB_WORDS * 32) {
        const int words = min(HB_WORDS, bitmap_words - (base >> 5));
        for (int i = threadIdx.x; i < words; i += HB_THREADS) {
            bm[i] = 0u;
        }
        __syncthreads();
        for (int t = threadIdx.x; t < step; t += HB_THREADS) {
            if (t >= input_length && t < max_input_length) {
                continue;
            }
            const int id = output_ids[(size_t)t * batch_size + row];
            if (id >= base && id < Vp && id < base + HB_WORDS * 32) {
                atomicOr(&bm[(id - base) >> 5], 1u << ((id - base) & 31));
            }
        }
        __syncthreads();
        for (int i = threadIdx.x; i < words; i += HB_THREADS) {
            out[(base >> 5) + i] = bm[i];
        }
        __syncthreads();
    }
}

struct FusedLaunch {
    int*             ids;
    int*             sequence_length;
    bool*            finished;
    RngState*        rng;
    const float*     uniforms;
    int              splits;
    int              tiles_per_wg;
    size_t           row_entries;
    TopkChunkHeader* headers;
    TopkEntry*       entries;
};

__device__ __forceinline__ float fused_row_draw(TopkShared& s, const FusedLaunch& l, int row)
{
    if (threadIdx.x == 0) {
        s.misc[0] = __float_as_int(row_uniform(l.rng, l.uniforms, row));
    }
    __syncthreads();
    return __int_as_float(s.misc[0]);
}

template<int DT, int BMW, int MANY = 0>
__global__ void __launch_bounds__(TK_THREADS, MANY > 0 ? TK_MIN_WGS_MANY : BMW <= FUSED_BITMAP_WORDS_SMALL ? TK_MIN_WGS : (TK_MIN_WGS * 3 + 3) / 4)
fused_row_kernel(FusedParams p, FusedLaunch l)
{
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    if (p.skip_decode != nullptr && p.skip_decode[row]) {
        return;
    }
    if (l.finished != nullptr && l.finished[row]) {
        if (threadIdx.x == 0) {
            l.ids[row] = p.end_ids[row];  // a finished row emits its end id without looking at the logits
        }
        return;
    }
    const int    k  = p.top_ks != nullptr ? p.top_ks[row] : p.max_top_k;
    const float  tp = p.top_ps != nullptr ? p.top_ps[row] : 1.0f;
    FTK_PHASE_BEGIN();
    const float  u  = fused_row_draw(s, l, row);
    const TopkOutputs out = topk_outputs(l.ids, l.sequence_length, l.finished, nullptr, nullptr, row, p.end_ids);
    FusedRow<DT, BMW> r(p, row);
    FTK_PHASE(0);
    uint32_t     thr = 0u;
    const int    n   = topk_stream<DT, FusedRow<DT, BMW>, MANY>(r, s, p.Vp, k, 0, topk_row_tiles<DT>(r.rowp, p.Vp), &thr);
    topk_select_lds<DT>(r, s, n, thr, row, p.Vp, k, tp, p.max_top_k, l.entries + (size_t)row * l.row_entries, false, u,
                        p.end_ids, out);
}

template<int DT, int BMW, int MANY = 0>
__global__ void __launch_bounds__(TK_THREADS, MANY > 0 ? TK_MIN_WGS_MANY : BMW <= FUSED_BITMAP_WORDS_SMALL ? TK_MIN_WGS : (TK_MIN_WGS * 3 + 3) / 4)
fused_gather_kernel(FusedParams p, FusedLaunch l)
{
    __shared__ TopkShared s;
    const int             row   = blockIdx.y;
    const int             chunk = blockIdx.x;
    if (p.skip_decode != nullptr && p.skip_decode[row]) {
        return;
    }
    if (p.finished_in != nullptr && p.finished_in[row]) {
        return;
    }
    const int    k = p.top_ks != nullptr ? p.top_ks[row] : p.max_top_k;
    FusedRow<DT, BMW> r(p, row);
    const int    tiles = topk_row_tiles<DT>(r.rowp, p.Vp);
    const int    t0    = min(tiles, chunk * l.tiles_per_wg);
    const int    t1    = min(tiles, t0 + l.tiles_per_wg);
    uint32_t     thr   = 0u;
    const int    n     = topk_stream<DT, FusedRow<DT, BMW>, MANY>(r, s, p.Vp, k, t0, t1, &thr);
    topk_dump_list(s, n, k, l.splits, thr, l.headers + (size_t)row * l.splits + chunk,
                   l.entries + (size_t)row * l.row_entries + (size_t)chunk * TK_CCAP);
}

template<int DT>
__global__ void __launch_bounds__(TK_THREADS) fused_select_kernel(FusedParams p, FusedLaunch l)
{
    constexpr int BMW = 0;  // the literal replay reads whole-row bitmaps from global memory
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    // everything the row needs is requested before the first decision: the arguments (scalar loads), the
    // chunk lists (vector loads), the draw
    TopkEntry*             row_entries = l.entries + (size_t)row * l.row_entries;
    const TopkListPrefetch pf          = topk_prefetch_lists(l.splits, row_entries);
    const bool   skip = p.skip_decode != nullptr && p.skip_decode[row];
    const bool   fin  = l.finished != nullptr && l.finished[row];
    const int    k    = p.top_ks != nullptr ? p.top_ks[row] : p.max_top_k;
    const float  tp   = p.top_ps != nullptr ? p.top_ps[row] : 1.0f;
    FusedRow<DT, BMW> r(p, row);
    if (skip) {
        return;
    }
    if (fin) {
        if (threadIdx.x == 0) {
            l.ids[row] = p.end_ids[row];
        }
        return;
    }
    const float  u  = fused_row_draw(s, l, row);
    const TopkOutputs out = topk_outputs(l.ids, l.sequence_length, l.finished, nullptr, nullptr, row, p.end_ids);
    uint32_t     thr         = 0u;
    const int    n = topk_merge_lists<DT>(s, k, l.splits, l.headers + (size_t)row * l.splits, row_entries, &thr, pf);
    topk_select_lds<DT, FusedRow<DT, BMW>, true>(r, s, n, thr, row, p.Vp, k, tp, p.max_top_k, row_entries, false, u, p.end_ids, out);
}

}  // namespace ftk

using namespace ftk;

// ---- optional per-kernel timing (HIP events on the caller's stream) ------------------------------
namespace {
struct KernelTimer {
    std::vector<hipEvent_t> start, stop;
    int                     used = 0;
};
KernelTimer g_timers[3];
bool        g_profile = false;

// Launches `kernel`; when timing is on, the launch itself carries a start and a stop event, so the
// pair brackets the kernel's execution and nothing else.
template<typename K, typename... Args>
void launch_timed(int which, K kernel, dim3 grid, dim3 block, hipStream_t st, Args... args)
{
    KernelTimer& t = g_timers[which];
    if (g_profile && t.used < (int)t.start.size()) {
        const int i = t.used++;
        hipExtLaunchKernelGGL(kernel, grid, block, 0, st, t.start[i], t.stop[i], 0, args...);
    }
    else {
        hipLaunchKernelGGL(kernel, grid, block, 0, st, args...);
    }
}
}  // namespace

#ifdef FTK_PHASE_TIMING
extern "C" int ftk_debug_read_phases_fused(unsigned long long* out, int reset)
{
    hipError_t e = hipMemcpyFromSymbol(out, HIP_SYMBOL(g_ftk_phase), sizeof(unsigned long long) * 32);
    if (e == hipSuccess && reset) {
        unsigned long long z[32] = {};
        e = hipMemcpyToSymbol(HIP_SYMBOL(g_ftk_phase), z, sizeof(z));
    }
    return (int)e;
}
#endif

extern "C" int ftk_profile_enable(int max_launches)
{
    for (auto& t : g_timers) {
        for (auto e : t.start) {
            (void)hipEventDestroy(e);
        }
        for (auto e : t.stop) {
            (void)hipEventDestroy(e);
        }
        t.start.clear();
        t.stop.clear();
        t.used = 0;
        for (int i = 0; i < max_launches; ++i) {
            hipEvent_t a, b;
            hipError_t e = hipEventCreate(&a);
            if (e != hipSuccess) {
                return (int)e;
            }
            e = hipEventCreate(&b);
            if (e != hipSuccess) {
                return (int)e;
            }
            t.start.push_back(a);
            t.stop.push_back(b);
        }
    }
    g_profile = max_launches > 0;
    return 0;
}

extern "C" int ftk_profile_read(int kernel, double* total_ms, int* launches)
{
    if (kernel < 0 || kernel > 2 || total_ms == nullptr || launches == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    KernelTimer& t = g_timers[kernel];
    double       sum = 0.0;
    for (int i = 0; i < t.used; ++i) {
        hipError_t e = hipEventSynchronize(t.stop[i]);
        if (e != hipSuccess) {
            return (int)e;
        }
        float ms = 0.0f;
        e        = hipEventElapsedTime(&ms, t.start[i], t.stop[i]);
        if (e != hipSuccess) {
            return (int)e;
        }
        sum += ms;
    }
    *total_ms = sum;
    *launches = t.used;
    t.used    = 0;
    return 0;
}

extern "C" int ftk_fused_topk_step(ftk_fused_topk_args* a, ftk_stream_t stream)
{
    if (a == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    if (a->dtype < 0 || a->dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (a->max_top_k < 1 || a->max_top_k > 1024) {
        return FTK_ERR_TOPK_DOMAIN;
    }
    const int      elem         = a->dtype == FTK_DTYPE_F32 ? 4 : 2;
    const int      rows         = a->local_batch_size;
    const TopkPlan plan         = topk_plan(a->vocab_size_padded, rows, a->max_top_k, elem);
    const int      many         = topk_many_level(a->max_top_k);  // > 0: the large-k kernels (whole-row bitmaps only)
    const int      bitmap_words = (a->vocab_size_padded + 31) / 32 + 1;  // +1: vector_bits may peek one word ahead
    const size_t   bitmap_bytes = ((size_t)rows * bitmap_words * sizeof(uint32_t) + 255) / 256 * 256;
    const size_t   need         = bitmap_bytes + plan.bytes;
    if (a->workspace == nullptr) {
        a->workspace_size = need;
        return 0;
    }
    if (a->workspace_size < need) {
        return FTK_ERR_WORKSPACE;
    }
    if (rows <= 0) {
        return 0;
    }
    if (a->logits == nullptr || a->ids == nullptr || a->end_ids == nullptr || a->top_ks == nullptr
        || (a->rng_state == nullptr && a->uniform_draws == nullptr)
        || (a->min_lengths != nullptr && a->sequence_length == nullptr)) {
        return FTK_ERR_ARGUMENT;
    }
    hipStream_t st = (hipStream_t)stream;
    FusedParams p{};
    p.logits             = a->logits;
    p.bias               = a->embedding_bias;
    p.V                  = a->vocab_size;
    p.Vp                 = a->vocab_size_padded;
    p.batch_size         = a->batch_size;
    p.step               = a->step;
    p.max_input_length   = a->max_input_length;
    p.temperatures       = a->temperatures;
    p.penalties          = a->penalty_type != FTK_PENALTY_NONE ? a->penalties : nullptr;
    p.penalty_type       = a->penalty_type;
    p.min_lengths        = a->min_lengths;
    p.end_ids            = a->end_ids;
    p.input_lengths      = a->input_lengths;
    p.output_ids         = a->output_ids;
    p.sequence_length_in = a->sequence_length;
    p.top_ks             = a->top_ks;
    p.top_ps             = a->top_ps;
    p.max_top_k          = a->max_top_k;
    p.skip_decode        = a->skip_decode;
    p.finished_in        = a->finished;
    p.bitmaps            = nullptr;
    p.bitmap_words       = bitmap_words;
    p.bitmaps_ready      = 0;
    p.lds_window         = 0;

    char* ws = (char*)a->workspace;
    if (p.penalties != nullptr && a->step > 0) {
        if (a->output_ids == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        p.bitmaps = (uint32_t*)ws;
        // columns one workgroup streams (upper bound): does its bitmap window fit in LDS?
        const int    epv        = 16 / elem;
        const size_t range_cols = (size_t)plan.tiles_per_wg * TK_THREADS * TK_NVT * epv + epv;
        const size_t words      = range_cols / 32 + 4;
        const bool   local      = words <= (size_t)FUSED_BITMAP_WORDS_LARGE && many == 0
                           && (plan.splits == 1 || a->step <= FUSED_SPLIT_BITMAP_MAX_STEP);
        if (local) {
            p.lds_window = words <= (size_t)FUSED_BITMAP_WORDS_SMALL ? 1 : 2;
        }
        else {
            launch_timed(0, history_bitmap_kernel, dim3(rows), dim3(HB_THREADS), st, p.bitmaps, bitmap_words, a->output_ids, a->batch_size,
                                                               a->vocab_size_padded, a->input_lengths,
                                                               a->max_input_length, a->step, a->skip_decode,
                                                               a->finished);
            FTK_LAUNCH_CHECK();
            p.bitmaps_ready = 1;
        }
    }
    else {
        p.penalties = nullptr;
    }
    FusedLaunch l;
    l.ids             = a->ids;
    l.sequence_length = a->sequence_length;
    l.finished        = a->finished;
    l.rng             = (RngState*)a->rng_state;
    l.uniforms        = a->uniform_draws;
    l.splits          = plan.splits;
    l.tiles_per_wg    = plan.tiles_per_wg;
    l.row_entries     = plan.row_entries;
    l.headers         = (TopkChunkHeader*)(ws + bitmap_bytes);
    l.entries         = (TopkEntry*)(l.headers + (size_t)rows * plan.splits);
    if (plan.splits == 1) {
        const dim3 grid1(rows), block(TK_THREADS);
        if (many == 2) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_row_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL, 2>, grid1,
                                                      block, st, p, l));
        }
        else if (many == 1) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_row_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL, 1>, grid1,
                                                      block, st, p, l));
        }
        else if (p.bitmaps_ready) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_row_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL>, grid1, block,
                                                      st, p, l));
        }
        else if (p.lds_window == 2) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_row_kernel<DT, FUSED_BITMAP_WORDS_LARGE>, grid1, block,
                                                      st, p, l));
        }
        else {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_row_kernel<DT, FUSED_BITMAP_WORDS_SMALL>, grid1, block,
                                                      st, p, l));
        }
        FTK_LAUNCH_CHECK();
        return 0;
    }
    dim3 grid(plan.splits, rows);
    {
        const dim3 block(TK_THREADS);
        if (many == 2) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_gather_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL, 2>, grid,
                                                      block, st, p, l));
        }
        else if (many == 1) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_gather_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL, 1>, grid,
                                                      block, st, p, l));
        }
        else if (p.bitmaps_ready) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_gather_kernel<DT, FUSED_BITMAP_WORDS_GLOBAL>, grid, block,
                                                      st, p, l));
        }
        else if (p.lds_window == 2) {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_gather_kernel<DT, FUSED_BITMAP_WORDS_LARGE>, grid, block,
                                                      st, p, l));
        }
        else {
            FTK_DISPATCH_DTYPE(a->dtype, launch_timed(1, fused_gather_kernel<DT, FUSED_BITMAP_WORDS_SMALL>, grid, block,
                                                      st, p, l));
        }
    }
    FTK_LAUNCH_CHECK();
    {
        FTK_DISPATCH_DTYPE(a->dtype,
                           launch_timed(2, fused_select_kernel<DT>, dim3(rows), dim3(TK_THREADS), st, p, l));
    }
    FTK_LAUNCH_CHECK();
    return 0;
}
