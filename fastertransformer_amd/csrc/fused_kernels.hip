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

#include <mutex>
#include <vector>

#include "ftk_sampling.h"
#ifdef FTK_TEST_HOOKS
#include "ftk_test_hooks.h"
#endif
#include "ftk_fused.cuh"
#include "ftk_largek.cuh"
#include "ftk_lean.cuh"
#include "ftk_logprob.cuh"
#include "ftk_rowwide.cuh"

namespace ftk {

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

}  // namespace ftk

using namespace ftk;

#define FTK_HIP_CHECK(call)                                                                                            \
    do {                                                                                                               \
        const hipError_t e_ = (call);                                                                                  \
        if (e_ != hipSuccess) {                                                                                        \
            return (int)e_;                                                                                            \
        }                                                                                                              \
    } while (0)

// ---- optional per-kernel timing (HIP events on the caller's stream) ------------------------------
namespace {
struct KernelTimer {
    std::vector<hipEvent_t> start, stop;
    int                     used = 0;
};
KernelTimer g_timers[4];
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
    if (kernel < 0 || kernel > 3 || total_ms == nullptr || launches == nullptr) {
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

// Threads per row of a log-prob step in one launch (lp_wide_kernel). Measured on MI355X (k = 64, us per step with 1024
// / 512 / 256 threads per row; the two-launch form in brackets): 256 x 152064 f16 59 / 66 / 96 (129); 512 x 152064 f16
// 109 / 96 / 110 (153); 1024 x 152064 f16 209 / 174 / 200 (218); 1024 x 128256 f32 206 / 177 / 217 (219); 1024 x 50264
// f32 114 / 89 / 88 (111); 1024 x 32000 bf16 94 / 72 / 64; 8 x 50264 f32 28 / 33 / 47 (58). One workgroup per compute
// unit wants all sixteen waves on its row; with more rows than compute units, two workgroups of eight waves overlap
// one's reading with the other's arithmetic; many short rows do best with four of four.
static int lp_threads_per_row(int rows, int vocab_size)
{
    if (rows <= 256) {
        return 1024;
    }
    return rows >= 1024 && vocab_size <= 65536 ? 256 : 512;
}

#ifdef FTK_TEST_HOOKS
// Test hook (hooks build of the library only): non-zero sends every launch through the general stream, so
// that it can be compared with the lean gather on the shapes the lean gather normally takes.
static int g_fused_force_general = 0;
extern "C" void ftk_test_set_fused_force_general(int v)
{
    g_fused_force_general = v;
}
// Test hook: the form of the log-prob step. 0: the product's choice, 1: two launches, 1024 / 512 / 256: one launch
// with that many threads per row.
static int g_lp_form = 0;
extern "C" void ftk_test_set_lp_form(int v)
{
    g_lp_form = (v == 1 || v == 1024 || v == 512 || v == 256) ? v : 0;
}
// Test hook: non-zero keeps launches with a large k on the two launches of the lean gather also where one
// 1024-thread workgroup per row would make their lists in one.
static int g_largek_two_launches = 0;
extern "C" void ftk_test_set_largek_two_launches(int v)
{
    g_largek_two_launches = v;
}
// Test hook: non-zero keeps the selection in a launch of its own also where one workgroup per row could do both.
static int g_fused_two_launches = 0;
extern "C" void ftk_test_set_fused_two_launches(int v)
{
    g_fused_two_launches = v;
}
// Test hook: which kernels the last fused step launched. 0: general stream, 1: lean gather + select, 2: lean gather
// that also selects (one 256-thread workgroup per row), 3: one 1024-thread workgroup per row, 4: log-prob step,
// 5: large-k lists in one launch + select.
static int g_fused_last_path = -1;
extern "C" int ftk_test_last_fused_path(void)
{
    return g_fused_last_path;
}
#define FTK_NOTE_PATH(v) (g_fused_last_path = (v))
#else
static constexpr int g_fused_force_general = 0;
static constexpr int g_fused_two_launches  = 0;
static constexpr int g_largek_two_launches = 0;
static constexpr int g_lp_form             = 0;
#define FTK_NOTE_PATH(v) ((void)0)
#endif

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
    // Almost every launch takes the lean gather, which cuts a row differently from the general stream: in one
    // read of the logits for a small k (lean_mode 1), in two for a large one (2) where a row yields at least
    // twice k maxima.
    const LeanPlan lplan      = lean_plan(a->vocab_size, rows > 0 ? rows : 1, elem, 256 * LG_OCCUPANCY);
    const int      slot_u     = lean_slot_u(lplan.splits);
    // (an embedding bias is read in 16-byte vectors next to the row: both must start on 16-byte boundaries)
    const bool     bias_ok    = a->embedding_bias == nullptr
                         || (((uintptr_t)a->embedding_bias | (uintptr_t)a->logits) & 15u) == 0
                                && ((size_t)a->vocab_size_padded * elem) % 16 == 0;
    const bool     lean_ok    = bias_ok && !g_fused_force_general;
    const bool     one_read   = lean_ok && a->max_top_k <= LG_MAX_K;
    const bool     two_reads  = lean_ok && !one_read && slot_u > 0
                           && (size_t)lplan.splits * slot_u * LG_THREADS >= (size_t)2 * a->max_top_k
                           && (size_t)a->vocab_size / (16 / elem) >= (size_t)lplan.splits * slot_u * LG_THREADS;
    const int      lean_mode  = one_read ? 1 : (two_reads ? 2 : 0);
    // Log-prob outputs: the two-read step covers what the lean gather covers, for vocabularies of at least 1024
    // columns (the reference's softmax block); rows may start anywhere an element may.
    const bool want_log_probs = a->cum_log_probs != nullptr || a->output_log_probs != nullptr;
    if (want_log_probs
        && (lean_mode != 1 || a->embedding_bias != nullptr || a->max_top_k > TK_STAGE || a->vocab_size < LP_BLOCK
            || ((uintptr_t)a->logits % (uintptr_t)elem) != 0)) {
        return FTK_ERR_UNSUPPORTED;
    }
    // Up to one row per compute unit, or a few nearly full rounds of that, a small k, no bias: a 1024-thread
    // workgroup per row does the whole step in one launch (ftk_rowwide.cuh), provided the row's history bitmap fits
    // its LDS window. With at most 256 rows it is the faster form at every size measured (MI355X, k = 64, one
    // launch / gather + select in us: 96 x 128256 f32 24.5 / 33.1, 192 x 128256 f32 27.8 / 41.4, 160 x 152064 f16
    // 25.7 / 33.7, 192 x 50264 f32 20.5 / 26.9; 16 to 64 rows, bound by latency either way, within 1 us); with more,
    // it pays when the rounds of 256 workgroups are nearly full and the rows are long.
    const int  rw_rounds = (rows + 255) / 256;
    const bool rw_full   = rows * 5 >= rw_rounds * 256 * 4
                         && (size_t)a->vocab_size / (16 / elem) >= (size_t)RW_MIN_SUBS * RW_SUB_VECS;
    const bool rw_small  = rows <= 256 && a->vocab_size >= 1024;
    const bool rowwide   = lean_mode == 1 && !want_log_probs && a->embedding_bias == nullptr && lplan.splits > 1
                         && g_fused_two_launches == 0 && (rw_full || rw_small)
                         && (size_t)a->vocab_size / 32 + 4 <= (size_t)FUSED_BITMAP_WORDS_LARGE
                         && ((uintptr_t)a->logits & 15u) == 0 && ((size_t)a->vocab_size_padded * elem) % 16 == 0
                         && (a->penalty_type == FTK_PENALTY_NONE || a->penalties == nullptr
                             || a->step <= RW_HIST_U * RW_THREADS);
    // A large k (the launch reads twice) on up to one row per compute unit: one 1024-thread workgroup per row makes
    // the row's list in one launch (ftk_largek.cuh) where the lean gather takes two launches of small workgroups.
    // Measured on MI355X with k = 1024 in every row, us per step, one launch / two: 256 x 51200 f16 70.7 / 79.3, 16 x
    // 51200 f16 65 / 67, 256 x 128256 f32 94 / 100, 128 x 128256 f32 83 / 85, 160 x 152064 f16 87 / 96; a few long
    // rows are better spread over several workgroups each (16 x 128256 f32 78 / 58, 96 x 152064 f16 85 / 78), and
    // so is more than one round of rows (320 x 51200 f16 93 / 90, 320 x 152064 f16 130 / 116).
    const bool largek = lean_mode == 2 && !want_log_probs && a->embedding_bias == nullptr && rows <= 256
                        && (rows >= 128 || (size_t)a->vocab_size * elem <= ((size_t)128 << 10))
                        && g_largek_two_launches == 0 && a->max_top_k <= 1024
                        && (size_t)a->vocab_size / (16 / elem) >= (size_t)LK_GROUPS * LK_THREADS
                        && (size_t)a->vocab_size / 32 + 4 <= (size_t)FUSED_BITMAP_WORDS_LARGE
                        && ((uintptr_t)a->logits & 15u) == 0 && ((size_t)a->vocab_size_padded * elem) % 16 == 0;
    // A frequency penalty needs the counts of the history's ids, which only that kernel keeps (a table in LDS).
    if (a->frequency_penalties != nullptr
        && (a->penalties == nullptr || a->penalty_type != FTK_PENALTY_ADDITIVE || a->output_ids == nullptr)) {
        return FTK_ERR_ARGUMENT;  // x - presence - frequency * count: the presence array comes with it
    }
    if (a->frequency_penalties != nullptr && (!rowwide || a->vocab_size_padded > FUSED_COUNT_MAX_VOCAB)) {
        return FTK_ERR_UNSUPPORTED;
    }
    const size_t   slot_bytes = lean_mode == 2 ? (size_t)lplan.splits * slot_u * LG_THREADS * sizeof(uint32_t) : 0;
    const size_t   lean_bytes =
        (size_t)(rows > 0 ? rows : 0)
        * (lplan.splits * (sizeof(TopkChunkHeader) + (size_t)TK_CCAP * sizeof(TopkEntry)) + slot_bytes);
    const size_t   need = bitmap_bytes + (lean_mode != 0 && lean_bytes > plan.bytes ? lean_bytes : plan.bytes);
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
    p.frequencies        = (p.penalties != nullptr && a->step > 0) ? a->frequency_penalties : nullptr;

    char* ws = (char*)a->workspace;
    if (p.penalties != nullptr && a->step > 0) {
        if (a->output_ids == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        p.bitmaps = (uint32_t*)ws;
        // columns one workgroup streams (upper bound): does its bitmap window fit in LDS?
        const int    epv        = 16 / elem;
        const size_t range_cols = lean_mode != 0 ? (size_t)lplan.subs_per_wg * LG_SUB_VECS * epv + 2 * epv :
                                                   (size_t)plan.tiles_per_wg * TK_THREADS * TK_NVT * epv + epv;
        const size_t words      = (want_log_probs ? (size_t)a->vocab_size : range_cols) / 32 + 4;
        const bool   local      = words <= (size_t)FUSED_BITMAP_WORDS_LARGE && (many == 0 || lean_mode != 0)
                           && ((lean_mode != 0 ? lplan.splits : plan.splits) == 1 && !want_log_probs
                               || a->step <= FUSED_SPLIT_BITMAP_MAX_STEP);
        if (rowwide || largek) {
            p.lds_window = (size_t)a->vocab_size / 32 + 4 <= (size_t)FUSED_BITMAP_WORDS_SMALL ? 1 : 2;
        }
        else if (local) {
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
    l.subs_per_wg     = 0;
    l.headers         = (TopkChunkHeader*)(ws + bitmap_bytes);
    l.entries         = (TopkEntry*)(l.headers + (size_t)rows * plan.splits);
    l.slots           = nullptr;
    l.slot_u          = 0;
    // events carried by a launch when per-kernel timing is on
    auto take_events = [&](int which, hipEvent_t* e0, hipEvent_t* e1) {
        KernelTimer& tm = g_timers[which];
        *e0 = *e1 = nullptr;
        if (g_profile && tm.used < (int)tm.start.size()) {
            *e0 = tm.start[tm.used];
            *e1 = tm.stop[tm.used];
            tm.used++;
        }
    };
    auto launch_general = [&](int kind, int window, dim3 grid) -> int {
        hipEvent_t e0, e1;
        take_events(kind == FUSED_KIND_SELECT ? 2 : 1, &e0, &e1);
        if (a->dtype == FTK_DTYPE_F32) {
            return fused_launch_f32(kind, window, many, grid, st, p, l, e0, e1);
        }
        if (a->dtype == FTK_DTYPE_F16) {
            return fused_launch_f16(kind, window, many, grid, st, p, l, e0, e1);
        }
        return fused_launch_bf16(kind, window, many, grid, st, p, l, e0, e1);
    };
    const int window = p.bitmaps_ready ? 0 : (p.lds_window == 2 ? 2 : 1);
    int       rc;
    if (lean_mode != 0) {
        l.splits       = lplan.splits;
        l.subs_per_wg  = lplan.subs_per_wg;
        l.row_entries  = (size_t)lplan.splits * TK_CCAP;
        l.entries      = (TopkEntry*)(l.headers + (size_t)rows * lplan.splits);
        const dim3 lgrid(lplan.splits, rows);
        if (want_log_probs) {
            FTK_NOTE_PATH(4);
            LogProbLaunch lp;
            lp.cum_log_probs    = a->cum_log_probs;
            lp.output_log_probs = a->output_log_probs;
            lp.partial_max      = (float*)l.headers;  // one float per list header slot: the lists are not used
            lp.splits           = lplan.splits;
            hipEvent_t e0, e1;
            const int lp_threads = g_lp_form == 0 ? lp_threads_per_row(rows, a->vocab_size) : (g_lp_form == 1 ? 0 : g_lp_form);
            if (lp_threads != 0) {
                take_events(1, &e0, &e1);
                if (e0 != nullptr) {
                    FTK_HIP_CHECK(hipEventRecord(e0, st));
                }
                rc = a->dtype == FTK_DTYPE_F32 ? lp_wide_launch_f32(window, lp_threads, rows, st, p, l, lp) :
                     a->dtype == FTK_DTYPE_F16 ? lp_wide_launch_f16(window, lp_threads, rows, st, p, l, lp) :
                                                 lp_wide_launch_bf16(window, lp_threads, rows, st, p, l, lp);
                if (rc == 0 && e1 != nullptr) {
                    FTK_HIP_CHECK(hipEventRecord(e1, st));
                }
                return rc;
            }
            take_events(1, &e0, &e1);
            if (e0 != nullptr) {
                FTK_HIP_CHECK(hipEventRecord(e0, st));
            }
            rc = a->dtype == FTK_DTYPE_F32 ? lp_rowmax_launch_f32(window, lgrid, st, p, l, lp) :
                 a->dtype == FTK_DTYPE_F16 ? lp_rowmax_launch_f16(window, lgrid, st, p, l, lp) :
                                             lp_rowmax_launch_bf16(window, lgrid, st, p, l, lp);
            if (rc != 0) {
                return rc;
            }
            if (e1 != nullptr) {
                FTK_HIP_CHECK(hipEventRecord(e1, st));
            }
            take_events(2, &e0, &e1);
            if (e0 != nullptr) {
                FTK_HIP_CHECK(hipEventRecord(e0, st));
            }
            rc = a->dtype == FTK_DTYPE_F32 ? lp_row_launch_f32(window, rows, st, p, l, lp) :
                 a->dtype == FTK_DTYPE_F16 ? lp_row_launch_f16(window, rows, st, p, l, lp) :
                                             lp_row_launch_bf16(window, rows, st, p, l, lp);
            if (rc == 0 && e1 != nullptr) {
                FTK_HIP_CHECK(hipEventRecord(e1, st));
            }
            return rc;
        }
        if (rowwide) {
            FTK_NOTE_PATH(3);
            hipEvent_t e0, e1;
            take_events(1, &e0, &e1);
            const int w = p.lds_window == 2 ? 2 : 1;
            return a->dtype == FTK_DTYPE_F32 ? rowwide_launch_f32(w, rows, st, p, l, e0, e1) :
                   a->dtype == FTK_DTYPE_F16 ? rowwide_launch_f16(w, rows, st, p, l, e0, e1) :
                                               rowwide_launch_bf16(w, rows, st, p, l, e0, e1);
        }
        if (largek) {
            // one list per row from one launch, then the selection
            FTK_NOTE_PATH(5);
            l.splits = 1;
            hipEvent_t e0, e1;
            take_events(1, &e0, &e1);
            const int w = p.lds_window == 2 ? 2 : 1;
            rc = a->dtype == FTK_DTYPE_F32 ? largek_gather_launch_f32(w, rows, st, p, l, e0, e1) :
                 a->dtype == FTK_DTYPE_F16 ? largek_gather_launch_f16(w, rows, st, p, l, e0, e1) :
                                             largek_gather_launch_bf16(w, rows, st, p, l, e0, e1);
            if (rc != 0) {
                return rc;
            }
            take_events(2, &e0, &e1);
            return a->dtype == FTK_DTYPE_F32 ? lean_select_launch_f32(rows, st, p, l, e0, e1) :
                   a->dtype == FTK_DTYPE_F16 ? lean_select_launch_f16(rows, st, p, l, e0, e1) :
                                               lean_select_launch_bf16(rows, st, p, l, e0, e1);
        }
        // one workgroup per row: it also orders and samples, the step is one launch
        const bool row_select =
            lean_mode == 1 && lplan.splits == 1 && a->embedding_bias == nullptr && g_fused_two_launches == 0;
        FTK_NOTE_PATH(row_select ? 2 : 1);
        auto launch_lean = [&](int mode, int timer) -> int {
            hipEvent_t e0, e1;
            take_events(timer, &e0, &e1);
            if (a->dtype == FTK_DTYPE_F32) {
                return lean_gather_launch_f32(mode, row_select, window, lgrid, st, p, l, e0, e1);
            }
            if (a->dtype == FTK_DTYPE_F16) {
                return lean_gather_launch_f16(mode, row_select, window, lgrid, st, p, l, e0, e1);
            }
            return lean_gather_launch_bf16(mode, row_select, window, lgrid, st, p, l, e0, e1);
        };
        if (lean_mode == 2) {
            l.slots  = (uint32_t*)(l.entries + (size_t)rows * l.row_entries);
            l.slot_u = slot_u;
            rc       = launch_lean(LG_MODE_SLOTS, 3);
            if (rc != 0) {
                return rc;
            }
        }
        rc = launch_lean(lean_mode == 2 ? LG_MODE_PRESET : LG_MODE_STREAM, 1);
        if (rc != 0 || row_select) {
            return rc;
        }
        hipEvent_t e0, e1;
        take_events(2, &e0, &e1);
        if (a->dtype == FTK_DTYPE_F32) {
            return lean_select_launch_f32(rows, st, p, l, e0, e1);
        }
        if (a->dtype == FTK_DTYPE_F16) {
            return lean_select_launch_f16(rows, st, p, l, e0, e1);
        }
        return lean_select_launch_bf16(rows, st, p, l, e0, e1);
    }
    FTK_NOTE_PATH(0);
    if (plan.splits == 1) {
        return launch_general(FUSED_KIND_ROW, window, dim3(rows));
    }
    rc = launch_general(FUSED_KIND_GATHER, window, dim3(plan.splits, rows));
    if (rc != 0) {
        return rc;
    }
    return launch_general(FUSED_KIND_SELECT, 0, dim3(rows));
}

// ---- producer hand-over: the step over vocabulary shards ------------------------------------------------------
// The reference writes the logits of a step from the last GEMM (under tensor parallelism one vocabulary shard per
// rank, gathered afterwards: src/fastertransformer/models/multi_gpu_gpt/ParallelGpt.cc:1374-1433) and reads them
// back in DynamicDecodeLayer::forward (:1436-1501). Here a producer - a GEMM epilogue, or a rank that holds one
// shard - can hand over columns [col_offset, col_offset + cols) of every row on their own: the gather below leaves,
// per row and shard, the bounded candidate lists of the lean gather (every element at or above a lower bound of the
// k-th largest value of the shard's own columns) and, on request, the shard's (maximum, sum of exp(x - maximum)) of
// the final values; the merge runs the selection over the lists of all shards, which is the same deterministic
// computation wherever it runs. What crosses between the two is at most lists_per_shard * (16 + 8 * 2048) bytes
// per row and shard, typically a few hundred entries, instead of the row.
namespace ftk {

struct ShardLayout {
    LeanPlan plan;   // how a shard of the widest kind is cut into workgroups
    int      total;  // lists per row over all shards
    size_t   bitmap_bytes, bytes;
};

static ShardLayout shard_layout(const ftk_fused_topk_args* a, const ftk_topk_shards* sh, int elem, int global_vp)
{
    ShardLayout y;
    const int   rows = a->local_batch_size > 0 ? a->local_batch_size : 1;
    y.plan           = lean_plan(sh->shard_width, rows, elem, 256 * LG_OCCUPANCY);
    const int most   = TK_MAXSPLIT / (sh->n_shards > 0 ? sh->n_shards : 1);
    if (y.plan.splits > most) {
        const int epv  = 16 / elem;
        const int nsub = (sh->shard_width / epv + 1 + LG_SUB_VECS - 1) / LG_SUB_VECS;
        y.plan.subs_per_wg = (nsub + most - 1) / most;
        y.plan.splits      = (nsub + y.plan.subs_per_wg - 1) / y.plan.subs_per_wg;
    }
    y.total        = y.plan.splits * sh->n_shards;
    const int words = (global_vp + 31) / 32 + 1;
    y.bitmap_bytes = ((size_t)rows * words * sizeof(uint32_t) + 255) / 256 * 256;  // the merge's recovery path
    y.bytes = y.bitmap_bytes + (size_t)rows * y.total * (sizeof(TopkChunkHeader) + (size_t)TK_CCAP * sizeof(TopkEntry));
    return y;
}

// (maximum, sum of exp(x - maximum)) over the final values of a shard's columns, one workgroup per row. The final
// value of a column is what top-k sees: temperature, history penalty, min-length and pad masks applied.
template<int DT>
__global__ void __launch_bounds__(256) shard_stats_kernel(FusedParams p, float* __restrict__ partials, int n_shards,
                                                          int shard)
{
    __shared__ float sh_m[4], sh_s[4];
    const int        row = blockIdx.x;
    if (row_flag_or(p.skip_decode, row, p.end_ids + row, false)
        || row_flag_or(p.finished_in, row, p.end_ids + row, false)) {
        if (threadIdx.x == 0) {  // rows that do not take part: an empty shard
            partials[((size_t)row * n_shards + shard) * 2 + 0] = -__builtin_inff();
            partials[((size_t)row * n_shards + shard) * 2 + 1] = 0.0f;
        }
        return;
    }
    FusedRow<DT, FUSED_BITMAP_WORDS_LARGE> r(p, row);
    r.prepare(0, p.V);
    __syncthreads();
    float m = -__builtin_inff(), sum = 0.0f;
    for (int v = threadIdx.x; v < p.V; v += 256) {
        if (r.never_selected(v)) {
            continue;
        }
        const float x = topk_value_at<DT>(r, v);
        if (x > m) {
            sum = sum * det_expf(m - x) + 1.0f;  // (exp(-inf) = 0 on the first element)
            m   = x;
        }
        else if (x > -__builtin_inff()) {
            sum += det_expf(x - m);
        }
    }
    auto merge = [](float& m0, float& s0, float m1, float s1) {
        const float mm = __builtin_fmaxf(m0, m1);
        if (mm > -__builtin_inff()) {
            s0 = s0 * det_expf(m0 - mm) + s1 * det_expf(m1 - mm);
        }
        m0 = mm;
    };
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        merge(m, sum, __shfl_xor(m, o, WAVE), __shfl_xor(sum, o, WAVE));
    }
    if (lane_id() == 0) {
        sh_m[wave_id()] = m;
        sh_s[wave_id()] = sum;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 4; ++w) {
            merge(m, sum, sh_m[w], sh_s[w]);
        }
        partials[((size_t)row * n_shards + shard) * 2 + 0] = m;
        partials[((size_t)row * n_shards + shard) * 2 + 1] = sum;
    }
}

__global__ void shard_stats_combine_kernel(const float* __restrict__ partials, float* __restrict__ row_stats, int rows,
                                           int n_shards)
{
    const int row = blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) {
        return;
    }
    float m = -__builtin_inff();
    for (int i = 0; i < n_shards; ++i) {
        m = __builtin_fmaxf(m, partials[((size_t)row * n_shards + i) * 2]);
    }
    float sum = 0.0f;
    for (int i = 0; i < n_shards; ++i) {
        const float mi = partials[((size_t)row * n_shards + i) * 2];
        if (mi > -__builtin_inff()) {
            sum += partials[((size_t)row * n_shards + i) * 2 + 1] * det_expf(mi - m);
        }
    }
    row_stats[2 * row]     = m;
    row_stats[2 * row + 1] = sum;
}

}  // namespace ftk

static int shard_common_checks(const ftk_fused_topk_args* a, const ftk_topk_shards* sh)
{
    if (a == nullptr || sh == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    if (a->dtype < 0 || a->dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    if (a->max_top_k < 1 || a->max_top_k > 1024) {
        return FTK_ERR_TOPK_DOMAIN;
    }
    if (sh->n_shards < 1 || sh->n_shards > 16 || sh->shard_width < 1) {
        return FTK_ERR_ARGUMENT;
    }
    if (a->max_top_k > LG_MAX_K || a->embedding_bias != nullptr || a->cum_log_probs != nullptr
        || a->output_log_probs != nullptr) {
        return FTK_ERR_UNSUPPORTED;  // one read of the shard, no bias, no log-prob outputs (see row_stats)
    }
    return 0;
}

extern "C" int ftk_fused_topk_shard_gather(ftk_fused_topk_args* a, const ftk_topk_shards* sh, ftk_stream_t stream)
{
    int rc = shard_common_checks(a, sh);
    if (rc != 0) {
        return rc;
    }
    const int elem = a->dtype == FTK_DTYPE_F32 ? 4 : 2;
    const int rows = a->local_batch_size;
    if (sh->shard < 0 || sh->shard >= sh->n_shards || sh->col_offset < 0 || a->vocab_size > sh->shard_width
        || a->vocab_size > a->vocab_size_padded) {
        return FTK_ERR_ARGUMENT;
    }
    const ShardLayout y = shard_layout(a, sh, elem, sh->global_vocab_size_padded);
    if (a->workspace == nullptr) {
        a->workspace_size = y.bytes;
        return 0;
    }
    if (a->workspace_size < y.bytes) {
        return FTK_ERR_WORKSPACE;
    }
    if (rows <= 0) {
        return 0;
    }
    if (a->logits == nullptr || a->end_ids == nullptr || a->top_ks == nullptr
        || (a->min_lengths != nullptr && a->sequence_length == nullptr)) {
        return FTK_ERR_ARGUMENT;
    }
    hipStream_t st = (hipStream_t)stream;
    FusedParams p{};
    p.logits             = a->logits;
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
    p.bitmap_words       = (sh->global_vocab_size_padded + 31) / 32 + 1;
    p.col_offset         = sh->col_offset;
    int window           = 1;
    if (p.penalties != nullptr && a->step > 0) {
        if (a->output_ids == nullptr) {
            return FTK_ERR_ARGUMENT;
        }
        // the history bitmap of a workgroup's columns lives in LDS (no whole-row bitmaps in this mode)
        const int    epv   = 16 / elem;
        const size_t words = ((size_t)y.plan.subs_per_wg * LG_SUB_VECS * epv + 2 * epv) / 32 + 4;
        if (words > (size_t)FUSED_BITMAP_WORDS_LARGE || a->step > FUSED_SPLIT_BITMAP_MAX_STEP) {
            return FTK_ERR_UNSUPPORTED;
        }
        p.bitmaps    = (uint32_t*)a->workspace;  // (marks "a history penalty applies"; the memory is not touched)
        p.lds_window = words <= (size_t)FUSED_BITMAP_WORDS_SMALL ? 1 : 2;
        window       = p.lds_window;
    }
    else {
        p.penalties = nullptr;
    }
    char*       ws = (char*)a->workspace;
    FusedLaunch l{};
    l.splits      = y.total;
    l.subs_per_wg = y.plan.subs_per_wg;
    l.row_entries = (size_t)y.total * TK_CCAP;
    // this shard's lists sit at [shard * lists_per_shard, ...) of every row's lists
    l.headers = (TopkChunkHeader*)(ws + y.bitmap_bytes) + (size_t)sh->shard * y.plan.splits;
    l.entries = (TopkEntry*)((TopkChunkHeader*)(ws + y.bitmap_bytes) + (size_t)rows * y.total)
                + (size_t)sh->shard * y.plan.splits * TK_CCAP;
    if (sh->partials != nullptr && p.penalties != nullptr
        && (size_t)a->vocab_size / 32 + 4 > (size_t)FUSED_BITMAP_WORDS_LARGE) {
        return FTK_ERR_UNSUPPORTED;  // (the statistics kernel keeps the bitmap of the shard's columns in LDS)
    }
    const dim3 grid(y.plan.splits, rows);  // (workgroups past a narrow shard's columns leave empty lists)
    rc = a->dtype == FTK_DTYPE_F32 ? lean_gather_launch_f32(LG_MODE_STREAM, false, window, grid, st, p, l, nullptr, nullptr) :
         a->dtype == FTK_DTYPE_F16 ? lean_gather_launch_f16(LG_MODE_STREAM, false, window, grid, st, p, l, nullptr, nullptr) :
                                     lean_gather_launch_bf16(LG_MODE_STREAM, false, window, grid, st, p, l, nullptr, nullptr);
    if (rc != 0 || sh->partials == nullptr) {
        return rc;
    }
    FTK_DISPATCH_DTYPE(a->dtype, hipLaunchKernelGGL((shard_stats_kernel<DT>), dim3(rows), dim3(256), 0, st, p,
                                                    sh->partials, sh->n_shards, sh->shard));
    FTK_LAUNCH_CHECK();
    return 0;
}

extern "C" int ftk_fused_topk_shard_merge(ftk_fused_topk_args* a, const ftk_topk_shards* sh, ftk_stream_t stream)
{
    int rc = shard_common_checks(a, sh);
    if (rc != 0) {
        return rc;
    }
    const int         elem = a->dtype == FTK_DTYPE_F32 ? 4 : 2;
    const int         rows = a->local_batch_size;
    const ShardLayout y    = shard_layout(a, sh, elem, a->vocab_size_padded);
    if (a->workspace == nullptr) {
        a->workspace_size = y.bytes;
        return 0;
    }
    if (a->workspace_size < y.bytes || sh->global_vocab_size_padded != a->vocab_size_padded) {
        return a->workspace_size < y.bytes ? FTK_ERR_WORKSPACE : FTK_ERR_ARGUMENT;
    }
    if (rows <= 0) {
        return 0;
    }
    if (a->ids == nullptr || a->end_ids == nullptr || a->top_ks == nullptr
        || (a->rng_state == nullptr && a->uniform_draws == nullptr)
        || (sh->row_stats != nullptr && sh->partials == nullptr)) {
        return FTK_ERR_ARGUMENT;
    }
    hipStream_t st = (hipStream_t)stream;
    FusedParams p{};
    p.logits             = a->logits;  // whole rows for the recovery of rows whose lists overflowed, or null
    p.V                  = a->vocab_size;
    p.Vp                 = a->vocab_size_padded;
    p.batch_size         = a->batch_size;
    p.step               = a->step;
    p.max_input_length   = a->max_input_length;
    p.temperatures       = a->temperatures;
    p.penalties          = (a->penalty_type != FTK_PENALTY_NONE && a->step > 0) ? a->penalties : nullptr;
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
    p.bitmaps            = p.penalties != nullptr ? (uint32_t*)a->workspace : nullptr;
    p.bitmap_words       = (a->vocab_size_padded + 31) / 32 + 1;
    char*       ws = (char*)a->workspace;
    FusedLaunch l{};
    l.ids             = a->ids;
    l.sequence_length = a->sequence_length;
    l.finished        = a->finished;
    l.rng             = (RngState*)a->rng_state;
    l.uniforms        = a->uniform_draws;
    l.splits          = y.total;
    l.row_entries     = (size_t)y.total * TK_CCAP;
    l.headers         = (TopkChunkHeader*)(ws + y.bitmap_bytes);
    l.entries         = (TopkEntry*)(l.headers + (size_t)rows * y.total);
    rc = a->dtype == FTK_DTYPE_F32 ? lean_select_launch_f32(rows, st, p, l, nullptr, nullptr) :
         a->dtype == FTK_DTYPE_F16 ? lean_select_launch_f16(rows, st, p, l, nullptr, nullptr) :
                                     lean_select_launch_bf16(rows, st, p, l, nullptr, nullptr);
    if (rc != 0 || sh->row_stats == nullptr) {
        return rc;
    }
    hipLaunchKernelGGL(shard_stats_combine_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, sh->partials,
                       sh->row_stats, rows, sh->n_shards);
    FTK_LAUNCH_CHECK();
    return 0;
}

// ---- plain read of a buffer: the yardstick of the streaming kernels ------------------------------------
// What the gather would cost if it did nothing but fetch: the same launch shape (256-thread workgroups, four
// per compute unit, each walking a contiguous share in sub-tiles of four 16-byte vectors per thread with two
// sub-tiles in flight, non-temporal loads), one maximum per vector, one float written per workgroup.
namespace ftk {
__global__ void __launch_bounds__(LG_THREADS, LG_OCCUPANCY)
read_yardstick_kernel(const uint4* __restrict__ data, size_t nvec, size_t vec_per_wg, float* __restrict__ sink)
{
    const int    t  = threadIdx.x;
    const size_t vb = (size_t)blockIdx.x * vec_per_wg;
    const size_t ve = vb + vec_per_wg < nvec ? vb + vec_per_wg : nvec;
    if (vb >= ve) {
        return;
    }
    const int nsub = (int)((ve - vb + LG_SUB_VECS - 1) / LG_SUB_VECS);
    uint4     raw[LG_RING][LG_NV];
    auto      load = [&](int slot, int q) {
#pragma unroll
        for (int j = 0; j < LG_NV; ++j) {
            size_t vi = vb + (size_t)q * LG_SUB_VECS + j * LG_THREADS + t;
            vi        = vi < ve ? vi : ve - 1;
            raw[slot][j] = lean_stream_load(data + vi);
        }
    };
#pragma unroll
    for (int r = 0; r < LG_RING; ++r) {
        if (r < nsub) {
            load(r, r);
        }
    }
    float m = -__builtin_inff();
    for (int q0 = 0; q0 < nsub; q0 += LG_RING) {
#pragma unroll
        for (int r = 0; r < LG_RING; ++r) {
            const int q = q0 + r;
            if (q < nsub) {
#pragma unroll
                for (int j = 0; j < LG_NV; ++j) {
                    m = __builtin_fmaxf(m, lean_raw_max<DT_F32>(raw[r][j]));
                }
                if (q + LG_RING < nsub) {
                    load(r, q + LG_RING);
                }
            }
        }
    }
    m = wave_max(m);
    if (lane_id() == 0) {
        sink[blockIdx.x * LG_WAVES + wave_id()] = m;
    }
}
}  // namespace ftk

extern "C" int ftk_measure_plain_read(const void* data, size_t bytes, float* sink, size_t sink_floats,
                                      ftk_stream_t stream, float* elapsed_ms)
{
    const int    wgs  = 256 * LG_OCCUPANCY;
    const size_t nvec = bytes / sizeof(uint4);
    if (data == nullptr || sink == nullptr || nvec == 0 || ((uintptr_t)data & 15u) != 0
        || sink_floats < (size_t)wgs * LG_WAVES) {
        return FTK_ERR_ARGUMENT;
    }
    const size_t vec_per_wg = ((nvec + wgs - 1) / wgs + LG_THREADS - 1) / LG_THREADS * LG_THREADS;
    hipStream_t  st         = (hipStream_t)stream;
    if (elapsed_ms == nullptr) {
        hipLaunchKernelGGL(read_yardstick_kernel, dim3(wgs), dim3(LG_THREADS), 0, st, (const uint4*)data, nvec,
                           vec_per_wg, sink);
        FTK_LAUNCH_CHECK();
        return 0;
    }
    hipEvent_t e0, e1;
    hipError_t e = hipEventCreate(&e0);
    if (e != hipSuccess) {
        return (int)e;
    }
    e = hipEventCreate(&e1);
    if (e != hipSuccess) {
        (void)hipEventDestroy(e0);
        return (int)e;
    }
    hipExtLaunchKernelGGL(read_yardstick_kernel, dim3(wgs), dim3(LG_THREADS), 0, st, e0, e1, 0, (const uint4*)data,
                          nvec, vec_per_wg, sink);
    e = hipGetLastError();
    if (e == hipSuccess) {
        e = hipEventSynchronize(e1);
    }
    if (e == hipSuccess) {
        e = hipEventElapsedTime(elapsed_ms, e0, e1);
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    return (int)e;
}

// ---- the fused step for callers that cannot allocate ------------------------------------------------
// Same step, with the workspace taken from a fixed array in device memory instead of the caller. Every GPU
// the library runs on holds its own copy of the array from the moment the code object is loaded until the
// process ends; its address on a device is looked up once, with that device current.
// (The test build of the library, which a test process loads next to the product library, keeps a token array and
// refuses every step: one 32 MiB array per GPU and process is enough.)
#ifdef FTK_TEST_HOOKS
constexpr size_t FTK_STATIC_BYTES = 256;
#else
constexpr size_t FTK_STATIC_BYTES = FTK_FUSED_STATIC_WORKSPACE_BYTES;
#endif
static __device__ __align__(256) unsigned char scratch[FTK_STATIC_BYTES];

namespace {
constexpr int FTK_MAX_DEVICES = 64;
std::mutex    g_scratch_mutex;
void*         g_scratch_ptr[FTK_MAX_DEVICES] = {};
}  // namespace

extern "C" int ftk_fused_topk_step_static(ftk_fused_topk_args* a, ftk_stream_t stream)
{
    if (a == nullptr) {
        return FTK_ERR_ARGUMENT;
    }
    int        device = -1;
    hipError_t e      = hipGetDevice(&device);
    if (e != hipSuccess) {
        return (int)e;
    }
    if (device < 0 || device >= FTK_MAX_DEVICES) {
        return FTK_ERR_ARGUMENT;
    }
    void* ptr = nullptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_ptr[device] == nullptr) {
            void* found = nullptr;
            e           = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
            if (e != hipSuccess) {
                return (int)e;
            }
            g_scratch_ptr[device] = found;
        }
        ptr = g_scratch_ptr[device];
    }
    // size the step exactly as the caller-workspace entry point would, and refuse what the array cannot hold
    ftk_fused_topk_args q = *a;
    q.workspace           = nullptr;
    q.workspace_size      = 0;
    const int rc          = ftk_fused_topk_step(&q, stream);
    if (rc != 0) {
        return rc;
    }
    a->workspace_size = q.workspace_size;  // reported back, so that the caller sees what was needed
    if (q.workspace_size > FTK_STATIC_BYTES) {
        return FTK_ERR_STATIC_WORKSPACE;
    }
    // Nothing in the workspace has to start at zero: list headers are written by every streaming workgroup
    // before the merging kernel reads them, lists are read up to the count in their header, and the history
    // bitmaps are cleared by the kernel that fills them.
    q.workspace      = ptr;
    q.workspace_size = FTK_STATIC_BYTES;
    return ftk_fused_topk_step(&q, stream);
}
