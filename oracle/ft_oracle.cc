// CPU ORACLE (test infrastructure only; never linked into or called by the product path).
//
// A plain, single-threaded restatement of the decode-step sampling path of
// NVIDIA/FasterTransformer: every function below follows one reference kernel or layer method
// and cites it. Thread-block shapes, tie resolution and floating-point summation orders of the
// reference kernels are restated literally (simulated thread partials, simulated cub trees),
// because sampled ids depend on them.
//
// Deliberate departures (reference behaviour is undefined or unavailable):
//  * `__expf` / `logf` are replaced by the deterministic det_expf / det_logf of oracle_math.h.
//  * cuRAND is replaced by an injected per-row uniform draw in (0, 1].
//  * Out-of-bounds accesses of the reference (exhausted top-k slices writing index -1, missing
//    bounds checks, history ids outside the vocabulary) are not replicated: an exhausted pick has
//    weight 0 and is never emitted; out-of-range history ids are skipped.
//  * Lanes that do not exist in a partially filled warp contribute the identity to
//    blockReduceSum / blockReduceMax (the reference shuffles from them, which is undefined).
//  * finalize: hypotheses from num_beams[b] on count as the lowest score (the reference scans
//    shared memory it never wrote for them).
//  * bfloat16 storage and the frequency penalty have no reference code ("parity unpinned");
//    they follow the generic `T` branches with fp32 arithmetic and one rounding per store.
//
// Pinning (tests/test_oracle.py, runs without a GPU):
//  * whole layer: the reference tests' known-answer id sets
//    (tests/unittests/test_sampling_layer.cu:318-592, 20 argument combinations x 3 dtypes) and the
//    Python known answers (tests/unittests/th_op/test_th_decode_op.py:233-324);
//  * top-k order and tie rule: a thread-by-thread Python simulation of topk_stage1 /
//    topk_stage2_sampling and of the cub reduction trees, written from the reference sources;
//    top-k set against numpy on distinct values; inverse CDF and log-probs against float64;
//  * temperature, repetition / presence, min-length, end mask, softmax, top-p walk and decay:
//    closed forms in float64 / exact binary cases; the softmax's summation order bit for bit against a
//    thread-by-thread float32 simulation; the rounding order of top-p's prefix sums
//    (cub::BlockScan<float, 256>::InclusiveSum with the running prefix, BLOCK_SCAN_RAKING) against a
//    thread-by-thread float32 simulation written from the vendored sources
//    (3rdparty/cub/block/specializations/block_scan_raking.cuh:601-655,
//    3rdparty/cub/warp/specializations/warp_scan_shfl.cuh:199-232, :465-487, :543-609), position for position, on
//    draws that a running sum or another raking split of the same terms would cross elsewhere
//    (tests/cub_block_scan.py); storage conversions against numpy and torch; det_expf / det_logf against float64;
//  * ban_bad_words, stop words, length criterion, finalize: no reference test exists, pinned by brute
//    force written from the source description only (finalize: a stable descending sort);
//  * beam search step (topk_softmax): no reference test exists; pinned by the definition it must reduce to
//    without hypotheses (the K largest of cum + log_softmax over all continuations, float64) and by
//    scenario checks of the hypothesis bookkeeping written from the source description; the penalties,
//    update and cache-indirection kernels around it, and the word lists with beams, by independent numpy
//    restatements of the description.
//  PARITY UNPINNED (no reference code or no way to run it here): bfloat16 storage, the frequency
//  penalty, the random stream (cuRAND XORWOW is replaced; draws are injected), the last-ulp
//  behaviour of __expf / logf (tolerance 1e-5 relative instead), and in the beam search step the
//  reference's pairwise (max, sum) merges in cub's order and its powf.
//
// Build: oracle/Makefile (g++ -O2 -ffp-contract=off).

#include "oracle_math.h"

#include <algorithm>
#include <cfloat>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <vector>

namespace oracle {

enum { DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2 };
enum { PEN_ADDITIVE = 0, PEN_MULTIPLICATIVE = 1, PEN_NONE = 2 };  // kernels/penalty_types.h:26-30

template<int DT>
struct St;
template<>
struct St<DT_F32> {
    typedef float T;
    static float  ld(T v) { return v; }
    static T      st(float f) { return f; }
    static float  max_t() { return FLT_MAX; }
};
template<>
struct St<DT_F16> {
    typedef uint16_t T;
    static float     ld(T v) { return half_to_float(v); }
    static T         st(float f) { return float_to_half(f); }
    static float     max_t() { return 65504.0f; }
};
template<>
struct St<DT_BF16> {
    typedef uint16_t T;
    static float     ld(T v) { return bf16_to_float(v); }
    static T         st(float f) { return float_to_bf16(f); }
    // largest finite bfloat16 (FLT_MAX itself would round to +inf)
    static float max_t() { return bf16_to_float(0x7F7F); }
};

// ------------------------------------------------------------------------------------------
// kernels/ban_bad_words.cu:22-86 (beam_width == 1)
// ------------------------------------------------------------------------------------------
template<int DT>
static void ban_bad_words(typename St<DT>::T* logits, const int* output_ids, int batch_size, int local_batch_size,
                          const int* bad_words, bool share_words, int bad_words_len, int id_offset,
                          int vocab_size_padded, int step)
{
    typedef St<DT> S;
    for (int row = 0; row < local_batch_size; ++row) {
        const int* base    = share_words ? bad_words : bad_words + (size_t)row * 2 * bad_words_len;
        const int* offsets = base + bad_words_len;
        for (int id = 0; id < bad_words_len; ++id) {
            if (offsets[id] < 0) {
                continue;
            }
            const int item_end   = offsets[id];
            const int item_start = id > 0 ? offsets[id - 1] : 0;
            const int item_size  = item_end - item_start;
            bool      should_ban = item_size == 1;
            if (item_size > 1 && step >= item_size - 1) {
                should_ban = true;
                for (int t = item_size - 2; t >= 0; --t) {
                    const int prev = output_ids[(size_t)(step - (item_size - 1) + t) * batch_size + id_offset + row];
                    if (prev != base[item_start + t]) {
                        should_ban = false;
                        break;
                    }
                }
            }
            if (should_ban) {
                const int tok = base[item_end - 1];
                if (0 < tok && tok < vocab_size_padded) {
                    logits[(size_t)row * vocab_size_padded + tok] = S::st(-INFINITY);
                }
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// kernels/sampling_penalty_kernels.cu:117-206 (batch) and :25-99 (scalar temperature)
// ------------------------------------------------------------------------------------------
template<int DT>
static void temperature_penalty(typename St<DT>::T* logits, const typename St<DT>::T* bias, const float* temperatures,
                                int temperatures_size, int batch, int V, int Vp, bool scalar_variant)
{
    typedef St<DT>        S;
    typedef typename S::T T;
    // half2 kernels are taken for T == half with even V and Vp (:87, :192); they leave pads alone.
    const bool h2 = (DT == DT_F16) && (V % 2 == 0) && (Vp % 2 == 0);
    for (int b = 0; b < batch; ++b) {
        const float temp = temperatures_size > 1 ? temperatures[b] : temperatures[0];
        const float inv  = 1.0f / (temp + 1e-6f);
        for (int v = 0; v < Vp; ++v) {
            T& x = logits[(size_t)b * Vp + v];
            if (v >= V) {
                if (!h2) {
                    x = S::st(-S::max_t());
                }
                continue;
            }
            if (DT == DT_F32) {
                float f = S::ld(x);
                if (bias != nullptr) {
                    f = f + S::ld(bias[v]);
                }
                else if (scalar_variant) {
                    f = f + 0.0f;  // generic scalar kernel always adds bias_val (:37-39)
                }
                x = S::st(f * inv);
            }
            else if (DT == DT_F16) {
                // arithmetic in half: hadd then hmul by half(inv)
                float f = S::ld(x);
                if (bias != nullptr) {
                    f = S::ld(S::st(f + S::ld(bias[v])));
                }
                else if (scalar_variant && !h2) {
                    f = S::ld(S::st(f + 0.0f));
                }
                const float inv_h = S::ld(S::st(inv));
                x                 = S::st(f * inv_h);
            }
            else {
                // bfloat16 extension: generic branch, fp32 multiply, one rounding per store
                float f = S::ld(x);
                if (bias != nullptr) {
                    f = S::ld(S::st(f + S::ld(bias[v])));
                }
                x = S::st(f * inv);
            }
        }
    }
}

// ------------------------------------------------------------------------------------------
// kernels/sampling_penalty_kernels.cu:367-459 (batch) / :224-337 (scalar)
// `vocab_stride` is the row stride the kernel is given (the layer passes vocab_size_padded,
// layers/sampling_layers/BaseSamplingLayer.cc:324).
// frequency != nullptr selects the frequency-penalty extension (additive only).
// ------------------------------------------------------------------------------------------
template<int DT>
static void repetition_penalty(typename St<DT>::T* logits, const float* penalties, int penalties_size,
                               const float* frequency, int frequency_size, const int* output_ids, int batch_size,
                               int local_batch_size, int vocab_stride, const int* input_lengths, int max_input_length,
                               int step, int type)
{
    typedef St<DT> S;
    if (type == PEN_NONE) {
        return;
    }
    std::vector<int>   ids;
    std::vector<float> vals;
    std::vector<int>   counts(frequency ? vocab_stride : 0);
    for (int b = 0; b < local_batch_size; ++b) {
        const float pen          = penalties_size > 1 ? penalties[b] : penalties[0];
        const float freq         = frequency ? (frequency_size > 1 ? frequency[b] : frequency[0]) : 0.0f;
        const int   input_length = input_lengths ? input_lengths[b] : max_input_length;
        auto*       row          = logits + (size_t)b * vocab_stride;
        ids.clear();
        vals.clear();
        if (frequency) {
            std::fill(counts.begin(), counts.end(), 0);
            for (int t = 0; t < step; ++t) {
                if (t >= input_length && t < max_input_length) {
                    continue;
                }
                const int id = output_ids[(size_t)t * batch_size + b];
                if (id >= 0 && id < vocab_stride) {
                    counts[id]++;
                }
            }
        }
        // phase 1: read every pre-penalty value
        for (int t = 0; t < step; ++t) {
            if (t >= input_length && t < max_input_length) {
                continue;
            }
            const int id = output_ids[(size_t)t * batch_size + b];
            if (id < 0 || id >= vocab_stride) {
                continue;
            }
            const float x = S::ld(row[id]);
            float       y;
            if (type == PEN_ADDITIVE) {
                y = x - pen;
                if (frequency) {
                    y = y - freq * (float)counts[id];
                }
            }
            else {
                y = x < 0.0f ? x * pen : x / pen;
            }
            ids.push_back(id);
            vals.push_back(y);
        }
        // phase 2: scatter
        for (size_t i = 0; i < ids.size(); ++i) {
            row[ids[i]] = S::st(vals[i]);
        }
    }
}

// kernels/sampling_penalty_kernels.cu:485-517
template<int DT>
static void min_length_penalty(typename St<DT>::T* logits, const int* min_lengths, const int* end_ids,
                               const int* sequence_lengths, int max_input_length, int batch, int Vp)
{
    typedef St<DT> S;
    for (int b = 0; b < batch; ++b) {
        if (sequence_lengths[b] + 1 - max_input_length < min_lengths[b]) {
            logits[(size_t)b * Vp + end_ids[b]] = S::st(-S::max_t());
        }
    }
}

// kernels/sampling_topk_kernels.cu:67-110
template<int DT>
static void add_bias_end_mask(typename St<DT>::T* logits, const typename St<DT>::T* bias, const int* end_ids,
                              const bool* finished, int batch, int V, int Vp)
{
    typedef St<DT> S;
    for (int b = 0; b < batch; ++b) {
        const bool fin = finished ? finished[b] : false;
        for (int v = 0; v < Vp; ++v) {
            auto& x = logits[(size_t)b * Vp + v];
            if (v >= V) {
                x = S::st(-S::max_t());
            }
            else if (fin) {
                x = S::st(v == end_ids[b] ? S::max_t() : -S::max_t());
            }
            else if (bias) {
                x = S::st(S::ld(x) + S::ld(bias[v]));
            }
        }
    }
}

// kernels/reduce_kernel_utils.cuh:73-103: xor butterfly (16,8,4,2,1) inside each 32-lane group,
// lane-0 partials to shared[warp], first warp butterflies again. Missing lanes add 0.
static float block_reduce_sum(const std::vector<float>& partial, int block)
{
    const int nwarps = (block + 31) / 32;
    float     shared[32];
    for (int w = 0; w < 32; ++w) {
        shared[w] = 0.0f;
    }
    for (int w = 0; w < nwarps; ++w) {
        float v[32];
        for (int l = 0; l < 32; ++l) {
            const int t = w * 32 + l;
            v[l]        = t < block ? partial[t] : 0.0f;
        }
        for (int mask = 16; mask > 0; mask >>= 1) {
            float nv[32];
            for (int l = 0; l < 32; ++l) {
                nv[l] = v[l] + v[l ^ mask];
            }
            std::memcpy(v, nv, sizeof(v));
        }
        shared[w] = v[0];
    }
    // val = threadIdx.x < blockDim.x / 32.f ? shared[lane] : 0
    float v[32];
    for (int l = 0; l < 32; ++l) {
        v[l] = ((float)l < (float)block / 32.0f) ? shared[l] : 0.0f;
    }
    for (int mask = 16; mask > 0; mask >>= 1) {
        float nv[32];
        for (int l = 0; l < 32; ++l) {
            nv[l] = v[l] + v[l ^ mask];
        }
        std::memcpy(v, nv, sizeof(v));
    }
    return v[0];
}

// kernels/sampling_topp_kernels.cu:1294-1361
template<int DT>
static void add_bias_softmax(typename St<DT>::T* logits, const typename St<DT>::T* bias, const int* end_ids,
                             const bool* finished, int m, int n_padded, int n)
{
    typedef St<DT> S;
    const int      block = std::min(n, 1024);
    std::vector<float> partial(block);
    for (int b = 0; b < m; ++b) {
        const bool fin = finished ? finished[b] : false;
        auto*      row = logits + (size_t)b * n_padded;
        float      mx  = -FLT_MAX;
        for (int v = 0; v < n_padded; ++v) {
            if (v < n) {
                if (fin) {
                    row[v] = S::st(v == end_ids[b] ? S::max_t() : -S::max_t());
                }
                else {
                    const float bv = bias ? S::ld(bias[v]) : 0.0f;
                    row[v]         = S::st(S::ld(row[v]) + bv);
                }
            }
            else {
                row[v] = S::st(-S::max_t());
            }
            mx = std::max(mx, S::ld(row[v]));  // fmaxf semantics for non-NaN inputs
        }
        // blockReduceMax pads the second stage with -1e20f when the block has < 32 warps
        // (reduce_kernel_utils.cuh:131)
        if (block < 1024) {
            mx = std::max(mx, -1e20f);
        }
        std::fill(partial.begin(), partial.end(), 0.0f);
        for (int v = 0; v < n_padded; ++v) {
            row[v] = S::st(det_expf(S::ld(row[v]) - mx));
            partial[v % block] += S::ld(row[v]);
        }
        const float s = block_reduce_sum(partial, block);
        for (int v = 0; v < n_padded; ++v) {
            row[v] = S::st(S::ld(row[v]) / (s + 1e-6f));
        }
    }
}

// ------------------------------------------------------------------------------------------
// cub::BlockReduce<TopK_2<T>, BLOCK> with reduce_topk_op_2 (a.u > b.u ? a : b):
// 3rdparty/cub/warp/specializations/warp_reduce_shfl.cuh:389-401 (lane l combines with l+offset,
// offsets 1,2,4,8,16), 3rdparty/cub/block/specializations/block_reduce_warp_reductions.cuh:113-160
// (thread 0 folds warp aggregates in ascending warp order).
// ------------------------------------------------------------------------------------------
struct Top2 {
    int   p;
    float u;
};
static inline Top2 top2_op(const Top2& a, const Top2& b)
{
    return a.u > b.u ? a : b;
}
static Top2 cub_block_reduce_top2(const Top2* partial, int block)
{
    const int nwarps = block / 32;
    Top2      agg{-1, 0.0f};
    for (int w = 0; w < nwarps; ++w) {
        Top2 v[32];
        for (int l = 0; l < 32; ++l) {
            v[l] = partial[w * 32 + l];
        }
        for (int offset = 1; offset < 32; offset <<= 1) {
            Top2 nv[32];
            for (int l = 0; l < 32; ++l) {
                nv[l] = (l + offset <= 31) ? top2_op(v[l], v[l + offset]) : v[l];
            }
            std::memcpy(v, nv, sizeof(v));
        }
        agg = (w == 0) ? v[0] : top2_op(agg, v[0]);
    }
    return agg;
}

// ------------------------------------------------------------------------------------------
// kernels/sampling_topk_kernels.cu:130-396 (topk_stage1, topk_stage2_sampling, dispatch)
// `uniforms[b]` replaces curand_uniform(curandstate + b).
// ------------------------------------------------------------------------------------------
template<int DT>
static int batch_topk_sampling(const typename St<DT>::T* log_probs, int* ids, int* sequence_length, bool* finished,
                               float* cum_log_probs, float* output_log_probs, const float* uniforms, int max_top_k,
                               const int* top_ks, float top_p, const float* top_ps, int vocab_size_padded,
                               const int* end_ids, int batch, const bool* skip_decode)
{
    typedef St<DT> S;
    if (max_top_k < 1 || max_top_k > 1024) {
        return 1;  // std::domain_error in the reference (:393-394)
    }
    const int   vocab = vocab_size_padded;
    const int   BS1   = max_top_k <= 16 ? 128 : 256;
    const int   BS2   = max_top_k <= 32 ? 128 : 256;
    const int   NB    = 8;
    const float MAXT  = S::max_t();
    const bool  probs_in = (cum_log_probs != nullptr || output_log_probs != nullptr);

    std::vector<float> tmp(vocab);
    std::vector<Top2>  partial(256);
    for (int b = 0; b < batch; ++b) {
        if (skip_decode && skip_decode[b]) {
            continue;
        }
        const int   k = top_ks ? top_ks[b] : max_top_k;
        const float p = top_ps ? top_ps[b] : top_p;
        if (finished && finished[b]) {
            ids[b] = end_ids[b];  // stage 2 early exit (:249-252)
            continue;
        }
        // ---- stage 1: per slice, k knock-out arg-max passes in type T
        std::vector<int>   cand_id((size_t)NB * k, -1);
        std::vector<float> cand_val((size_t)NB * k, -MAXT);
        const auto*        row = log_probs + (size_t)b * vocab;
        for (int v = 0; v < vocab; ++v) {
            tmp[v] = S::ld(row[v]);
        }
        for (int s = 0; s < NB; ++s) {
            auto thread_partial = [&](int t) {
                Top2 pt{-1, -MAXT};
                for (int e = t + s * BS1; e < vocab; e += BS1 * NB) {
                    if (tmp[e] > pt.u) {
                        pt.u = tmp[e];
                        pt.p = e;
                    }
                }
                return pt;
            };
            for (int t = 0; t < BS1; ++t) {
                partial[t] = thread_partial(t);
            }
            for (int ite = 0; ite < k; ++ite) {
                const Top2 total      = cub_block_reduce_top2(partial.data(), BS1);
                cand_id[s * k + ite]  = total.p;
                cand_val[s * k + ite] = total.u;
                if (total.p >= 0) {
                    tmp[total.p] = -MAXT;
                    // only the owning thread's partial changes on the next pass
                    partial[total.p % BS1] = thread_partial(total.p % BS1);
                }
            }
        }
        // ---- stage 2: k knock-out passes over 8k candidates in fp32
        // A slot that stage 1 could not fill (id -1) is not a candidate; for half its filler value
        // -65504 would otherwise compare above the fp32 sentinel.
        for (size_t i = 0; i < cand_id.size(); ++i) {
            if (cand_id[i] < 0) {
                cand_val[i] = -FLT_MAX;
            }
        }
        const int          size = k * NB;
        std::vector<int>   s_id(k, -1);
        std::vector<float> s_val2(k, 0.0f);
        float              s_sum = 0.0f, s_max = 0.0f;
        int                n_valid = 0;
        {
            auto thread_partial = [&](int t) {
                Top2 pt{-1, -FLT_MAX};
                for (int i = t; i < size; i += BS2) {
                    if (cand_val[i] > pt.u) {
                        pt.u = cand_val[i];
                        pt.p = i;
                    }
                }
                return pt;
            };
            for (int t = 0; t < BS2; ++t) {
                partial[t] = thread_partial(t);
            }
            for (int ite = 0; ite < k; ++ite) {
                Top2 total = cub_block_reduce_top2(partial.data(), BS2);
                if (ite == 0) {
                    s_max = total.u;
                }
                s_id[ite] = total.p;
                float w   = 0.0f;  // an exhausted pick carries no weight
                if (total.p >= 0) {
                    cand_val[total.p]      = -FLT_MAX;
                    partial[total.p % BS2] = thread_partial(total.p % BS2);
                    w                      = probs_in ? total.u : det_expf(total.u - s_max);
                    n_valid++;
                }
                s_val2[ite] = w;
                s_sum += w;
            }
        }
        // ---- sample (:282-311)
        if (n_valid == 0) {
            ids[b] = 0;
        }
        else {
            float rand_num = uniforms[b] * p * s_sum;
            for (int i = 0; i < k; ++i) {
                const float w = s_val2[i];
                rand_num      = rand_num - w;
                if (rand_num <= 0.0f || i == k - 1) {
                    int j = i;
                    while (s_id[j] < 0) {
                        j--;  // never emit an exhausted pick
                    }
                    ids[b] = cand_id[s_id[j]] % vocab;
                    if (probs_in) {
                        const float lp = det_logf(s_val2[j]);
                        if (cum_log_probs) {
                            cum_log_probs[b] += lp;
                        }
                        if (output_log_probs) {
                            output_log_probs[b] = lp - det_logf(s_sum);
                        }
                    }
                    break;
                }
            }
        }
        if (sequence_length && finished) {
            sequence_length[b] = finished[b] ? sequence_length[b] : sequence_length[b] + 1;
            finished[b]        = ids[b] == end_ids[b];
        }
    }
    return 0;
}

// ------------------------------------------------------------------------------------------
// kernels/sampling_topp_kernels.cu:801-860 (top-1 shortcut), :1106-1119 (stable descending
// segmented sort), :877-1004 (tile scan and pick). Scan rounding order:
// 3rdparty/cub/block/specializations/block_scan_raking.cuh:608-660 with 256 threads =
// 32 raking threads x 8 items (3rdparty/cub/block/block_raking_layout.cuh:79-85).
// ------------------------------------------------------------------------------------------
template<int DT>
static void batch_topp_sampling(const typename St<DT>::T* probs, int* ids, int* sequence_length, bool* finished,
                                float* cum_log_probs, float* output_log_probs, const float* uniforms, int batch,
                                int vocab, const int* end_ids, float top_p, const float* top_ps,
                                const bool* skip_decode)
{
    typedef St<DT>     S;
    std::vector<int>   order(vocab);
    std::vector<float> val(vocab);
    for (int b = 0; b < batch; ++b) {
        if (skip_decode && skip_decode[b]) {
            continue;
        }
        const float p   = top_ps ? top_ps[b] : top_p;
        const auto* row = probs + (size_t)b * vocab;
        for (int v = 0; v < vocab; ++v) {
            val[v] = S::ld(row[v]);
        }
        // arg-max, ties to the lowest index (TopK<T,1>::insert, reduce_kernel_utils.cuh:280-300)
        int best = 0;
        for (int v = 1; v < vocab; ++v) {
            if (val[v] > val[best]) {
                best = v;
            }
        }
        const float rand_num = uniforms[b] * p;  // drawn for every non-skipped row (:910-913)

        auto emit = [&](int id, float prob) {
            ids[b] = id;
            if (cum_log_probs || output_log_probs) {
                const float lp = det_logf(prob);
                if (cum_log_probs) {
                    cum_log_probs[b] += lp;
                }
                if (output_log_probs) {
                    output_log_probs[b] = lp;
                }
            }
            if (sequence_length && finished) {
                sequence_length[b] = finished[b] ? sequence_length[b] : sequence_length[b] + 1;
                finished[b]        = ids[b] == end_ids[b];
            }
        };
        // sum_prob = T(0) + max prob, compared as float (:842-849)
        const float sum_prob = S::ld(S::st(0.0f + val[best]));
        if (sum_prob >= p) {
            emit(best, val[best]);
            continue;
        }
        for (int v = 0; v < vocab; ++v) {
            order[v] = v;
        }
        std::stable_sort(order.begin(), order.end(), [&](int a, int c) { return val[a] > val[c]; });
        ids[b] = order[0];  // written before the loop (:954)

        float     carry  = 0.0f;
        const int ntiles = (vocab + 255) / 256;
        bool      done   = false;
        for (int tile = 0; tile < ntiles && !done; ++tile) {
            float x[256], c[256];
            for (int i = 0; i < 256; ++i) {
                const int g = tile * 256 + i;
                x[i]        = g < vocab ? val[order[g]] : 0.0f;
            }
            float seg[32], incl[32];
            for (int g = 0; g < 32; ++g) {
                float a = x[g * 8];
                for (int j = 1; j < 8; ++j) {
                    a = a + x[g * 8 + j];
                }
                seg[g] = a;
            }
            std::memcpy(incl, seg, sizeof(seg));
            for (int d = 1; d < 32; d <<= 1) {
                float nv[32];
                for (int l = 0; l < 32; ++l) {
                    nv[l] = l >= d ? incl[l - d] + incl[l] : incl[l];
                }
                std::memcpy(incl, nv, sizeof(nv));
            }
            const float block_aggregate = incl[31];
            const float block_prefix    = carry;
            carry                       = carry + block_aggregate;
            for (int g = 0; g < 32; ++g) {
                float a = g == 0 ? block_prefix : block_prefix + incl[g - 1];
                for (int j = 0; j < 8; ++j) {
                    a            = a + x[g * 8 + j];
                    c[g * 8 + j] = a;
                }
            }
            for (int w = 0; w < 8; ++w) {
                uint32_t mask = 0;
                for (int l = 0; l < 32; ++l) {
                    if (rand_num <= c[w * 32 + l]) {
                        mask |= 1u << l;
                    }
                }
                if (mask != 0) {
                    const int lane = 32 - __builtin_popcount(mask);
                    int       i    = tile * 256 + w * 32 + lane;
                    if (i >= vocab) {
                        i = vocab - 1;
                    }
                    emit(order[i], val[order[i]]);
                    done = true;
                    break;
                }
            }
        }
        // no crossing: ids[b] keeps the arg-max and nothing else is updated (:978-1003)
    }
}

// kernels/sampling_topp_kernels.cu:1381-1427
static void compute_topp_decay(float* runtime_top_p, const float* initial_top_p, const int* output_ids,
                               const float* decay, const float* top_p_min, const int32_t* reset_ids, int n)
{
    for (int i = 0; i < n; ++i) {
        if (output_ids[i] == reset_ids[i]) {
            runtime_top_p[i] = initial_top_p[i];
        }
        else {
            runtime_top_p[i] = std::max(runtime_top_p[i] * decay[i], top_p_min[i]);
        }
    }
}

// kernels/stop_criteria_kernels.cu:24-104 (beam_width == 1; rows of the local window only)
static void stop_words_criterion(const int* output_ids, const int* stop_words, bool* finished, int id_offset,
                                 int stop_words_len, int batch_size, int local_batch_size, int step)
{
    for (int row = 0; row < local_batch_size; ++row) {
        const int* base    = stop_words + (size_t)row * 2 * stop_words_len;
        const int* offsets = base + stop_words_len;
        for (int id = 0; id < stop_words_len; ++id) {
            if (offsets[id] < 0) {
                continue;
            }
            const int item_end   = offsets[id];
            const int item_start = id > 0 ? offsets[id - 1] : 0;
            const int item_size  = item_end - item_start;
            bool      should     = false;
            if (step + 1 >= item_size) {
                should = true;
                for (int t = item_size - 1; t >= 0; --t) {
                    const int prev = output_ids[(size_t)(step - (item_size - 1) + t) * batch_size + id_offset + row];
                    if (prev != base[item_start + t]) {
                        should = false;
                        break;
                    }
                }
            }
            if (should) {
                finished[row] = true;
            }
        }
    }
}

// The two word-list kernels with beams (kernels/ban_bad_words.cu:22-86, kernels/stop_criteria_kernels.cu:24-81 with
// beam_width > 1): the history of a beam is read backwards, the token of a time from the beam reached so far, then
// that time's parent; a parent outside [0, beam_width) ends the match. `id_offset` is added as given (the layer
// passes ite * local_batch_size, without the beam width). with_last: the n-gram includes the token written at
// `step` (stop words) or ends one before it and bans its last token (bad words).
static bool beam_history_matches(const int* output_ids, const int* parent_ids, const int* tokens, int count, int last,
                                 size_t stride, size_t base, int beam, int K)
{
    for (int t = count - 1; t >= 0; --t) {
        const size_t at = (size_t)(last - (count - 1) + t) * stride + base;
        if (output_ids[at + beam] != tokens[t]) {
            return false;
        }
        if (K > 1) {
            beam = parent_ids[at + beam];
            if (beam < 0 || beam >= K) {
                return false;
            }
        }
    }
    return true;
}

template<int DT>
static void ban_bad_words_beams(typename St<DT>::T* logits, const int* output_ids, const int* parent_ids,
                                int batch_size, int local_batch_size, int K, const int* bad_words, bool share_words,
                                int bad_words_len, int id_offset, int vocab_size_padded, int step)
{
    typedef St<DT> S;
    for (int row = 0; row < local_batch_size * K; ++row) {
        const int  b       = row / K;
        const int* base    = share_words ? bad_words : bad_words + (size_t)b * 2 * bad_words_len;
        const int* offsets = base + bad_words_len;
        for (int id = 0; id < bad_words_len; ++id) {
            if (offsets[id] < 0) {
                continue;
            }
            const int start = id > 0 ? offsets[id - 1] : 0;
            const int size  = offsets[id] - start;
            bool      ban   = size == 1;
            if (size > 1 && step >= size - 1) {
                ban = beam_history_matches(output_ids, parent_ids, base + start, size - 1, step - 1,
                                           (size_t)batch_size * K, (size_t)id_offset + (size_t)b * K, row % K, K);
            }
            const int tok = size >= 1 ? base[offsets[id] - 1] : 0;
            if (ban && 0 < tok && tok < vocab_size_padded) {
                logits[(size_t)row * vocab_size_padded + tok] = S::st(-INFINITY);
            }
        }
    }
}

static void stop_words_criterion_beams(const int* output_ids, const int* parent_ids, const int* stop_words,
                                       bool* finished, int id_offset, int stop_words_len, int batch_size, int rows,
                                       int K, int step)
{
    for (int row = 0; row < rows * K; ++row) {
        const int  b       = row / K;
        const int* base    = stop_words + (size_t)b * 2 * stop_words_len;
        const int* offsets = base + stop_words_len;
        for (int id = 0; id < stop_words_len; ++id) {
            if (offsets[id] < 0) {
                continue;
            }
            const int start = id > 0 ? offsets[id - 1] : 0;
            const int size  = offsets[id] - start;
            if (step + 1 >= size
                && beam_history_matches(output_ids, parent_ids, base + start, size, step, (size_t)batch_size * K,
                                        (size_t)id_offset + (size_t)b * K, row % K, K)) {
                finished[row] = true;
            }
        }
    }
}

// kernels/stop_criteria_kernels.cu:106-157
static void length_criterion(bool* finished, bool* should_stop, const uint32_t* sequence_limit_length, int batch_size,
                             int step)
{
    int sum = 0;
    for (int i = 0; i < batch_size; ++i) {
        finished[i] = finished[i] || ((uint32_t)step >= sequence_limit_length[i]);
        sum += finished[i] ? 1 : 0;
    }
    *should_stop = sum == batch_size;
}

// layers/sampling_layers/TopKSamplingLayer.cu:28-77
static void setup_topk_runtime_args(int batch, uint32_t top_k, uint32_t* top_ks, int top_ks_size, float top_p,
                                    float* top_ps, int top_ps_size, bool* skip_decode)
{
    for (int i = 0; i < batch; ++i) {
        uint32_t k = top_ks_size > 1 ? top_ks[i] : top_k;
        float    p = top_ps_size > 1 ? top_ps[i] : top_p;
        if (k == 0 && p == 0.0f) {
            k = 1;
        }
        if (k > 0 && p == 0.0f) {
            p = 1.0f;
        }
        top_ks[i]      = k > 1024 ? 1024 : k;
        top_ps[i]      = p < 0.0f ? 0.0f : (p > 1.0f ? 1.0f : p);
        skip_decode[i] = k == 0;
    }
}

// layers/sampling_layers/TopPSamplingLayer.cu:30-109
static void set_topp_runtime_args(int batch, uint32_t top_k, uint32_t* top_ks, int top_ks_size, float top_p,
                                  float* top_ps, int top_ps_size, bool* skip_decode, float* initial_top_p,
                                  float* decay_buf, const float* decay, float* min_buf, const float* top_p_min,
                                  int32_t* reset_buf, const uint32_t* reset_ids)
{
    for (int i = 0; i < batch; ++i) {
        uint32_t k = top_ks_size > 1 ? top_ks[i] : top_k;
        float    p = top_ps_size > 1 ? top_ps[i] : top_p;
        if (k == 0 && p == 0.0f) {
            k = 1;
        }
        top_ks[i]        = k;
        top_ps[i]        = p < 0.0f ? 0.0f : (p > 1.0f ? 1.0f : p);
        skip_decode[i]   = k > 0;
        initial_top_p[i] = top_ps[i];
        decay_buf[i]     = decay == nullptr ? 1.0f : decay[i];
        if (decay_buf[i] > 1.0f || decay_buf[i] <= 0.0f) {
            decay_buf[i] = 1.0f;
        }
        min_buf[i] = top_p_min == nullptr ? 1e-6f : top_p_min[i];
        if (min_buf[i] > 1.0f || min_buf[i] <= 0.0f) {
            min_buf[i] = 0.5f;
        }
        reset_buf[i] = (int32_t)(reset_ids == nullptr ? (uint32_t)-1 : reset_ids[i]);
    }
}

// ------------------------------------------------------------------------------------------
// Layer state: what BaseSamplingLayer / TopKSamplingLayer / TopPSamplingLayer keep between
// setup() and forward() (layers/sampling_layers/BaseSamplingLayer.cc:112-206,
// TopKSamplingLayer.cu:134-186, TopPSamplingLayer.cu:184-253).
// ------------------------------------------------------------------------------------------
struct SamplingState {
    std::vector<float>    temperature, penalty, frequency;
    std::vector<int>      min_length;
    int                   penalty_type = PEN_NONE;
    bool                  has_frequency = false;
    std::vector<uint32_t> top_ks;
    std::vector<float>    top_ps;
    std::vector<uint8_t>  skip;  // bool
    // top-k
    int max_top_k = 1;
    // top-p
    std::vector<float>   initial_top_p, decay, top_p_min;
    std::vector<int32_t> reset_ids;
};

struct Layer {
    int           dtype, V, Vp;
    int           batch = 0;
    SamplingState topk, topp;
};

// ------------------------------------------------------------------------------------------
// Steps either side of the sampling path.
//   kernels/logprob_kernels.cu:35-135   log_probs_kernel + accumulate_log_probs (beam folded into batch)
// ------------------------------------------------------------------------------------------
template<int DT>
void log_prob_from_logits(float* cum_log_probs, float* log_probs, const void* logits_v, const int* ids,
                          const int* lengths, size_t max_len, size_t batch, size_t V, size_t Vp, bool batch_first)
{
    typedef St<DT>       S;
    const typename S::T* logits = (const typename S::T*)logits_v;
    for (size_t b = 0; b < batch; ++b) {
        float accum = 0.0f;
        for (size_t step = 0; step + 1 < max_len; ++step) {
            if ((int)step >= lengths[b] - 1) {
                continue;
            }
            const size_t         off = batch_first ? (b * max_len + step) * Vp : (step * batch + b) * Vp;
            const typename S::T* row = logits + off;
            float                mx  = -S::max_t();
            for (size_t v = 0; v < V; ++v) {
                mx = fmaxf(mx, S::ld(row[v]));
            }
            float sum = 0.0f;
            for (size_t v = 0; v < V; ++v) {
                sum += det_expf(S::ld(row[v]) - mx);
            }
            const size_t tok = batch_first ? b * max_len + step + 1 : (step + 1) * batch + b;
            const float  lp  = S::ld(row[ids[tok]]) - mx - det_logf(sum + 1e-9f);
            if (log_probs != nullptr) {
                log_probs[batch_first ? b * (max_len - 1) + step : step * batch + b] = lp;
            }
            accum += lp;
        }
        cum_log_probs[b] = accum;
    }
}

// ------------------------------------------------------------------------------------------
// Beam search step: kernels/online_softmax_beamsearch_kernels.cu:296-739 (invokeTopkSoftMax) with the
// TopK<T, MAX_K> insert rule of kernels/reduce_kernel_utils.cuh:275-322 and BeamHypotheses of
// kernels/beam_search_topk_kernels.h:31-58.
//   rows:   per (batch, beam) row the 2K best of elem = T(x + bias) (a finished row: MAX_T at its end id,
//           -MAX_T elsewhere) by (value descending, id ascending), which is what any merge order of the insert
//           rule gives on distinct ids, and val = u - m - log(d) + cum_log_probs[row], stored as T
//           (:336-349, :500-511);
//   batch:  per batch entry the 2 * MAX_K best of the K * 2K candidates by (score descending, candidate index
//           ascending), score = val with length penalty and diversity term in T arithmetic (:146-160), then the
//           single-thread walk of :163-249 over them, literally (including its use of finished[] and
//           sequence_lengths[] at the batch index and of num_beams / is_done at the block index).
// Departures: m and d are the row's exact maximum and the sum of det_expf(elem - m) accumulated in double
// precision, not the reference's chain of pairwise (m, d) merges with __expf in cub's order; powf is
// det_expf(p * det_logf(length)); a NaN orders below every number.
// ------------------------------------------------------------------------------------------
struct BeamHyps {
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
    const int*   sequence_lengths_src;
    const int*   end_ids;
    const float* log_probs_src;
    int          step;
    int          ite;
    int          batch_size;
    int          local_batch_size;
    int          max_seq_len;
    float        length_penalty;
    int          early_stopping;
};

static int beam_max_k(int beam_width)
{
    // CASE_K of :650-688
    return beam_width <= 4 ? 4 : beam_width <= 8 ? 8 : beam_width <= 16 ? 16 : beam_width <= 32 ? 32 : 64;
}

static bool order_before(float va, int ia, float vb, int ib)
{
    // a NaN never wins a comparison of the insert rule; it is placed last here
    const bool na = va != va, nb = vb != vb;
    if (na != nb) {
        return nb;
    }
    if (!na && va != vb) {
        return va > vb;
    }
    return ia < ib;
}

template<int DT>
static int topk_softmax(const typename St<DT>::T* log_probs, const typename St<DT>::T* bias, const bool* finished,
                        const int* sequence_lengths, float* cum_log_probs, float* output_log_probs, int* ids,
                        const BeamHyps* hyps, int batch_size, int K, int V, const int* end_ids, float diversity_rate,
                        float length_penalty)
{
    typedef St<DT> S;
    if (K < 2 || K > 64 || V < 2 * K) {
        return -1;
    }
    auto        rt    = [](float f) { return S::ld(S::st(f)); };
    const float MAXT  = S::max_t();
    const int   N     = 2 * K;
    const int   rows  = batch_size * K;
    std::vector<int>   cand_id((size_t)rows * N);
    std::vector<float> cand_val((size_t)rows * N);  // values of T
    for (int r = 0; r < rows; ++r) {
        std::vector<float> e(V);
        if (finished[r]) {
            for (int v = 0; v < V; ++v) {
                e[v] = v == end_ids[r / K] ? MAXT : -MAXT;
            }
        }
        else {
            for (int v = 0; v < V; ++v) {
                const float b = bias != nullptr ? S::ld(bias[v]) : 0.0f;
                e[v]          = rt(S::ld(log_probs[(size_t)r * V + v]) + b);
            }
        }
        float m = -MAXT;
        for (int v = 0; v < V; ++v) {
            m = e[v] > m ? e[v] : m;
        }
        double d = 0.0;
        for (int v = 0; v < V; ++v) {
            d += (double)det_expf(e[v] - m);
        }
        const float      logd = det_logf((float)d);
        std::vector<int> order(V);
        for (int v = 0; v < V; ++v) {
            order[v] = v;
        }
        std::partial_sort(order.begin(), order.begin() + N, order.end(),
                          [&](int a, int b) { return order_before(e[a], a, e[b], b); });
        for (int i = 0; i < N; ++i) {
            const int   v   = order[i];
            const float val = e[v] - m - logd;
            cand_id[(size_t)r * N + i]  = v + r * V;
            cand_val[(size_t)r * N + i] = rt(val + cum_log_probs[r]);
        }
    }

    const int   MAX_K2 = 2 * beam_max_k(K);
    const int   C      = K * N;
    const float div_t  = rt(diversity_rate);
    for (int b = 0; b < batch_size; ++b) {
        const int*   x = cand_id.data() + (size_t)b * C;
        const float* y = cand_val.data() + (size_t)b * C;
        std::vector<float> old_cum(K);
        for (int i = 0; i < K; ++i) {
            old_cum[i] = cum_log_probs[b * K + i];
        }
        const bool with_hyps = hyps != nullptr && hyps->num_beams != nullptr;
        if (with_hyps) {
            const int g = hyps->ite * hyps->local_batch_size + b;
            if (hyps->num_beams[g] == 0) {
                hyps->min_normed_scores[g] = FLT_MAX;
            }
            else if (hyps->num_beams[g] == K) {
                continue;
            }
        }
        std::vector<float> score(C);
        for (int c = 0; c < C; ++c) {
            float elem = y[c];
            if (length_penalty != 0.0f) {
                const int length = finished[b] ? sequence_lengths[b] : sequence_lengths[b] + 1;
                if (length != 1) {
                    elem = rt(elem / rt(det_expf(length_penalty * det_logf((float)length))));
                }
            }
            score[c] = rt(elem + rt(div_t * rt((float)(c % K))));
        }
        std::vector<int> order(C);
        for (int c = 0; c < C; ++c) {
            order[c] = c;
        }
        const int take = MAX_K2 < C ? MAX_K2 : C;
        std::partial_sort(order.begin(), order.begin() + take, order.end(),
                          [&](int a, int c) { return order_before(score[a], a, score[c], c); });
        int*   z        = ids + (size_t)b * K;
        float* v        = cum_log_probs + (size_t)b * K;
        int    selected = 0;
        for (int i = 0; i < take; ++i) {
            const int p = order[i];
            if (with_hyps && x[p] % V == hyps->end_ids[b]) {
                if (i < K) {
                    const int   g            = hyps->ite * hyps->local_batch_size + b;
                    const float normed_score = score[p];
                    const int   num_beam     = hyps->num_beams[g];
                    int         beam_idx     = num_beam;
                    if (num_beam == K) {
                        if (normed_score < hyps->min_normed_scores[g]) {
                            selected = K;
                            break;
                        }
                        for (int j = 0; j < K; ++j) {
                            if (hyps->normed_scores[g * (K * 2) + j] == hyps->min_normed_scores[g]) {
                                beam_idx = j;
                                hyps->num_beams[g]--;
                                hyps->min_normed_scores[g]           = FLT_MAX;
                                hyps->normed_scores[g * (K * 2) + j] = normed_score;
                                for (int l = 0; l < K; ++l) {
                                    hyps->min_normed_scores[g] =
                                        std::min(hyps->min_normed_scores[g], hyps->normed_scores[g * (K * 2) + l]);
                                }
                                break;
                            }
                        }
                    }
                    const size_t tgt = ((size_t)(b + hyps->ite * hyps->local_batch_size) * (K * 2) + beam_idx)
                                       * hyps->max_seq_len;
                    hyps->output_ids_tgt[tgt + hyps->step] = hyps->end_ids[b];
                    if (hyps->log_probs != nullptr) {
                        hyps->log_probs[tgt + hyps->step] = y[p] - old_cum[(x[p] / V) % K];
                    }
                    int prev_id = (x[p] / V) % K;
                    for (int j = hyps->step - 1; j >= 0; --j) {
                        const size_t src = (size_t)j * hyps->batch_size * K
                                           + (size_t)hyps->ite * hyps->local_batch_size * K + (size_t)b * K + prev_id;
                        hyps->output_ids_tgt[tgt + j] = hyps->output_ids_src[src];
                        if (hyps->log_probs != nullptr && hyps->log_probs_src != nullptr) {
                            hyps->log_probs[tgt + j] = hyps->log_probs_src[src];
                        }
                        prev_id = hyps->parent_ids_src[src];
                    }
                    const int tgt_beam                   = g * (K * 2) + beam_idx;
                    hyps->sequence_lengths_tgt[tgt_beam] = hyps->step;
                    hyps->normed_scores[tgt_beam]        = normed_score;
                    hyps->min_normed_scores[g] = std::min(hyps->min_normed_scores[g], hyps->normed_scores[tgt_beam]);
                    hyps->num_beams[g]++;
                    hyps->cum_log_probs[tgt_beam] = y[p];
                }
            }
            else if ((with_hyps && i < 2 * K) || (!with_hyps && i < K)) {
                z[selected] = x[p];
                if (output_log_probs != nullptr) {
                    output_log_probs[b * K + selected] = y[p] - old_cum[(z[selected] / V) % K];
                }
                v[selected] = y[p];
                selected++;
            }
            if (selected >= K) {
                break;
            }
        }
        if (with_hyps) {
            if (hyps->num_beams[b] < K) {
                hyps->is_done[b] = false;
            }
            else if (hyps->early_stopping) {
                hyps->is_done[b] = true;
            }
        }
    }
    return 0;
}

// ------------------------------------------------------------------------------------------
// kernels/beam_search_penalty_kernels.cu:24-267 (invokeAddBiasApplyPenalties): bias and temperature over
// [local_batch * beam_width, vocab_size_padded] logits with pad columns masked, the repetition / presence penalty
// over a beam's own history (followed back through parent_ids, every token penalised from the value it had before
// the kernel), the min-length mask. Literal, including: previous_ids is indexed with the local batch index
// (the launcher offsets parent_ids by `ite` but not previous_ids), and the half2 kernel adds the bias only when
// there is one while the generic kernel adds T(0) (a difference for -0 only).
// ------------------------------------------------------------------------------------------
template<int DT>
static void beam_add_bias_apply_penalties(int step, typename St<DT>::T* logits, const int* current_ids,
                                          const int* previous_ids, const int* parent_ids, const int* input_lengths,
                                          const int* sequence_lengths, const typename St<DT>::T* bias, int ite,
                                          int max_input_length, int local_batch_size, int batch_size, int K, int V,
                                          int Vp, const int* end_ids, float temperature, float repetition_penalty,
                                          int penalty_type, int min_length)
{
    typedef St<DT> S;
    auto        rt   = [](float f) { return S::ld(S::st(f)); };
    const int   rows = local_batch_size * K;
    const float MAXT = S::max_t();
    if (bias != nullptr || temperature != 1.0f || V != Vp) {
        const float inv   = 1.0f / (temperature + 1e-6f);
        const float inv_t = rt(inv);
        const bool  pairs = DT == DT_F16 && V % 2 == 0 && Vp % 2 == 0;
        for (int r = 0; r < rows; ++r) {
            for (int v = 0; v < Vp; ++v) {
                typename S::T& x = logits[(size_t)r * Vp + v];
                if (v >= V) {
                    x = S::st(-MAXT);
                }
                else if (pairs) {
                    float y = S::ld(x);
                    if (bias != nullptr) {
                        y = rt(y + S::ld(bias[v]));
                    }
                    x = S::st(y * inv_t);
                }
                else {
                    const float b = bias != nullptr ? S::ld(bias[v]) : 0.0f;
                    x             = S::st(rt(S::ld(x) + b) * (DT == DT_F32 ? inv : inv_t));
                }
            }
        }
    }
    const float neutral = penalty_type == PEN_MULTIPLICATIVE ? 1.0f : 0.0f;
    if (penalty_type != PEN_NONE && step > 0 && repetition_penalty != neutral) {
        const int*  parents = parent_ids + (size_t)ite * K * local_batch_size;
        const int   bbsize  = batch_size * K;
        const float pen     = rt(repetition_penalty);
        for (int r = 0; r < rows; ++r) {
            typename S::T*     row = logits + (size_t)r * Vp;
            const int          b   = r / K;
            const int          len = input_lengths != nullptr ? input_lengths[r] : max_input_length;
            std::vector<int>   idx(step, -1);
            std::vector<float> val(step, 0.0f);
            auto               penalised = [&](float x) {
                if (penalty_type == PEN_ADDITIVE) {
                    return rt(x - pen);
                }
                return x > 0.0f ? rt(x / pen) : rt(x * pen);
            };
            int prev_id   = current_ids[r];
            idx[step - 1] = prev_id;
            val[step - 1] = penalised(S::ld(row[prev_id]));
            int beam      = r % K;
            for (int i = step - 2; i >= 0; --i) {
                if (i >= len && i < max_input_length) {
                    continue;
                }
                beam    = parents[(size_t)i * bbsize + b * K + beam];
                prev_id = previous_ids[(size_t)i * bbsize + b * K + beam];
                idx[i]  = prev_id;
                val[i]  = penalised(S::ld(row[prev_id]));
            }
            for (int i = 0; i < step; ++i) {
                if (i >= len && i < max_input_length) {
                    continue;
                }
                row[idx[i]] = S::st(val[i]);
            }
        }
    }
    if (step - max_input_length < min_length) {
        for (int r = 0; r < rows; ++r) {
            if (sequence_lengths[r] + 1 - max_input_length < min_length) {
                logits[(size_t)r * Vp + end_ids[r / K]] = S::st(-MAXT);
            }
        }
    }
}

// layers/beam_search_layers/OnlineBeamSearchLayer.cu:24-61 (update_kernel). The reference's threads read
// sequence_length and write finished of other rows of their batch entry inside one launch; the order restated here
// is what a warp in lockstep does when an entry's rows share it: every row counts its token first, then every row
// takes the length of the beam it continues, then an entry that has collected beam_width hypotheses is finished.
static void beam_update(bool* finished, int* parent_ids, int* sequence_length, int* word_ids, int* output_ids,
                        const BeamHyps* hyps, int local_batch_size, int K, int Vp, const int* end_ids)
{
    const int        rows = local_batch_size * K;
    std::vector<int> counted(rows);
    for (int i = 0; i < rows; ++i) {
        counted[i] = finished[i] ? sequence_length[i] : sequence_length[i] + 1;
    }
    for (int i = 0; i < rows; ++i) {
        const int b = i / K;
        // a slot the step left untouched holds the caller's old contents: a negative value counts as "this beam,
        // its end token" (the reference indexes other rows' memory with it)
        const bool valid   = word_ids[i] >= 0;
        const int  beam_id = valid ? (word_ids[i] / Vp) % K : i % K;
        const int  word_id = valid ? word_ids[i] % Vp : end_ids[b];
        sequence_length[i] = counted[b * K + beam_id];
        finished[i]        = word_id == end_ids[b];
        parent_ids[i]      = beam_id;
        word_ids[i]        = word_id;
        output_ids[i]      = word_id;
    }
    if (hyps != nullptr && hyps->num_beams != nullptr) {
        for (int b = 0; b < local_batch_size; ++b) {
            if (hyps->num_beams[hyps->ite * hyps->local_batch_size + b] == K) {
                for (int i = 0; i < K; ++i) {
                    finished[b * K + i] = true;
                }
            }
        }
    }
}

// layers/beam_search_layers/BaseBeamSearchLayer.cu:22-77
static void update_indir_cache(int* tgt, const int* src, const int* beam_ids, const bool* finished,
                               int local_batch_size, int K, int max_seq_len, int step)
{
    const int start_step = std::max(0, step + 1 - max_seq_len);
    const int num_steps  = std::min(step + 1, max_seq_len);
    for (int bb = 0; bb < local_batch_size * K; ++bb) {
        if (finished[bb]) {
            continue;
        }
        const int b = bb / K, beam = bb % K;
        const int src_beam = beam_ids[b * K + beam];
        for (int ts = 0; ts < num_steps; ++ts) {
            const int    time_step = ts + start_step;
            const int    circ      = time_step % max_seq_len;
            const size_t t_off     = (size_t)b * K * max_seq_len + (size_t)beam * max_seq_len + circ;
            const size_t s_off     = (size_t)b * K * max_seq_len + (size_t)src_beam * max_seq_len + circ;
            tgt[t_off]             = time_step == step ? beam : src[s_off];
        }
    }
}

}  // namespace oracle

using namespace oracle;

#define DISPATCH(dt, CALL)                                                                                             \
    switch (dt) {                                                                                                      \
        case DT_F32: {                                                                                                 \
            constexpr int DT = DT_F32;                                                                                 \
            CALL;                                                                                                      \
        } break;                                                                                                       \
        case DT_F16: {                                                                                                 \
            constexpr int DT = DT_F16;                                                                                 \
            CALL;                                                                                                      \
        } break;                                                                                                       \
        case DT_BF16: {                                                                                                \
            constexpr int DT = DT_BF16;                                                                                \
            CALL;                                                                                                      \
        } break;                                                                                                       \
        default:                                                                                                       \
            return -1;                                                                                                 \
    }

// Arguments of one DynamicDecodeLayer::forward call (layers/DynamicDecodeLayer.cc:191-474),
// all host pointers. Pointers that are null mean "tensor absent".
struct OracleForwardArgs {
    void*           logits;           // [batch, Vp], mutated as the reference mutates it
    const void*     embedding_bias;   // [Vp] or null
    const int*      end_ids;          // [batch]
    const int*      input_lengths;    // [batch] or null
    const uint32_t* sequence_limit_length;  // [batch] or null
    const int*      stop_words;       // [batch, 2, stop_words_len] or null
    const int*      bad_words;        // [2, L] or [batch, 2, L] or null
    const float*    uniform_draws;    // [batch], injected draws in (0, 1]
    int*            output_ids;       // [max_seq_len, batch]
    bool*           finished;         // [batch] or null
    int*            sequence_length;  // [batch] or null
    float*          cum_log_probs;    // [batch] or null
    float*          output_log_probs; // [gen_len, batch] or null
    bool*           should_stop;      // [1] or null
    int             step, max_input_length, ite, local_batch_size, batch_size;
    int             stop_words_len, bad_words_len, bad_words_shared;
};

template<int DT>
static void sampling_layer_forward(Layer* L, SamplingState& st, bool is_topk, const OracleForwardArgs* a)
{
    // layers/sampling_layers/BaseSamplingLayer.cc:255-359
    typedef St<DT>        S;
    typedef typename S::T T;
    const int             local = a->local_batch_size, ite = a->ite, Vp = L->Vp, V = L->V;
    const int             off   = ite * local;
    const uint8_t*        skip  = st.skip.data() + off;
    if (std::all_of(skip, skip + local, [](uint8_t s) { return s != 0; })) {
        return;
    }
    const bool skip_any = std::any_of(skip, skip + local, [](uint8_t s) { return s != 0; });
    T*         logits   = (T*)a->logits + (size_t)off * Vp;
    std::vector<T> copy;
    if (skip_any) {
        copy.assign(logits, logits + (size_t)local * Vp);
        logits = copy.data();
    }
    const T*     bias      = (const T*)a->embedding_bias;
    const float* temps     = st.temperature.data() + off;
    const bool   all_one   = std::all_of(temps, temps + local, [](float t) { return t == 1.0f; });
    if (bias != nullptr || !all_one) {
        temperature_penalty<DT>(logits, bias, temps, local, local, V, Vp, false);
    }
    if (a->step > 1 && st.penalty_type != PEN_NONE) {
        const float  dflt = st.penalty_type == PEN_MULTIPLICATIVE ? 1.0f : 0.0f;
        const float* pens = st.penalty.data() + off;
        bool         all_default = std::all_of(pens, pens + local, [&](float x) { return x == dflt; });
        if (st.has_frequency) {
            const float* fr = st.frequency.data() + off;
            all_default     = all_default && std::all_of(fr, fr + local, [](float x) { return x == 0.0f; });
        }
        if (!all_default) {
            repetition_penalty<DT>(logits, pens, local, st.has_frequency ? st.frequency.data() + off : nullptr, local,
                                   a->output_ids + off, a->batch_size, local, Vp,
                                   a->input_lengths ? a->input_lengths + off : nullptr, a->max_input_length, a->step,
                                   st.penalty_type);
        }
    }
    const int  num_generated = a->step - a->max_input_length;
    const int* minl          = st.min_length.data() + off;
    if (std::any_of(minl, minl + local, [&](int m) { return m > num_generated; })) {
        min_length_penalty<DT>(logits, minl, a->end_ids + off, a->sequence_length + off, a->max_input_length, local,
                               Vp);
    }
    int*   ids     = a->output_ids + (size_t)a->step * a->batch_size + off;
    int*   seqlen  = a->sequence_length ? a->sequence_length + off : nullptr;
    bool*  fin     = a->finished ? a->finished + off : nullptr;
    float* cum     = a->cum_log_probs ? a->cum_log_probs + off : nullptr;
    float* outlp   = a->output_log_probs ?
                         a->output_log_probs + (size_t)(a->step - a->max_input_length) * a->batch_size + off :
                         nullptr;
    const float* u = a->uniform_draws + off;
    if (is_topk) {
        // TopKSamplingLayer::runSampling (TopKSamplingLayer.cu:189-268)
        add_bias_end_mask<DT>(logits, nullptr, a->end_ids + off, fin, local, V, Vp);
        if (cum || outlp) {
            add_bias_softmax<DT>(logits, nullptr, a->end_ids + off, fin, local, Vp, V);
        }
        batch_topk_sampling<DT>(logits, ids, seqlen, fin, cum, outlp, u, st.max_top_k,
                                (const int*)st.top_ks.data() + off, 1.0f, st.top_ps.data() + off, Vp,
                                a->end_ids + off, local, (const bool*)skip);
    }
    else {
        // TopPSamplingLayer::runSampling (TopPSamplingLayer.cu:256-343)
        add_bias_softmax<DT>(logits, nullptr, a->end_ids + off, fin, local, Vp, V);
        batch_topp_sampling<DT>(logits, ids, seqlen, fin, cum, outlp, u, local, Vp, a->end_ids + off, 0.0f,
                                st.top_ps.data() + off, (const bool*)skip);
        compute_topp_decay(st.top_ps.data() + off, st.initial_top_p.data() + off, ids, st.decay.data() + off,
                           st.top_p_min.data() + off, st.reset_ids.data() + off, local);
    }
}

extern "C" {

float oracle_expf(float x)
{
    return det_expf(x);
}
float oracle_logf(float x)
{
    return det_logf(x);
}
void oracle_expf_array(const float* x, float* y, long n)
{
    for (long i = 0; i < n; ++i) {
        y[i] = det_expf(x[i]);
    }
}
void oracle_logf_array(const float* x, float* y, long n)
{
    for (long i = 0; i < n; ++i) {
        y[i] = det_logf(x[i]);
    }
}
void oracle_float_to_half(const float* x, uint16_t* y, long n)
{
    for (long i = 0; i < n; ++i) {
        y[i] = float_to_half(x[i]);
    }
}
void oracle_half_to_float(const uint16_t* x, float* y, long n)
{
    for (long i = 0; i < n; ++i) {
        y[i] = half_to_float(x[i]);
    }
}
void oracle_float_to_bf16(const float* x, uint16_t* y, long n)
{
    for (long i = 0; i < n; ++i) {
        y[i] = float_to_bf16(x[i]);
    }
}

int oracle_ban_bad_words(int dtype, void* logits, const int* output_ids, int batch_size, int local_batch_size,
                         const int* bad_words, int share_words, int bad_words_len, int id_offset,
                         int vocab_size_padded, int step)
{
    DISPATCH(dtype, ban_bad_words<DT>((St<DT>::T*)logits, output_ids, batch_size, local_batch_size, bad_words,
                                      share_words != 0, bad_words_len, id_offset, vocab_size_padded, step));
    return 0;
}

int oracle_apply_temperature_penalty(int dtype, void* logits, const void* bias, float temperature, int batch, int V,
                                     int Vp)
{
    DISPATCH(dtype, temperature_penalty<DT>((St<DT>::T*)logits, (const St<DT>::T*)bias, &temperature, 1, batch, V, Vp,
                                            true));
    return 0;
}

int oracle_batch_apply_temperature_penalty(int dtype, void* logits, const void* bias, const float* temperatures,
                                           int batch, int V, int Vp)
{
    DISPATCH(dtype, temperature_penalty<DT>((St<DT>::T*)logits, (const St<DT>::T*)bias, temperatures, batch, batch, V,
                                            Vp, false));
    return 0;
}

int oracle_batch_apply_repetition_penalty(int dtype, void* logits, const float* penalties, const int* output_ids,
                                          int batch_size, int local_batch_size, int vocab_stride,
                                          const int* input_lengths, int max_input_length, int step, int type)
{
    DISPATCH(dtype, repetition_penalty<DT>((St<DT>::T*)logits, penalties, local_batch_size, nullptr, 0, output_ids,
                                           batch_size, local_batch_size, vocab_stride, input_lengths,
                                           max_input_length, step, type));
    return 0;
}

// scalar-penalty variant (kernels/sampling_penalty_kernels.cu:224-337): same arithmetic, one penalty
int oracle_apply_repetition_penalty(int dtype, void* logits, float penalty, const int* output_ids, int batch_size,
                                    int local_batch_size, int vocab_size, int vocab_size_padded,
                                    const int* input_lengths, int max_input_length, int step, int type)
{
    // ids >= vocab_size are skipped by this variant (:250-252); emulate by a pre-filtered id table
    std::vector<int> filtered((size_t)step * batch_size);
    for (size_t i = 0; i < filtered.size(); ++i) {
        filtered[i] = output_ids[i] >= vocab_size ? -1 : output_ids[i];
    }
    DISPATCH(dtype, repetition_penalty<DT>((St<DT>::T*)logits, &penalty, 1, nullptr, 0, filtered.data(), batch_size,
                                           local_batch_size, vocab_size_padded, input_lengths, max_input_length, step,
                                           type));
    return 0;
}

int oracle_batch_apply_frequency_penalty(int dtype, void* logits, const float* presence, const float* frequency,
                                         const int* output_ids, int batch_size, int local_batch_size,
                                         int vocab_stride, const int* input_lengths, int max_input_length, int step)
{
    DISPATCH(dtype, repetition_penalty<DT>((St<DT>::T*)logits, presence, local_batch_size, frequency,
                                           local_batch_size, output_ids, batch_size, local_batch_size, vocab_stride,
                                           input_lengths, max_input_length, step, PEN_ADDITIVE));
    return 0;
}

int oracle_min_length_penalty(int dtype, void* logits, const int* min_lengths, const int* end_ids,
                              const int* sequence_lengths, int max_input_length, int batch, int Vp)
{
    DISPATCH(dtype, min_length_penalty<DT>((St<DT>::T*)logits, min_lengths, end_ids, sequence_lengths,
                                           max_input_length, batch, Vp));
    return 0;
}

int oracle_add_bias_end_mask(int dtype, void* logits, const void* bias, const int* end_ids, const bool* finished,
                             int batch, int V, int Vp)
{
    DISPATCH(dtype, add_bias_end_mask<DT>((St<DT>::T*)logits, (const St<DT>::T*)bias, end_ids, finished, batch, V,
                                          Vp));
    return 0;
}

int oracle_add_bias_softmax(int dtype, void* logits, const void* bias, const int* end_ids, const bool* finished, int m,
                            int n_padded, int n)
{
    DISPATCH(dtype,
             add_bias_softmax<DT>((St<DT>::T*)logits, (const St<DT>::T*)bias, end_ids, finished, m, n_padded, n));
    return 0;
}

int oracle_batch_topk_sampling(int dtype, const void* log_probs, int* ids, int* sequence_length, bool* finished,
                               float* cum_log_probs, float* output_log_probs, const float* uniforms, int max_top_k,
                               const int* top_ks, float top_p, const float* top_ps, int vocab_size_padded,
                               const int* end_ids, int batch, const bool* skip_decode)
{
    int rc = 0;
    DISPATCH(dtype, rc = batch_topk_sampling<DT>((const St<DT>::T*)log_probs, ids, sequence_length, finished,
                                                 cum_log_probs, output_log_probs, uniforms, max_top_k, top_ks, top_p,
                                                 top_ps, vocab_size_padded, end_ids, batch, skip_decode));
    return rc;
}

int oracle_batch_topp_sampling(int dtype, const void* probs, int* ids, int* sequence_length, bool* finished,
                               float* cum_log_probs, float* output_log_probs, const float* uniforms, int batch,
                               int vocab_size_padded, const int* end_ids, float top_p, const float* top_ps,
                               const bool* skip_decode)
{
    DISPATCH(dtype, batch_topp_sampling<DT>((const St<DT>::T*)probs, ids, sequence_length, finished, cum_log_probs,
                                            output_log_probs, uniforms, batch, vocab_size_padded, end_ids, top_p,
                                            top_ps, skip_decode));
    return 0;
}

void oracle_compute_topp_decay(float* runtime_top_p, const float* initial_top_p, const int* output_ids,
                               const float* decay, const float* top_p_min, const int32_t* reset_ids, int n)
{
    compute_topp_decay(runtime_top_p, initial_top_p, output_ids, decay, top_p_min, reset_ids, n);
}

void oracle_stop_words_criterion(const int* output_ids, const int* stop_words, bool* finished, int id_offset,
                                 int stop_words_len, int batch_size, int local_batch_size, int step)
{
    stop_words_criterion(output_ids, stop_words, finished, id_offset, stop_words_len, batch_size, local_batch_size,
                         step);
}

void oracle_length_criterion(bool* finished, bool* should_stop, const uint32_t* sequence_limit_length, int batch_size,
                             int step)
{
    length_criterion(finished, should_stop, sequence_limit_length, batch_size, step);
}

void oracle_setup_topk_runtime_args(int batch, uint32_t top_k, uint32_t* top_ks, int top_ks_size, float top_p,
                                    float* top_ps, int top_ps_size, bool* skip_decode)
{
    setup_topk_runtime_args(batch, top_k, top_ks, top_ks_size, top_p, top_ps, top_ps_size, skip_decode);
}

// ---- layer object ------------------------------------------------------------------------
void* oracle_layer_create(int dtype, int vocab_size, int vocab_size_padded)
{
    Layer* L = new Layer();
    L->dtype = dtype;
    L->V     = vocab_size;
    L->Vp    = vocab_size_padded;
    return L;
}

void oracle_layer_destroy(void* h)
{
    delete (Layer*)h;
}

// DynamicDecodeLayer::setup for beam_width == 1 (layers/DynamicDecodeLayer.cc:153-178). Every
// runtime argument is (pointer, element count); count 0 = absent. top_p_decay / top_p_min /
// top_p_reset_ids are [batch] or null. Returns 0, or a negative code for the argument errors the
// reference raises (-2: both penalties, -3: bad array size).
int oracle_layer_setup(void* h, int batch, const uint32_t* runtime_top_k, int top_k_size, const float* runtime_top_p,
                       int top_p_size, const float* temperature, int temperature_size,
                       const float* repetition_penalty, int repetition_size, const float* presence_penalty,
                       int presence_size, const float* frequency_penalty, int frequency_size, const int* min_length,
                       int min_length_size, const float* top_p_decay, const float* top_p_min,
                       const uint32_t* top_p_reset_ids)
{
    Layer* L = (Layer*)h;
    L->batch = batch;
    if (repetition_size > 0 && presence_size > 0) {
        return -2;
    }
    if ((top_k_size > 1 && top_k_size != batch) || (top_p_size > 1 && top_p_size != batch)) {
        return -3;
    }
    for (int which = 0; which < 2; ++which) {
        SamplingState& st = which == 0 ? L->topk : L->topp;
        st                = SamplingState();
        // BaseSamplingLayer::setup (BaseSamplingLayer.cc:156-205)
        st.temperature.assign(batch, 1.0f);
        for (int i = 0; i < batch && temperature_size > 0; ++i) {
            st.temperature[i] = temperature_size == 1 ? temperature[0] : temperature[i];
        }
        st.penalty.assign(batch, 0.0f);
        st.frequency.assign(batch, 0.0f);
        if (repetition_size > 0 || presence_size > 0 || frequency_size > 0) {
            const bool   mult = repetition_size > 0;
            st.penalty_type   = mult ? PEN_MULTIPLICATIVE : PEN_ADDITIVE;
            const float* src  = mult ? repetition_penalty : presence_penalty;
            const int    n    = mult ? repetition_size : presence_size;
            for (int i = 0; i < batch && n > 0; ++i) {
                st.penalty[i] = n == 1 ? src[0] : src[i];
            }
            if (frequency_size > 0) {
                if (mult) {
                    return -2;
                }
                st.has_frequency = true;
                for (int i = 0; i < batch; ++i) {
                    st.frequency[i] = frequency_size == 1 ? frequency_penalty[0] : frequency_penalty[i];
                }
            }
        }
        st.min_length.assign(batch, 0);
        for (int i = 0; i < batch && min_length_size > 0; ++i) {
            st.min_length[i] = min_length_size == 1 ? min_length[0] : min_length[i];
        }
        st.top_ks.assign(batch, 0);
        st.top_ps.assign(batch, 0.0f);
        st.skip.assign(batch, 0);
        if (top_k_size > 1) {
            std::copy(runtime_top_k, runtime_top_k + batch, st.top_ks.begin());
        }
        if (top_p_size > 1) {
            std::copy(runtime_top_p, runtime_top_p + batch, st.top_ps.begin());
        }
    }
    // TopKSamplingLayer::setup (TopKSamplingLayer.cu:146-185)
    {
        SamplingState& st    = L->topk;
        uint32_t       top_k = 0;
        for (int i = 0; i < top_k_size; ++i) {
            top_k = std::max(top_k, runtime_top_k[i]);  // runtime_top_k.max<uint>()
        }
        const float top_p = top_p_size == 0 ? 0.0f : runtime_top_p[0];
        setup_topk_runtime_args(batch, top_k, st.top_ks.data(), top_k_size, top_p, st.top_ps.data(), top_p_size,
                                (bool*)st.skip.data());
        st.max_top_k = (int)*std::max_element(st.top_ks.begin(), st.top_ks.end());
    }
    // TopPSamplingLayer::setup (TopPSamplingLayer.cu:200-252)
    {
        SamplingState& st = L->topp;
        if (top_p_size == 0) {
            st.skip.assign(batch, 1);
        }
        else {
            const uint32_t top_k = top_k_size > 0 ? runtime_top_k[0] : 0;
            const float    top_p = runtime_top_p[0];
            st.initial_top_p.assign(batch, 0.0f);
            st.decay.assign(batch, 1.0f);
            st.top_p_min.assign(batch, 0.0f);
            st.reset_ids.assign(batch, -1);
            set_topp_runtime_args(batch, top_k, st.top_ks.data(), top_k_size, top_p, st.top_ps.data(), top_p_size,
                                  (bool*)st.skip.data(), st.initial_top_p.data(), st.decay.data(), top_p_decay,
                                  st.top_p_min.data(), top_p_min, st.reset_ids.data(), top_p_reset_ids);
        }
    }
    return 0;
}

// read back the per-row state (tests compare it with the product's device buffers)
void oracle_layer_get_state(void* h, int which, uint32_t* top_ks, float* top_ps, uint8_t* skip)
{
    Layer*         L  = (Layer*)h;
    SamplingState& st = which == 0 ? L->topk : L->topp;
    for (int i = 0; i < L->batch; ++i) {
        top_ks[i] = st.top_ks[i];
        top_ps[i] = st.top_ps[i];
        skip[i]   = st.skip[i];
    }
}

int oracle_layer_forward(void* h, const OracleForwardArgs* a)
{
    Layer*    L     = (Layer*)h;
    const int local = a->local_batch_size, off = a->ite * local;
    // 1. bad words on the caller's buffer, all local rows (DynamicDecodeLayer.cc:247-283)
    if (a->bad_words != nullptr) {
        const int* bw = a->bad_words_shared ? a->bad_words : a->bad_words + (size_t)off * 2 * a->bad_words_len;
        DISPATCH(L->dtype, ban_bad_words<DT>((St<DT>::T*)a->logits + (size_t)off * L->Vp, a->output_ids, a->batch_size,
                                             local, bw, a->bad_words_shared != 0, a->bad_words_len, off, L->Vp,
                                             a->step));
    }
    // 2./3. top-k layer then top-p layer (DynamicDecodeLayer.cc:443-444)
    DISPATCH(L->dtype, sampling_layer_forward<DT>(L, L->topk, true, a));
    DISPATCH(L->dtype, sampling_layer_forward<DT>(L, L->topp, false, a));
    // 4. stop words, local rows (DynamicDecodeLayer.cc:447-462)
    if (a->stop_words != nullptr) {
        stop_words_criterion(a->output_ids, a->stop_words + (size_t)off * 2 * a->stop_words_len, a->finished + off,
                             off, a->stop_words_len, a->batch_size, local, a->step);
    }
    // 5. length criterion over the whole batch (DynamicDecodeLayer.cc:464-473)
    if (a->sequence_limit_length != nullptr) {
        length_criterion(a->finished, a->should_stop, a->sequence_limit_length, a->batch_size, a->step);
    }
    return 0;
}

// kernels/logprob_kernels.cu:137-183
void oracle_log_prob_from_logits(int dtype, float* cum_log_probs, float* log_probs, const void* logits, const int* ids,
                                 const int* lengths, size_t max_len, size_t batch, size_t V, size_t Vp, int batch_first)
{
    const bool bf = batch_first != 0;
    switch (dtype) {
        case DT_F32:
            log_prob_from_logits<DT_F32>(cum_log_probs, log_probs, logits, ids, lengths, max_len, batch, V, Vp, bf);
            break;
        case DT_F16:
            log_prob_from_logits<DT_F16>(cum_log_probs, log_probs, logits, ids, lengths, max_len, batch, V, Vp, bf);
            break;
        default:
            log_prob_from_logits<DT_BF16>(cum_log_probs, log_probs, logits, ids, lengths, max_len, batch, V, Vp, bf);
            break;
    }
}

// kernels/decoding_kernels.cu:26-47; cum_log_probs as fp32 images of T: 0 for the first beam,
// -MAX_T_VAL otherwise (65504 for half, 1e20 for float / bfloat16)
void oracle_decoding_initialize(int dtype, bool* finished, int* sequence_length, int* word_ids, float* cum_log_probs,
                                const int* sentence_ids, int batch, int beam, int max_input_length)
{
    const float max_t = dtype == DT_F16 ? 65504.0f : 1e20f;
    for (int i = 0; i < batch * beam; ++i) {
        finished[i]        = false;
        sequence_length[i] = max_input_length;
        if (word_ids != nullptr) {
            word_ids[i] = sentence_ids[i / beam];
        }
        cum_log_probs[i] = (i % beam == 0) ? 0.0f : -max_t;
    }
}

// kernels/decoding_kernels.cu:680-694
void oracle_plus_scalar(int* buf, int val, int size)
{
    for (int i = 0; i < size; ++i) {
        buf[i] += val;
    }
}

// kernels/gpt_kernels.cu:329-345 (out [dim1, dim0], in [dim0, dim1], optional per-column source offsets)
void oracle_transpose_axis01(int* out, const int* in, const int* in_skipping_dim1, int dim0, int dim1)
{
    for (int i0 = 0; i0 < dim0; ++i0) {
        for (int i1 = 0; i1 < dim1; ++i1) {
            const int off       = in_skipping_dim1 == nullptr ? 0 : in_skipping_dim1[i1] * dim1;
            out[i1 * dim0 + i0] = in[off + i0 * dim1 + i1];
        }
    }
}

// kernels/decoding_kernels.cu:697-785 (finalize): rank i is the hypothesis with the largest remaining score, found
// by the scan from index 0 (:738-745); hypotheses from num_beams[b] on count as -FLT_MAX here (the reference reads
// shared memory it never wrote for them). Copies skip the first position of the source rows (:768-771).
void oracle_finalize(int* output_ids, int* sequence_lengths, float* cum_log_probs, float* output_log_probs,
                     const int* topk_output_ids, const int* topk_sequence_lengths, const float* scores,
                     const float* topk_cum_log_probs, const float* topk_log_probs, const int* num_beams,
                     int beam_width, int max_seq_len, int batch_size)
{
    const int hyps = 2 * beam_width;
    for (int b = 0; b < batch_size; ++b) {
        std::vector<float> s(hyps, -FLT_MAX);
        for (int j = 0; j < hyps && j < num_beams[b]; ++j) {
            s[j] = scores[(size_t)b * hyps + j];
        }
        std::vector<int> rank(beam_width, 0);
        for (int i = 0; i < beam_width; ++i) {
            float mx = -FLT_MAX;
            for (int j = 0; j < hyps; ++j) {
                mx = s[j] > mx ? s[j] : mx;
            }
            for (int j = 0; j < hyps; ++j) {
                if (s[j] == mx) {
                    rank[i] = j;
                    s[j]    = -FLT_MAX;
                    break;
                }
            }
        }
        for (int i = 0; i < beam_width; ++i) {
            const size_t src                            = (size_t)b * hyps + rank[i];
            sequence_lengths[(size_t)b * beam_width + i] = topk_sequence_lengths[src];
            if (cum_log_probs != nullptr) {
                cum_log_probs[(size_t)b * beam_width + i] = topk_cum_log_probs[src];
            }
            const size_t from = src * (max_seq_len + 1) + 1;
            const size_t to   = ((size_t)b * beam_width + i) * max_seq_len;
            for (int t = 0; t < topk_sequence_lengths[src]; ++t) {
                output_ids[to + t] = topk_output_ids[from + t];
                if (output_log_probs != nullptr) {
                    output_log_probs[to + t] = topk_log_probs[from + t];
                }
            }
        }
    }
}


// kernels/online_softmax_beamsearch_kernels.cu:671-701; `hyps` may be NULL (the reference always passes one whose
// num_beams may be NULL)
int oracle_topk_softmax(int dt, const void* log_probs, const void* bias, const bool* finished,
                        const int* sequence_lengths, float* cum_log_probs, float* output_log_probs, int* ids,
                        const BeamHyps* hyps, int batch_size, int beam_width, int vocab_size, const int* end_ids,
                        float diversity_rate, float length_penalty)
{
    int rc = -1;
    DISPATCH(dt, rc = topk_softmax<DT>((const St<DT>::T*)log_probs, (const St<DT>::T*)bias, finished, sequence_lengths,
                                       cum_log_probs, output_log_probs, ids, hyps, batch_size, beam_width, vocab_size,
                                       end_ids, diversity_rate, length_penalty));
    return rc;
}


int oracle_beam_add_bias_apply_penalties(int dt, int step, void* logits, const int* current_ids,
                                         const int* previous_ids, const int* parent_ids, const int* input_lengths,
                                         const int* sequence_lengths, const void* bias, int ite, int max_input_length,
                                         int local_batch_size, int batch_size, int beam_width, int vocab_size,
                                         int vocab_size_padded, const int* end_ids, float temperature,
                                         float repetition_penalty, int penalty_type, int min_length)
{
    DISPATCH(dt, beam_add_bias_apply_penalties<DT>(step, (St<DT>::T*)logits, current_ids, previous_ids, parent_ids,
                                                   input_lengths, sequence_lengths, (const St<DT>::T*)bias, ite,
                                                   max_input_length, local_batch_size, batch_size, beam_width,
                                                   vocab_size, vocab_size_padded, end_ids, temperature,
                                                   repetition_penalty, penalty_type, min_length));
    return 0;
}

void oracle_beam_update(bool* finished, int* parent_ids, int* sequence_length, int* word_ids, int* output_ids,
                        const BeamHyps* hyps, int local_batch_size, int beam_width, int vocab_size_padded,
                        const int* end_ids)
{
    beam_update(finished, parent_ids, sequence_length, word_ids, output_ids, hyps, local_batch_size, beam_width,
                vocab_size_padded, end_ids);
}

void oracle_update_indir_cache(int* tgt, const int* src, const int* beam_ids, const bool* finished,
                               int local_batch_size, int beam_width, int max_seq_len, int step)
{
    update_indir_cache(tgt, src, beam_ids, finished, local_batch_size, beam_width, max_seq_len, step);
}


int oracle_ban_bad_words_beams(int dtype, void* logits, const int* output_ids, const int* parent_ids, int batch_size,
                               int local_batch_size, int beam_width, const int* bad_words, int share_words,
                               int bad_words_len, int id_offset, int vocab_size_padded, int step)
{
    DISPATCH(dtype, ban_bad_words_beams<DT>((St<DT>::T*)logits, output_ids, parent_ids, batch_size, local_batch_size,
                                            beam_width, bad_words, share_words != 0, bad_words_len, id_offset,
                                            vocab_size_padded, step));
    return 0;
}

void oracle_stop_words_criterion_beams(const int* output_ids, const int* parent_ids, const int* stop_words,
                                       bool* finished, int id_offset, int stop_words_len, int batch_size, int rows,
                                       int beam_width, int step)
{
    stop_words_criterion_beams(output_ids, parent_ids, stop_words, finished, id_offset, stop_words_len, batch_size,
                               rows, beam_width, step);
}

}  // extern "C"
