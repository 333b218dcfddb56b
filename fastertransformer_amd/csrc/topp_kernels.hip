// Masked softmax and top-p (nucleus) sampling.
//
// Reference behaviour restated (src/fastertransformer/kernels/sampling_topp_kernels.cu):
//   :1294-1345 addBiasSoftMax          - in-place masked softmax, result rounded to T
//   :801-860   topp_beam_topk_kernel   - arg-max shortcut when max prob >= top_p
//   :1106-1119 cub segmented sort      - stable descending sort of every row
//   :877-1004  topp_sampling           - inclusive prefix sum over 256-wide tiles, first crossing
//   :1381-1412 computeToppDecay
//
// The replacement never sorts a whole row unless it has to. One 1024-thread workgroup per row:
//   1. one pass: arg-max (ties to the lowest id), number of positive entries, per-thread maxima;
//   2. a lower bound t0 on the ~500th largest value from the order statistics of the thread maxima;
//      one pass gathers every entry >= t0 (<= 4096) into LDS; bitonic sort by (prob desc, id asc);
//   3. the reference's tile scan is replayed on the sorted prefix with its exact rounding order
//      (32 raking lanes x 8 items, Kogge-Stone over the 32 partials, sequential carry over tiles).
//   If the draw is not crossed inside the sorted prefix (deep draws on flat distributions) the row
//   falls back to a stable LSD radix sort of all positive entries in the caller's workspace and
//   replays the scan from the start.
#include "ftk_device.cuh"
#include "ftk_sampling.h"
#include "ftk_transform.cuh"

namespace ftk {

// =============================================================================================
// softmax
// =============================================================================================
constexpr int SM_THREADS = 1024;

// The reference block has BLK = min(n, 1024) threads and thread t owns columns t, t+BLK, ...;
// summation order (reduce_kernel_utils.cuh:73-103) = sequential per thread, xor butterfly
// (16,8,4,2,1) inside each 32-lane group, lane-0 partials through shared memory, butterfly again.
template<int DT>
__global__ void __launch_bounds__(SM_THREADS)
softmax_kernel(typename Storage<DT>::T* __restrict__ logits, const typename Storage<DT>::T* __restrict__ bias,
               const int* __restrict__ end_ids, const bool* __restrict__ finished, int n_padded, int n)
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

    float mx = -3.402823466e+38f;
    if (active) {
        for (int v = t; v < n_padded; v += BLK) {
            mx = __builtin_fmaxf(mx, masked(v));
        }
    }
    mx = block_max<float>(mx, sh, -3.402823466e+38f);
    if (BLK < 1024) {
        mx = __builtin_fmaxf(mx, -1e20f);  // blockReduceMax pads its second stage with -1e20f
    }

    float sum = 0.0f;
    if (active) {
        for (int v = t; v < n_padded; v += BLK) {
            sum += round_t<DT>(det_expf(masked(v) - mx));
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
    if (active) {
        for (int v = t; v < n_padded; v += BLK) {
            const float e = round_t<DT>(det_expf(masked(v) - mx));
            rowp[v]       = S::st(e / denom);
        }
    }
}

// =============================================================================================
// top-p
// =============================================================================================
constexpr int      TP_THREADS = 1024;
constexpr int      TP_BUF     = 4096;         // sorted-prefix capacity (LDS)
constexpr int      TP_TILE    = 256;          // the reference's scan tile
constexpr int      TP_MAXT    = TP_BUF / TP_TILE;
constexpr uint32_t ZERO_KEY   = 0x80000000u;  // order_key(+0.0f); entries at or below never join the scan

struct TopPShared {
    unsigned long long buf[TP_BUF];
    unsigned long long red64[16];
    uint32_t           red32[16];
    float              agg[TP_MAXT];
    float              carry[TP_MAXT + 1];
    uint32_t           tilemask[TP_MAXT][8];
    int                wtot[256];
    int                counter;
    int                misc[8];
    float              fmisc[4];
};

__device__ __forceinline__ float key64_prob(unsigned long long k)
{
    return key_to_float(~(uint32_t)(k >> 32));
}

// Replays the reference scan over `nt` tiles held in s.buf (entries >= n_in_buf count as 0).
// Returns the sorted position (relative to the buffer start) the reference would pick, or -1;
// s.carry[nt] is the running total afterwards. All threads must call; result is block-uniform.
__device__ int eval_tiles(TopPShared& s, int n_in_buf, int nt, float carry_in, float rand_num)
{
    const int t     = threadIdx.x;
    const int group = t >> 5;   // one 32-lane group per tile
    const int l     = t & 31;   // raking lane: items 8l .. 8l+7 of the tile
    float     x[8];
    float     incl = 0.0f;
    if (group < nt) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = group * TP_TILE + l * 8 + j;
            x[j]        = i < n_in_buf ? key64_prob(s.buf[i]) : 0.0f;
        }
        float seg = x[0];
#pragma unroll
        for (int j = 1; j < 8; ++j) {
            seg = seg + x[j];
        }
        incl = seg;
#pragma unroll
        for (int d = 1; d < 32; d <<= 1) {
            const float up = __shfl_up(incl, d, 32);
            if (l >= d) {
                incl = up + incl;
            }
        }
        if (l == 31) {
            s.agg[group] = incl;
        }
    }
    __syncthreads();
    if (t == 0) {
        float c    = carry_in;
        s.carry[0] = c;
        for (int g = 0; g < nt; ++g) {
            c              = c + s.agg[g];
            s.carry[g + 1] = c;
        }
    }
    __syncthreads();
    if (group < nt) {
        const float excl   = __shfl_up(incl, 1, 32);
        const float prefix = s.carry[group];
        float       a      = l == 0 ? prefix : prefix + excl;
        uint32_t    m8     = 0;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            a = a + x[j];
            if (rand_num <= a) {
                m8 |= 1u << j;
            }
        }
        reinterpret_cast<unsigned char*>(&s.tilemask[group][0])[l] = (unsigned char)m8;
    }
    __syncthreads();
    if (t == 0) {
        int found = -1;
        for (int g = 0; g < nt && found < 0; ++g) {
            for (int w = 0; w < 8; ++w) {
                const uint32_t m = s.tilemask[g][w];
                if (m != 0u) {
                    found = g * TP_TILE + w * 32 + (32 - __popc(m));
                    break;
                }
            }
        }
        s.misc[0] = found;
    }
    __syncthreads();
    const int found = s.misc[0];
    __syncthreads();
    return found;
}

// id of the `nth` (0-based) entry with probability exactly zero, in ascending id order: what a
// stable descending sort leaves behind the positive entries. Single thread; reached only when a
// draw lands within rounding distance of the total mass.
template<int DT>
__device__ int nth_zero_entry(const typename Storage<DT>::T* __restrict__ rowp, int vocab, int nth)
{
    int seen = 0, last = vocab - 1;
    for (int v = 0; v < vocab; ++v) {
        if (order_key(Storage<DT>::ld(rowp[v])) <= ZERO_KEY) {
            last = v;
            if (seen == nth) {
                return v;
            }
            seen++;
        }
    }
    return last;
}

template<int DT>
__global__ void __launch_bounds__(TP_THREADS)
topp_kernel(const typename Storage<DT>::T* __restrict__ probs, int* __restrict__ ids,
            int* __restrict__ sequence_length, bool* __restrict__ finished, float* __restrict__ cum_log_probs,
            float* __restrict__ output_log_probs, RngState* rng, const float* __restrict__ uniforms, int vocab,
            const int* __restrict__ end_ids, float top_p, const float* __restrict__ top_ps,
            const bool* __restrict__ skip_decode, unsigned long long* __restrict__ workspace, int force_deep)
{
    typedef Storage<DT>            S;
    __shared__ TopPShared          s;
    const int                      row = blockIdx.x;
    const int                      t   = threadIdx.x;
    if (skip_decode != nullptr && skip_decode[row]) {
        return;
    }
    const typename S::T* rowp = probs + (size_t)row * vocab;
    const float          p    = top_ps != nullptr ? top_ps[row] : top_p;

    // ---- pass 1: arg-max (lowest id on ties), positive count, thread maximum
    uint32_t tmax = 0;
    int      tidx = 0x7FFFFFFF;
    int      npos = 0;
    for (int v = t; v < vocab; v += TP_THREADS) {
        const uint32_t k = order_key(S::ld(rowp[v]));
        if (k > tmax) {
            tmax = k;
            tidx = v;
        }
        npos += k > ZERO_KEY ? 1 : 0;
    }
    // (key, ~id) packs "largest key, then lowest id" into one max-reduction
    unsigned long long best = ((unsigned long long)tmax << 32) | (uint32_t)(~(uint32_t)tidx);
    best                    = block_max<unsigned long long>(best, s.red64, 0ull);
    const int n_pos         = block_sum_i(npos, (int*)s.red32);
    int       best_id       = (int)(~(uint32_t)best);
    if ((uint32_t)(best >> 32) == 0u) {
        best_id = 0;  // nothing comparable in the row (all NaN): the reference keeps index 0
    }
    const float best_prob = S::ld(rowp[best_id]);

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

    bool done = false;
    if (!force_deep) {
        // ---- threshold from the order statistics of the 1024 thread maxima: every wave sorts its
        // 64 maxima; the q-th largest of each wave, minimised over the 16 waves, has at least 16q
        // entries above it. Four candidates, tightest first.
        const uint32_t sorted = wave_sort_desc(tmax);
        const int      qs[4]  = {30, 16, 6, 1};
        for (int a = 0; a < 4 && !done; ++a) {
            uint32_t cand = __shfl(sorted, qs[a] - 1, WAVE);
            uint32_t t0   = block_min<uint32_t>(cand, s.red32, 0xFFFFFFFFu);
            if (t0 <= ZERO_KEY) {
                t0 = ZERO_KEY + 1;
            }
            if (t == 0) {
                s.counter = 0;
            }
            __syncthreads();
            for (int v = t; v < vocab; v += TP_THREADS) {
                const uint32_t k = order_key(S::ld(rowp[v]));
                if (k >= t0) {
                    const int slot = atomicAdd(&s.counter, 1);
                    if (slot < TP_BUF) {
                        s.buf[slot] = ((unsigned long long)(~k) << 32) | (uint32_t)v;
                    }
                }
            }
            __syncthreads();
            const int n = s.counter;
            __syncthreads();
            if (n > TP_BUF) {
                continue;  // too many ties / too flat at this quantile: try a tighter threshold
            }
            const int np2 = max(2, next_pow2(n));
            for (int i = n + t; i < np2; i += TP_THREADS) {
                s.buf[i] = ~0ull;
            }
            __syncthreads();
            block_bitonic_sort_u64(s.buf, np2);
            const bool all = n == n_pos;
            const int  nt  = all ? (n + TP_TILE - 1) / TP_TILE : n / TP_TILE;
            if (nt > 0) {
                const int found = eval_tiles(s, n, nt, 0.0f, rand_num);
                if (found >= 0) {
                    if (t == 0) {
                        if (found < n) {
                            const unsigned long long e = s.buf[found];
                            emit((int)(uint32_t)e, key64_prob(e));
                        }
                        else {
                            const int id = nth_zero_entry<DT>(rowp, vocab, found - n);
                            emit(id, S::ld(rowp[id]));
                        }
                    }
                    return;
                }
            }
            if (all) {
                return;  // every positive entry scanned, never crossed: ids keeps the arg-max
            }
            break;  // sorted prefix exhausted without crossing: deep path
        }
    }

    // ---- deep path: stable LSD radix sort (4-bit digits) of all positive entries in `workspace`
    // (2 * vocab 64-bit slots per row), then the same scan over the whole sorted row.
    unsigned long long* A = workspace + (size_t)row * 2 * vocab;
    unsigned long long* B = A + vocab;
    // stable compaction in id order, 1024 consecutive ids per round
    if (t == 0) {
        s.misc[1] = 0;
    }
    __syncthreads();
    for (int base = 0; base < vocab; base += TP_THREADS) {
        const int      v    = base + t;
        const uint32_t k    = v < vocab ? order_key(S::ld(rowp[v])) : 0u;
        const bool     keep = k > ZERO_KEY;
        const unsigned long long bal = __ballot(keep);
        const int      below = __popcll(bal & ((1ull << lane_id()) - 1ull));
        if (lane_id() == 0) {
            s.red32[wave_id()] = (uint32_t)__popcll(bal);
        }
        __syncthreads();
        int off = s.misc[1];
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
            s.misc[1] += tot;
        }
        __syncthreads();
    }
    const int n = s.misc[1];  // == n_pos
    // digit passes over bits 32..63; thread t owns the contiguous slice [t*chunk, (t+1)*chunk)
    {
        // [16][1024] 16-bit counters alias the (idle) sort buffer; a slice holds <= 65535 entries
        unsigned short* cnt16 = reinterpret_cast<unsigned short*>(s.buf);
        const int       chunk = (n + TP_THREADS - 1) / TP_THREADS;
        const int       lo    = min(n, t * chunk);
        const int       hi    = min(n, lo + chunk);
        // digits that are constant over the whole row need no pass
        unsigned long long vor = 0ull, vand = ~0ull;
        for (int i = lo; i < hi; ++i) {
            vor |= A[i];
            vand &= A[i];
        }
        for (int o = 32; o > 0; o >>= 1) {
            vor |= __shfl_xor(vor, o, WAVE);
            vand &= __shfl_xor(vand, o, WAVE);
        }
        if (lane_id() == 0) {
            s.red64[wave_id()] = vor;
        }
        __syncthreads();
        unsigned long long all_or = 0ull;
        for (int w = 0; w < TP_THREADS / WAVE; ++w) {
            all_or |= s.red64[w];
        }
        __syncthreads();
        if (lane_id() == 0) {
            s.red64[wave_id()] = vand;
        }
        __syncthreads();
        unsigned long long all_and = ~0ull;
        for (int w = 0; w < TP_THREADS / WAVE; ++w) {
            all_and &= s.red64[w];
        }
        __syncthreads();
        const unsigned long long diff = all_or ^ all_and;

        unsigned long long* src = A;
        unsigned long long* dst = B;
        for (int shift = 32; shift < 64; shift += 4) {
            if (((diff >> shift) & 0xFull) == 0ull) {
                continue;
            }
            // 1. private digit counts
            for (int d = 0; d < 16; ++d) {
                cnt16[d * TP_THREADS + t] = 0;
            }
            for (int i = lo; i < hi; ++i) {
                const int d = (int)((src[i] >> shift) & 0xFull);
                cnt16[d * TP_THREADS + t]++;
            }
            // 2. exclusive prefix over (digit major, thread minor)
            int base_off[16];
#pragma unroll
            for (int d = 0; d < 16; ++d) {
                const int val = cnt16[d * TP_THREADS + t];
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
                    s.wtot[d * 16 + wave_id()] = inc;
                }
            }
            __syncthreads();
            {
                int digit_base = 0;
#pragma unroll
                for (int d = 0; d < 16; ++d) {
                    int pre = 0, tot = 0;
                    for (int w = 0; w < TP_THREADS / WAVE; ++w) {
                        const int x = s.wtot[d * 16 + w];
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
        // sorted data is in `src`
        float carry_in = 0.0f;
        for (int base = 0; base < n; base += TP_BUF) {
            const int m = min(TP_BUF, n - base);
            for (int i = t; i < m; i += TP_THREADS) {
                s.buf[i] = src[base + i];
            }
            __syncthreads();
            const bool last = base + m == n;
            const int  nt   = last ? (m + TP_TILE - 1) / TP_TILE : m / TP_TILE;  // m == TP_BUF unless last
            const int  found = eval_tiles(s, m, nt, carry_in, rand_num);
            if (found >= 0) {
                if (t == 0) {
                    if (found < m) {
                        const unsigned long long e = s.buf[found];
                        emit((int)(uint32_t)e, key64_prob(e));
                    }
                    else {
                        const int id = nth_zero_entry<DT>(rowp, vocab, base + found - n);
                        emit(id, S::ld(rowp[id]));
                    }
                }
                return;
            }
            carry_in = s.carry[nt];
            __syncthreads();
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
    FTK_DISPATCH_DTYPE(dtype, softmax_kernel<DT><<<m, SM_THREADS, 0, (hipStream_t)stream>>>(
                                  (Storage<DT>::T*)logits, (const Storage<DT>::T*)bias, end_ids, finished, n_padded, n));
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

// Test hook: a non-zero value routes every row through the radix-sort fallback.
static int g_topp_force_deep = 0;
void       ftk_test_set_topp_force_deep(int v)
{
    g_topp_force_deep = v;
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
    if (dtype < 0 || dtype > 2) {
        return FTK_ERR_DTYPE;
    }
    // fallback sort: two 64-bit (key, id) arrays per row
    const size_t need = (size_t)batch_size * vocab_size_padded * 2 * sizeof(unsigned long long);
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
    if (vocab_size_padded > (size_t)65535 * TP_THREADS) {
        return FTK_ERR_ARGUMENT;
    }
    FTK_DISPATCH_DTYPE(dtype, topp_kernel<DT><<<batch_size, TP_THREADS, 0, (hipStream_t)stream>>>(
                                  (const Storage<DT>::T*)log_probs, output_ids, sequence_length, finished,
                                  cum_log_probs, output_log_probs, (RngState*)rng_state, uniform_draws,
                                  (int)vocab_size_padded, end_ids, max_top_p, top_ps, skip_decode,
                                  (unsigned long long*)workspace, g_topp_force_deep));
    FTK_LAUNCH_CHECK();
    return 0;
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
