// Candidate lists for launches whose largest k is beyond what one read of a row can bound (k > 192), in one launch.
//
// The lean gather takes two launches for them (lean_gather_kernel in its SLOTS and PRESET modes: maxima of column
// groups first, then every workgroup of a row works out the row's bound from all of them and gathers). With up to a
// few rows per compute unit that pair is bound by the latency of its many small workgroups. Here one 1024-thread
// workgroup per row reads the row twice (the second time from the caches):
//   1. every thread takes the exact maxima of three disjoint groups of its columns (3072 per row, each the final
//      value of a column of its own, after temperature, history penalty and masks);
//   2. the row's bound: the largest P, to within its low sixteen bits, that at least k of those maxima reach (two
//      rounds of a 256-bin count over the keys' top bytes) - at least k columns lie at or above it;
//   3. everything at or above the bound goes to the row's list in the format of the lean gather (one list per row),
//      which lean_select_kernel orders and samples from.
// Preconditions (checked by the host, which otherwise takes the two launches): no embedding bias, rows on 16-byte
// boundaries with at least 3072 whole vectors, the row's history bitmap fits the LDS window.
#pragma once
#include "ftk_lean.cuh"

namespace ftk {

constexpr int LK_THREADS = 1024;
constexpr int LK_GROUPS  = 3;  // maxima per thread
constexpr int LK_RING    = 8;  // vectors a thread keeps in flight

// The lane of wave 0 that holds bins 4 lane .. 4 lane + 3 of a 256-bin count finds the highest bin b with at least
// `want` entries in bins b .. 255. Returns true in the lane that found it, with the bin and the number of entries
// above it; false everywhere when there are fewer than `want` entries.
__device__ __forceinline__ bool largek_bin_of_rank(const uint32_t* hist, int lane, uint32_t want, uint32_t* bin,
                                                   uint32_t* above_out)
{
    const uint32_t c0 = hist[4 * lane], c1 = hist[4 * lane + 1], c2 = hist[4 * lane + 2], c3 = hist[4 * lane + 3];
    const uint32_t s    = c0 + c1 + c2 + c3;
    uint32_t       incl = s;  // entries in this lane's bins and in those of higher lanes
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const uint32_t v = __shfl_down(incl, d, WAVE);
        if (lane + d < WAVE) {
            incl += v;
        }
    }
    const uint32_t above = incl - s;
    if (!(above < want && want <= incl)) {
        return false;
    }
    uint32_t run = above;
    if (run + c3 >= want) {
        *bin       = 4 * lane + 3;
        *above_out = run;
        return true;
    }
    run += c3;
    if (run + c2 >= want) {
        *bin       = 4 * lane + 2;
        *above_out = run;
        return true;
    }
    run += c2;
    if (run + c1 >= want) {
        *bin       = 4 * lane + 1;
        *above_out = run;
        return true;
    }
    run += c1;
    *bin       = 4 * lane;
    *above_out = run;
    return true;
}

#ifdef FTK_LK_STAMPS  // development builds: wall-clock stamps of a row's phases behind its list
#define LK_STAMP(i) if (threadIdx.x == 0) { reinterpret_cast<unsigned long long*>(l.entries + (size_t)blockIdx.x * l.row_entries + TK_CCAP)[i] = wall_clock64(); }
#else
#define LK_STAMP(i)
#endif

template<int DT, int BMW>
__global__ void __launch_bounds__(LK_THREADS) largek_gather_kernel(FusedParams p, FusedLaunch l)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    __shared__ uint32_t   hist[256];
    __shared__ uint32_t   pick[4];
    __shared__ int        n_out;
    const int             t    = threadIdx.x;
    const int             lane = t & (WAVE - 1);
    const int             row  = blockIdx.x;
    const T*              rowp = (const T*)p.logits + (size_t)row * p.Vp;
    const uint4*          base = reinterpret_cast<const uint4*>(rowp);  // (the host checked the alignment)
    const int             nvec  = p.V / EPV;                            // whole vectors inside the vocabulary
    const int             turns = (nvec + LK_THREADS - 1) / LK_THREADS;
    uint4                 ring[LK_RING];
    // (every load is issued whatever the turn, one past the last fetches the last again, unused: with the same number
    // of loads on every path the waits can name the oldest load instead of everything in flight)
    auto vload = [&](int slot, int q) { ring[slot] = base[min(min(q, turns - 1) * LK_THREADS + t, nvec - 1)]; };
#pragma unroll
    for (int r = 0; r < LK_RING; ++r) {
        vload(r, r);
    }
    const bool        skip = row_flag_or(p.skip_decode, row, p.end_ids + row, false);
    const bool        fin  = row_flag_or(p.finished_in, row, p.end_ids + row, false);
    const int         k    = row_arg_or(p.top_ks, row, p.end_ids + row, p.max_top_k);
    FusedRow<DT, BMW> rowctx(p, row);
    LK_STAMP(0)
    if (skip || fin) {
        return;  // (the select kernel does what such a row needs)
    }
    if (t == 0) {
        n_out = 0;
    }
    if (t < 256) {
        hist[t] = 0u;
    }
    rowctx.prepare(0, p.V);  // the row's history bitmap in LDS
    __syncthreads();
    LK_STAMP(1)
    const bool     bitsv   = rowctx.has_vector_bits();
    const float    mul     = rowctx.fast_mul;
    const bool     ordered = mul > 0.0f && mul < __builtin_inff();  // the plain transform keeps the order
    const float    NEG_INF = -__builtin_inff();
    const uint32_t KMIN    = min_valid_key<DT>();
    // history flags of the vector whose first column is `first` (a multiple of EPV: never across a bitmap word)
    auto flags_of = [&](int first) -> uint32_t {
        if (!bitsv) {
            return 0u;
        }
        if constexpr (BMW > 0) {
            const int rel = first - rowctx.bm_origin;
            return (rowctx.bm_word(rel >> 5) >> (rel & 31)) & ((1u << EPV) - 1u);
        }
        else {
            return rowctx.vector_bits(first, EPV);
        }
    };
    // the final values of a vector's columns; the masked end id counts as -MAX_T like in the reference
    auto values_of = [&](const uint4& v, int first, uint32_t bits, float* x) {
#pragma unroll
        for (int c = 0; c < EPV; ++c) {
            x[c] = rowctx.fast(vector_element<DT>(v, c));
            if ((bits >> c) & 1u) {
                x[c] = rowctx.flagged(x[c], first + c);
            }
            if (first + c == rowctx.masked_end_id) {
                x[c] = -S::max_t();
            }
        }
    };
    auto value_of = [&](int v) -> float {
        float x = rowctx.fast(S::ld(rowp[v]));
        if (bitsv && rowctx.vector_bits(v, 1) != 0u) {
            x = rowctx.flagged(x, v);
        }
        return v == rowctx.masked_end_id ? -S::max_t() : x;
    };

    // ---- 1. three maxima per thread: of the first, the second and the last third of its vectors
    float     g0 = NEG_INF, g1 = NEG_INF, g2 = NEG_INF;
    const int third = (turns + LK_GROUPS - 1) / LK_GROUPS;
    for (int q0 = 0; q0 < turns; q0 += LK_RING) {
#pragma unroll
        for (int r = 0; r < LK_RING; ++r) {
            const int q = q0 + r;
            if (q < turns) {
                const int      rel     = q * LK_THREADS + t;
                const int      first   = min(rel, nvec - 1) * EPV;
                const uint32_t bits    = flags_of(first);
                const uint32_t rel_end = (uint32_t)(rowctx.masked_end_id - first);
                float          vm;
                if (bits == 0u && rel_end >= (uint32_t)EPV && ordered) {
                    vm = rowctx.fast(lean_raw_max<DT>(ring[r]));
                }
                else {
                    float x[EPV];
                    values_of(ring[r], first, bits, x);
                    vm = NEG_INF;
#pragma unroll
                    for (int c = 0; c < EPV; ++c) {
                        vm = __builtin_fmaxf(vm, x[c]);
                    }
                }
                vm           = rel < nvec ? vm : NEG_INF;
                const int g  = q / third;  // (the same for every thread)
                g0           = g == 0 ? __builtin_fmaxf(g0, vm) : g0;
                g1           = g == 1 ? __builtin_fmaxf(g1, vm) : g1;
                g2           = g >= 2 ? __builtin_fmaxf(g2, vm) : g2;
            }
            vload(r, q + LK_RING);
        }
    }
    // the columns behind the last whole vector join their thread's last group
    for (int v = nvec * EPV + t; v < p.V; v += LK_THREADS) {
        g2 = __builtin_fmaxf(g2, value_of(v));
    }
    LK_STAMP(2)
    const uint32_t key[LK_GROUPS] = {order_key(g0), order_key(g1), order_key(g2)};
    // (the second read's first vectors are requested now: they arrive while the bound is worked out)
#pragma unroll
    for (int r = 0; r < LK_RING; ++r) {
        vload(r, r);
    }

    // ---- 2. the bound: the top byte of the k-th largest key, then its second byte among the keys that share the first
#pragma unroll
    for (int g = 0; g < LK_GROUPS; ++g) {
        atomicAdd(&hist[key[g] >> 24], 1u);
    }
    __syncthreads();
    if (t < WAVE) {
        uint32_t   bin = 0u, above = 0u;
        const bool mine = largek_bin_of_rank(hist, lane, (uint32_t)k, &bin, &above);
        if (__ballot(mine) == 0ull) {
            if (lane == 0) {
                pick[0] = 0xFFFFFFFFu;  // fewer than k maxima at all (cannot happen with 3072 of them and k <= 1024)
            }
        }
        else if (mine) {
            pick[0] = bin;
            pick[1] = (uint32_t)k - above;  // rank inside the bin
        }
    }
    __syncthreads();
    const uint32_t top_byte = pick[0];
    const uint32_t want     = pick[1];
    if (t < 256) {
        hist[t] = 0u;
    }
    __syncthreads();
    if (top_byte != 0xFFFFFFFFu) {
#pragma unroll
        for (int g = 0; g < LK_GROUPS; ++g) {
            if ((key[g] >> 24) == top_byte) {
                atomicAdd(&hist[(key[g] >> 16) & 255u], 1u);
            }
        }
    }
    __syncthreads();
    if (t < WAVE) {
        uint32_t   bin = 0u, above = 0u;
        const bool mine = top_byte != 0xFFFFFFFFu && largek_bin_of_rank(hist, lane, want, &bin, &above);
        if (__ballot(mine) == 0ull) {
            if (lane == 0) {
                pick[2] = 0u;
            }
        }
        else if (mine) {
            pick[2] = (top_byte << 24) | (bin << 16);
        }
    }
    __syncthreads();
    LK_STAMP(3)
    const uint32_t P     = pick[2];
    const bool     valid = P >= KMIN;  // at least k columns with a valid value at or above it
    const uint32_t thr   = valid ? P : KMIN;
    const float    thr_f = key_to_float(thr);  // x >= thr_f  <=>  order_key(x) >= thr (a NaN fails both)

    // ---- 3. what reaches the bound goes to the list (the row comes from the caches this time)
    TopkEntry* out  = l.entries + (size_t)row * l.row_entries;
    auto       push = [&](float x, int v) {
        const int slot = atomicAdd(&n_out, 1);
        if (slot < TK_CCAP) {
            out[slot] = TopkEntry{order_key(x), (uint32_t)(v + p.col_offset)};
        }
    };
    for (int q0 = 0; q0 < turns; q0 += LK_RING) {
#pragma unroll
        for (int r = 0; r < LK_RING; ++r) {
            const int q = q0 + r;
            if (q < turns) {
                const int      rel     = q * LK_THREADS + t;
                const int      first   = min(rel, nvec - 1) * EPV;
                const uint32_t bits    = flags_of(first);
                const uint32_t rel_end = (uint32_t)(rowctx.masked_end_id - first);
                const bool     plain   = bits == 0u && rel_end >= (uint32_t)EPV && ordered;
                // (a plain vector whose largest element stays under the bound holds no candidate)
                if (rel < nvec && !(plain && !(rowctx.fast(lean_raw_max<DT>(ring[r])) >= thr_f))) {
                    float    x[EPV];
                    uint32_t hit = 0u;
                    if (plain) {  // (the common case without the history and end-id arithmetic)
#pragma unroll
                        for (int c = 0; c < EPV; ++c) {
                            x[c] = rowctx.fast(vector_element<DT>(ring[r], c));
                        }
                    }
                    else {
                        values_of(ring[r], first, bits, x);
                    }
#pragma unroll
                    for (int c = 0; c < EPV; ++c) {
                        hit |= (x[c] >= thr_f && (uint32_t)c != rel_end) ? (1u << c) : 0u;  // (the masked end id is no candidate)
                    }
                    while (hit != 0u) {  // as many rounds as the lane of the wave with the most candidates has
                        const int c = __builtin_ctz(hit);
                        hit &= hit - 1u;
                        float xc = x[0];
#pragma unroll
                        for (int j = 1; j < EPV; ++j) {
                            xc = j == c ? x[j] : xc;
                        }
                        push(xc, first + c);
                    }
                }
            }
            vload(r, q + LK_RING);
        }
    }
    for (int v = nvec * EPV + t; v < p.V; v += LK_THREADS) {
        const float x = value_of(v);
        if (x >= thr_f && v != rowctx.masked_end_id) {
            push(x, v);
        }
    }
    LK_STAMP(4)
    __syncthreads();
    LK_STAMP(5)
    if (t == 0) {
        const int       n = n_out;
        TopkChunkHeader h;
        h.count     = n > TK_CCAP ? 0u : (uint32_t)n;
        h.threshold = thr;
        h.flags     = n > TK_CCAP ? 2u : (valid ? 1u : 0u);
        h.share     = 0u;
        l.headers[(size_t)row * l.splits] = h;  // (the launch has one list per row)
    }
}

// Launchers, one translation unit per element type (lean_kernels.hip). window: 1 = small LDS window, 2 = large.
int largek_gather_launch_f32(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                             hipEvent_t start, hipEvent_t stop);
int largek_gather_launch_f16(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                             hipEvent_t start, hipEvent_t stop);
int largek_gather_launch_bf16(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                              hipEvent_t start, hipEvent_t stop);

}  // namespace ftk
