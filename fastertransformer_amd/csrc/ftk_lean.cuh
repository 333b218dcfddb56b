// Streaming candidate gather of the fused decode step for launches without an embedding bias: in one read of
// the logits when the largest k is at most 192, in two (maxima first, see LG_MODE_*) for a larger k.
//
// Same contract as the stream of ftk_topk.cuh (reference behaviour: topk_stage1 of
// src/fastertransformer/kernels/sampling_topk_kernels.cu:130-202 after the penalty kernels of
// src/fastertransformer/kernels/sampling_penalty_kernels.cu): a workgroup walks its share of a row once and
// leaves, in the workspace, every element at or above a lower bound of the row's k-th largest value. What
// differs is how the walk is organised, so that the memory system never waits for the arithmetic:
//   - a thread keeps a ring of R sub-tiles (4 vectors of 16 bytes each) in registers; the loads of all R are
//     issued before anything else happens, from kernel arguments alone (the per-row arguments arrive while
//     they are in flight), and a slot is refilled as soon as it has been examined;
//   - the inner loop is a maximum, a multiply and a compare per vector, without barriers and without looking
//     at the history bitmap: a vector is parked when its largest element, taken as if no history penalty
//     applied, reaches a threshold that no penalised or rounded value can get past; parked vectors are
//     evaluated exactly, by the wave that parked them, when its parking list fills up;
//   - the bound is the k-th largest of 256 values of distinct elements - first the thread maxima over the
//     first two sub-tiles, later the largest candidate each lane has evaluated - found by every wave on its
//     own with 16 rounds of ballots (one workgroup barrier per bound, no sort);
//   - candidates go straight to the workgroup's list in the workspace.
// A workgroup that cannot keep its list inside the workspace slot says so in the header; the merging kernel
// then walks that row again with the general stream.
#pragma once
#include <hip/hip_ext.h>

#include "ftk_fused.cuh"

namespace ftk {

constexpr int LG_THREADS  = 256;
constexpr int LG_WAVES    = LG_THREADS / WAVE;
constexpr int LG_NV       = 4;                   // 16-byte vectors per thread and sub-tile
constexpr int LG_SUB_VECS = LG_THREADS * LG_NV;  // a sub-tile: 16 KB
constexpr int LG_DRAIN_AT = 64;                  // parked vectors at which a wave evaluates them (checked once per sub-tile)
constexpr int LG_STAGE    = LG_DRAIN_AT + LG_NV * WAVE;  // vectors a wave can park between two evaluations
constexpr int LG_MAX_K    = 192;  // largest k of a launch that reads the logits once (the bound is the k-th of 256 values)

struct LeanShared {
    uint4    stage_raw[LG_WAVES][LG_STAGE];
    int      stage_first[LG_WAVES][LG_STAGE];
    uint32_t slot_key[2][LG_THREADS];
    int      n_out;
};

struct LeanPlan {
    int splits;       // workgroups per row
    int subs_per_wg;  // sub-tiles each of them streams
};

// `fill`: workgroups the chip holds at once
inline LeanPlan lean_plan(int vocab, int rows, int elem_bytes, int fill)
{
    const int epv  = 16 / elem_bytes;
    const int nvec = vocab / epv + 1;
    const int nsub = (nvec + LG_SUB_VECS - 1) / LG_SUB_VECS;
    int       s    = (fill + rows - 1) / (rows > 0 ? rows : 1);
    const int most = nsub / 2 > 1 ? nsub / 2 : 1;  // a workgroup takes its first bound from two sub-tiles
    s              = s > most ? most : s;
    s              = s > TK_MAXSPLIT ? TK_MAXSPLIT : s;
    s              = s < 1 ? 1 : s;
    LeanPlan p;
    p.subs_per_wg = (nsub + s - 1) / s;
    p.splits      = (nsub + p.subs_per_wg - 1) / p.subs_per_wg;
    return p;
}

// The largest value P, to within its low sixteen bits, such that at least k of the 256 keys are >= P
// (0 when fewer than k keys are non-zero): sign, exponent and seven bits of mantissa decide, which admits a
// few per cent more candidates than the exact k-th largest would. Every wave calls it on the same keys and
// gets the same answer.
__device__ __forceinline__ uint32_t lean_kth_of_slots(const uint32_t* keys, int k)
{
    uint32_t kk[LG_WAVES];
#pragma unroll
    for (int g = 0; g < LG_WAVES; ++g) {
        kk[g] = keys[lane_id() + g * WAVE];
    }
    uint32_t P = 0u;
#pragma unroll
    for (int bit = 31; bit >= 16; --bit) {
        const uint32_t cand = P | (1u << bit);
        int            c    = 0;
#pragma unroll
        for (int g = 0; g < LG_WAVES; ++g) {
            c += (int)__builtin_popcountll(__ballot(kk[g] >= cand));
        }
        P = c >= k ? cand : P;
    }
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)P);
}

// largest element of a 16-byte vector as stored (no transform); NaN elements are ignored
template<int DT>
__device__ __forceinline__ float lean_raw_max(const uint4& v)
{
    if constexpr (DT == DT_F32) {
        return __builtin_fmaxf(__builtin_fmaxf(__uint_as_float(v.x), __uint_as_float(v.y)),
                               __builtin_fmaxf(__uint_as_float(v.z), __uint_as_float(v.w)));
    }
    else if constexpr (DT == DT_F16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        const h2         a = __builtin_bit_cast(h2, v.x), b = __builtin_bit_cast(h2, v.y);
        const h2         c = __builtin_bit_cast(h2, v.z), d = __builtin_bit_cast(h2, v.w);
        const h2 m = __builtin_elementwise_max(__builtin_elementwise_max(a, b), __builtin_elementwise_max(c, d));
        return __builtin_fmaxf((float)m.x, (float)m.y);
    }
    else {
        auto pair_max = [](uint32_t w) -> float {
            return __builtin_fmaxf(__uint_as_float(w << 16), __uint_as_float(w & 0xFFFF0000u));
        };
        return __builtin_fmaxf(__builtin_fmaxf(pair_max(v.x), pair_max(v.y)),
                               __builtin_fmaxf(pair_max(v.z), pair_max(v.w)));
    }
}

// A value that an unrounded product must reach before its rounding to T can reach `x`.
template<int DT>
__device__ __forceinline__ float lean_below_rounding(float x)
{
    if constexpr (DT == DT_F32) {
        return x;
    }
    else {
        const float rel  = DT == DT_F16 ? 0.0009765625f : 0.0078125f;             // one unit in the last place of T
        const float tiny = DT == DT_F16 ? 5.9604644775390625e-08f : 1.0e-38f;  // ... of T's subnormals
        return x - __builtin_fmaxf(__builtin_fabsf(x) * rel, tiny);
    }
}

// a 16-byte load that is read once: it does not displace what the caches hold for others
__device__ __forceinline__ uint4 lean_stream_load(const uint4* p)
{
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    const u4             v = __builtin_nontemporal_load(reinterpret_cast<const u4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}

constexpr int LG_HIST_U = 8;  // history ids a thread requests before the logits (2048 positions per workgroup)

// What a launch of lean_gather_kernel does.
//   STREAM: one read of the row. Every workgroup bounds the k-th largest of its own columns as it goes
//           (k <= LG_MAX_K: the bound is the k-th largest of 256 values, which gets loose as k approaches 256).
//   SLOTS / PRESET: two reads, for any k up to 1024. The first launch (SLOTS) only takes maxima: 256 * slot_u
//           per workgroup, each over a group of columns of its own. The k-th largest of a row's maxima bounds
//           the row's k-th largest value from below, and with two to four times k maxima only little more than
//           k columns reach it. The second launch (PRESET) finds that bound first and gathers against it.
enum { LG_MODE_STREAM = 0, LG_MODE_SLOTS = 1, LG_MODE_PRESET = 2 };
constexpr int LG_SLOT_U_MAX    = 4;   // maxima a thread delivers: one per vector of a sub-tile
constexpr int LG_SLOT_KEYS_MAX = 32;  // maxima of a row a thread of the PRESET launch holds: splits * slot_u

// slot_u for a row cut into `splits`; 0: too many workgroups per row for the two-read selection
inline int lean_slot_u(int splits)
{
    const int u = LG_SLOT_KEYS_MAX / (splits > 0 ? splits : 1);
    return u >= 4 ? 4 : (u >= 2 ? 2 : u);
}

constexpr int LS_PF_LISTS  = 2;  // lists a wave requests up front (wave w: lists w and w + 4)
constexpr int LS_PF_ROUNDS = 4;  // 64 entries each: the first 256 entries of a list

struct LeanListPrefetch {
    TopkEntry e[LS_PF_LISTS][LS_PF_ROUNDS];
};

// Requested at the top of the kernel, before anything is known about the row: the loads are in flight while
// the row's arguments and the list headers arrive. Reads stay inside the row's slots of the workspace.
__device__ __forceinline__ LeanListPrefetch lean_prefetch_lists(int splits, const TopkEntry* entries)
{
    LeanListPrefetch pf;
#pragma unroll
    for (int m = 0; m < LS_PF_LISTS; ++m) {
        const int        c = wave_id() + m * TK_WAVES;
        const TopkEntry* e = entries + (size_t)(c < splits ? c : 0) * TK_CCAP;
#pragma unroll
        for (int r = 0; r < LS_PF_ROUNDS; ++r) {
            pf.e[m][r] = e[r * WAVE + lane_id()];
        }
    }
    return pf;
}

template<int DT>
__device__ __forceinline__ void lean_select_row(TopkShared& s, const FusedParams& p, const FusedLaunch& l, int row, int k,
                                                float tp, const LeanListPrefetch& pf);

union LeanTopkShared {
    LeanShared lean;  // while the row is read
    TopkShared topk;  // while a row's list is ordered and sampled (ROWSEL)
};

// BIAS: the launch has an embedding bias (a variant of its own: the common kernels do not carry its registers).
// ROWSEL: every row belongs to one workgroup (gridDim.x == 1), which goes on to order its list and sample:
// the step is this one launch, and the selection of one row overlaps with the reading of others.
template<int DT, int BMW, int OCC, int R, int MODE, bool BIAS, bool ROWSEL>
__global__ void __launch_bounds__(LG_THREADS, OCC) lean_gather_kernel(FusedParams p, FusedLaunch l)
{
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    static_assert(R >= 2, "the first bound reads two sub-tiles");
    static_assert(!ROWSEL || LG_THREADS == TK_THREADS, "the selection runs in the gather's workgroup");
    __shared__ LeanTopkShared sh;
    LeanShared&               s     = sh.lean;
    const int                 t     = threadIdx.x;
    const int                 row   = blockIdx.y;
    const int                 chunk = blockIdx.x;
    const int             lane  = lane_id();
    const int             wv    = wave_id();

    // ---- geometry, from kernel arguments alone: the first loads leave before anything is read from memory
    const T*     rowp     = (const T*)p.logits + (size_t)row * p.Vp;
    const int    a        = (int)(((uintptr_t)rowp & 15u) / sizeof(T));
    const uint4* base     = reinterpret_cast<const uint4*>(reinterpret_cast<const char*>(rowp) - a * sizeof(T));
    const int    vfull_lo = (a + EPV - 1) / EPV;  // vectors [vfull_lo, vfull_hi) lie inside columns [0, V)
    const int    vfull_hi = max(vfull_lo, (a + p.V) / EPV);
    const int    vb       = min(vfull_hi, vfull_lo + chunk * l.subs_per_wg * LG_SUB_VECS);
    const int    ve       = min(vfull_hi, vb + l.subs_per_wg * LG_SUB_VECS);
    const int    nvec     = ve - vb;
    const int    nsub     = (nvec + LG_SUB_VECS - 1) / LG_SUB_VECS;

    // The token history comes first (it is time-major: every id is a cache line of its own), so that the
    // bitmap of penalised columns is built while the logits are still on their way.
    const bool hist = BMW > 0 && p.bitmaps != nullptr && p.penalties != nullptr;
    int        hist_ids[LG_HIST_U];
    if (hist) {
#pragma unroll
        for (int u = 0; u < LG_HIST_U; ++u) {
            const int pos = t + u * LG_THREADS;
            hist_ids[u]   = pos < p.step ? p.output_ids[(size_t)pos * p.batch_size + row] - p.col_offset : -1;
        }
    }
    // An embedding bias (rows and bias on 16-byte boundaries: the launcher checks) is read alongside: the same
    // vector of every row, so it comes from the caches.
    constexpr bool has_bias  = BIAS;
    const uint4*   bias_base = reinterpret_cast<const uint4*>(p.bias);
    uint4          raw[R][LG_NV];
    uint4          rawb[BIAS ? R : 1][LG_NV];
    auto         load = [&](int slot, int q) {
#pragma unroll
        for (int j = 0; j < LG_NV; ++j) {
            const int vi = min(vb + q * LG_SUB_VECS + j * LG_THREADS + t, ve - 1);  // past the end: a harmless vector
            raw[slot][j] = lean_stream_load(base + vi);
            if constexpr (BIAS) {
                rawb[slot][j] = bias_base[vi];
            }
        }
    };
    // largest element of a vector before the temperature: as stored, or stored + bias (unrounded for 16-bit
    // types: the thresholds allow for that rounding)
    auto vector_max = [&](const uint4& v, const uint4& b) -> float {
        if (!has_bias) {
            return lean_raw_max<DT>(v);
        }
        float m = -__builtin_inff();
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
            m = __builtin_fmaxf(m, vector_element<DT>(v, e) + vector_element<DT>(b, e));
        }
        return m;
    };
    // element e of a vector as the temperature sees it: T(stored + bias)
    auto biased_element = [&](const uint4& v, const uint4& b, int e) -> float {
        const float x = vector_element<DT>(v, e);
        return has_bias ? round_t<DT>(x + vector_element<DT>(b, e)) : x;
    };
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r < nsub) {
            load(r, r);
        }
    }

    // PRESET: the row's maxima from the SLOTS launch, thread t looks at slot t of every group
    uint32_t  slot_keys[MODE == LG_MODE_PRESET ? LG_SLOT_KEYS_MAX : 1];
    const int n_slot_keys = MODE == LG_MODE_PRESET ? (int)gridDim.x * l.slot_u : 0;
    if constexpr (MODE == LG_MODE_PRESET) {
        const uint32_t* mine = l.slots + (size_t)row * gridDim.x * l.slot_u * LG_THREADS + t;
#pragma unroll
        for (int i = 0; i < LG_SLOT_KEYS_MAX; ++i) {
            slot_keys[i] = i < n_slot_keys ? mine[(size_t)i * LG_THREADS] : 0u;
        }
    }

    // ---- per-row arguments
    // (all requested together; a row that does not take part leaves once they are here)
    const bool        skip = row_flag_or(p.skip_decode, row, p.end_ids + row, false);
    const bool        fin  = row_flag_or(p.finished_in, row, p.end_ids + row, false);
    const int         k    = row_arg_or(p.top_ks, row, p.end_ids + row, p.max_top_k);
    const float       tp   = ROWSEL ? row_arg_or(p.top_ps, row, p.end_ids + row, 1.0f) : 1.0f;
    FusedRow<DT, BMW> rowctx(p, row);
    if (skip || fin) {
        if (ROWSEL && fin && !skip && t == 0) {
            l.ids[row] = p.end_ids[row];  // (what the select kernel does for a finished row)
        }
        return;
    }
    if (t == 0) {
        s.n_out = 0;
    }
    // columns this workgroup looks at: its vectors, plus the few columns in front of the first whole vector
    // (first workgroup of the row) and behind the last one (last workgroup)
    const bool first_wg = chunk == 0;
    const bool last_wg  = chunk == (int)gridDim.x - 1;
    const int  lo_col   = first_wg ? 0 : vb * EPV - a;
    const int  hi_col   = last_wg ? p.V : ve * EPV - a;
    if (hist) {
        // the window of the history bitmap that covers [lo_col, hi_col), in LDS
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
            mark(pos, p.output_ids[(size_t)pos * p.batch_size + row] - p.col_offset);
        }
        rowctx.bm_mode   = 1;
        rowctx.bm_origin = origin;
    }
    lds_barrier();
    const bool     bitsv = rowctx.has_vector_bits();
    // Rows that start on a 16-byte boundary: the flags of a vector never straddle a word of the bitmap.
    const bool     aligned_bits = bitsv && a == 0 && BMW > 0;
    const uint32_t KMIN  = min_valid_key<DT>();
    const float    NEG_INF = -__builtin_inff();
    const float    mul   = rowctx.fast_mul;
    // a multiplier that is not positive and finite does not keep the order: every vector is evaluated exactly
    const bool all_hit = !(mul > 0.0f && mul < __builtin_inff());

    uint32_t thr   = KMIN;   // candidates are the elements with key >= thr
    bool     valid = false;  // at least k elements of this workgroup's columns have key >= thr
    float    thr_f = key_to_float(thr);
    float    thr_hot;
    auto     set_threshold = [&](uint32_t key) {
        thr        = key;
        thr_f      = key_to_float(key);
        // What the unrounded, unpenalised product of an element must reach for its final value to reach thr_f:
        // rounding to T can lift a product by half a unit of T, and a history penalty that raises values
        // (a multiplicative one below 1, a negative additive one) can lift it further.
        float h = lean_below_rounding<DT>(thr_f);
        if (has_bias) {
            h = lean_below_rounding<DT>(h);  // stored + bias is rounded to T as well
        }
        if (bitsv) {
            const float pen = rowctx.penalty;
            float       g   = h;
            bool        raises;
            if (rowctx.penalty_type == 0) {
                raises = !(pen >= 0.0f);
                g      = h + pen;
            }
            else {
                raises = !(pen >= 1.0f);
                g      = (pen > 0.0f && pen < 1.0f) ? (h > 0.0f ? h * pen : h / pen) : NEG_INF;
            }
            if (raises) {
                g = g - (__builtin_fabsf(g) * 9.5367431640625e-07f + 1.0e-37f);
                g = lean_below_rounding<DT>(g);
                h = __builtin_fminf(h, g);
            }
        }
        if (!(h == h) || !(__builtin_fabsf(thr_f) < __builtin_inff())) {
            h = NEG_INF;
        }
        thr_hot = uniform_f(h);
    };
    set_threshold(KMIN);

    // flags of the vector that starts at column `first`: one bit per column of the history
    auto vector_flags = [&](int first) -> uint32_t {
        if (aligned_bits) {
            const int brel = max(first - rowctx.bm_origin, 0);
            return (rowctx.bm_word(brel >> 5) >> (brel & 31)) & ((1u << EPV) - 1u);
        }
        return bitsv ? rowctx.vector_bits(first, EPV) : 0u;
    };

    if constexpr (MODE == LG_MODE_SLOTS) {
        // ---- maxima only. Vectors whose elements all take the plain transform count (no history column, not
        // the masked end id): the transform keeps the order, so the maximum of the stored values gives the
        // largest final value of the group.
        float sm[LG_NV];
#pragma unroll
        for (int j = 0; j < LG_NV; ++j) {
            sm[j] = NEG_INF;
        }
        for (int q0 = 0; q0 < nsub; q0 += R) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
                const int q = q0 + r;
                if (q < nsub) {
#pragma unroll
                    for (int j = 0; j < LG_NV; ++j) {
                        const int  rel   = q * LG_SUB_VECS + j * LG_THREADS + t;
                        const int  first = (vb + rel) * EPV - a;
                        const bool clean = rel < nvec && rowctx.interior_vector(first, EPV) && vector_flags(first) == 0u;
                        float      vm    = NEG_INF;
                        if (has_bias) {
#pragma unroll
                            for (int e = 0; e < EPV; ++e) {
                                vm = __builtin_fmaxf(vm, biased_element(raw[r][j], rawb[BIAS ? r : 0][j], e));
                            }
                        }
                        else {
                            vm = lean_raw_max<DT>(raw[r][j]);
                        }
                        sm[j] = __builtin_fmaxf(sm[j], clean ? vm : NEG_INF);
                    }
                    if (q + R < nsub) {
                        load(r, q + R);
                    }
                }
            }
        }
        uint32_t key[LG_NV];
#pragma unroll
        for (int j = 0; j < LG_NV; ++j) {
            key[j] = all_hit ? 0u : order_key(rowctx.fast(sm[j]));
        }
        uint32_t* dst = l.slots + ((size_t)row * gridDim.x + chunk) * l.slot_u * LG_THREADS + t;
        if (l.slot_u == 4) {
#pragma unroll
            for (int j = 0; j < LG_NV; ++j) {
                dst[j * LG_THREADS] = key[j];
            }
        }
        else if (l.slot_u == 2) {
            dst[0]          = max(key[0], key[1]);
            dst[LG_THREADS] = max(key[2], key[3]);
        }
        else {
            dst[0] = max(max(key[0], key[1]), max(key[2], key[3]));
        }
        return;
    }

    if constexpr (MODE == LG_MODE_PRESET) {
        // ---- the bound of the row: the largest P, to within its low sixteen bits, that at least k of the
        // row's maxima reach. Every workgroup of the row finds the same one.
        uint32_t P  = 0u;
        int      pp = 0;
#pragma unroll 1
        for (int bit = 31; bit >= 16; --bit) {
            const uint32_t cand = P | (1u << bit);
            int            c    = 0;
#pragma unroll
            for (int i = 0; i < LG_SLOT_KEYS_MAX; ++i) {
                if (i < n_slot_keys) {
                    c += slot_keys[i] >= cand ? 1 : 0;
                }
            }
            c = wave_sum_i(c);
            if (lane == 0) {
                s.slot_key[pp][wv] = (uint32_t)c;
            }
            lds_barrier();
            int total = 0;
#pragma unroll
            for (int g = 0; g < LG_WAVES; ++g) {
                total += (int)s.slot_key[pp][g];
            }
            pp ^= 1;
            P = total >= k ? cand : P;
        }
        if (P >= KMIN) {
            set_threshold(P);
            valid = true;
        }
    }

    // ---- first bound: the k-th largest of the thread maxima over the first two sub-tiles. Only vectors whose
    // elements all take the plain transform count (no history column, not the masked end id), so every
    // maximum is the final value of an element.
    if (MODE == LG_MODE_STREAM && nsub > 0) {
        float tmax = NEG_INF;
#pragma unroll
        for (int sb = 0; sb < 2; ++sb) {
            if (sb < nsub) {
#pragma unroll
                for (int j = 0; j < LG_NV; ++j) {
                    const int  rel   = sb * LG_SUB_VECS + j * LG_THREADS + t;
                    const int  first = (vb + rel) * EPV - a;
                    const bool clean = rel < nvec && rowctx.interior_vector(first, EPV) && vector_flags(first) == 0u;
                    float vm = NEG_INF;
#pragma unroll
                    for (int e = 0; e < EPV; ++e) {
                        vm = __builtin_fmaxf(vm, rowctx.fast(biased_element(raw[sb][j], rawb[BIAS ? sb : 0][j], e)));
                    }
                    tmax = __builtin_fmaxf(tmax, clean ? vm : NEG_INF);
                }
            }
        }
        s.slot_key[0][t] = order_key(tmax);
        lds_barrier();
        const uint32_t P = lean_kth_of_slots(s.slot_key[0], k);
        if (P >= KMIN) {
            set_threshold(P);
            valid = true;
        }
    }
    int par = 1;  // which half of slot_key the next bound uses

    // ---- parking and exact evaluation
    TopkEntry* out    = l.entries + (size_t)row * l.row_entries + (size_t)chunk * TK_CCAP;
    int        wcount = 0;   // vectors parked by this wave (wave-uniform)
    int        rot    = 0;   // spreads the evaluated vectors over the lanes from one evaluation to the next
    uint32_t   dmax   = 0u;  // largest key this lane has put on the list
    // Evaluate what the wave has parked: one vector per lane and round. The elements that reach the bound get
    // their slots on the workgroup's list with one LDS atomic per round (prefix sums of the per-lane counts,
    // which are at most EPV, from one ballot per bit of the count).
    auto drain = [&]() {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront", "local");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront", "local");
        const int staged = wcount;
        for (int e0 = 0; e0 < staged; e0 += WAVE) {
            const int  e    = e0 + ((lane - rot) & (WAVE - 1));
            const bool have = e < staged;
            float      x[EPV];
            uint32_t   mask  = 0u;
            int        first = 0;
            if (have) {
                const uint4 v = s.stage_raw[wv][e];
                first         = s.stage_first[wv][e];
                const uint4 bias_vec = has_bias ? bias_base[first / EPV] : v;  // (first is a multiple of EPV with a bias)
                uint32_t bits = 0u;
                if (aligned_bits) {
                    const int rel = first - rowctx.bm_origin;
                    bits          = (rowctx.bm_word(rel >> 5) >> (rel & 31)) & ((1u << EPV) - 1u);
                }
                else if (bitsv) {
                    bits = rowctx.vector_bits(first, EPV);
                }
#pragma unroll
                for (int c = 0; c < EPV; ++c) {
                    x[c] = rowctx.fast(biased_element(v, bias_vec, c));
                }
                if (bits != 0u) {  // rare: a column of the history
#pragma unroll
                    for (int c = 0; c < EPV; ++c) {
                        if ((bits >> c) & 1u) {
                            x[c] = rowctx.flagged(x[c], first + c);
                        }
                    }
                }
#pragma unroll
                for (int c = 0; c < EPV; ++c) {
                    mask |= x[c] >= thr_f ? (1u << c) : 0u;
                }
                const uint32_t rel_end = (uint32_t)(rowctx.masked_end_id - first);  // the masked end id is no candidate
                mask &= rel_end < (uint32_t)EPV ? ~(1u << rel_end) : ~0u;
            }
            const int cnt = __builtin_popcount(mask);
            int       pre = 0, total = 0;
#pragma unroll
            for (int bit = 0; (1 << bit) <= EPV; ++bit) {
                const unsigned long long bm = __ballot((cnt >> bit) & 1);
                pre += (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(bm >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)bm, 0u))
                       << bit;
                total += (int)__builtin_popcountll(bm) << bit;
            }
            if (total > 0) {
                int base_slot = 0;
                if (lane == 0) {
                    base_slot = atomicAdd(&s.n_out, total);
                }
                int slot = __builtin_amdgcn_readfirstlane(base_slot) + pre;
#pragma unroll
                for (int c = 0; c < EPV; ++c) {
                    if ((mask >> c) & 1u) {
                        const uint32_t key = order_key(x[c]);
                        if (slot < TK_CCAP) {
                            out[slot] = TopkEntry{key, (uint32_t)(first + c + p.col_offset)};
                        }
                        dmax = key > dmax ? key : dmax;
                        ++slot;
                    }
                }
            }
        }
        rot    = (rot + staged) & (WAVE - 1);
        wcount = 0;
    };
    // The parking list holds what is left from before a sub-tile (fewer than LG_DRAIN_AT vectors) plus every
    // vector of a sub-tile: it cannot overflow.
    static_assert(LG_STAGE >= LG_DRAIN_AT - 1 + LG_NV * WAVE, "a sub-tile always fits the parking list");
    auto park = [&](bool hit, const uint4& v, int first) {
        const unsigned long long m = __ballot(hit);
        if (m != 0ull) {
            if (hit) {
                const int slot = wcount
                                 + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                                                  __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                s.stage_raw[wv][slot]   = v;
                s.stage_first[wv][slot] = first;
            }
            wcount += (int)__builtin_popcountll(m);
        }
    };

    // ---- the stream. The bound is raised again after 4, 8, 16, ... sub-tiles: the k-th largest of the lanes'
    // largest candidates bounds the k-th largest of everything seen so far.
    int next_tighten = 4;
    for (int q0 = 0; q0 < nsub; q0 += R) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int q = q0 + r;
            if (q < nsub) {
#pragma unroll
                for (int j = 0; j < LG_NV; ++j) {
                    const int   rel = q * LG_SUB_VECS + j * LG_THREADS + t;
                    const float m   = vector_max(raw[r][j], rawb[BIAS ? r : 0][j]) * mul;
                    park((all_hit || m >= thr_hot) && rel < nvec, raw[r][j], (vb + rel) * EPV - a);
                }
                if (q + R < nsub) {
                    load(r, q + R);
                }
                const bool tighten = MODE == LG_MODE_STREAM && q + 1 == next_tighten && q + 1 < nsub;
                if (wcount >= LG_DRAIN_AT || tighten || q + 1 == nsub) {
                    drain();
                }
                if (tighten) {
                    next_tighten *= 2;
                    s.slot_key[par][t] = dmax;
                    lds_barrier();
                    const uint32_t P = lean_kth_of_slots(s.slot_key[par], k);
                    par ^= 1;
                    if (P > thr) {
                        set_threshold(P);
                        valid = true;
                    }
                }
            }
        }
    }

    // ---- the columns outside whole vectors, one by one
    auto edge = [&](int v0, int v1) {
        for (int v = v0 + t; v < v1; v += LG_THREADS) {
            if (!rowctx.never_selected(v)) {
                const float xv = topk_value_at<DT>(rowctx, v);
                if (xv >= thr_f) {
                    const int slot = atomicAdd(&s.n_out, 1);
                    if (slot < TK_CCAP) {
                        out[slot] = TopkEntry{order_key(xv), (uint32_t)(v + p.col_offset)};
                    }
                }
            }
        }
    };
    if (first_wg) {
        edge(0, min(p.V, vfull_lo * EPV - a));
    }
    if (last_wg) {
        edge(max(vfull_hi * EPV - a, first_wg ? min(p.V, vfull_lo * EPV - a) : 0), p.V);
    }
    lds_barrier();
    if (t == 0) {
        const int       n = s.n_out;
        TopkChunkHeader h;
        h.count     = n > TK_CCAP ? 0u : (uint32_t)n;
        h.threshold = thr;
        h.flags     = n > TK_CCAP ? 2u : (valid ? 1u : 0u);
        h.share     = 0u;
        l.headers[(size_t)row * l.splits + chunk] = h;
    }
    if constexpr (ROWSEL) {
        __syncthreads();  // list and header are written; the gather's view of the shared memory is dead
        const TopkEntry*       row_entries = l.entries + (size_t)row * l.row_entries;
        const LeanListPrefetch pf          = lean_prefetch_lists(l.splits, row_entries);
        lean_select_row<DT>(sh.topk, p, l, row, k, tp, pf);
    }
}

// -------------------------------------------------------------------------------------------
// merge + select for the lists of the lean gather
// -------------------------------------------------------------------------------------------
// The union of a row's lists at or above the row's bound -> s.cand, cut to the k largest keys (and ties).
// Returns the count, or -1 when a workgroup of the gather gave up on its list.
// `my_header`: header of list t, loaded by thread t < splits (requested with the prefetch). `draw_bits`: the
// row's uniform draw, held by thread 0; it is handed to every thread through the barrier that publishes the
// headers.
template<int DT>
__device__ __forceinline__ int lean_merge_lists(TopkShared& s, int k, int splits, const TopkChunkHeader& my_header,
                                                const TopkEntry* entries, uint32_t* thr_out,
                                                const LeanListPrefetch& pf, int* draw_bits)
{
    const int t = threadIdx.x;
    // headers through LDS: one load per list, every thread then looks at all of them
    TopkChunkHeader* hdr = reinterpret_cast<TopkChunkHeader*>(&s.stage.raw[0][0]);
    static_assert(sizeof(s.stage.raw) >= TK_MAXSPLIT * sizeof(TopkChunkHeader) + TK_THREADS * sizeof(uint32_t),
                  "headers and 256 slot maxima fit the staging area");
    if (t < splits) {
        hdr[t] = my_header;
    }
    if (t == 0) {
        s.n_cand  = 0;
        s.misc[0] = *draw_bits;
    }
    __syncthreads();
    *draw_bits = s.misc[0];
    uint32_t T0       = min_valid_key<DT>();
    bool     overflow = false;
    int      total    = 0;
    for (int c = 0; c < splits; ++c) {
        const TopkChunkHeader h = hdr[c];
        overflow                = overflow || (h.flags & 2u) != 0u;
        total += (int)h.count;
        if ((h.flags & 1u) && h.threshold > T0) {
            T0 = h.threshold;
        }
    }
    if (overflow) {
        return -1;
    }
    if (total > TK_CCAP && k <= LG_MAX_K) {
        // Many lists that each hold the best of their own columns: together they may not fit the list in LDS.
        // Raise the bound first: every thread takes the largest key among the entries it is about to look at
        // (they are entries of its own), and at least k of these 256 maxima reach the k-th largest of them.
        uint32_t mx = 0u;
#pragma unroll
        for (int m = 0; m < LS_PF_LISTS; ++m) {
            const int c   = wave_id() + m * TK_WAVES;
            const int cnt = c < splits ? (int)hdr[c].count : 0;
#pragma unroll
            for (int r = 0; r < LS_PF_ROUNDS; ++r) {
                const uint32_t key = r * WAVE + lane_id() < cnt ? pf.e[m][r].key : 0u;
                mx                 = key > mx ? key : mx;
            }
        }
        for (int c = wave_id(); c < splits; c += TK_WAVES) {
            const int        cnt   = (int)hdr[c].count;
            const TopkEntry* e     = entries + (size_t)c * TK_CCAP;
            const int        begin = c < LS_PF_LISTS * TK_WAVES ? LS_PF_ROUNDS * WAVE : 0;
            for (int i = begin + lane_id(); i < cnt; i += WAVE) {
                const uint32_t key = e[i].key;
                mx                 = key > mx ? key : mx;
            }
        }
        uint32_t* slot_key = reinterpret_cast<uint32_t*>(&s.stage.raw[0][0]) + 4 * TK_MAXSPLIT;  // behind the headers
        slot_key[t]        = mx;
        lds_barrier();
        const uint32_t P = lean_kth_of_slots(slot_key, k);
        if (P > T0) {
            T0 = P;
        }
    }
    // what was requested up front: one slot reservation per wave
    unsigned long long keepm[LS_PF_LISTS][LS_PF_ROUNDS];
    int                wave_total = 0;
#pragma unroll
    for (int m = 0; m < LS_PF_LISTS; ++m) {
        const int c   = wave_id() + m * TK_WAVES;
        const int cnt = c < splits ? (int)hdr[c].count : 0;
#pragma unroll
        for (int r = 0; r < LS_PF_ROUNDS; ++r) {
            keepm[m][r] = __ballot(r * WAVE + lane_id() < cnt && pf.e[m][r].key >= T0);
            wave_total += (int)__builtin_popcountll(keepm[m][r]);
        }
    }
    int wave_base = 0;
    if (lane_id() == 0 && wave_total > 0) {
        wave_base = atomicAdd(&s.n_cand, wave_total);
    }
    wave_base = __builtin_amdgcn_readfirstlane(wave_base);
#pragma unroll
    for (int m = 0; m < LS_PF_LISTS; ++m) {
#pragma unroll
        for (int r = 0; r < LS_PF_ROUNDS; ++r) {
            const unsigned long long mk = keepm[m][r];
            if ((mk >> lane_id()) & 1ull) {
                const int slot = wave_base
                                 + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mk >> 32),
                                                                  __builtin_amdgcn_mbcnt_lo((uint32_t)mk, 0u));
                if (slot < TK_CCAP) {
                    s.cand.key[slot] = pf.e[m][r].key;
                    s.cand.idx[slot] = pf.e[m][r].idx;
                }
            }
            wave_base += (int)__builtin_popcountll(mk);
        }
    }
    // the rest: lists beyond the eighth, entries beyond the first 256 of a list; four rounds of loads in flight
    for (int c = wave_id(); c < splits; c += TK_WAVES) {
        const int        cnt   = (int)hdr[c].count;
        const TopkEntry* e     = entries + (size_t)c * TK_CCAP;
        const int        begin = c < LS_PF_LISTS * TK_WAVES ? LS_PF_ROUNDS * WAVE : 0;
        for (int i0 = begin; i0 < cnt; i0 += 4 * WAVE) {
            TopkEntry en[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = i0 + r * WAVE + lane_id();
                en[r]       = e[min(i, TK_CCAP - 1)];
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int                i    = i0 + r * WAVE + lane_id();
                const bool               keep = i < cnt && en[r].key >= T0;
                const unsigned long long mk   = __ballot(keep);
                int                      base = 0;
                if (lane_id() == 0 && mk != 0ull) {
                    base = atomicAdd(&s.n_cand, (int)__builtin_popcountll(mk));
                }
                base = __builtin_amdgcn_readfirstlane(base);
                if (keep) {
                    const int slot = base
                                     + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(mk >> 32),
                                                                      __builtin_amdgcn_mbcnt_lo((uint32_t)mk, 0u));
                    if (slot < TK_CCAP) {
                        s.cand.key[slot] = en[r].key;
                        s.cand.idx[slot] = en[r].idx;
                    }
                }
            }
        }
    }
    __syncthreads();
    int n = s.n_cand;
    __syncthreads();
    (void)total;
    if (n > TK_CCAP) {
        return -2;  // the union does not fit the list: the caller merges with the general routine
    }
    if (n > k + k / 2 && n <= 4 * TK_THREADS && k <= LG_MAX_K && k <= TK_THREADS) {
        // Far more candidates than needed (every workgroup of the gather reports the best of its own columns):
        // raise the bound to the k-th largest of 256 slot maxima (slot t: entries t, t + 256, ...), which at
        // least k entries reach, and keep what reaches it. The replay of the tie orders below ranks every
        // candidate against every other one; this keeps it short.
        uint32_t mx = 0u;
        for (int i = t; i < n; i += TK_THREADS) {
            const uint32_t key = s.cand.key[i];
            mx                 = key > mx ? key : mx;
        }
        uint32_t* slot_key = reinterpret_cast<uint32_t*>(&s.stage.raw[0][0]);
        slot_key[t]        = mx;
        lds_barrier();
        const uint32_t P = lean_kth_of_slots(slot_key, k);
        lds_barrier();
        if (P > T0) {
            T0 = P;
            n  = topk_prune(s, n, P);
        }
    }
    *thr_out = T0;
    return n;
}

// Merge the lists of a row, replay the tie orders, sample, write the row's outputs. Every thread of the workgroup
// calls it, for a row that takes part; `k`, `tp`: the row's top-k and top-p; `pf`: lean_prefetch_lists of the row.
template<int DT>
__device__ __forceinline__ void lean_select_row(TopkShared& s, const FusedParams& p, const FusedLaunch& l, int row, int k,
                                                float tp, const LeanListPrefetch& pf)
{
    constexpr int          BMW         = 0;  // the recovery paths read whole-row bitmaps from global memory
    TopkEntry*             row_entries = l.entries + (size_t)row * l.row_entries;
    const TopkChunkHeader* headers     = l.headers + (size_t)row * l.splits;
    TopkChunkHeader        my_header{};
    if ((int)threadIdx.x < l.splits) {
        my_header = headers[threadIdx.x];
    }
    int draw_bits = 0;
    if (threadIdx.x == 0) {
        draw_bits = __float_as_int(row_uniform(l.rng, l.uniforms, row));
    }
    FusedRow<DT, BMW> r(p, row);
    const TopkOutputs out = topk_outputs(l.ids, l.sequence_length, l.finished, nullptr, nullptr, row, p.end_ids);
    uint32_t          thr = 0u;
    int               n   = lean_merge_lists<DT>(s, k, l.splits, my_header, row_entries, &thr, pf, &draw_bits);
    const float       u   = __int_as_float(draw_bits);
    if (n == -2) {
        const TopkListPrefetch none{};
        n = topk_merge_lists<DT>(s, k, l.splits, headers, row_entries, &thr, none, false);
    }
    if (n < 0) {
        // A workgroup of the gather could not hold its candidates. Walk the whole row again, here, with the
        // stream that recovers from overfull tiles; only rows it cannot bound either take the literal replay.
        if (p.logits == nullptr) {
            // (lists merged from vocabulary shards without the rows at hand: the row is reported as not sampled)
            if (threadIdx.x == 0) {
                l.ids[row] = -1;
            }
            return;
        }
        r.prepare_whole_row();
        __syncthreads();
        n = topk_stream<DT, FusedRow<DT, BMW>, 0>(r, s, p.Vp, k, 0, topk_row_tiles<DT>(r.rowp, p.Vp), &thr);
    }
    topk_select_lds<DT, FusedRow<DT, BMW>, true>(r, s, n, thr, row, p.Vp, k, tp, p.max_top_k, row_entries, false, u,
                                                 p.end_ids, out);
}

template<int DT>
__global__ void __launch_bounds__(TK_THREADS) lean_select_kernel(FusedParams p, FusedLaunch l)
{
    __shared__ TopkShared s;
    const int             row = blockIdx.x;
    // everything the row needs is requested before the first decision: the lists (vector loads), the
    // arguments (scalar loads)
    const LeanListPrefetch pf   = lean_prefetch_lists(l.splits, l.entries + (size_t)row * l.row_entries);
    const bool             skip = row_flag_or(p.skip_decode, row, p.end_ids + row, false);
    const bool             fin  = row_flag_or(l.finished, row, p.end_ids + row, false);
    const int              k    = row_arg_or(p.top_ks, row, p.end_ids + row, p.max_top_k);
    const float            tp   = row_arg_or(p.top_ps, row, p.end_ids + row, 1.0f);
    if (skip) {
        return;
    }
    if (fin) {
        if (threadIdx.x == 0) {
            l.ids[row] = p.end_ids[row];
        }
        return;
    }
    lean_select_row<DT>(s, p, l, row, k, tp, pf);
}

// Launchers, one translation unit per element type (lean_kernels.hip built with FTK_LEAN_DT = 0, 1, 2).
// mode: LG_MODE_*; row_select: one workgroup per row that also orders and samples (LG_MODE_STREAM without a
// bias only); window: 0 = history bitmaps in global memory, 1 = small LDS window, 2 = large.
// start / stop: optional events carried by the launch.
int lean_gather_launch_f32(int mode, bool row_select, int window, dim3 grid, hipStream_t st, const FusedParams& p,
                           const FusedLaunch& l, hipEvent_t start, hipEvent_t stop);
int lean_select_launch_f32(int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start,
                           hipEvent_t stop);
int lean_select_launch_f16(int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start,
                           hipEvent_t stop);
int lean_select_launch_bf16(int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start,
                            hipEvent_t stop);
int lean_gather_launch_f16(int mode, bool row_select, int window, dim3 grid, hipStream_t st, const FusedParams& p,
                           const FusedLaunch& l, hipEvent_t start, hipEvent_t stop);
int lean_gather_launch_bf16(int mode, bool row_select, int window, dim3 grid, hipStream_t st, const FusedParams& p,
                            const FusedLaunch& l, hipEvent_t start, hipEvent_t stop);

// workgroups per compute unit the lean gather is built for, and sub-tiles in flight per thread
constexpr int LG_OCCUPANCY = 4;
constexpr int LG_RING      = 2;

}  // namespace ftk
