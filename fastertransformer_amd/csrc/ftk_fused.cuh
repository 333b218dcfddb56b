// Types shared by the kernels of the fused decode step (fused_kernels.hip, lean_kernels.hip): the launch
// arguments and the row accessor that applies the penalty and mask arithmetic of
// src/fastertransformer/layers/sampling_layers/BaseSamplingLayer.cc:302-352 to a column on the fly.
#pragma once
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
    // A launch over a vocabulary shard (a producer hands over columns [col_offset, col_offset + V) of every row:
    // `logits` points at the shard's first column, Vp is the pitch of its rows): token ids in the history and the
    // end ids are global, and so are the column numbers the launch reports. 0 for whole rows.
    int          col_offset;
    // Frequency penalty (an extension of the additive rule): a column that occurs `count` times in the row's history
    // gets x - penalty - frequency * count. Null: none. Only the kernels that keep a table of the counts in LDS take it.
    const float* frequencies;
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
// One flag of a bool array at an index that is the same for the whole workgroup, read through the aligned
// 32-bit word that holds it: a scalar load, which does not queue behind the vector loads in flight (a byte
// load would, and its consumer would wait for all of them).
__device__ __forceinline__ bool uniform_flag(const bool* flags, int index)
{
    const bool*    flag = flags + index;
    const uint32_t mis  = (uint32_t)(reinterpret_cast<uintptr_t>(flag) & 3u);
    const uint32_t word = *reinterpret_cast<const uint32_t*>(flag - mis);  // stays inside the flag's own word
    return ((word >> (8u * mis)) & 0xFFu) != 0u;
}

// Per-row arguments are optional arrays. Reading them behind their null checks makes a chain of loads that
// each wait for the one before; these helpers always load - from the array when it exists, from `safe` (any
// valid 4-byte aligned address, the row's end id) when it does not - so that all of a row's arguments are
// requested together and cost one trip to memory.
template<typename V>
__device__ __forceinline__ V row_arg_or(const V* array, int row, const void* safe, V otherwise)
{
    static_assert(sizeof(V) == 4, "32-bit arguments");
    const V* from = array != nullptr ? array + row : reinterpret_cast<const V*>(safe);
    const V  v    = *from;
    return array != nullptr ? v : otherwise;
}
__device__ __forceinline__ bool row_flag_or(const bool* flags, int row, const void* safe, bool otherwise)
{
    const bool* from = flags != nullptr ? flags + row : reinterpret_cast<const bool*>(safe);
    const bool  v    = uniform_flag(from, 0);
    return flags != nullptr ? v : otherwise;
}

__device__ __forceinline__ float uniform_f(float x)
{
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(x)));
}

// A row's per-row arguments, requested in one block without control flow so that they share one trip to memory
// (the arithmetic on them, which waits for the values, comes afterwards).
struct FusedRowArgs {
    float temperature, penalty, frequency;
    int   input_length, min_length, sequence_length, end_id;
};
__device__ __forceinline__ FusedRowArgs fused_row_args(const FusedParams& p, int row)
{
    const void*  safe = p.end_ids + row;
    FusedRowArgs a;
    a.temperature     = row_arg_or(p.temperatures, row, safe, 1.0f);
    a.penalty         = row_arg_or(p.penalties, row, safe, 0.0f);
    a.frequency       = row_arg_or(p.frequencies, row, safe, 0.0f);
    a.input_length    = row_arg_or(p.input_lengths, row, safe, p.max_input_length);
    a.min_length      = row_arg_or(p.min_lengths, row, safe, 0);
    a.sequence_length = row_arg_or(p.min_lengths != nullptr ? p.sequence_length_in : nullptr, row, safe, 0);
    a.end_id          = p.end_ids[row];
    return a;
}

// How often each token id occurs in a row's history: an open-addressing table in LDS, one 32-bit word per distinct
// id, (id + 1) << 13 | count. Ids below 2^18 and at most 4096 history positions (half the slots), which the
// launcher checks.
constexpr int      FUSED_COUNT_SLOTS = 8192;
constexpr int      FUSED_COUNT_BITS  = 13;
constexpr int      FUSED_COUNT_MAX_VOCAB = 1 << 18;
__device__ __forceinline__ uint32_t fused_count_hash(int id)
{
    return ((uint32_t)id * 2654435761u) >> (32 - FUSED_COUNT_BITS);
}
__device__ __forceinline__ void fused_count_insert(uint32_t* table, int id)
{
    const uint32_t tag = (uint32_t)(id + 1) << FUSED_COUNT_BITS;
    uint32_t       h   = fused_count_hash(id);
#pragma unroll 1
    for (int probe = 0; probe < FUSED_COUNT_SLOTS; ++probe) {
        const uint32_t old = atomicCAS(&table[h], 0u, tag | 1u);
        if (old == 0u) {
            return;
        }
        if ((old >> FUSED_COUNT_BITS) == (uint32_t)(id + 1)) {
            atomicAdd(&table[h], 1u);
            return;
        }
        h = (h + 1) & (FUSED_COUNT_SLOTS - 1);
    }
}
__device__ __forceinline__ int fused_count_lookup(const uint32_t* table, int id)
{
    uint32_t h = fused_count_hash(id);
#pragma unroll 1
    for (int probe = 0; probe < FUSED_COUNT_SLOTS; ++probe) {
        const uint32_t e = table[h];
        if (e == 0u) {
            return 0;
        }
        if ((e >> FUSED_COUNT_BITS) == (uint32_t)(id + 1)) {
            return (int)(e & ((1u << FUSED_COUNT_BITS) - 1u));
        }
        h = (h + 1) & (FUSED_COUNT_SLOTS - 1);
    }
    return 0;
}

// What a FusedRow works out from the row's arguments, as ten 32-bit words: one wave can do the arithmetic and hand
// the result to the others of a large workgroup.
struct FusedRowDerived {
    static constexpr int WORDS = 10;
    float inv, fast_mul, penalty, frequency, up_mul_neg, up_mul_pos, up_add;
    int   masked_end_id, input_length;
    int   flags;  // bit 0: keep_pads, bit 1: up_ok
};

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
    int             col_offset;  // global number of column 0 (a vocabulary shard), see FusedParams
    int             team;        // threads that call prepare() / prepare_whole_row() together (the whole workgroup
                                 // unless the caller says otherwise: some of a workgroup's waves may have left)
    float           frequency;   // frequency penalty of the row (with count_table), see FusedParams
    const uint32_t* count_table; // null: no frequency penalty

    __device__ __forceinline__ FusedRow(const FusedParams& p, int row): FusedRow(p, row, fused_row_args(p, row)) {}
    // what does not depend on the row's own arguments
    __device__ __forceinline__ void from_launch(const FusedParams& p, int row)
    {
        rowp             = (const T*)p.logits + (size_t)row * p.Vp;
        bias             = (const T*)p.bias;
        V                = p.V;
        Vp               = p.Vp;
        temp_active      = p.temperatures != nullptr;
        penalty_type     = p.penalties != nullptr ? p.penalty_type : 2;
        global_bm        = (p.bitmaps != nullptr && penalty_type != 2) ? p.bitmaps + (size_t)row * p.bitmap_words : nullptr;
        global_ready     = p.bitmaps_ready != 0;
        bm_mode          = (BMW == 0 && global_bm != nullptr && global_ready) ? 1 : 0;
        bm_origin        = 0;
        history          = p.output_ids != nullptr ? p.output_ids + row : nullptr;
        batch_size       = p.batch_size;
        step             = p.step;
        max_input_length = p.max_input_length;
        col_offset       = p.col_offset;
        team             = (int)blockDim.x;
        count_table      = nullptr;  // (the kernel that keeps the table sets it)
    }
    // from what another wave worked out with the constructor below (and derived())
    __device__ __forceinline__ FusedRow(const FusedParams& p, int row, const FusedRowDerived& d)
    {
        from_launch(p, row);
        inv           = d.inv;
        fast_mul      = d.fast_mul;
        penalty       = d.penalty;
        frequency     = d.frequency;
        up_mul_neg    = d.up_mul_neg;
        up_mul_pos    = d.up_mul_pos;
        up_add        = d.up_add;
        masked_end_id = d.masked_end_id;
        input_length  = d.input_length;
        keep_pads     = (d.flags & 1) != 0;
        up_ok         = (d.flags & 2) != 0;
    }
    __device__ __forceinline__ FusedRowDerived derived() const
    {
        FusedRowDerived d;
        d.inv           = inv;
        d.fast_mul      = fast_mul;
        d.penalty       = penalty;
        d.frequency     = frequency;
        d.up_mul_neg    = up_mul_neg;
        d.up_mul_pos    = up_mul_pos;
        d.up_add        = up_add;
        d.masked_end_id = masked_end_id;
        d.input_length  = input_length;
        d.flags         = (keep_pads ? 1 : 0) | (up_ok ? 2 : 0);
        return d;
    }
    __device__ __forceinline__ FusedRow(const FusedParams& p, int row, const FusedRowArgs& args)
    {
        from_launch(p, row);
        const TemperatureCtx<DT> tc(args.temperature, V, Vp, false);
        inv           = tc.inv;
        fast_mul      = temp_active ? tc.inv : 1.0f;
        keep_pads     = tc.keep_pads;
        penalty       = args.penalty;
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
        input_length  = args.input_length;
        // values that are the same for every lane of the workgroup but come out of floating-point
        // arithmetic: move them to scalar registers, they stay live for the whole kernel
        inv        = uniform_f(inv);
        fast_mul   = uniform_f(fast_mul);
        penalty    = uniform_f(penalty);
        up_mul_neg = uniform_f(up_mul_neg);
        up_mul_pos = uniform_f(up_mul_pos);
        up_add     = uniform_f(up_add);
        frequency     = uniform_f(args.frequency);
        masked_end_id = (p.min_lengths != nullptr
                         && min_length_masks(args.sequence_length, p.max_input_length, args.min_length)
                         && args.end_id >= p.col_offset) ?
                            args.end_id - p.col_offset :  // (beyond the shard: no column of it matches)
                            -1;
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
        for (int i = threadIdx.x; i < words; i += team) {
            window[i] = 0u;
        }
        __syncthreads();
        // the history is time-major: every id is a cache line of its own, so the reads are issued eight
        // deep before the first one is used
        constexpr int U = 8;
        for (int t0 = threadIdx.x; t0 < step; t0 += U * team) {
            int ids[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int t = t0 + u * team;
                ids[u] = (t < step && history_position_counts(t)) ? history[(size_t)t * batch_size] - col_offset : -1;
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
        for (int i = threadIdx.x; i < words; i += team) {
            global_bm[i] = 0u;
        }
        __threadfence_block();
        __syncthreads();
        for (int t = threadIdx.x; t < step; t += team) {
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
        return bias == nullptr && interior_vector(first, n);
    }
    // columns of the vocabulary proper, none of them the masked end id (a bias may still apply)
    __device__ __forceinline__ bool interior_vector(int first, int n) const
    {
        return first + n <= V && !(masked_end_id >= first && masked_end_id < first + n);
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
    // the same column (number v) when it is in the history
    __device__ __forceinline__ float flagged(float xf, int v) const
    {
        if (count_table != nullptr) {
            return round_t<DT>(frequency_value(xf, penalty, frequency, fused_count_lookup(count_table, v + col_offset)));
        }
        return round_t<DT>(repetition_value(xf, penalty, penalty_type));
    }
    // the kernel's table of counts is in place: columns of the history take the frequency rule from here on
    __device__ __forceinline__ void use_count_table(const uint32_t* table)
    {
        count_table = table;
        // (the cheap upper bound of flagged_upper holds while neither term raises a value)
        up_ok = up_ok && penalty >= 0.0f && frequency >= 0.0f;
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
            x = flagged(x, v);
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

struct FusedLaunch {
    int*             ids;
    int*             sequence_length;
    bool*            finished;
    RngState*        rng;
    const float*     uniforms;
    int              splits;
    int              tiles_per_wg;
    int              subs_per_wg;  // lean_gather_kernel: sub-tiles per workgroup
    size_t           row_entries;
    TopkChunkHeader* headers;
    TopkEntry*       entries;
    // two-read selection for a large k (lean_gather_kernel, slots and preset modes): per row and workgroup,
    // 256 * slot_u maxima of disjoint groups of columns
    uint32_t* slots;
    int       slot_u;
};

__device__ __forceinline__ float fused_row_draw(TopkShared& s, const FusedLaunch& l, int row)
{
    if (threadIdx.x == 0) {
        s.misc[0] = __float_as_int(row_uniform(l.rng, l.uniforms, row));
    }
    __syncthreads();
    return __int_as_float(s.misc[0]);
}

// Launchers of the general-stream kernels, one translation unit per element type (fused_dtype_kernels.hip).
// kind: which kernel; window: 0 = history bitmaps in global memory, 1 = small LDS window, 2 = large;
// many: the large-k level of the launch (topk_many_level); start / stop: optional events carried by the launch.
enum { FUSED_KIND_ROW = 0, FUSED_KIND_GATHER = 1, FUSED_KIND_SELECT = 2 };
int fused_launch_f32(int kind, int window, int many, dim3 grid, hipStream_t st, const FusedParams& p,
                     const FusedLaunch& l, hipEvent_t start, hipEvent_t stop);
int fused_launch_f16(int kind, int window, int many, dim3 grid, hipStream_t st, const FusedParams& p,
                     const FusedLaunch& l, hipEvent_t start, hipEvent_t stop);
int fused_launch_bf16(int kind, int window, int many, dim3 grid, hipStream_t st, const FusedParams& p,
                      const FusedLaunch& l, hipEvent_t start, hipEvent_t stop);

}  // namespace ftk
