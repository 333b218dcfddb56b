// The fused decode step in one launch for batches of about one row per compute unit (and for any small launch): a
// 1024-thread workgroup owns a whole row. It streams the row once like the lean gather of ftk_lean.cuh (a ring of
// sub-tiles in registers, parking of the vectors that may hold a candidate, exact evaluation of what was parked), but
//   - the bound is one per row instead of one per share of a row: the k-th largest of 256 maxima over the first
//     sub-tile, raised once more two sub-tiles before the end from the list itself, which is pruned with it (about
//     1.5 k candidates per row instead of 4 x 3 k at k = 64 over 128 Ki columns),
//   - candidates go to a list in LDS, never to memory: no list headers, no second launch, no trip to memory between
//     the read of the row and its selection,
//   - after the row's last column twelve of the sixteen waves leave; the first four (one per SIMD) cut the list to
//     little more than k entries and replay the reference's tie orders (topk_stage1 / topk_stage2_sampling of
//     src/fastertransformer/kernels/sampling_topk_kernels.cu:130-312) by counting, in one pass when all keys differ,
//   - what is the same for the whole row (its arguments and what follows from them, its draw, every bound) is worked
//     out by one wave and handed to the others through LDS: sixteen waves in lock-step pay sixteen issue slots for
//     every instruction.
// Rows the kernel cannot bound (a list that outgrows LDS) are walked again by the first four waves with the general
// stream of ftk_topk.cuh, as the merging kernel of the lean gather does.
#pragma once
#include "ftk_lean.cuh"

namespace ftk {

constexpr int RW_THREADS    = 1024;
constexpr int RW_WAVES      = RW_THREADS / WAVE;
constexpr int RW_NV         = 4;                    // 16-byte vectors per thread and sub-tile
constexpr int RW_SUB_VECS   = RW_THREADS * RW_NV;   // a sub-tile: 64 KB
#ifndef FTK_RW_RING
#define FTK_RW_RING 2
#endif
constexpr int RW_RING       = FTK_RW_RING;          // sub-tiles in flight per thread
constexpr int RW_PARK_GROUP = 2;                    // vectors a wave parks between two looks at its list's fill
constexpr int RW_STAGE      = LG_DRAIN_AT + RW_PARK_GROUP * WAVE;
constexpr int RW_HIST_U     = 4;                    // history ids a thread requests before the logits: the longest
                                                    // history the kernel takes is RW_HIST_U * RW_THREADS positions
#ifndef FTK_RW_T1
#define FTK_RW_T1 6
#endif
#ifndef FTK_RW_GAP
#define FTK_RW_GAP 2
#endif
constexpr int RW_FIRST_TIGHTEN = FTK_RW_T1;
constexpr int RW_TAIL_GAP      = FTK_RW_GAP;
constexpr int RW_MIN_SUBS   = 4;                    // shortest row that a batch of full rounds sends here, in sub-tiles

struct RowwideShared {
    uint32_t count_table[FUSED_COUNT_SLOTS];  // occurrences of the history's ids (rows with a frequency penalty)
    uint4    stage_raw[RW_WAVES][RW_STAGE];
    int      stage_first[RW_WAVES][RW_STAGE];
    uint32_t slot_key[RW_THREADS];
    uint32_t bound;
    float    bound_hot;  // what a raw maximum times the multiplier must reach under that bound
    int      setup[16];  // what the first wave made of the row's arguments, see the kernel
    int      n_list[2];  // length of the row's list; the second counter takes over when the list is pruned
};

// The largest value P, to within its low sixteen bits, such that at least k of 256 keys are >= P (0 when fewer
// than k are non-zero); slot i of the 256 is the largest of keys i, i + 256, i + 512, i + 768 of the workgroup, all
// of them keys of distinct elements. The first wave finds it and what follows from it for the stream (hot_of(P), a
// few dozen instructions that sixteen waves in lock-step would each pay for); every thread gets both. Two barriers.
template<typename HotOf>
__device__ __forceinline__ uint32_t rowwide_bound(RowwideShared& s, uint32_t my_key, int k, HotOf hot_of, float& hot)
{
    s.slot_key[threadIdx.x] = my_key;
    lds_barrier();
    if (wave_id() == 0) {
        uint32_t kk[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int i = lane_id() + g * WAVE;
            kk[g]       = max(max(s.slot_key[i], s.slot_key[i + 256]), max(s.slot_key[i + 512], s.slot_key[i + 768]));
        }
        uint32_t P = 0u;
#pragma unroll
        for (int bit = 31; bit >= 16; --bit) {
            const uint32_t cand = P | (1u << bit);
            int            c    = 0;
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                c += (int)__builtin_popcountll(__ballot(kk[g] >= cand));
            }
            P = c >= k ? cand : P;
        }
        const float h = hot_of(P);
        if (lane_id() == 0) {
            s.bound     = P;
            s.bound_hot = h;
        }
    }
    lds_barrier();
    hot = uniform_f(s.bound_hot);
    return (uint32_t)__builtin_amdgcn_readfirstlane((int)s.bound);
}

// Both tie orders of the reference by counting, for a list of at most 256 candidates, by the first TK_THREADS threads
// of the workgroup (the others have left): the composite keys and the counting of the small case of topk_select_lds.
// Candidates are in s.cand; on return the ordered list is in s.sel (values in w, columns in idx); returns its length.
__device__ __forceinline__ int rowwide_rank(TopkShared& s, int n, int k, int max_top_k)
{
    const int t       = threadIdx.x;
    const int bs1_log = max_top_k <= 16 ? 7 : 8;
    const int BS1     = 1 << bs1_log;
    const int BS2     = max_top_k <= 32 ? 128 : 256;
    constexpr int CAP = 256;
    const uint32_t      my_key = t < n ? s.cand.key[t] : 0u;
    const uint32_t      my_idx = t < n ? s.cand.idx[t] : 0u;
    unsigned long long* A      = s.keys;                                    // stage-1 keys  [0, 256)
    unsigned long long* B      = s.keys + CAP;                              // stage-2 keys  [256, 512)
    int*                cnt    = reinterpret_cast<int*>(s.keys + 2 * CAP);  // 3 x 256 counts
    const int           n2     = (n + 1) & ~1;
    int                 CP     = 2;
    while (CP < n) {
        CP <<= 1;
    }
    const int parts = TK_THREADS / CP;  // CP <= 256
    const int c     = t & (CP - 1);
    const int part  = t / CP;
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
    cnt[t]           = 0;
    cnt[CAP + t]     = 0;
    cnt[2 * CAP + t] = 0;
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
            atomicAdd(&cnt[CAP + c], qs);
        }
    }
    lds_barrier();
    unsigned long long k2 = ~0ull;
    if (t < n) {
        const int slice = (int)(mine >> 61);
        const int r     = cnt[t] - cnt[CAP + t];  // rank inside the slice
        if (r < k) {
            const int pos = slice * k + r;
            k2 = ((unsigned long long)(uint32_t)(mine >> 29) << 32) | ((unsigned long long)(BS2 - 1 - pos % BS2) << 24)
                 | ((unsigned long long)(pos / BS2) << 12);
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
            atomicAdd(&cnt[2 * CAP + c], q);
        }
        if (c == 0 && jhi > jlo) {
            atomicAdd(&s.misc[1], kept);  // entries that stage 1 kept, over all parts
        }
    }
    lds_barrier();
    const int n_list = min(k, s.misc[1]);
    if (t < n && k2 != ~0ull) {
        const int q2 = cnt[2 * CAP + t];
        if (q2 < n_list) {
            s.sel.w[q2]   = key_to_float(~(uint32_t)(k2 >> 32));
            s.sel.idx[q2] = (int)my_idx;
        }
    }
    lds_barrier();
    return n_list;
}

// The usual case of rowwide_rank in one counting pass over 32-bit keys: when the candidates' keys are all different
// and no stage-1 slice holds more than k of them, stage 1 drops none of them and both tie rules are idle, so the
// reference's list is the candidates in descending order of value, cut at k. Returns the length of the list (in
// s.sel, like rowwide_rank), or -1 when one of the two conditions fails (s.cand is left as it was). Called by the
// first TK_THREADS threads; n <= 256.
__device__ __forceinline__ int rowwide_rank_distinct(TopkShared& s, int n, int k, int max_top_k)
{
    const int      t       = threadIdx.x;
    const int      bs1_log = max_top_k <= 16 ? 7 : 8;
    const uint32_t my_key  = t < n ? s.cand.key[t] : 0u;
    const uint32_t my_idx  = t < n ? s.cand.idx[t] : 0u;
    int*           cnt     = s.sel.idx + 1024;  // 256 counts and 256 marks, clear of the list this function writes
    int            CP      = 4;
    while (CP < n) {
        CP <<= 1;
    }
    const int parts = TK_THREADS / CP;
    const int c     = t & (CP - 1);
    const int part  = t / CP;
    const int quads = (n + 3) >> 2;
    const int per   = (quads + parts - 1) / parts;
    const int jlo   = min(quads, part * per) * 4;
    const int jhi   = min(quads, part * per + per) * 4;
    if (t < 4) {
        s.cand.key[n + t] = 0u;  // the last four keys read may lie past the list: a key that is above nothing
    }
    if (t < 8) {
        s.slice_count[t] = 0;
    }
    cnt[t]              = 0;
    cnt[TK_THREADS + t] = 0;
    if (t == 0) {
        s.misc[1] = 0;
    }
    lds_barrier();
    if (t < n) {
        atomicAdd(&s.slice_count[(my_idx >> bs1_log) & 7u], 1);
    }
    {
        const uint32_t key   = c < n ? s.cand.key[c] : 0xFFFFFFFFu;
        int            above = 0;
#pragma unroll 2
        for (int j = jlo; j < jhi; j += 4) {
            const uint4 kk = *reinterpret_cast<const uint4*>(&s.cand.key[j]);
            above += (kk.x > key ? 1 : 0) + (kk.y > key ? 1 : 0) + (kk.z > key ? 1 : 0) + (kk.w > key ? 1 : 0);
        }
        if (c < n && jhi > jlo) {
            atomicAdd(&cnt[c], above);
        }
    }
    lds_barrier();
    // Keys that are all different give n different counts: two candidates with the same count have the same key.
    int rank = 0;
    if (t < n) {
        rank = cnt[t];
        if (atomicAdd(&cnt[TK_THREADS + rank], 1) != 0 || s.slice_count[(my_idx >> bs1_log) & 7u] > k) {
            s.misc[1] = 1;
        }
    }
    lds_barrier();
    if (s.misc[1] != 0) {
        return -1;
    }
    const int n_list = min(k, n);
    if (t < n && rank < n_list) {
        s.sel.w[rank]   = key_to_float(my_key);
        s.sel.idx[rank] = (int)my_idx;
    }
    lds_barrier();
    return n_list;
}

// The kernel's arguments as one block, so that code that is rarely reached can read them again from the
// kernel-argument segment instead of keeping some fifty scalar registers alive through the whole kernel for it.
struct RowwideArgs {
    FusedParams p;
    FusedLaunch l;
};
typedef const __attribute__((address_space(4))) void* RowwideArgSegment;

// What is left to the first four waves when a row's list is still longer than 256 entries after the cut (the
// selection of topk_select_lds for long lists) or outgrew LDS (the whole row is walked again with the stream that
// recovers from overfull tiles; rows it cannot bound either take the literal replay). Not inlined, so that the
// kernel's registers are planned for its stream, and it takes the launch arguments and the row's own from memory
// again (passed by reference they would move the kernel's copy from scalar registers to scratch memory; passed by
// value they stay live, and spill, all the way through the kernel).
template<int DT>
__device__ __noinline__ void rowwide_rare(TopkShared& ts, RowwideArgSegment segment, int row, int n, uint32_t thr, int k,
                                          float tp, float u, const uint32_t* count_table)
{
    RowwideArgs a;
    __builtin_memcpy(&a, (const void*)segment, sizeof(a));
    const FusedParams& p    = a.p;
    const FusedLaunch& l    = a.l;
    const FusedRowArgs args = fused_row_args(p, row);
    TopkOutputs        out;
    out.ids                = l.ids;
    out.sequence_length    = l.sequence_length;
    out.finished           = l.finished;
    out.cum_log_probs      = nullptr;
    out.output_log_probs   = nullptr;
    out.sequence_length_in = l.sequence_length != nullptr ? l.sequence_length[row] : 0;  // (not written yet)
    out.cum_log_prob_in    = 0.0f;
    out.end_id_in          = args.end_id;
    TopkEntry*      row_entries = l.entries + (size_t)row * l.row_entries;
    FusedRow<DT, 0> r0(p, row, args);
    r0.team = TK_THREADS;  // (the other waves of the workgroup have left)
    if (count_table != nullptr) {
        r0.use_count_table(count_table);
    }
    if (n > TK_CCAP) {
        r0.prepare_whole_row();
        __syncthreads();
        n = topk_stream<DT, FusedRow<DT, 0>, 0>(r0, ts, p.Vp, k, 0, topk_row_tiles<DT>(r0.rowp, p.Vp), &thr);
    }
    topk_select_lds<DT, FusedRow<DT, 0>, true>(r0, ts, n, thr, row, p.Vp, k, tp, p.max_top_k, row_entries, false, u,
                                               p.end_ids, out);
}

// Requirements the launcher checks: rows start on 16-byte boundaries (so a vector never straddles a word of the
// history bitmap and there are no columns in front of the first vector), no embedding bias, the largest k at most
// LG_MAX_K, at least one whole vector per row, the row's history bitmap fits BMW words, and a history of at most
// RW_HIST_U * RW_THREADS positions.
// Keeps a launch argument in a scalar register of its own from here on. Without it the compiler, short of scalar
// registers, reads arguments again from the kernel-argument segment wherever they are used, and every such read
// issued after the bulk of the row has been requested queues behind it.
template<typename V>
__device__ __forceinline__ void rowwide_pin(V& v)
{
    asm("" : "+s"(v));  // (not volatile: a volatile statement counts as a store to any address, and loads behind
                        // such a store are no longer scalar loads)
}

template<int DT, int BMW>
__global__ void __launch_bounds__(RW_THREADS) rowwide_step_kernel(const RowwideArgs a_in)
{
    const FusedLaunch& l_in = a_in.l;
    FusedParams        p    = a_in.p;
    FusedLaunch        l    = a_in.l;
    rowwide_pin(p.V);
    rowwide_pin(p.Vp);
    rowwide_pin(p.step);
    rowwide_pin(p.max_input_length);
    rowwide_pin(p.max_top_k);
    rowwide_pin(p.penalty_type);
    rowwide_pin(p.col_offset);
    // (pointers that are only stored through, at the end: a pinned pointer is a generic one to the compiler)
    rowwide_pin(l.ids);
    rowwide_pin(l.sequence_length);
    rowwide_pin(l.finished);
    typedef Storage<DT>   S;
    typedef typename S::T T;
    constexpr int         EPV = (int)(16 / sizeof(T));
    constexpr int         R   = RW_RING;
    static_assert(BMW > 0, "the history bitmap of the whole row lives in LDS");
    __shared__ RowwideShared s;
    __shared__ TopkShared    ts;
    const int                t    = threadIdx.x;
    const int                row  = blockIdx.x;
    const int                lane = lane_id();
    const int                wv   = wave_id();
#ifdef FTK_RW_STAMPS
    unsigned long long* stamps = reinterpret_cast<unsigned long long*>(l.entries + (size_t)blockIdx.x * l.row_entries);
#define RW_STAMP(i) if (threadIdx.x == 0) { stamps[i] = wall_clock64(); }
#else
#define RW_STAMP(i)
#endif

    // the row's address, pinned as a number and used as a pointer to global memory
    typedef unsigned int                                  u4 __attribute__((ext_vector_type(4)));
    typedef const __attribute__((address_space(1))) u4*   GlobalVec;
    unsigned long long base_addr = (unsigned long long)((const T*)p.logits + (size_t)row * p.Vp);
    rowwide_pin(base_addr);
    const int nvec = p.V / EPV;  // whole vectors inside columns [0, V)
    const int    nsub = (nvec + RW_SUB_VECS - 1) / RW_SUB_VECS;

    // ---- Everything the row needs from memory is requested at once: the per-row arguments (scalar loads, ahead of
    // everything else), the token history (time-major: every id is a cache line of its own; positions past the step
    // re-read the last one), then the first sub-tile of the row. Sixteen waves in lock-step pay sixteen issue slots
    // for every instruction, so what is the same for the whole row is worked out by one wave and handed to the others
    // through LDS: the first wave takes the row's arguments and what follows from them, the second the row's draw.
    const int           wv_s = __builtin_amdgcn_readfirstlane(wv);
    const void*         safe = p.end_ids + row;
    // (Only the loads themselves sit in the two branches: anything computed there from a loaded value would wait
    // for it, in front of the wave's own loads of the history and the row.)
    auto word_at = [&](const void* array, size_t offset) -> const uint32_t* {
        return reinterpret_cast<const uint32_t*>(array != nullptr ? (const char*)array + offset : (const char*)safe);
    };
    auto flag_word_at = [&](const bool* flags) -> const uint32_t* {  // the aligned word that holds the row's flag
        const char* flag = flags != nullptr ? (const char*)flags + row : (const char*)safe;
        return reinterpret_cast<const uint32_t*>(flag - (reinterpret_cast<uintptr_t>(flag) & 3u));
    };
    auto flag_of = [&](const bool* flags, uint32_t word) -> bool {
        const uint32_t mis = (uint32_t)(reinterpret_cast<uintptr_t>(flags + row) & 3u);
        return flags != nullptr && ((word >> (8u * mis)) & 0xFFu) != 0u;
    };
    const int* seq_from_array = p.min_lengths != nullptr ? p.sequence_length_in : nullptr;
    uint32_t   w_skip = 0u, w_fin = 0u, w_k = 0u, w_tp = 0u, w_temp = 0u, w_pen = 0u, w_freq = 0u, w_in = 0u, w_min = 0u,
             w_seq = 0u, w_end = 0u, w_seq_in = 0u;
    RowDrawSource      draw         = {};
    unsigned long long counter_addr = 0ull;
    if (wv_s == 0) {
        w_skip   = *flag_word_at(p.skip_decode);
        w_fin    = *flag_word_at(p.finished_in);
        w_k      = *word_at(p.top_ks, (size_t)row * 4);
        w_tp     = *word_at(p.top_ps, (size_t)row * 4);
        w_temp   = *word_at(p.temperatures, (size_t)row * 4);
        w_pen    = *word_at(p.penalties, (size_t)row * 4);
        w_freq   = *word_at(p.frequencies, (size_t)row * 4);
        w_in     = *word_at(p.input_lengths, (size_t)row * 4);
        w_min    = *word_at(p.min_lengths, (size_t)row * 4);
        w_seq    = *word_at(seq_from_array, (size_t)row * 4);
        w_end    = *word_at(p.end_ids, (size_t)row * 4);
        w_seq_in = *word_at((const int*)l_in.sequence_length, (size_t)row * 4);  // (the unpinned copy: a load through
                                                                                // a pointer known to be global)
    }
    else if (wv_s == 1) {
        w_skip       = *flag_word_at(p.skip_decode);
        w_fin        = *flag_word_at(p.finished_in);
        draw         = row_draw_source(l.rng, l.uniforms, row, safe);
        counter_addr = (unsigned long long)(l.rng != nullptr ? &l.rng[row].offset : nullptr);
    }
    const bool injected = l.uniforms != nullptr;
    const bool hist     = p.bitmaps != nullptr && p.penalties != nullptr;
    // (the instruction scheduler keeps the argument loads above in front of the vector loads below: requested behind
    // them, they would also arrive behind them)
    __builtin_amdgcn_sched_barrier(0);
    RW_STAMP(0)  // (behind the argument loads: a store in front of them would make vector loads of them)
    int                hist_ids[RW_HIST_U];
    {
        const int* column = hist ? p.output_ids + row : p.end_ids;  // (without a history: any valid address)
        const int  last   = hist ? p.step - 1 : 0;
        const int  stride = hist ? p.batch_size : 0;
#pragma unroll
        for (int u = 0; u < RW_HIST_U; ++u) {
            hist_ids[u] = column[(size_t)min(t + u * RW_THREADS, last) * stride];
        }
    }
    uint4 raw[R][RW_NV];
    auto  load = [&](int slot, int q) {
#pragma unroll
        for (int j = 0; j < RW_NV; ++j) {
            const int vi = min(q * RW_SUB_VECS + j * RW_THREADS + t, nvec - 1);  // past the end: a harmless vector
            const u4  v  = __builtin_nontemporal_load((GlobalVec)(base_addr + (unsigned long long)vi * 16ull));
            raw[slot][j] = make_uint4(v.x, v.y, v.z, v.w);
        }
    };
    // Only the first sub-tile for now: a compute unit holds about that much in flight, further loads would wait at
    // issue until data returns and hold up the barriers of the set-up below. The rest of the ring follows once the
    // bitmap is built.
    load(0, 0);
    // while all that is on its way: an empty bitmap of the row's history
    uint32_t* window = fused_lds_bitmap<BMW>();
    const bool counting = hist && p.frequencies != nullptr;  // a frequency penalty: the history's ids are counted too
    if (hist) {
        const int words = min(BMW, (p.V + 31) / 32 + 1);
        for (int i = t; i < words; i += RW_THREADS) {
            window[i] = 0u;
        }
        if (counting) {
#pragma unroll
            for (int i = 0; i < FUSED_COUNT_SLOTS / RW_THREADS; ++i) {
                s.count_table[t + i * RW_THREADS] = 0u;
            }
        }
    }
    // (a fixed point in the program: no arithmetic on the loaded words moves up from here into the branches above)
    asm volatile("" : "+s"(w_skip), "+s"(w_fin), "+s"(w_temp), "+s"(w_pen), "+s"(w_freq), "+s"(w_k), "+s"(w_tp));
    asm volatile("" : "+s"(w_in), "+s"(w_min), "+s"(w_seq), "+s"(w_end), "+s"(w_seq_in));
    const bool skip01 = flag_of(p.skip_decode, w_skip), fin01 = flag_of(p.finished_in, w_fin);
    if (wv_s == 0) {
        FusedRowArgs args0;
        args0.temperature     = p.temperatures != nullptr ? __uint_as_float(w_temp) : 1.0f;
        args0.penalty         = p.penalties != nullptr ? __uint_as_float(w_pen) : 0.0f;
        args0.frequency       = p.frequencies != nullptr ? __uint_as_float(w_freq) : 0.0f;
        args0.input_length    = p.input_lengths != nullptr ? (int)w_in : p.max_input_length;
        args0.min_length      = p.min_lengths != nullptr ? (int)w_min : 0;
        args0.sequence_length = seq_from_array != nullptr ? (int)w_seq : 0;
        args0.end_id          = (int)w_end;
        const FusedRow<DT, BMW> first(p, row, args0);
        const FusedRowDerived   d = first.derived();
        if (lane == 0) {
            s.n_list[0]  = 0;
            s.n_list[1]  = 0;
            s.setup[0]   = __float_as_int(d.inv);
            s.setup[1]   = __float_as_int(d.fast_mul);
            s.setup[2]   = __float_as_int(d.penalty);
            s.setup[3]   = __float_as_int(d.frequency);
            s.setup[4]   = __float_as_int(d.up_mul_neg);
            s.setup[5]   = __float_as_int(d.up_mul_pos);
            s.setup[6]   = __float_as_int(d.up_add);
            s.setup[7]   = d.masked_end_id;
            s.setup[8]   = d.input_length;
            s.setup[9]   = d.flags;
            s.setup[10]  = p.top_ks != nullptr ? (int)w_k : p.max_top_k;
            s.setup[11]  = (skip01 ? 1 : 0) | (fin01 ? 2 : 0);
            s.setup[12]  = p.top_ps != nullptr ? (int)w_tp : __float_as_int(1.0f);
            s.setup[13]  = l_in.sequence_length != nullptr ? (int)w_seq_in : 0;
            s.setup[14]  = (int)w_end;
        }
    }
    // The row's draw: taken once, by the rows that take part (like the reference's curand_uniform).
    if (wv_s == 1 && !(skip01 || fin01) && lane == 0) {
        float u = draw.injected;
        if (!injected) {
            uint64_t next;
            u = row_draw_generate(draw, &next);
            *(__attribute__((address_space(1))) uint64_t*)counter_addr = next;
        }
        ts.misc[0] = __float_as_int(u);
    }
    lds_barrier();

    const int       rec = s.setup[lane & 15];
    FusedRowDerived d;
    d.inv           = __int_as_float(__builtin_amdgcn_readlane(rec, 0));
    d.fast_mul      = __int_as_float(__builtin_amdgcn_readlane(rec, 1));
    d.penalty       = __int_as_float(__builtin_amdgcn_readlane(rec, 2));
    d.frequency     = __int_as_float(__builtin_amdgcn_readlane(rec, 3));
    d.up_mul_neg    = __int_as_float(__builtin_amdgcn_readlane(rec, 4));
    d.up_mul_pos    = __int_as_float(__builtin_amdgcn_readlane(rec, 5));
    d.up_add        = __int_as_float(__builtin_amdgcn_readlane(rec, 6));
    d.masked_end_id = __builtin_amdgcn_readlane(rec, 7);
    d.input_length  = __builtin_amdgcn_readlane(rec, 8);
    d.flags         = __builtin_amdgcn_readlane(rec, 9);
    const int  k    = __builtin_amdgcn_readlane(rec, 10);
    const int  gone = __builtin_amdgcn_readlane(rec, 11);
    FusedRow<DT, BMW> rowctx(p, row, d);
    if (gone != 0) {  // the row is skipped or has finished
        if (gone == 2 && t == 0) {
            l.ids[row] = __builtin_amdgcn_readlane(rec, 14);
        }
        return;
    }
    if (hist) {
#pragma unroll
        for (int u = 0; u < RW_HIST_U; ++u) {
            const int pos = t + u * RW_THREADS;
            const int id  = hist_ids[u];
            if (pos < p.step && id >= 0 && id < p.V && rowctx.history_position_counts(pos)) {
                atomicOr(&window[id >> 5], 1u << (id & 31));
                if (counting) {
                    fused_count_insert(s.count_table, id);
                }
            }
        }
        rowctx.bm_mode   = 1;
        rowctx.bm_origin = 0;
        if (counting) {
            rowctx.use_count_table(s.count_table);  // (read after the barrier below)
        }
    }
    lds_barrier();
#pragma unroll
    for (int r = 1; r < R; ++r) {
        load(r, r);  // (past the row's end: the last vector again, never looked at)
    }
    RW_STAMP(1)
    const bool     bitsv   = hist;
    const uint32_t KMIN    = min_valid_key<DT>();
    const float    NEG_INF = -__builtin_inff();
    const float    mul     = rowctx.fast_mul;
    // a multiplier that is not positive and finite does not keep the order: every vector is evaluated exactly
    const bool all_hit = !(mul > 0.0f && mul < __builtin_inff());

    uint32_t thr     = KMIN;  // candidates are the elements with key >= thr
    float    thr_f   = key_to_float(thr);
    float    thr_hot = NEG_INF;  // (without a bound every vector is looked at exactly)
    auto     set_threshold = [&](uint32_t key, float hot) {
        thr     = key;
        thr_f   = key_to_float(key);
        thr_hot = hot;
    };
    auto hot_of = [&](uint32_t key) -> float {
        const float thr_f = key_to_float(key);
        // What the unrounded, unpenalised product of an element must reach for its final value to reach thr_f:
        // rounding to T can lift a product by half a unit of T, and a history penalty that raises values
        // (a multiplicative one below 1, a negative additive one) can lift it further.
        float h = lean_below_rounding<DT>(thr_f);
        if (bitsv) {
            const float pen = rowctx.penalty;
            float       g   = h;
            bool        raises;
            if (rowctx.penalty_type == 0) {
                // (with a frequency penalty a column loses pen + frequency * count, count between 1 and the step)
                const float per_count = counting ? __builtin_fminf(rowctx.frequency, rowctx.frequency * (float)p.step) : 0.0f;
                g                     = h + (pen + per_count);
                raises                = !(g >= h);
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
        return h;
    };

    // flags of the vector that starts at column `first` (a multiple of EPV): one bit per column of the history
    auto vector_flags = [&](int first) -> uint32_t {
        return bitsv ? (window[first >> 5] >> (first & 31)) & ((1u << EPV) - 1u) : 0u;
    };

    // ---- first bound: the k-th largest of 256 maxima over the first sub-tile (the first of the row to arrive).
    // Only vectors whose elements all take the plain transform count (no history column in the 32-column word of
    // the bitmap around them, not the masked end id), so that every maximum is the final value of an element.
    {
        uint32_t word[RW_NV];
#pragma unroll
        for (int j = 0; j < RW_NV; ++j) {
            word[j] = bitsv ? window[(min(j * RW_THREADS + t, nvec - 1) * EPV) >> 5] : 0u;
        }
        float tmax = NEG_INF;
#pragma unroll
        for (int j = 0; j < RW_NV; ++j) {
            const int   first = (j * RW_THREADS + t) * EPV;
            const bool  clean = j * RW_THREADS + t < nvec && word[j] == 0u && rowctx.interior_vector(first, EPV);
            const float vm    = lean_raw_max<DT>(raw[0][j]);
            tmax              = __builtin_fmaxf(tmax, clean ? vm : NEG_INF);
        }
        tmax = all_hit ? NEG_INF : rowctx.fast(tmax);  // (the transform keeps the order)
        float          hot;
        const uint32_t P = rowwide_bound(s, order_key(tmax), k, hot_of, hot);
        if (P >= KMIN) {
            set_threshold(P, hot);
        }
    }

    RW_STAMP(2)
    // ---- parking and exact evaluation
    int      cur    = 0;   // which counter holds the length of the list
    int      wcount = 0;   // vectors parked by this wave (wave-uniform)
    int      rot    = 0;   // spreads the evaluated vectors over the lanes from one evaluation to the next
    uint32_t dmax   = 0u;  // largest key this lane has put on the list
    // Evaluate what the wave has parked: one vector per lane and round. The elements that reach the bound get
    // their slots on the row's list with one LDS atomic per round.
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
                const uint4 v       = s.stage_raw[wv][e];
                first               = s.stage_first[wv][e];
                const uint32_t bits = vector_flags(first);
#pragma unroll
                for (int c = 0; c < EPV; ++c) {
                    x[c] = rowctx.fast(vector_element<DT>(v, c));
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
                    base_slot = atomicAdd(&s.n_list[cur], total);
                }
                int slot = __builtin_amdgcn_readfirstlane(base_slot) + pre;
#pragma unroll
                for (int c = 0; c < EPV; ++c) {
                    if ((mask >> c) & 1u) {
                        const uint32_t key = order_key(x[c]);
                        if (slot < TK_CCAP) {
                            ts.cand.key[slot] = key;
                            ts.cand.idx[slot] = (uint32_t)(first + c);
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
    static_assert(RW_STAGE >= LG_DRAIN_AT - 1 + RW_PARK_GROUP * WAVE, "a group of vectors always fits the parking list");
    static_assert(RW_NV % RW_PARK_GROUP == 0, "whole groups per sub-tile");
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

    // ---- the stream. The bound is raised again on the way (see below): the k-th largest of disjoint groups of
    // the list's entries bounds the k-th largest of everything seen so far.
    int next_tighten = RW_FIRST_TIGHTEN;  // then twice that plus two, ...
    for (int q0 = 0; q0 < nsub; q0 += R) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int q = q0 + r;
            if (q < nsub) {
#pragma unroll
                for (int j = 0; j < RW_NV; ++j) {
                    const int   rel = q * RW_SUB_VECS + j * RW_THREADS + t;
                    const float m   = lean_raw_max<DT>(raw[r][j]) * mul;
                    park((all_hit || m >= thr_hot) && rel < nvec, raw[r][j], rel * EPV);
                    if ((j + 1) % RW_PARK_GROUP == 0 && j + 1 < RW_NV && wcount >= LG_DRAIN_AT) {
                        drain();
                    }
                }
                if (q + R < nsub) {
                    load(r, q + R);
                }
                // Once or twice per row the bound is raised and the list pruned (after 6, 14, 30, ... sub-tiles while
                // more than four remain, and two sub-tiles before the end, so that the selection at the end starts
                // from little more than k candidates). Every pause of the whole workgroup costs about a
                // microsecond of the stream, which is why there are so few.
                const int  done    = q + 1;
                const bool tighten = (done == next_tighten && done + RW_TAIL_GAP + 2 <= nsub) || (done + RW_TAIL_GAP == nsub && nsub >= 4);
                if (wcount >= LG_DRAIN_AT || tighten || done == nsub) {
                    drain();
                }
                if (tighten) {
                    if (done == next_tighten) {
                        next_tighten = 2 * next_tighten + 2;
                    }
                    lds_barrier();  // every wave has evaluated what it had parked: the list is complete so far
                    const int      n_now   = s.n_list[cur];
                    const bool     listed  = n_now <= RW_THREADS;  // one entry per thread
                    const uint32_t key     = t < n_now ? ts.cand.key[t] : 0u;
                    const uint32_t idx     = t < n_now ? ts.cand.idx[t] : 0u;
                    // the k-th largest of 256 disjoint groups of the list's entries; of the lanes' largest entries when
                    // the list is longer than the workgroup
                    float          hot;
                    const uint32_t P = rowwide_bound(s, listed ? key : dmax, k, hot_of, hot);
                    if (P > thr) {
                        set_threshold(P, hot);
                        if (listed) {
                            // entries below the new bound (collected under an older one) leave the list
                            const bool               keep = key >= P;  // (P > 0: the slots past the list drop out)
                            const unsigned long long m    = __ballot(keep);
                            int                      at   = 0;
                            if (lane == 0 && m != 0ull) {
                                at = atomicAdd(&s.n_list[cur ^ 1], (int)__builtin_popcountll(m));
                            }
                            at = __builtin_amdgcn_readfirstlane(at);
                            if (keep) {
                                const int slot = at
                                                 + (int)__builtin_amdgcn_mbcnt_hi(
                                                     (uint32_t)(m >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                                ts.cand.key[slot] = key;
                                ts.cand.idx[slot] = idx;
                            }
                            lds_barrier();
                            if (t == 0) {
                                s.n_list[cur] = 0;  // (not looked at before the next pruning, several barriers away)
                            }
                            cur ^= 1;
                        }
                    }
                }
            }
        }
    }

    RW_STAMP(3)
    // ---- the columns behind the last whole vector, one by one (fewer than a vector's worth)
    {
        const int v = nvec * EPV + t;
        if (v < p.V && !rowctx.never_selected(v)) {
            const float xv = topk_value_at<DT>(rowctx, v);
            if (xv >= thr_f) {
                const int slot = atomicAdd(&s.n_list[cur], 1);
                if (slot < TK_CCAP) {
                    ts.cand.key[slot] = order_key(xv);
                    ts.cand.idx[slot] = (uint32_t)v;
                }
            }
        }
    }
    lds_barrier();
    RW_STAMP(4)
    if (wv >= TK_WAVES) {
        return;  // the first four waves, one per SIMD, select
    }
    TopkOutputs out;
    out.ids                = l.ids;
    out.sequence_length    = l.sequence_length;
    out.finished           = l.finished;
    out.cum_log_probs      = nullptr;
    out.output_log_probs   = nullptr;
    out.sequence_length_in = __builtin_amdgcn_readfirstlane(s.setup[13]);
    out.cum_log_prob_in    = 0.0f;
    out.end_id_in          = __builtin_amdgcn_readfirstlane(s.setup[14]);
    const float tp_late    = uniform_f(__int_as_float(s.setup[12]));
    int         n = s.n_list[cur];
    const float u = __int_as_float(ts.misc[0]);
    if (n > k + k / 2 && n > 96 && n <= 4 * TK_THREADS) {
        // Far more candidates than needed: raise the bound once more, to the k-th largest of 256 disjoint groups of
        // the list's own entries (at least k entries reach it), and keep what reaches it. The ranking compares every
        // candidate with every other one; this keeps it short.
        uint32_t ck[4], ci[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int i = t + r * TK_THREADS;
            ck[r]       = i < n ? ts.cand.key[i] : 0u;
            ci[r]       = i < n ? ts.cand.idx[i] : 0u;
        }
        s.slot_key[t] = max(max(ck[0], ck[1]), max(ck[2], ck[3]));
        if (t == 0) {
            ts.n_cand = 0;
        }
        lds_barrier();
        const uint32_t P = lean_kth_of_slots(s.slot_key, k);
        if (P > thr) {
            thr = P;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool               keep = ck[r] >= P;  // (the slots past the list hold 0 < P)
                const unsigned long long m    = __ballot(keep);
                int                      at   = 0;
                if (lane == 0 && m != 0ull) {
                    at = atomicAdd(&ts.n_cand, (int)__builtin_popcountll(m));
                }
                at = __builtin_amdgcn_readfirstlane(at);
                if (keep) {
                    const int slot = at
                                     + (int)__builtin_amdgcn_mbcnt_hi((uint32_t)(m >> 32),
                                                                      __builtin_amdgcn_mbcnt_lo((uint32_t)m, 0u));
                    ts.cand.key[slot] = ck[r];
                    ts.cand.idx[slot] = ci[r];
                }
            }
            lds_barrier();
            n = ts.n_cand;
        }
    }
    if (n <= 256) {
        RW_STAMP(5)
        int n_list = rowwide_rank_distinct(ts, n, k, p.max_top_k);
        if (n_list < 0) {
            n_list = rowwide_rank(ts, n, k, p.max_top_k);
        }
        RW_STAMP(7)
#ifdef FTK_RW_STAMPS
        if (threadIdx.x == 0) { stamps[9] = (unsigned long long)n; }
#endif
        topk_finish_list<DT>(ts, n_list, row, p.Vp, tp_late, false, u, p.end_ids, out);
    }
    else {
        rowwide_rare<DT>(ts, (RowwideArgSegment)__builtin_amdgcn_kernarg_segment_ptr(), row, n, thr, k, tp_late, u,
                         counting ? s.count_table : nullptr);
    }
    RW_STAMP(6)
}

// Launchers, one per element type (lean_kernels.hip). window: 1 = the row's bitmap fits the small LDS window,
// 2 = the large one. start / stop: optional events carried by the launch.
int rowwide_launch_f32(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start,
                       hipEvent_t stop);
int rowwide_launch_f16(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l, hipEvent_t start,
                       hipEvent_t stop);
int rowwide_launch_bf16(int window, int rows, hipStream_t st, const FusedParams& p, const FusedLaunch& l,
                        hipEvent_t start, hipEvent_t stop);

}  // namespace ftk
