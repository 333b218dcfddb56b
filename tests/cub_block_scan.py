"""Thread-by-thread float32 simulation of the prefix sums inside the reference's top-p pick kernel, written from the
vendored cub sources and independent of the oracle. Test infrastructure: it fixes the rounding order that
`topp_sampling` (src/fastertransformer/kernels/sampling_topp_kernels.cu:877-1004) inherits from
`cub::BlockScan<float, 256>::InclusiveSum(input, output, prefix_callback)`.

What the sources say, in the order a tile of 256 values goes through them:

* `BlockScan<float, 256>` defaults to `BLOCK_SCAN_RAKING` (3rdparty/cub/block/block_scan.cuh:189, :214-225).
* Layout (3rdparty/cub/block/block_raking_layout.cuh:79-85): 256 shared elements, 32 raking threads,
  SEGMENT_LENGTH = 8; thread t places its input at grid slot t (padding moves addresses, not values), raking
  thread g owns slots 8g .. 8g+7.
* `InclusiveScan(input, output, scan_op, prefix_callback)`
  (3rdparty/cub/block/specializations/block_scan_raking.cuh:601-655): place, barrier, then the 32 raking threads:
  `Upsweep` (:173-185 with `GuardedReduce` :121-135): partial = seg[0]; partial = partial + seg[i] for i = 1..7;
  warp `ExclusiveScan(upsweep_partial, exclusive_partial, scan_op, block_aggregate)`; lane 0 calls the callback with
  the aggregate, the returned prefix is broadcast; `downsweep_prefix = block_prefix + exclusive_partial`, for
  thread 0 the bare `block_prefix`; `InclusiveDownsweep` (:211-228) -> `ThreadScanInclusive` with a prefix
  (3rdparty/cub/thread/thread_scan.cuh:220-236, :147-162): inclusive = prefix + seg[0]; then
  inclusive = inclusive + seg[i]; every thread reads its slot back.
* The warp scan is `WarpScanShfl<float, 32>` (3rdparty/cub/warp/specializations/warp_scan_shfl.cuh):
  `InclusiveScan` (:465-487) runs STEPS = 5 `InclusiveScanStep`s with offsets 1, 2, 4, 8, 16; the fp32 step
  (:199-232) is `shfl.up` by `offset` and, where the source lane exists, `shuffled + own`; the exclusive value is
  the inclusive one shuffled up by one lane, the aggregate lane 31's inclusive value (`Update`, :543-552, :599-609).
* The callback (sampling_topp_kernels.cu:862-875) returns the old running total and adds the aggregate to it.
* Pick (sampling_topp_kernels.cu:953-1003): per tile every 32-lane warp ballots `rand_num <= thread_offset`; after
  the first tile in which any warp has a vote, the lowest such warp takes lane `32 - popc(mask)`.
"""
import numpy as np

f32 = np.float32
BLOCK = 256
RAKING_THREADS = 32
SEGMENT = 8


class _PrefixCallback:
    """BlockPrefixCallbackOp, sampling_topp_kernels.cu:862-875"""

    def __init__(self):
        self.running_total = f32(0.0)

    def __call__(self, block_aggregate):
        old = self.running_total
        self.running_total = f32(self.running_total + block_aggregate)
        return old


def _warp_inclusive_scan(values):
    """WarpScanShfl<float, 32>::InclusiveScan: five shuffle-up steps, all lanes of a step at once"""
    lanes = [f32(v) for v in values]
    for step in range(5):
        offset = 1 << step
        shuffled = list(lanes)
        for lane in range(32):
            if lane - offset >= 0:  # predicate of shfl.up with first_lane 0
                shuffled[lane] = f32(lanes[lane - offset] + lanes[lane])  # add.f32 r0, r0, input
        lanes = shuffled
    return lanes


def block_inclusive_sum(thread_inputs, prefix_op):
    """one call of BlockScan<float, 256>::InclusiveSum(input, output, prefix_op) by all 256 threads"""
    assert len(thread_inputs) == BLOCK
    grid = [f32(v) for v in thread_inputs]                 # *placement_ptr = input
    # raking threads: upsweep
    upsweep = []
    for g in range(RAKING_THREADS):
        seg = grid[g * SEGMENT:(g + 1) * SEGMENT]          # CopySegment
        partial = seg[0]
        for i in range(1, SEGMENT):                        # GuardedReduce, UNGUARDED
            partial = f32(partial + seg[i])
        upsweep.append(partial)
    inclusive = _warp_inclusive_scan(upsweep)
    block_aggregate = inclusive[31]                        # ShuffleIndex(inclusive, 31)
    exclusive = [None] + inclusive[:31]                    # ShuffleUp(inclusive, 1); lane 0 undefined
    block_prefix = prefix_op(block_aggregate)              # lane 0, then Broadcast
    for g in range(RAKING_THREADS):
        downsweep_prefix = block_prefix if g == 0 else f32(block_prefix + exclusive[g])
        seg = grid[g * SEGMENT:(g + 1) * SEGMENT]
        running = f32(downsweep_prefix + seg[0])           # ThreadScanInclusive, apply_prefix
        grid[g * SEGMENT] = running
        for i in range(1, SEGMENT):
            running = f32(running + seg[i])
            grid[g * SEGMENT + i] = running
    return grid                                            # output = *placement_ptr


def prefix_sums(sorted_probs):
    """thread_offset of every position of a sorted row, tile after tile (positions beyond the row read 0)"""
    n = len(sorted_probs)
    op = _PrefixCallback()
    out = []
    for base in range(0, n, BLOCK):
        tile = [f32(sorted_probs[i]) if i < n else f32(0.0) for i in range(base, base + BLOCK)]
        out.extend(block_inclusive_sum(tile, op))
    return np.array(out, f32)


def pick_position(thread_offsets, rand_num):
    """the position topp_sampling emits for prefix sums `thread_offsets` (a multiple of 256 long), or None when
    no tile has a vote"""
    rand_num = f32(rand_num)
    for base in range(0, len(thread_offsets), BLOCK):
        selected = []
        for warp in range(BLOCK // 32):
            mask = 0
            for lane in range(32):
                if rand_num <= thread_offsets[base + warp * 32 + lane]:
                    mask |= 1 << lane
            selected.append(mask)
        for warp, mask in enumerate(selected):
            if mask:
                return base + warp * 32 + 32 - bin(mask).count("1")
    return None


# ---- other rounding orders of the same sums: what a restatement might do instead ----------------------------

def prefix_sums_running(sorted_probs):
    """one running fp32 sum over the whole row"""
    n_padded = -(-len(sorted_probs) // BLOCK) * BLOCK
    out = np.zeros(n_padded, f32)
    s = f32(0.0)
    for i in range(n_padded):
        s = f32(s + (f32(sorted_probs[i]) if i < len(sorted_probs) else f32(0.0)))
        out[i] = s
    return out


def prefix_sums_other_raking(sorted_probs, raking_threads):
    """the same reduce-then-scan scheme with another split of the tile (64 x 4, 16 x 16): a Kogge-Stone scan over
    `raking_threads` segment sums and a sequential walk through each segment"""
    seg_len = BLOCK // raking_threads
    n = len(sorted_probs)
    carry = f32(0.0)
    out = []
    for base in range(0, n, BLOCK):
        tile = [f32(sorted_probs[i]) if i < n else f32(0.0) for i in range(base, base + BLOCK)]
        sums = []
        for g in range(raking_threads):
            a = tile[g * seg_len]
            for i in range(1, seg_len):
                a = f32(a + tile[g * seg_len + i])
            sums.append(a)
        incl = list(sums)
        d = 1
        while d < raking_threads:
            incl = [f32(incl[l - d] + incl[l]) if l >= d else incl[l] for l in range(raking_threads)]
            d *= 2
        for g in range(raking_threads):
            a = carry if g == 0 else f32(carry + incl[g - 1])
            for i in range(seg_len):
                a = f32(a + tile[g * seg_len + i])
                out.append(a)
        carry = f32(carry + incl[-1])
    return np.array(out, f32)


def discriminating_draws(sorted_probs, max_draws=6, lo=0.05, hi=0.9):
    """Draws r for which the reference's order and another rounding order of the same prefix sums pick different
    positions. Returns a list of (r, position under the reference's order, {name: position under another order})
    in which at least one other order disagrees. Candidates are the prefix sums themselves: where two orders differ
    in the last bit at position i, a draw equal to the larger of the two values is crossed at i by one order only."""
    ref = prefix_sums(sorted_probs)
    others = {"running": prefix_sums_running(sorted_probs),
              "raking64x4": prefix_sums_other_raking(sorted_probs, 64),
              "raking16x16": prefix_sums_other_raking(sorted_probs, 16)}
    n = len(sorted_probs)
    found = []
    for name, alt in others.items():
        differ = np.nonzero((alt != ref) & (ref > lo) & (ref < hi))[0]
        differ = differ[differ < n - 64]
        taken = 0
        stride = max(1, len(differ) // (2 * max_draws))     # spread over the row: carries of many tiles take part
        for i in differ[::stride]:
            r = max(ref[i], alt[i])
            pos = pick_position(ref, r)
            alt_pos = {k: pick_position(v, r) for k, v in others.items()}
            if pos is not None and pos < n and alt_pos[name] != pos:
                found.append((f32(r), pos, alt_pos))
                taken += 1
                if taken >= max_draws:
                    break
    return found
