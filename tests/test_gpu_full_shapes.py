"""The benchmark configurations at their stated sizes, through DynamicDecodeLayer, against the CPU oracle with
injected draws: the launch geometries that bench.py times (rows split over several workgroups that stream
several tiles each, one workgroup per row at batch 1024) are the ones compared here. ids / finished /
sequence_length / should_stop bit-exact, log-probs within 1e-5 relative (fp32) or 2e-3 (fp16 / bf16), mutated
logits bit-exact on the kernel-by-kernel path."""
import numpy as np
import pytest

import ft_oracle as O
from decode_harness import Case, OracleRunner, ProductRunner, compare, kernel_sequence
from helpers import DTYPES, DTYPE_NAMES, make_word_list, uniforms

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


def _normal(rng, dt, B, Vp, sigma):
    return O.to_storage(rng.standard_normal((B, Vp), dtype=np.float32) * np.float32(sigma), dt)


def _history(rng, steps, batch, V, zipf=None):
    if zipf:
        return np.minimum(rng.zipf(zipf, (steps, batch)), V - 1).astype(np.int32)
    return rng.integers(0, V, (steps, batch)).astype(np.int32)


def _run(c, rng, steps, logits_fn, check_logits):
    p, o = ProductRunner(c), OracleRunner(c)
    for i in range(steps):
        step = c.max_input_length + i
        logits = logits_fn(i)
        u = uniforms(rng, c.batch)
        p.step(step, logits, u)
        o.step(step, logits, u)
        compare(p.snapshot(), o.snapshot(), c.dt, check_logits, where="step %d" % step)
    return p.snapshot()


def test_headline_b256_v128256_f32():
    """bench.py's default workload as it is timed: 256 x 128256 fp32, k = 64, p = 0.9, temperature 0.8, repetition
    penalty 1.1 over a 64-token history, fused step; three steps."""
    rng = np.random.default_rng(101)
    B, V, H = 256, 128256, 64
    c = Case(O.F32, B, V, V, max_input_length=H, gen_len=3, runtime_top_k=[64], runtime_top_p=[0.9],
             temperature=[0.8], repetition_penalty=[1.1], prompt=_history(rng, H, B, V))
    _run(c, rng, 3, lambda i: _normal(rng, O.F32, B, V, 2.5), check_logits=False)


@pytest.mark.parametrize("logprobs", [False, True], ids=["fused", "logprobs"])
def test_config2_b256_v51200_f16(logprobs):
    """Configuration 2 at full size: 256 rows, vocabulary 50257 padded to 51200 fp16, N(0, 3) plus 8 spikes of +12
    per row, per-row k from {1, 4, 16, 40, 64, 1024}, per-row temperature U[0.5, 1.5]."""
    rng = np.random.default_rng(102)
    B, V, Vp = 256, 50257, 51200
    ks = rng.choice([1, 4, 16, 40, 64, 1024], B).astype(np.uint32)
    c = Case(O.F16, B, V, Vp, gen_len=2, runtime_top_k=ks, temperature=rng.uniform(0.5, 1.5, B),
             end_ids=np.full(B, 50256, np.int32), with_cum=logprobs, with_out_lp=logprobs)

    def logits_fn(i):
        x = rng.standard_normal((B, Vp), dtype=np.float32) * np.float32(3.0)
        for b in range(B):
            x[b, rng.integers(0, V, 8)] += 12.0
        return O.to_storage(x, O.F16)

    _run(c, rng, 2, logits_fn, check_logits=logprobs)


def test_config3_b256_v128256_f32_topp_16_steps():
    """Configuration 3 at full size: 256 rows, vocabulary 128256 fp32, log-softmax of Zipf(1.1) over a seeded
    permutation plus N(0, 0.5), top_k 0, per-row top_p U[0.5, 0.99], decay 0.9, minimum 0.3, reset id 13,
    16 consecutive steps with fresh logits."""
    rng = np.random.default_rng(103)
    B, V = 256, 128256
    base = -1.1 * np.log(np.arange(1, V + 1, dtype=np.float64))
    base = (base - np.log(np.exp(base).sum())).astype(np.float32)

    def logits_fn(i):
        x = rng.standard_normal((B, V), dtype=np.float32) * np.float32(0.5)
        for b in range(B):
            x[b] += base[rng.permutation(V)]
        if i % 5 == 2:
            x[::7, 13] = 3.0  # the reset id becomes likely in some rows, so that the reset branch runs
        return x

    c = Case(O.F32, B, V, V, gen_len=16, runtime_top_k=[0], runtime_top_p=rng.uniform(0.5, 0.99, B),
             top_p_decay=np.full(B, 0.9), top_p_min=np.full(B, 0.3), top_p_reset_ids=np.full(B, 13),
             end_ids=np.full(B, V - 1, np.int32), with_cum=True, with_out_lp=True)
    _run(c, rng, 12, logits_fn, check_logits=False)  # straight from the logits, which are left alone
    with kernel_sequence():  # the reference's side effect: the logits end up as probabilities, bit for bit
        _run(c, rng, 4, logits_fn, check_logits=True)


@pytest.mark.parametrize("freq", [None, 0.3], ids=["presence", "presence+frequency"])
def test_config4_b128_v32000_bf16_history_2048(freq):
    """Configuration 4 at full size: 128 rows, vocabulary 32000 bf16, a 2048-token Zipf(1.2) history per row,
    min_length 2100 against step 2048 (the end id 2 stays masked), presence 0.5 (+ frequency 0.3), 64 bad-word
    n-grams of length 1-4, 16 stop-word n-grams of length 1-3, top_k 50."""
    rng = np.random.default_rng(104)
    B, V, H = 128, 32000, 2048
    prompt = _history(rng, H, B, V, zipf=1.2)
    bad = np.stack([make_word_list(rng, 64, 4, V, L=256, history=np.vstack([prompt, prompt[:2]]), step=H, row=b)[0]
                    for b in range(B)])
    stop = np.stack([make_word_list(rng, 16, 3, V, L=48)[0] for b in range(B)])
    c = Case(O.BF16, B, V, V, max_input_length=H, gen_len=3, runtime_top_k=[50], presence_penalty=[0.5],
             frequency_penalty=None if freq is None else [freq], min_length=[2100],
             end_ids=np.full(B, 2, np.int32), prompt=prompt, bad_words=bad, stop_words=stop)
    snap = _run(c, rng, 3, lambda i: _normal(rng, O.BF16, B, V, 2.0), check_logits=False)
    assert not (snap["output_ids"][H:] == 2).any()


@pytest.mark.parametrize("logprobs", [False, True], ids=["fused", "logprobs"])
def test_config5_b1024_v152064_f16(logprobs):
    """Configuration 5 at its real batch: 1024 rows, vocabulary 152064 fp16, k = 64 then p = 0.9, temperature 0.8,
    repetition penalty 1.1, finished / sequence_length / length-criterion updates, with and without log-probs;
    three steps, some rows finishing on the way."""
    rng = np.random.default_rng(105)
    B, V, H = 1024, 152064, 8
    end = 7
    c = Case(O.F16, B, V, V, max_input_length=H, gen_len=3, runtime_top_k=[64], runtime_top_p=[0.9],
             temperature=[0.8], repetition_penalty=[1.1], end_ids=np.full(B, end, np.int32),
             prompt=_history(rng, H, B, V), with_cum=logprobs, with_out_lp=logprobs,
             sequence_limit_length=rng.integers(H + 1, H + 6, B))

    def logits_fn(i):
        x = rng.standard_normal((B, V), dtype=np.float32) * np.float32(2.5)
        x[rng.random(B) < 0.1, end] = 30.0
        return O.to_storage(x, O.F16)

    _run(c, rng, 3, logits_fn, check_logits=False)  # fused step: one read, two with log-probs, nothing mutated
    if logprobs:
        with kernel_sequence():  # the reference's kernel sequence: logits end up as probabilities, bit for bit
            _run(c, rng, 2, logits_fn, check_logits=True)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("B", [320, 600, 1100])
def test_small_k_many_tiles_per_workgroup(dt, B):
    """k <= 128 at batches where every streaming workgroup walks three or more tiles of its row (a few
    workgroups per row at 320 and 600 rows, one per row at 1100), all dtypes; per-row k in [1, 128], top-p,
    temperature, repetition penalty over a short history; two steps."""
    rng = np.random.default_rng(300 + 7 * dt + B)
    V, H = 131071, 12  # an odd vocabulary: rows start at every alignment
    ks = rng.integers(1, 129, B).astype(np.uint32)
    ks[0] = 128
    c = Case(dt, B, V, V, max_input_length=H, gen_len=2, runtime_top_k=ks,
             runtime_top_p=rng.uniform(0.3, 1.0, B).astype(np.float32), temperature=rng.uniform(0.6, 1.3, B),
             repetition_penalty=rng.uniform(1.0, 1.4, B), prompt=_history(rng, H, B, V),
             end_ids=rng.integers(0, V, B).astype(np.int32))
    _run(c, rng, 2, lambda i: _normal(rng, dt, B, V, 2.0), check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_rows_whose_late_columns_dominate(dt):
    """Rows whose bound from the first columns is useless further on: logits that climb with the column index,
    a plateau of equal large values in the middle of the row, and a row where only the last thousand columns
    matter. The candidate list of a streaming workgroup overflows in a tile that is not its first; the recovery
    must give the reference's picks."""
    rng = np.random.default_rng(400 + dt)
    B, V, H = 260, 120000, 6
    x = rng.standard_normal((B, V), dtype=np.float32)
    ramp = np.linspace(-30.0, 30.0, V, dtype=np.float32)
    x[0::4] += ramp                      # ascending rows
    x[1::4, 50000:90000] += 25.0         # a wide plateau of large values after quiet columns
    x[2::4, V - 1000:] += 40.0           # everything happens at the end of the row
    x[3::4, 70000:70000 + 3000] = 9.0    # thousands of identical values above everything else
    c = Case(dt, B, V, V, max_input_length=H, gen_len=2, runtime_top_k=[50], runtime_top_p=[0.95],
             temperature=[0.9], repetition_penalty=[1.2], prompt=_history(rng, H, B, V))
    xs = O.to_storage(x, dt)
    _run(c, rng, 2, lambda i: xs, check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_large_k_two_reads_and_lopsided_slices(dt):
    """Launches whose largest k is beyond 128 read the logits twice (maxima of column groups bound the k-th
    largest, then a gather against that bound) and order the candidates slice by slice. Rows here: k from 1 to
    1024 over plain noise with many equal values (fp16 / bf16), rows whose large values all sit in the columns of
    one stage-1 slice (more than 256 candidates in it: the whole-list sorts take over), and constant rows."""
    rng = np.random.default_rng(900 + dt)
    B, V, H = 64, 51200, 5
    x = rng.standard_normal((B, V), dtype=np.float32) * np.float32(2.0)
    cols = np.arange(V)
    one_slice = ((cols >> 8) & 7) == 3          # BS1 = 256 for k > 16
    x[1::8][:, one_slice] += 9.0                # every candidate of these rows lies in slice 3
    x[2::8] = np.round(x[2::8])                 # few distinct values: long runs of equal candidates
    x[3::8] = 1.5                               # a constant row
    ks = np.array([1024, 1000, 777, 300, 129, 64, 7, 1] * (B // 8), dtype=np.uint32)
    c = Case(dt, B, V, V, max_input_length=H, gen_len=2, runtime_top_k=ks, runtime_top_p=[0.9],
             temperature=[0.8], repetition_penalty=[1.1], prompt=_history(rng, H, B, V))
    xs = O.to_storage(x, dt)
    _run(c, rng, 2, lambda i: xs, check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("B,k", [(1, 128), (3, 100), (4, 192), (70, 150), (2, 1024), (5, 400), (3, 193)])
def test_few_rows_many_lists_per_row(dt, B, k):
    """A handful of rows of a long vocabulary: every row is cut into the largest number of workgroups, each of which
    reports at least k candidates of its own, so the union of a row's lists is longer than the 2048 entries the
    select kernel holds at once (k up to 192, one read of the logits) and the bound is raised before the lists are
    merged; with k beyond 192 the same geometry goes through the two reads with two maxima per thread."""
    rng = np.random.default_rng(7000 + 10 * B + dt)
    V, H = 128256, 4
    c = Case(dt, B, V, V, max_input_length=H, gen_len=2, runtime_top_k=[k], runtime_top_p=[0.95],
             temperature=[0.7], repetition_penalty=[1.3], prompt=_history(rng, H, B, V))
    _run(c, rng, 2, lambda i: _normal(rng, dt, B, V, 3.0), check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("k", [50, 600])
def test_embedding_bias_through_the_fused_step(dt, k):
    """An embedding bias (added before the temperature, rounded to T) with rows and bias on 16-byte boundaries goes
    through the same streaming kernels as rows without one: one read of the logits (k = 50) and two (k = 600)."""
    rng = np.random.default_rng(8100 + dt + k)
    B, V, H = 48, 65536 + 8 * 5, 6
    bias = O.to_storage(rng.standard_normal(V).astype(np.float32) * np.float32(1.5), dt)
    c = Case(dt, B, V, V, max_input_length=H, gen_len=2, runtime_top_k=[k], runtime_top_p=[0.9], temperature=[0.7],
             repetition_penalty=[1.2], embedding_bias=bias, prompt=_history(rng, H, B, V))
    _run(c, rng, 2, lambda i: _normal(rng, dt, B, V, 2.0), check_logits=False)
