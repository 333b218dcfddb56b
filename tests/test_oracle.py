"""Pins the CPU oracle (oracle/ft_oracle.cc) without a GPU: against the reference's known-answer sets, against
closed forms evaluated independently in float64 / numpy / torch, and against a literal thread-by-thread
simulation of the reference's two-stage top-k written from its source description.

Every function the GPU parity tests lean on has a check here that a plausible mistake (a wrong sign, a
swapped operand, a dropped term, a different tie rule) would fail.
"""
import json
import os

import numpy as np
import pytest

import ft_oracle as O
from decode_harness import Case, OracleRunner
from helpers import DTYPE_NAMES, DTYPES, make_word_list, uniforms

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "sampling_layer_kat.json")))
FLT_MAX = np.finfo(np.float32).max


# ---- elementary functions and storage conversions ------------------------------------------------
def test_expf_logf_against_float64():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.uniform(-87, 88, 20000), rng.uniform(-1, 1, 20000), [0.0, -0.0, 1.0, -1.0]])
    x = x.astype(np.float32)
    got = O.expf(x)
    ref = np.exp(x.astype(np.float64))
    assert np.max(np.abs(got - ref) / ref) < 2.5e-7
    assert O.expf(np.array([0.0], np.float32))[0] == 1.0
    assert O.expf(np.array([-np.inf], np.float32))[0] == 0.0
    assert O.expf(np.array([-200.0], np.float32))[0] == 0.0
    y = np.concatenate([np.exp(rng.uniform(-80, 80, 20000)), rng.uniform(0.5, 2.0, 20000), [1.0]]).astype(np.float32)
    got = O.logf(y)
    ref = np.log(y.astype(np.float64))
    err = np.abs(got - ref)
    assert np.max(err / np.maximum(np.abs(ref), 1e-3)) < 3e-7
    assert O.logf(np.array([1.0], np.float32))[0] == 0.0
    assert O.logf(np.array([0.0], np.float32))[0] == -np.inf


def test_storage_conversions_against_numpy_and_torch():
    import torch
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(50000) * 10, rng.standard_normal(20000) * 1e-6,
                        rng.standard_normal(20000) * 6e4, [0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8, 3e38,
                                                           -3.4e38, np.inf, -np.inf]]).astype(np.float32)
    with np.errstate(over="ignore"):
        ref16 = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(O.to_storage(x, O.F16).view(np.uint16), ref16)
    refbf = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.to_storage(x, O.BF16), refbf)
    # widening is exact
    assert np.array_equal(O.to_f32(ref16.view(np.float16), O.F16), ref16.view(np.float16).astype(np.float32))
    assert np.array_equal(O.to_f32(refbf, O.BF16),
                          torch.from_numpy(refbf.view(np.int16)).view(torch.bfloat16).float().numpy())


# ---- the reference's known-answer sets --------------------------------------------------------------
def _kat_logits(dt):
    rows = [[-FLT_MAX if v == "-FLT_MAX" else v for v in row] for row in KAT["logits_per_step"]]
    return [O.to_storage(np.tile(np.array(r, np.float32), (KAT["batch_size"], 1)), dt) for r in rows]


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("kat", KAT["cases"], ids=lambda c: c["name"])
@pytest.mark.parametrize("logprobs", [True, False], ids=["logprobs", "plain"])
def test_known_answer_sets(dt, kat, logprobs):
    """tests/unittests/test_sampling_layer.cu:318-592: whatever the draw, the sampled id lies in the set."""
    B, V = KAT["batch_size"], KAT["vocab_size"]
    logits = _kat_logits(dt)
    local = B // 3 if kat["use_local_batch"] else B
    ite = 1 if kat["use_local_batch"] else 0
    rng = np.random.default_rng(11)
    for trial in range(30):
        c = Case(dt, B, V, V, gen_len=3, local_batch=local, runtime_top_k=kat["top_k"], runtime_top_p=kat["top_p"],
                 end_ids=np.full(B, KAT["end_id"], np.int32), with_finished=False, with_seq_len=False,
                 with_cum=logprobs, with_out_lp=logprobs)
        o = OracleRunner(c)
        for step in range(3):
            u = uniforms(rng, B)
            if trial == 0:
                u[:] = 1.0  # the largest draw curand_uniform can return
            if trial == 1:
                u[:] = np.float32(2.0 ** -32)
            o.step(step, logits[step], u, ite=ite)
        ids = o.snapshot()["output_ids"]
        rows = range(ite * local, ite * local + local)
        for step in range(3):
            for b in rows:
                assert int(ids[step, b]) in kat["expected"][step][b], (kat["name"], trial, step, b)


# ---- top-k: literal simulation of the two-stage scheme --------------------------------------------------
def _block_reduce_top1(cands):
    """cub::BlockReduce over (value, id) pairs with the reference's `a.u > b.u ? a : b`
    (reduce_kernel_utils.cuh:345-348): 32-lane shuffle-down trees (the lower lane is the left operand,
    warp_reduce_shfl.cuh:389-401), then warps folded in ascending order
    (block_reduce_warp_reductions.cuh:113-125)."""
    def comb(a, b):
        return a if a[0] > b[0] else b
    warps = []
    for w in range(len(cands) // 32):
        lanes = list(cands[32 * w:32 * w + 32])
        for off in (1, 2, 4, 8, 16):
            new = list(lanes)
            for lane in range(32):
                if lane + off < 32:
                    new[lane] = comb(lanes[lane], lanes[lane + off])
            lanes = new
        warps.append(lanes[0])
    agg = warps[0]
    for w in warps[1:]:
        agg = comb(agg, w)
    return agg


def _simulate_reference_topk(row, k, max_top_k):
    """sampling_topk_kernels.cu:130-280 for one fp32 row: returns the ordered candidate list [(id, value)]."""
    V = len(row)
    bs1 = 128 if max_top_k <= 16 else 256
    bs2 = 128 if max_top_k <= 32 else 256
    tmp = np.array(row, np.float32).copy()
    neg = np.float32(-FLT_MAX)
    ids = np.full(8 * k, -1, np.int64)
    vals = np.full(8 * k, neg, np.float32)
    for block in range(8):
        for ite in range(k):
            cands = []
            for tid in range(bs1):
                u, p = neg, -1
                for e in range(tid + block * bs1, V, bs1 * 8):
                    if tmp[e] > u:
                        u, p = tmp[e], e
                cands.append((u, p))
            u, p = _block_reduce_top1(cands)
            ids[block * k + ite] = p
            vals[block * k + ite] = u
            if p >= 0:
                tmp[p] = neg
    out = []
    s_val = vals.copy()
    for ite in range(k):
        cands = []
        for tid in range(bs2):
            u, p = neg, -1
            for i in range(tid, 8 * k, bs2):
                if s_val[i] > u:
                    u, p = s_val[i], i
            cands.append((u, p))
        u, p = _block_reduce_top1(cands)
        if p < 0:
            break
        out.append((int(ids[p]), float(u)))
        s_val[p] = neg
    return out


def _oracle_topk_pick(row, k, max_top_k, u, p=1.0):
    V = len(row)
    lp = np.ascontiguousarray(np.asarray(row, np.float32).reshape(1, V))
    ids = np.zeros(1, np.int32)
    O.batch_topk_sampling(O.F32, lp, ids, None, None, None, None, np.array([u], np.float32), max_top_k,
                          np.array([k], np.int32), p, None, V, np.array([V - 1], np.int32), 1, None)
    return int(ids[0])


@pytest.mark.parametrize("case", ["ties", "distinct", "few_valid", "two_values"])
def test_topk_order_against_thread_level_simulation(case):
    rng = np.random.default_rng({"ties": 3, "distinct": 4, "few_valid": 5, "two_values": 6}[case])
    for trial in range(3):
        V = int(rng.integers(300, 2600))
        k = int(rng.integers(1, 7))
        max_top_k = int(rng.choice([k, 16, 17, 32, 33, 64]))
        max_top_k = max(max_top_k, k)
        if case == "ties":
            row = rng.integers(0, 4, V).astype(np.float32)
        elif case == "two_values":
            row = np.where(rng.random(V) < 0.02, 5.0, 1.0).astype(np.float32)
        elif case == "few_valid":
            row = np.full(V, -FLT_MAX, np.float32)
            row[rng.choice(V, 3, replace=False)] = rng.standard_normal(3).astype(np.float32)
            row[rng.integers(0, V)] = -np.inf
        else:
            row = rng.standard_normal(V).astype(np.float32)
        order = _simulate_reference_topk(row, k, max_top_k)
        assert len(order) >= 1
        # draws that land in the middle of each position's share of the cumulative weight
        x0 = order[0][1]
        w = np.array([np.exp(np.float64(v) - np.float64(x0)) for _, v in order])
        cum = np.concatenate([[0.0], np.cumsum(w)])
        for j, (tok, _) in enumerate(order):
            u = (cum[j] + 0.5 * w[j]) / cum[-1]
            assert _oracle_topk_pick(row, k, max_top_k, np.float32(u)) == tok, (case, trial, j, order)


def test_topk_set_is_the_k_largest_when_values_are_distinct():
    rng = np.random.default_rng(8)
    V, k = 5000, 37
    row = rng.permutation(V).astype(np.float32) / 64.0
    want = set(np.argsort(-row)[:k].tolist())
    seen = set()
    for u in np.linspace(1e-6, 1.0, 400):
        seen.add(_oracle_topk_pick(row, k, 64, np.float32(u)))
    assert seen <= want
    assert _oracle_topk_pick(row, k, 64, np.float32(1e-9)) == int(np.argmax(row))
    # all k positions are reachable when the weights are equal
    flat = np.zeros(V, np.float32)
    flat[rng.choice(V, k, replace=False)] = 1.0
    got = {_oracle_topk_pick(flat, k, 64, np.float32((j + 0.5) / k)) for j in range(k)}
    assert got == set(np.nonzero(flat)[0].tolist())


def test_topk_inverse_cdf_and_logprobs_closed_form():
    """sampling_topk_kernels.cu:264-311: r = u*p*S walked down the ordered list; log-prob outputs."""
    rng = np.random.default_rng(9)
    B, V, k = 64, 3000, 12
    logits = (rng.standard_normal((B, V)) * 2).astype(np.float32)
    top_p = 0.8
    u = rng.random(B).astype(np.float32) * 0.98 + 0.01
    # probabilities in, as the layer does when log-probs are requested
    m = logits.max(axis=1, keepdims=True).astype(np.float64)
    e = np.exp(logits.astype(np.float64) - m)
    probs = (e / (e.sum(axis=1, keepdims=True) + 1e-6)).astype(np.float32)
    ids = np.zeros(B, np.int32)
    cum = np.zeros(B, np.float32)
    out = np.zeros(B, np.float32)
    seq = np.full(B, 5, np.int32)
    fin = np.zeros(B, np.bool_)
    end = rng.integers(0, V, B).astype(np.int32)
    O.batch_topk_sampling(O.F32, probs, ids, seq, fin, cum, out, u, k, np.full(B, k, np.int32), top_p, None, V, end,
                          B, None)
    mismatch = 0
    for b in range(B):
        order = np.argsort(-probs[b].astype(np.float64), kind="stable")[:k]
        w = probs[b][order].astype(np.float64)
        r = np.float64(u[b]) * top_p * w.sum()
        j = int(np.searchsorted(np.cumsum(w), r, side="left"))
        j = min(j, k - 1)
        if ids[b] != order[j]:
            mismatch += 1  # a draw within rounding of a boundary may fall either way
            assert abs(int(np.nonzero(order == ids[b])[0][0]) - j) == 1
            continue
        np.testing.assert_allclose(cum[b], np.log(w[j]), rtol=2e-6, atol=1e-6)
        np.testing.assert_allclose(out[b], np.log(w[j]) - np.log(w.sum()), rtol=2e-6, atol=2e-6)
    assert mismatch <= 1
    assert np.array_equal(seq, np.full(B, 6, np.int32))
    assert np.array_equal(fin, ids == end)


def test_topk_finished_and_skipped_rows():
    B, V = 4, 100
    rng = np.random.default_rng(10)
    lp = rng.standard_normal((B, V)).astype(np.float32)
    ids = np.full(B, -7, np.int32)
    seq = np.full(B, 3, np.int32)
    fin = np.array([False, True, False, True])
    skip = np.array([False, False, True, True])
    end = np.array([9, 8, 7, 6], np.int32)
    O.batch_topk_sampling(O.F32, lp, ids, seq, fin, None, None, np.full(B, 0.5, np.float32), 1,
                          np.full(B, 1, np.int32), 1.0, None, V, end, B, skip)
    assert ids[0] == int(np.argmax(lp[0])) and seq[0] == 4
    assert ids[1] == 8 and seq[1] == 3 and fin[1]          # finished: end id, nothing else moves
    assert ids[2] == -7 and ids[3] == -7 and seq[2] == 3   # skipped rows are untouched


# ---- penalties ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("with_bias", [False, True])
def test_temperature_closed_form(dt, with_bias):
    """sampling_penalty_kernels.cu:134-146 / :171-177, and the reference test's own expectation
    (tests/unittests/test_penalty_kernels.cu:188-208: (logit + bias) / temperature within tolerance)."""
    rng = np.random.default_rng(12)
    B, V, Vp = 6, 50, 56
    x = O.to_storage((rng.standard_normal((B, Vp)) * 3).astype(np.float32), dt)
    bias = O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt) if with_bias else None
    temps = rng.uniform(0.5, 2.0, B).astype(np.float32)
    got = x.copy()
    O.batch_apply_temperature_penalty(dt, got, bias, temps, B, V, Vp)
    gf = O.to_f32(got, dt)
    xf = O.to_f32(x, dt).astype(np.float64)
    bf = O.to_f32(bias, dt).astype(np.float64) if with_bias else np.zeros(Vp)
    want = (xf + bf) / temps[:, None].astype(np.float64)
    tol = {O.F32: 1e-5, O.F16: 4e-3, O.BF16: 2e-2}[dt]
    np.testing.assert_allclose(gf[:, :V], want[:, :V], rtol=tol, atol=tol)
    if dt == O.F16:
        assert np.array_equal(got[:, V:], x[:, V:])  # the half2 kernel leaves pad columns alone (V, Vp even)
    else:
        assert np.all(gf[:, V:] == -O.max_t(dt))
    if dt == O.F32:
        # operation by operation in float32: bit-exact
        inv = (np.float32(1.0) / (temps + np.float32(1e-6))).astype(np.float32)
        step = O.to_f32(x, dt)[:, :V]
        if with_bias:
            step = (step + O.to_f32(bias, dt)[None, :V]).astype(np.float32)
        step = (step * inv[:, None]).astype(np.float32)
        assert np.array_equal(gf[:, :V].view(np.uint32), step.view(np.uint32))


def _reference_repetition(x, ids_col, penalty, multiplicative, input_length, max_input_length):
    """the reference test's host expectation (tests/unittests/test_penalty_kernels.cu:58-119), in float64"""
    y = x.astype(np.float64).copy()
    seen = set()
    for t, tok in enumerate(ids_col):
        if input_length <= t < max_input_length:
            continue
        tok = int(tok)
        if tok in seen:
            continue
        seen.add(tok)
        v = float(x[tok])
        y[tok] = (v * penalty if v < 0 else v / penalty) if multiplicative else v - penalty
    return y


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("multiplicative", [True, False])
def test_repetition_penalty_closed_form(dt, multiplicative):
    rng = np.random.default_rng(13)
    B, V, step, max_in = 5, 40, 30, 12
    x = O.to_storage((rng.standard_normal((B, V)) * 2).astype(np.float32), dt)
    out_ids = rng.integers(0, V, (step, B)).astype(np.int32)
    out_ids[3] = out_ids[7]                      # repeated tokens are penalised once
    input_lengths = rng.integers(4, max_in + 1, B).astype(np.int32)
    pens = rng.uniform(1.1, 2.0, B).astype(np.float32) if multiplicative else rng.uniform(0.1, 2.0, B).astype(np.float32)
    got = x.copy()
    O.batch_apply_repetition_penalty(dt, got, pens, out_ids, B, B, V, input_lengths, max_in, step,
                                     O.PEN_MULTIPLICATIVE if multiplicative else O.PEN_ADDITIVE)
    gf = O.to_f32(got, dt)
    xf = O.to_f32(x, dt)
    tol = {O.F32: 1e-6, O.F16: 2e-3, O.BF16: 1.6e-2}[dt]
    for b in range(B):
        want = _reference_repetition(xf[b], out_ids[:, b], float(pens[b]), multiplicative, int(input_lengths[b]),
                                     max_in)
        np.testing.assert_allclose(gf[b], want, rtol=tol, atol=tol)
        untouched = np.ones(V, bool)
        hist = [int(t) for i, t in enumerate(out_ids[:, b]) if not (input_lengths[b] <= i < max_in)]
        untouched[hist] = False
        assert np.array_equal(got[b][untouched], x[b][untouched])


def test_frequency_penalty_reduces_to_presence():
    """extension (no reference code): with frequency 0 it must equal the additive penalty bit for bit"""
    rng = np.random.default_rng(14)
    B, V, step = 4, 64, 40
    for dt in DTYPES:
        x = O.to_storage((rng.standard_normal((B, V)) * 2).astype(np.float32), dt)
        out_ids = rng.integers(0, V, (step, B)).astype(np.int32)
        pres = rng.uniform(0.1, 1.0, B).astype(np.float32)
        a, b = x.copy(), x.copy()
        O.batch_apply_repetition_penalty(dt, a, pres, out_ids, B, B, V, None, 0, step, O.PEN_ADDITIVE)
        O.batch_apply_frequency_penalty(dt, b, pres, np.zeros(B, np.float32), out_ids, B, B, V, None, 0, step)
        assert np.array_equal(a.view(np.uint8), b.view(np.uint8))
        # and with a frequency term: x - presence - frequency * count, in float64
        freq = rng.uniform(0.1, 0.5, B).astype(np.float32)
        c = x.copy()
        O.batch_apply_frequency_penalty(dt, c, pres, freq, out_ids, B, B, V, None, 0, step)
        xf, cf = O.to_f32(x, dt).astype(np.float64), O.to_f32(c, dt)
        for r in range(B):
            counts = np.bincount(out_ids[:, r], minlength=V)
            want = np.where(counts > 0, xf[r] - pres[r] - freq[r] * counts, xf[r])
            tol = {O.F32: 1e-6, O.F16: 2e-3, O.BF16: 1.6e-2}[dt]
            np.testing.assert_allclose(cf[r], want, rtol=tol, atol=tol)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_min_length_and_end_mask(dt):
    rng = np.random.default_rng(15)
    B, V, Vp, max_in = 6, 30, 32, 4
    x = O.to_storage(rng.standard_normal((B, Vp)).astype(np.float32), dt)
    end = rng.integers(0, V, B).astype(np.int32)
    seq = np.array([3, 4, 5, 6, 7, 8], np.int32)
    min_len = np.array([3, 3, 3, 3, 3, 3], np.int32)
    got = x.copy()
    O.min_length_penalty(dt, got, min_len, end, seq, max_in, B, Vp)
    gf = O.to_f32(got, dt)
    for b in range(B):
        masked = seq[b] + 1 - max_in < min_len[b]   # sampling_penalty_kernels.cu:493-499
        assert (gf[b, end[b]] == -O.max_t(dt)) == masked
        keep = np.ones(Vp, bool)
        keep[end[b]] = False
        assert np.array_equal(got[b][keep], x[b][keep])
    fin = np.array([False, True, False, True, False, False])
    got = x.copy()
    O.add_bias_end_mask(dt, got, None, end, fin, B, V, Vp)
    gf = O.to_f32(got, dt)
    for b in range(B):
        assert np.all(gf[b, V:] == -O.max_t(dt))
        if fin[b]:
            want = np.full(V, -O.max_t(dt), np.float32)
            want[end[b]] = O.max_t(dt)
            assert np.array_equal(gf[b, :V], want)
        else:
            assert np.array_equal(got[b, :V], x[b, :V])


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_softmax_closed_form(dt):
    """sampling_topp_kernels.cu:1308-1344 against float64; the reference's own host check
    (tests/unittests/test_sampling_kernels.cu:51-104) agrees to the same tolerance"""
    rng = np.random.default_rng(16)
    B, V, Vp = 5, 700, 704
    x = O.to_storage((rng.standard_normal((B, Vp)) * 3).astype(np.float32), dt)
    end = rng.integers(0, V, B).astype(np.int32)
    fin = np.array([False, False, True, False, False])
    got = x.copy()
    O.add_bias_softmax(dt, got, None, end, fin, B, Vp, V)
    gf = O.to_f32(got, dt).astype(np.float64)
    xf = O.to_f32(x, dt).astype(np.float64)
    tol = {O.F32: 2e-6, O.F16: 2e-3, O.BF16: 1.6e-2}[dt]
    for b in range(B):
        assert np.all(gf[b, V:] == 0.0)
        if fin[b]:
            assert abs(gf[b, end[b]] - 1.0) < 4e-3 and np.count_nonzero(gf[b]) == 1
            continue
        e = np.exp(xf[b, :V] - xf[b, :V].max())
        want = e / (e.sum() + 1e-6)
        np.testing.assert_allclose(gf[b, :V], want, rtol=tol, atol=1e-7 if dt == O.F32 else 1e-4)
        assert abs(gf[b].sum() - 1.0) < (1e-4 if dt == O.F32 else 3e-2)


# ---- top-p ----------------------------------------------------------------------------------------------
def _oracle_topp(probs, u, top_p, end=None):
    B, V = probs.shape
    ids = np.full(B, -1, np.int32)
    seq = np.zeros(B, np.int32)
    fin = np.zeros(B, np.bool_)
    cum = np.zeros(B, np.float32)
    out = np.zeros(B, np.float32)
    end = np.full(B, V - 1, np.int32) if end is None else end
    O.batch_topp_sampling(O.F32, np.ascontiguousarray(probs, np.float32), ids, seq, fin, cum, out,
                          np.asarray(u, np.float32), B, V, end, 0.0, np.asarray(top_p, np.float32), None)
    return ids, seq, fin, cum, out


def test_topp_exact_cases():
    """probabilities that are exact in binary make every comparison of the walk exact
    (sampling_topp_kernels.cu:958-1003): stable descending order, first i with r <= c_i"""
    probs = np.array([[0.25, 0.25, 0.25, 0.25],        # ties keep ascending id order
                      [0.125, 0.5, 0.125, 0.25],
                      [0.125, 0.5, 0.125, 0.25],
                      [0.125, 0.5, 0.125, 0.25],
                      [0.125, 0.5, 0.125, 0.25]], np.float32)
    p = np.array([1.0, 1.0, 1.0, 1.0, 0.5], np.float32)
    u = np.array([0.5, 0.5, 0.75, 0.875, 0.99], np.float32)
    ids, seq, fin, cum, out = _oracle_topp(probs, u, p)
    # row 0: r = 0.5 -> c = .25, .5 -> second entry of the stable order -> id 1
    # row 1: order 1,3,0,2 with c = .5,.75,.875,1; r = .5 -> id 1
    # row 2: r = .75 -> id 3;  row 3: r = .875 -> id 0
    # row 4: max prob 0.5 >= p = 0.5 -> arg-max shortcut whatever the draw
    assert ids.tolist() == [1, 1, 3, 0, 1]
    assert np.allclose(cum, np.log([0.25, 0.5, 0.25, 0.125, 0.5]))
    assert np.array_equal(cum, out)          # no renormalisation for top-p (:986-990)
    assert seq.tolist() == [1, 1, 1, 1, 1]
    assert fin.tolist() == [False, False, True, False, False]


def test_topp_nucleus_property_random_rows():
    rng = np.random.default_rng(17)
    B, V = 48, 2000
    x = rng.standard_normal((B, V)) * 2.5
    e = np.exp(x - x.max(axis=1, keepdims=True))
    probs = (e / e.sum(axis=1, keepdims=True)).astype(np.float32)
    p = rng.uniform(0.3, 0.99, B).astype(np.float32)
    u = (rng.random(B) * 0.98 + 0.01).astype(np.float32)
    ids, _, _, cum, _ = _oracle_topp(probs, u, p)
    for b in range(B):
        pr = probs[b].astype(np.float64)
        order = np.argsort(-pr, kind="stable")
        if pr[order[0]] >= p[b]:
            assert ids[b] == order[0]
            continue
        c = np.cumsum(pr[order])
        r = np.float64(u[b]) * np.float64(p[b])
        j = int(np.searchsorted(c, r, side="left"))
        pos = int(np.nonzero(order == ids[b])[0][0])
        assert abs(pos - j) <= 1 and (pos == j or abs(c[min(pos, j)] - r) < 1e-5)
        np.testing.assert_allclose(cum[b], np.log(pr[ids[b]]), rtol=1e-5, atol=1e-6)


def _topp_rows_for_scan_order():
    """sorted-descending rows whose prefix sums round differently under different summation orders"""
    rng = np.random.default_rng(2024)
    rows = []
    for V, scale in ((2000, 2.5), (3000, 1.0), (1500, 0.3), (5000, 4.0), (6000, 0.05)):
        x = rng.standard_normal(V) * scale
        e = np.exp(x - x.max())
        rows.append((e / e.sum()).astype(np.float32))
    ranks = rng.permutation(4000) + 1.0                     # Zipf(1.1) over a permutation, with noise
    z = np.exp(-1.1 * np.log(ranks) + rng.standard_normal(4000) * 0.5)
    rows.append((z / z.sum()).astype(np.float32))
    return rows


def test_topp_prefix_sum_order_bit_for_bit():
    """The position top-p emits is the first one whose fp32 prefix sum reaches the draw, so the rounding order of
    those sums (cub's BLOCK_SCAN_RAKING with a running prefix over tiles of 256) decides ids whenever a draw
    lies within a bit of a prefix sum. tests/cub_block_scan.py simulates that scan thread by thread from the
    vendored cub sources; on draws chosen so that a plain running sum, a 64 x 4 and a 16 x 16 raking of the same
    terms cross at another position, the oracle must emit exactly the simulated position."""
    import cub_block_scan as C
    disagree = {"running": 0, "raking64x4": 0, "raking16x16": 0}
    checked = deepest = 0
    for probs in _topp_rows_for_scan_order():
        order = np.argsort(-probs, kind="stable")           # the stable descending sort of :1106-1119
        draws = C.discriminating_draws(probs[order])
        assert draws
        for r, pos, alt_pos in draws:
            ids, seq, fin, cum, out = _oracle_topp(probs.reshape(1, -1), [r], [1.0])
            assert ids[0] == order[pos], (len(probs), float(r), pos, alt_pos)
            np.testing.assert_allclose(cum[0], np.log(np.float64(probs[order[pos]])), rtol=1e-5, atol=1e-6)
            checked += 1
            deepest = max(deepest, pos)                     # running totals of many tiles take part
            for name, other in alt_pos.items():
                disagree[name] += int(other != pos)
    # the draw set separates the reference's order from each of the three other orders
    assert checked >= 60 and deepest >= 8 * 256 and all(n >= 15 for n in disagree.values()), (checked, disagree)


def test_topp_prefix_sums_whole_rows_bit_for_bit():
    """every prefix sum of a row, not only the crossing: a draw equal to the simulated c_i must be crossed at the
    first position whose simulated sum reaches it, for a spread of positions along the row (tile seams, segment
    seams of the raking grid, positions inside a segment)"""
    import cub_block_scan as C
    probs = _topp_rows_for_scan_order()[0]
    order = np.argsort(-probs, kind="stable")
    c = C.prefix_sums(probs[order])
    positions = [0, 1, 7, 8, 9, 31, 32, 33, 63, 64, 255, 256, 257, 263, 264, 511, 512, 700, 1023, 1024, 1500]
    rows = np.repeat(probs.reshape(1, -1), len(positions), axis=0)
    u = np.array([c[i] for i in positions], np.float32)
    ids, _, _, _, _ = _oracle_topp(rows, u, np.ones(len(positions), np.float32))
    for b, i in enumerate(positions):
        assert ids[b] == order[C.pick_position(c, c[i])], i


def test_topp_decay_closed_form():
    n = 7
    initial = np.linspace(0.5, 0.95, n).astype(np.float32)
    runtime = (initial * 0.8).astype(np.float32)
    decay = np.full(n, 0.9, np.float32)
    pmin = np.full(n, 0.45, np.float32)
    reset = np.array([5, 5, -1, 5, 5, 5, 5], np.int32)
    ids = np.array([5, 4, 5, 5, 0, 1, 2], np.int32)
    want = np.where(ids == reset, initial, np.maximum((runtime * decay).astype(np.float32), pmin))
    O.compute_topp_decay(runtime, initial, ids, decay, pmin, reset, n)
    assert np.array_equal(runtime, want.astype(np.float32))


# ---- word lists and stop criteria -------------------------------------------------------------------------
def _words(word_list):
    ids, offs = word_list
    out, start = [], 0
    for o in offs:
        if o < 0:
            break
        out.append([int(t) for t in ids[start:o]])
        start = o
    return out


def test_bad_words_against_brute_force():
    rng = np.random.default_rng(18)
    B, V, step = 6, 50, 9
    history = rng.integers(1, V, (step + 1, B)).astype(np.int32)
    for shared in (True, False):
        lists = []
        for b in range(1 if shared else B):
            wl, _ = make_word_list(rng, 10, 4, V, L=48, history=history, step=step - 1, row=b)
            lists.append(wl)
        bad = np.ascontiguousarray(lists[0] if shared else np.stack(lists))
        for dt in DTYPES:
            x = O.to_storage(rng.standard_normal((B, V)).astype(np.float32), dt)
            got = x.copy()
            O.ban_bad_words(dt, got, history, B, B, bad, shared, bad.shape[-1], 0, V, step)
            gf, xf = O.to_f32(got, dt), O.to_f32(x, dt)
            for b in range(B):
                banned = set()
                for w in _words(lists[0] if shared else lists[b]):
                    n = len(w)
                    if n == 0:
                        continue
                    ok = n == 1 or (step >= n - 1 and all(history[step - (n - 1) + t, b] == w[t] for t in range(n - 1)))
                    if ok and 0 < w[-1] < V:
                        banned.add(w[-1])
                for v in range(V):
                    if v in banned:
                        assert gf[b, v] == -np.inf
                    else:
                        assert gf[b, v] == xf[b, v]


def test_stop_words_and_length_against_brute_force():
    rng = np.random.default_rng(19)
    B, V, step = 8, 30, 7
    history = rng.integers(1, V, (step + 1, B)).astype(np.int32)
    lists = []
    for b in range(B):
        wl, words = make_word_list(rng, 6, 3, V, L=24)
        lists.append(wl)
    # plant matches: row 1 ends with its first word, row 4 with its second
    for b, wi in ((1, 0), (4, 1)):
        w = _words(lists[b])[wi]
        history[step - len(w) + 1:step + 1, b] = w
    stop = np.ascontiguousarray(np.stack(lists))
    fin = np.zeros(B, np.bool_)
    O.stop_words_criterion(history, stop, fin, 0, stop.shape[-1], B, B, step)
    for b in range(B):
        want = any(step + 1 >= len(w) and len(w) > 0
                   and all(history[step - (len(w) - 1) + t, b] == w[t] for t in range(len(w)))
                   for w in _words(lists[b]))
        assert fin[b] == want
    assert fin[1] and fin[4]
    limit = np.array([3, 8, 7, 100, 6, 7, 8, 9], np.uint32)
    fin2 = np.array([False, False, False, True, False, False, False, False])
    should = np.zeros(1, np.bool_)
    O.length_criterion(fin2, should, limit, B, step)
    assert fin2.tolist() == [True, False, True, True, True, True, False, False] and not should[0]
    O.length_criterion(fin2, should, np.zeros(B, np.uint32), B, step)
    assert fin2.all() and should[0]


# ---- the layer restatement: routing of (k, p) and the reference's Python known answers ------------------------
def test_python_known_answers_repetition_and_min_length():
    """tests/unittests/th_op/test_th_decode_op.py:233-324: with logits 2 / 1.8 / 1.6 on the last three ids and
    greedy decoding, a repetition penalty of 2 (or presence 0.5 / 1.0) must produce v-1, v-2, v-3, v-1, v-1;
    with the end id made the most probable token, min_length must hold generation open."""
    V = 1024
    for B, kwargs in [(4, dict(repetition_penalty=[2.0])), (256, dict(repetition_penalty=[2.0])),
                      (4, dict(presence_penalty=[0.5])), (4, dict(presence_penalty=[1.0]))]:
        H = 4
        x = np.zeros((B, V), np.float32)
        x[:, V - 1], x[:, V - 2], x[:, V - 3] = 2.0, 1.8, 1.6
        c = Case(O.F32, B, V, V, max_input_length=H, gen_len=5, runtime_top_k=[1], runtime_top_p=[0.0],
                 end_ids=np.zeros(B, np.int32), prompt=np.ones((H, B), np.int32),
                 input_lengths=np.full(B, H, np.int32), **kwargs)
        o = OracleRunner(c)
        for i in range(5):
            o.step(H + i, x, np.full(B, 0.5, np.float32))
        ids = o.snapshot()["output_ids"][H:]
        expect = np.array([V - 1, V - 2, V - 3, V - 1, V - 1], np.int32)
        assert (ids == expect[:, None]).all(), kwargs
    rng = np.random.default_rng(0)
    for method in (dict(runtime_top_k=[1], runtime_top_p=[0.0]), dict(runtime_top_k=[0], runtime_top_p=[0.8])):
        for B, H, min_len, gen in [(4, 4, 2, 4), (4, 4, 32, 40), (64, 6, 4, 8)]:
            c = Case(O.F32, B, V, V, max_input_length=H, gen_len=gen, min_length=[min_len],
                     end_ids=np.zeros(B, np.int32), prompt=rng.integers(1, V, (H, B)).astype(np.int32), **method)
            o = OracleRunner(c)
            for i in range(gen):
                x = rng.standard_normal((B, V)).astype(np.float32)
                x[:, 0] = x.max(axis=1) + 1  # end id is the most probable token
                o.step(H + i, x, uniforms(rng, B))
            snap = o.snapshot()
            assert ((snap["sequence_length"] + 1) >= H + min_len).all(), (method, B, min_len)
            if method["runtime_top_k"] == [1]:
                assert snap["finished"].all()  # greedy: it does stop as soon as it is allowed to


# ---- the steps either side of the path -------------------------------------------------------------------
@pytest.mark.parametrize("batch_first", [False, True])
@pytest.mark.parametrize("shape", [(1, 32, 16), (33, 4, 1000), (9, 3, 5001)])
def test_log_prob_from_logits_closed_form(batch_first, shape):
    """kernels/logprob_kernels.cu:35-135 against the reference test's host expectation
    (tests/unittests/test_logprob_kernels.cu:39-75) evaluated in float64"""
    max_len, batch, V = shape
    Vp = (V + 7) // 8 * 8
    rng = np.random.default_rng(21)
    for dt in DTYPES:
        shp = (batch, max_len, Vp) if batch_first else (max_len, batch, Vp)
        logits = O.to_storage((rng.standard_normal(shp) * 3).astype(np.float32), dt)
        ids = rng.integers(0, V, (batch, max_len) if batch_first else (max_len, batch)).astype(np.int32)
        lengths = rng.integers(1, max_len + 1, batch).astype(np.int32)
        cum, lp = O.log_prob_from_logits(dt, logits, ids, lengths, max_len, batch, V, Vp, batch_first)
        x = O.to_f32(logits, dt).astype(np.float64)
        want = np.zeros(batch)
        for b in range(batch):
            for step in range(1, max_len):
                if step < lengths[b]:
                    vec = (x[b, step - 1] if batch_first else x[step - 1, b])[:V]
                    tok = ids[b, step] if batch_first else ids[step, b]
                    v = vec[tok] - vec.max() - np.log(np.exp(vec - vec.max()).sum())
                    want[b] += v
                    got = lp[b * (max_len - 1) + step - 1] if batch_first else lp[(step - 1) * batch + b]
                    assert abs(got - v) < 1e-5 * max(1.0, abs(v))
        np.testing.assert_allclose(cum, want, rtol=2e-6 * max_len, atol=1e-5)


def test_decode_state_helpers():
    """kernels/decoding_kernels.cu:26-47, :680-694 and kernels/gpt_kernels.cu:329-345"""
    rng = np.random.default_rng(22)
    sent = rng.integers(0, 100, 5).astype(np.int32)
    for dt in DTYPES:
        fin, seq, ids, cum = O.decoding_initialize(dt, sent, 5, 3, 17)
        assert not fin.any() and (seq == 17).all()
        assert np.array_equal(ids, np.repeat(sent, 3))
        big = 65504.0 if dt == O.F16 else 1e20
        assert np.array_equal(cum.reshape(5, 3), np.tile(np.array([0.0, -big, -big], np.float32), (5, 1)))
    buf = rng.integers(0, 50, 77).astype(np.int32)
    want = buf + 9
    O.plus_scalar(buf, 9)
    assert np.array_equal(buf, want)
    a = rng.integers(0, 1000, (37, 53)).astype(np.int32)
    assert np.array_equal(O.transpose_axis01(a, None, 37, 53), a.T)
    # with per-column offsets the source of column i1 starts skipping[i1] rows further down
    big_in = rng.integers(0, 1000, (37 + 4, 53)).astype(np.int32)
    skip = rng.integers(0, 5, 53).astype(np.int32)
    got = O.transpose_axis01(big_in, skip, 37, 53)
    want = np.stack([big_in[skip[i1]:skip[i1] + 37, i1] for i1 in range(53)])
    assert np.array_equal(got, want)


def _finalize_case(rng, batch, beam_width, max_seq_len, ties):
    hyps = 2 * beam_width
    ids = rng.integers(0, 30000, (batch, hyps, max_seq_len + 1)).astype(np.int32)
    lens = rng.integers(0, max_seq_len + 1, (batch, hyps)).astype(np.int32)
    scores = rng.standard_normal((batch, hyps)).astype(np.float32)
    if ties:
        scores = np.round(scores)  # many equal scores: the smaller index must win
    cum = rng.standard_normal((batch, hyps)).astype(np.float32)
    lps = rng.standard_normal((batch, hyps, max_seq_len + 1)).astype(np.float32)
    num = rng.integers(beam_width, hyps + 1, batch).astype(np.int32)
    return ids, lens, scores, cum, lps, num


def finalize_by_numpy(ids, lens, scores, cum, lps, num, beam_width, max_seq_len):
    """the definition, written independently: a stable sort of the valid hypotheses by descending score"""
    batch = ids.shape[0]
    out_ids = np.zeros((batch, beam_width, max_seq_len), np.int32)
    out_lp = np.zeros((batch, beam_width, max_seq_len), np.float32)
    out_len = np.zeros((batch, beam_width), np.int32)
    out_cum = np.zeros((batch, beam_width), np.float32)
    for b in range(batch):
        order = np.argsort(-scores[b, :num[b]].astype(np.float64), kind="stable")[:beam_width]
        for i, j in enumerate(order):
            n = lens[b, j]
            out_len[b, i], out_cum[b, i] = n, cum[b, j]
            out_ids[b, i, :n] = ids[b, j, 1:n + 1]
            out_lp[b, i, :n] = lps[b, j, 1:n + 1]
    return out_ids, out_len, out_cum, out_lp


@pytest.mark.parametrize("beam_width,ties", [(1, False), (2, True), (4, False), (16, True), (100, True)])
def test_finalize_against_a_stable_sort(beam_width, ties):
    """invokeFinalize (kernels/decoding_kernels.cu:697-813; no test of it exists in the reference): the oracle's
    repeated arg-max with the scan from index 0 equals a stable descending sort of the valid hypotheses; the first
    position of every source row is dropped; optional outputs may be absent."""
    rng = np.random.default_rng(900 + beam_width)
    batch, max_seq_len = 5, 23
    ids, lens, scores, cum, lps, num = _finalize_case(rng, batch, beam_width, max_seq_len, ties)
    want = finalize_by_numpy(ids, lens, scores, cum, lps, num, beam_width, max_seq_len)
    got_ids, got_len, got_cum, got_lp = O.finalize(ids, lens, scores, cum, lps, num, beam_width, max_seq_len, batch)
    assert np.array_equal(got_ids, want[0]) and np.array_equal(got_len, want[1])
    assert np.array_equal(got_cum, want[2]) and np.array_equal(got_lp, want[3])
    only_ids = O.finalize(ids, lens, scores, None, None, num, beam_width, max_seq_len, batch)
    assert np.array_equal(only_ids[0], want[0]) and only_ids[2] is None and only_ids[3] is None


def _softmax_by_thread_simulation(x, n, n_padded, max_t):
    """addBiasSoftMax (sampling_topp_kernels.cu:1308-1344) for one unfinished fp32 row without a bias, written
    from the reference source independently of the oracle: BLK = min(n, 1024) threads, thread t walks columns
    t, t + BLK, ...; blockReduceSum (reduce_kernel_utils.cuh:73-103) = xor butterfly 16, 8, 4, 2, 1 inside each warp
    of 32, lane-0 partials to shared memory, the first warp adds them with the same butterfly. All arithmetic in
    np.float32, exp from the oracle (the one departure both sides share)."""
    f32 = np.float32
    blk = min(n, 1024)
    vals = np.full(n_padded, -max_t, f32)
    vals[:n] = x[:n]
    mx = vals.max()  # (a maximum does not depend on its order)
    if blk < 1024:
        mx = max(mx, f32(-1e20))  # blockReduceMax fills missing warps with -1e20f
    e = O.expf((vals - mx).astype(f32))
    part = np.zeros(((blk + 31) // 32) * 32, f32)
    for t in range(blk):
        s = f32(0.0)
        for v in range(t, n_padded, blk):
            s = f32(s + e[v])
        part[t] = s

    def butterfly(a):  # every lane adds its partner's value, all lanes at once, inside warps of 32
        a = a.copy()
        lanes = np.arange(a.size)
        for mask in (16, 8, 4, 2, 1):
            a = (a + a[lanes ^ mask]).astype(f32)
        return a
    warp_sums = butterfly(part)[0::32]  # lane 0 of every warp
    second = np.zeros(32, f32)
    for lane in range(32):
        if lane < blk / 32.0:  # (threadIdx.x < blockDim.x / 32.f)
            second[lane] = warp_sums[lane]
    total = butterfly(second)[0]
    denom = f32(total + f32(1e-6))
    return (e / denom).astype(f32), total


def test_softmax_summation_order_bit_for_bit():
    """The order of the softmax's sum decides the last bits of every probability, and sampled ids depend on them.
    Rows whose terms span many orders of magnitude make the order visible: the oracle must equal the thread-by-thread
    simulation bit for bit, and on the same rows a plain running sum of the same terms ends in other bits (so the
    test would catch a different order). Full blocks, a block shorter than 1024 threads with a partial warp, padding."""
    rng = np.random.default_rng(77)
    max_t = np.float32(3.4028234663852886e38)
    seen_other_order_differs = 0
    for n, n_padded in ((5000, 5000), (4097, 4104), (1000, 1000), (70, 72), (33000, 33024)):
        x = (rng.standard_normal(n_padded) * 6.0 + rng.integers(-3, 4, n_padded) * 4.0).astype(np.float32)
        got = x.copy().reshape(1, n_padded)
        O.add_bias_softmax(O.F32, got, None, np.zeros(1, np.int32), np.zeros(1, np.bool_), 1, n_padded, n)
        want, total = _softmax_by_thread_simulation(x, n, n_padded, max_t)
        assert np.array_equal(got[0].view(np.uint32), want.view(np.uint32)), (n, n_padded)
        # sensitivity: other summation orders of the same terms end in other bits
        vals = np.full(n_padded, -max_t, np.float32)
        vals[:n] = x[:n]
        mx = vals.max() if min(n, 1024) == 1024 else max(vals.max(), np.float32(-1e20))
        e = O.expf((vals - mx).astype(np.float32))
        running = np.float32(0.0)
        for v in e:
            running = np.float32(running + v)
        seen_other_order_differs += int(running != total)
    assert seen_other_order_differs >= 3


# ---- beam search step (invokeTopkSoftMax) -----------------------------------------------------------------------
def _log_softmax64(x):
    x = x.astype(np.float64)
    m = x.max(axis=-1, keepdims=True)
    return x - m - np.log(np.exp(x - m).sum(axis=-1, keepdims=True))


def _run_oracle_beam(c, dt, batch, K, V, diversity=0.0, length_penalty=0.0):
    rc = O.topk_softmax(dt, c["log_probs"], None, c["finished"], c["sequence_lengths"], c["cum_log_probs"],
                        c["output_log_probs"], c["ids"], c["hyps"], batch, K, V, c["end_ids"], diversity,
                        length_penalty)
    assert rc == 0


@pytest.mark.parametrize("K,V", [(2, 50), (3, 1000), (4, 50257), (8, 3000), (17, 700), (64, 2000)])
def test_beam_step_without_hypotheses_is_the_global_top_k(K, V):
    """No hypotheses, no penalties: the next beams are the K largest of cum_log_probs[beam] + log_softmax(row)
    over all K * V continuations of a batch entry (a definition that knows nothing of the 2K candidates per beam),
    in descending order, and the step's log-prob is the difference of the cumulative ones."""
    from helpers import make_beam_case
    rng = np.random.default_rng(K * 1000 + V)
    batch = 3
    c = make_beam_case(rng, O.F32, batch, K, V, with_hyps=False, finished_frac=0.0)
    old_cum = c["cum_log_probs"].copy()
    total = old_cum.reshape(batch, K, 1).astype(np.float64) + _log_softmax64(c["log_probs"]).reshape(batch, K, V)
    _run_oracle_beam(c, O.F32, batch, K, V)
    for b in range(batch):
        flat = total[b].reshape(-1)
        order = np.argsort(-flat, kind="stable")[:K]
        got = c["ids"][b] - b * K * V
        assert len(set(got.tolist())) == K and got.min() >= 0 and got.max() < K * V
        # the same continuations in the same order, except where two of them are closer than fp32 resolves
        np.testing.assert_allclose(flat[got], flat[order], rtol=2e-6, atol=0)
        distinct = np.abs(np.diff(flat[np.argsort(-flat, kind="stable")[:K + 1]])) > 1e-4
        clear = np.concatenate([[True], distinct[:-1]]) & distinct
        assert np.array_equal(got[clear], order[clear]), b
        np.testing.assert_allclose(c["cum_log_probs"][b * K:(b + 1) * K], flat[got], rtol=1e-5)
        np.testing.assert_allclose(c["output_log_probs"][b], flat[got] - old_cum[b * K + got // V], rtol=1e-4,
                                   atol=1e-5)


def test_beam_step_finished_beams_offer_their_end_token_only():
    """A finished beam's row is MAX_T at its end id and -MAX_T elsewhere: its only finite continuation is the end
    token at an unchanged cumulative log-prob (no hypotheses kept here, so it stays a beam)."""
    from helpers import make_beam_case
    rng = np.random.default_rng(5)
    batch, K, V = 2, 4, 300
    c = make_beam_case(rng, O.F32, batch, K, V, with_hyps=False, finished_frac=0.0)
    c["finished"][[1, 6]] = True
    c["cum_log_probs"][[1, 6]] = np.float32(-0.25)   # better than anything a live beam can reach
    _run_oracle_beam(c, O.F32, batch, K, V)
    assert c["ids"][0, 0] == 1 * V + c["end_ids"][0] and c["cum_log_probs"][0] == np.float32(-0.25)
    assert c["ids"][1, 0] == 6 * V + c["end_ids"][1] and c["cum_log_probs"][4] == np.float32(-0.25)
    assert c["output_log_probs"][0, 0] == 0.0 and c["output_log_probs"][1, 0] == 0.0
    # no other continuation of a finished beam is ever chosen
    for b in range(batch):
        for i in range(1, K):
            assert c["ids"][b, i] // V not in (1, 6)


@pytest.mark.parametrize("length_penalty", [0.0, 0.7])
def test_beam_step_moves_end_tokens_to_the_hypotheses(length_penalty):
    """The best continuation of entry 0 is its beam 2 ending: it becomes hypothesis number num_beams with the
    beam's history traced back through parent_ids, the step as its length, cum / length^penalty as its score
    (float64 here), and it is not among the next beams; entry 1 already holds K hypotheses and is left alone."""
    from helpers import make_beam_case
    rng = np.random.default_rng(11)
    batch, K, V, step, L = 2, 3, 400, 4, 9
    c = make_beam_case(rng, O.F32, batch, K, V, step=step, max_seq_len=L, finished_frac=0.0, full_frac=0.0,
                       end_spike=0.0)
    h = c["hyps"]
    h["num_beams"][:] = [1, K]
    h["min_normed_scores"][:] = [h["normed_scores"][0, 0], h["normed_scores"][1, :K].min()]
    c["sequence_lengths"][:] = step
    end = int(c["end_ids"][0])
    c["log_probs"][2, end] = 40.0           # beam 2 of entry 0 ends with near certainty
    c["cum_log_probs"][2] = np.float32(-0.5)
    before = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in h.items()}
    old_ids, old_cum = c["ids"].copy(), c["cum_log_probs"].copy()
    _run_oracle_beam(c, O.F32, batch, K, V, length_penalty=length_penalty)
    assert h["num_beams"].tolist() == [2, K]
    lsm = _log_softmax64(c["log_probs"][2])[end]
    cum = -0.5 + lsm
    np.testing.assert_allclose(h["cum_log_probs"][0, 1], cum, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(h["normed_scores"][0, 1], cum / (step + 1) ** length_penalty, rtol=1e-5, atol=1e-6)
    assert h["sequence_lengths_tgt"][0, 1] == step and h["output_ids_tgt"][0, 1, step] == end
    beam = 2
    for j in range(step - 1, -1, -1):       # the path, followed independently
        assert h["output_ids_tgt"][0, 1, j] == before["output_ids_src"][j, 0, beam]
        assert h["log_probs"][0, 1, j] == before["log_probs_src"][j, 0, beam]
        beam = before["parent_ids_src"][j, 0, beam]
    np.testing.assert_allclose(h["log_probs"][0, 1, step], lsm, atol=1e-5)
    assert h["min_normed_scores"][0] == min(before["min_normed_scores"][0], h["normed_scores"][0, 1])
    assert all(int(t) % V != end or int(t) // V != 2 for t in c["ids"][0])
    assert not h["is_done"][0]
    # entry 1: K hypotheses already: nothing of it moves (the kernel returns before it selects)
    assert np.array_equal(c["ids"][1], old_ids[1]) and np.array_equal(c["cum_log_probs"][K:], old_cum[K:])
    assert np.array_equal(h["output_ids_tgt"][1], before["output_ids_tgt"][1])


# ---- the kernels around the beam search step ---------------------------------------------------------------------
def _beam_penalties_by_numpy(x, bias, V, Vp, K, step, out_ids, parents, input_lengths, seq, end_ids, max_input,
                             temperature, penalty, multiplicative, min_length):
    """the description, independently: (x + bias) * 1/(T + 1e-6) with pads masked, every token of a beam's own
    history (followed back through the parent beams, prompt padding skipped) penalised once from its value before
    the penalty, the end id masked while the sequence is shorter than min_length; fp32 operation by operation"""
    f = np.float32
    rows = x.shape[0]
    y = x.astype(f).copy()
    if bias is not None or temperature != 1.0 or V != Vp:
        inv = f(1.0) / (f(temperature) + f(1e-6))
        b = bias.astype(f) if bias is not None else np.zeros(Vp, f)
        y[:, :V] = (y[:, :V] + b[:V]) * inv
        y[:, V:] = -np.finfo(f).max
    if penalty is not None and step > 0:
        before = y.copy()
        for r in range(rows):
            b_, beam = r // K, r % K
            tokens = [out_ids[step - 1, r]]
            for i in range(step - 2, -1, -1):
                if input_lengths[r] <= i < max_input:
                    continue
                beam = parents[i, b_ * K + beam]
                tokens.append(out_ids[i, b_ * K + beam])
            for tok in set(int(t) for t in tokens):
                v = before[r, tok]
                y[r, tok] = (v / f(penalty) if v > 0 else v * f(penalty)) if multiplicative else v - f(penalty)
    if step - max_input < min_length:
        for r in range(rows):
            if seq[r] + 1 - max_input < min_length:
                y[r, end_ids[r // K]] = -np.finfo(f).max
    return y


@pytest.mark.parametrize("multiplicative", [True, False])
@pytest.mark.parametrize("with_bias,temperature,V,Vp", [(False, 1.0, 300, 300), (True, 0.7, 300, 300),
                                                        (False, 1.3, 301, 304), (True, 1.0, 1000, 1024)])
def test_beam_penalties_against_the_description(multiplicative, with_bias, temperature, V, Vp):
    from helpers import make_beam_history
    rng = np.random.default_rng(V + Vp + int(multiplicative))
    batch, K, step, L, max_input = 3, 4, 7, 12, 4
    out_ids, parents, input_lengths = make_beam_history(rng, batch, K, V, step, L, max_input)
    x = (rng.standard_normal((batch * K, Vp)) * 3).astype(np.float32)
    bias = rng.standard_normal(Vp).astype(np.float32) if with_bias else None
    seq = rng.integers(max_input, max_input + 5, batch * K).astype(np.int32)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    penalty, min_length = (1.3 if multiplicative else 0.6), 5
    want = _beam_penalties_by_numpy(x, bias, V, Vp, K, step, out_ids, parents, input_lengths, seq, end_ids, max_input,
                                    temperature, penalty, multiplicative, min_length)
    got = x.copy()
    O.beam_add_bias_apply_penalties(O.F32, step, got, out_ids[step - 1].copy(), out_ids, parents, input_lengths, seq,
                                    bias, 0, max_input, batch, batch, K, V, Vp, end_ids, temperature, penalty,
                                    1 if multiplicative else 0, min_length)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the neutral penalty and a step past min_length leave the row alone
    same = x.copy()
    O.beam_add_bias_apply_penalties(O.F32, 50, same, out_ids[step - 1].copy(),
                                    out_ids, parents, input_lengths, seq, None, 0, max_input, batch, batch, K, Vp, Vp,
                                    end_ids, 1.0, 1.0 if multiplicative else 0.0, 1 if multiplicative else 0, 0)
    assert np.array_equal(same, x)


def test_beam_update_and_cache_indirection_against_the_description():
    rng = np.random.default_rng(21)
    batch, K, Vp, L, step = 4, 3, 500, 9, 5
    word = (rng.integers(0, K, (batch, K)) + np.arange(batch)[:, None] * K) * Vp + rng.integers(0, Vp, (batch, K))
    word = word.astype(np.int32).reshape(-1)
    end_ids = rng.integers(0, Vp, batch).astype(np.int32)
    word[2] = (2 // K * K + 1) * Vp + end_ids[0]     # row 2 continues beam 1 of entry 0 with the end token
    word[7] = -7                                      # a slot the step never wrote: the caller's old contents
    finished = rng.random(batch * K) < 0.3
    seq = rng.integers(3, 9, batch * K).astype(np.int32)
    num_beams = np.array([0, K, 1, 2], np.int32)
    f, s_, w = finished.copy(), seq.copy(), word.copy()
    parent, out = np.full(batch * K, -1, np.int32), np.full(batch * K, -1, np.int32)
    O.beam_update(f, parent, s_, w, out, num_beams, 0, batch, K, Vp, end_ids)
    counted = np.where(finished, seq, seq + 1)
    for i in range(batch * K):
        b = i // K
        beam, tok = ((word[i] // Vp) % K, word[i] % Vp) if word[i] >= 0 else (i % K, end_ids[b])
        assert parent[i] == beam and w[i] == tok and out[i] == tok
        assert s_[i] == counted[b * K + beam]
        assert f[i] == (tok == end_ids[b] or num_beams[b] == K)
    assert f[2] and f[K:2 * K].all()
    # cache indirection: position `step` names the beam itself, earlier ones come from the parent beam's row
    src = rng.integers(0, K, (batch, K, L)).astype(np.int32)
    tgt = np.full((batch, K, L), -7, np.int32)
    O.update_indir_cache(tgt, src, parent, f, batch, K, L, step)
    for b in range(batch):
        for k in range(K):
            if f[b * K + k]:
                assert (tgt[b, k] == -7).all()
                continue
            assert tgt[b, k, step] == k
            assert np.array_equal(tgt[b, k, :step], src[b, parent[b * K + k], :step])
            assert (tgt[b, k, step + 1:] == -7).all()
    # a step beyond the window wraps around: every position of the window is rewritten
    tgt2 = np.full((batch, K, L), -7, np.int32)
    O.update_indir_cache(tgt2, src, parent, np.zeros(batch * K, bool), batch, K, L, L + 3)
    assert (tgt2 != -7).all() and all(tgt2[b, k, (L + 3) % L] == k for b in range(batch) for k in range(K))


def test_word_lists_with_beams_against_the_description():
    """bad words and stop words with beam_width > 1: a word matches a beam when the beam's own history, read backwards
    through the parent beams, ends with it (bad words: with all but its last token, one step earlier); restated here
    by building every beam's history first and comparing lists"""
    rng = np.random.default_rng(31)
    batch, K, V, step, L = 3, 4, 30, 6, 48
    rows = batch * K
    out_ids = rng.integers(1, V, (step + 1, rows)).astype(np.int32)
    parents = rng.integers(0, K, (step + 1, rows)).astype(np.int32)

    def history(row, last, n):
        """the n tokens ending at time `last` of the beam `row`, oldest first; None if the chain leaves the beams"""
        b, beam, toks = row // K, row % K, []
        for t in range(last, last - n, -1):
            toks.append(int(out_ids[t, b * K + beam]))
            beam = int(parents[t, b * K + beam])
            if not 0 <= beam < K:
                return None
        return toks[::-1]

    lists = np.zeros((batch, 2, L), np.int32)
    lists[:, 1, :] = -1
    words = {}
    for b in range(batch):
        flat, ends, words[b] = [], [], []
        for w in range(10):
            n = int(rng.integers(1, 4))
            if rng.random() < 0.6:
                word = history(b * K + int(rng.integers(0, K)), step - 1, n - 1) + [int(rng.integers(1, V))]
            else:
                word = [int(x) for x in rng.integers(1, V, n)]
            words[b].append(word)
            flat += word
            ends.append(len(flat))
        lists[b, 0, :len(flat)], lists[b, 1, :len(ends)] = flat, ends
    x = np.zeros((rows, V), np.float32)
    O.ban_bad_words_beams(O.F32, x, out_ids, parents, batch, batch, K, lists, False, L, 0, V, step)
    for r in range(rows):
        banned = {w[-1] for w in words[r // K] if len(w) == 1 or history(r, step - 1, len(w) - 1) == w[:-1]}
        assert set(np.nonzero(np.isinf(x[r]))[0].tolist()) == banned, r
    # stop words: the same lists, now matched including the token of `step`
    fin = np.zeros(rows, np.bool_)
    stop = lists.copy()
    for b in range(batch):      # make some of them end with what a beam just wrote
        w0 = history(b * K + 1, step, 2)
        stop[b, 0, :2], stop[b, 1, 0] = w0, 2
        words[b][0] = w0
        rest = [w for w in words[b][1:]]
        flat = w0 + [t for w in rest for t in w]
        stop[b, 0, :len(flat)] = flat
        stop[b, 1, :len(words[b])] = np.cumsum([len(w) for w in words[b]])
    O.stop_words_criterion_beams(out_ids, parents, stop, fin, 0, L, batch, batch, K, step)
    for r in range(rows):
        want = any(history(r, step, len(w)) == w for w in words[r // K])
        assert fin[r] == want, r
    assert fin.any()

