"""DynamicDecodeLayer end to end on the GPU (C handle API -> host C++ layers -> C ABI -> HIP kernels)
against (a) the reference tests' known-answer id sets and (b) the CPU oracle on seeded scenarios shaped
like the benchmark configurations, with injected draws. ids / flags / lengths: bit-exact; log-probs:
1e-5 relative (fp32), 2e-3 (fp16 / bf16)."""
import json
import os

import numpy as np
import pytest

import ft_oracle as O
from decode_harness import Case, OracleRunner, ProductRunner, compare, kernel_sequence
from helpers import DTYPES, DTYPE_NAMES, make_logits, make_word_list, to_numpy, to_torch, uniforms

pytestmark = pytest.mark.gpu

KAT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "sampling_layer_kat.json")))


def _kat_logits(dt):
    rows = []
    for row in KAT["logits_per_step"]:
        rows.append([-np.finfo(np.float32).max if v == "-FLT_MAX" else v for v in row])
    return [O.to_storage(np.tile(np.array(r, np.float32), (KAT["batch_size"], 1)), dt) for r in rows]


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("kat", KAT["cases"], ids=lambda c: c["name"])
@pytest.mark.parametrize("logprobs", [True, False], ids=["logprobs", "fused"])
def test_reference_known_answer_sets(dt, kat, logprobs):
    """tests/unittests/test_sampling_layer.cu:271-313: every draw must land in the expected set; here the
    layer's own generator supplies the draws (seeds 0..9) and, separately, the oracle must agree id for id
    on injected draws."""
    B, V = KAT["batch_size"], KAT["vocab_size"]
    logits = _kat_logits(dt)
    local = B // 3 if kat["use_local_batch"] else B
    ite = 1 if kat["use_local_batch"] else 0
    for seed in range(10):
        c = Case(dt, B, V, V, gen_len=3, local_batch=local, runtime_top_k=kat["top_k"], runtime_top_p=kat["top_p"],
                 end_ids=np.full(B, KAT["end_id"], np.int32), with_finished=False, with_seq_len=False,
                 with_cum=logprobs, with_out_lp=logprobs, random_seed=[seed])
        p = ProductRunner(c)
        for step in range(3):
            p.step(step, logits[step], None, ite=ite)
        ids = p.snapshot()["output_ids"]
        for step in range(3):
            for b in range(B):
                assert int(ids[step, b]) in kat["expected"][step][b], (kat["name"], seed, step, b, ids)
    rng = np.random.default_rng(5)
    for trial in range(4):
        c = Case(dt, B, V, V, gen_len=3, local_batch=local, runtime_top_k=kat["top_k"], runtime_top_p=kat["top_p"],
                 end_ids=np.full(B, KAT["end_id"], np.int32), with_finished=False, with_seq_len=False,
                 with_cum=logprobs, with_out_lp=logprobs)
        p, o = ProductRunner(c), OracleRunner(c)
        for step in range(3):
            u = uniforms(rng, B)
            p.step(step, logits[step], u, ite=ite)
            o.step(step, logits[step], u, ite=ite)
            compare(p.snapshot(), o.snapshot(), dt, check_logits=False, where="%s step %d" % (kat["name"], step))
        ids = o.snapshot()["output_ids"]
        for step in range(3):
            for b in range(B):
                assert int(ids[step, b]) in kat["expected"][step][b]  # pins the oracle as well


def _history(rng, steps, batch, V, zipf=None):
    if zipf:
        return np.minimum(rng.zipf(zipf, (steps, batch)), V - 1).astype(np.int32)
    return rng.integers(0, V, (steps, batch)).astype(np.int32)


def _run_case(c, rng, steps, logits_fn, check_logits, ite=0):
    p, o = ProductRunner(c), OracleRunner(c)
    for i in range(steps):
        step = c.max_input_length + i
        logits = logits_fn(i)
        u = uniforms(rng, c.batch)
        p.step(step, logits, u, ite=ite)
        o.step(step, logits, u, ite=ite)
        compare(p.snapshot(), o.snapshot(), c.dt, check_logits, where="step %d" % step)
    return p.snapshot()


@pytest.mark.parametrize("logprobs", [True, False], ids=["logprobs", "fused"])
def test_config1_cpu_reference_step(logprobs):
    """Benchmark configuration 1: batch 8, vocab 50257 fp32 N(0,2), repetition penalty 1.2 over 64 prior ids,
    top_k 40, end_id 50256, log-probs on."""
    rng = np.random.default_rng(1)
    B, V = 8, 50257
    c = Case(O.F32, B, V, V, max_input_length=64, gen_len=3, runtime_top_k=[40], runtime_top_p=[0.0],
             temperature=[1.0], repetition_penalty=[1.2], end_ids=np.full(B, 50256, np.int32),
             prompt=_history(rng, 64, B, V), with_cum=logprobs, with_out_lp=logprobs)
    # (rows of 50257 fp32 columns start off 16-byte boundaries; both variants take a fused step, which leaves the
    # caller's logits alone)
    _run_case(c, rng, 3, lambda i: make_logits(rng, O.F32, B, V, V, 2.0), check_logits=False)


@pytest.mark.parametrize("logprobs", [False, True], ids=["fused", "logprobs"])
def test_config2_batched_topk_fp16_padded(logprobs):
    """Benchmark configuration 2 (rows cut to 48): vocab 50257 padded to 51200 fp16, N(0,3) + spikes, per-row
    k in {1,4,16,40,64,1024}, per-row temperature U[0.5,1.5]."""
    rng = np.random.default_rng(2)
    B, V, Vp = 48, 50257, 51200
    ks = rng.choice([1, 4, 16, 40, 64, 1024], B).astype(np.uint32)
    c = Case(O.F16, B, V, Vp, gen_len=2, runtime_top_k=ks, temperature=rng.uniform(0.5, 1.5, B),
             end_ids=np.full(B, 50256, np.int32), with_cum=logprobs, with_out_lp=logprobs)
    _run_case(c, rng, 2, lambda i: make_logits(rng, O.F16, B, V, Vp, 3.0, spikes=8), check_logits=logprobs)


def _zipf_logits(rng, dt, B, V):
    base = -1.1 * np.log(np.arange(1, V + 1, dtype=np.float64))
    base = base - np.log(np.exp(base).sum())
    x = np.empty((B, V), np.float32)
    for b in range(B):
        x[b] = (base[rng.permutation(V)] + rng.standard_normal(V) * 0.5).astype(np.float32)
    return O.to_storage(x, dt)


def test_config3_batched_topp_decay():
    """Benchmark configuration 3 (rows cut to 24, 6 steps): vocab 128256 fp32 Zipf(1.1) log-softmax + N(0,0.5),
    top_k 0, per-row top_p U[0.5,0.99], decay 0.9, min 0.3, reset id 13."""
    rng = np.random.default_rng(3)
    B, V = 24, 128256
    c = Case(O.F32, B, V, V, gen_len=6, runtime_top_k=[0], runtime_top_p=rng.uniform(0.5, 0.99, B),
             top_p_decay=np.full(B, 0.9), top_p_min=np.full(B, 0.3), top_p_reset_ids=np.full(B, 13),
             end_ids=np.full(B, V - 1, np.int32), with_cum=True, with_out_lp=True)
    # by default the step samples straight from the logits and leaves them alone; with the switch that asks for the
    # reference's side effects the logits end up as probabilities, bit for bit
    _run_case(c, rng, 6, lambda i: _zipf_logits(rng, O.F32, B, V), check_logits=False)
    with kernel_sequence():
        _run_case(c, rng, 3, lambda i: _zipf_logits(rng, O.F32, B, V), check_logits=True)


@pytest.mark.parametrize("freq", [None, 0.3], ids=["presence", "presence+frequency"])
def test_config4_penalty_mask_heavy(freq):
    """Benchmark configuration 4 (rows cut to 32, history 512): vocab 32000 bf16, Zipf(1.2) history, min_length beyond
    the current step (end id masked), presence (+frequency) penalty, bad words len 1-4, stop words len 1-3,
    top_k 50."""
    rng = np.random.default_rng(4)
    B, V, H = 32, 32000, 512
    prompt = _history(rng, H, B, V, zipf=1.2)
    bad = np.stack([make_word_list(rng, 64, 4, V, L=200, history=np.vstack([prompt, prompt[:2]]), step=H, row=b)[0]
                    for b in range(B)])
    stop = np.stack([make_word_list(rng, 16, 3, V, L=48)[0] for b in range(B)])
    c = Case(O.BF16, B, V, V, max_input_length=H, gen_len=3, runtime_top_k=[50], presence_penalty=[0.5],
             frequency_penalty=None if freq is None else [freq], min_length=[H + 52],
             end_ids=np.full(B, 2, np.int32), prompt=prompt, bad_words=bad, stop_words=stop,
             input_lengths=rng.integers(H // 2, H + 1, B))
    snap = _run_case(c, rng, 3, lambda i: make_logits(rng, O.BF16, B, V, V, 2.0), check_logits=False)
    assert not (snap["output_ids"][H:] == 2).any()  # min_length keeps the end id away


def test_config4_stop_words_fire_and_shared_bad_words():
    rng = np.random.default_rng(44)
    B, V, H = 8, 500, 6
    prompt = _history(rng, H, B, V)
    bad, _ = make_word_list(rng, 20, 3, V, L=64)
    c0 = Case(O.F32, B, V, V, max_input_length=H, gen_len=4, runtime_top_k=[1], prompt=prompt, bad_words=bad)
    # greedy first, to learn which token each row produces; then make it (and a 2-gram) a stop word
    o = OracleRunner(c0)
    logits = [make_logits(rng, O.F32, B, V, V, 2.0) for _ in range(4)]
    u = np.ones(B, np.float32)
    o.step(H, logits[0], u)
    first = o.snapshot()["output_ids"][H]
    stop = np.zeros((B, 2, 8), np.int32)
    stop[:, 1, :] = -1
    for b in range(B):
        if b % 2 == 0:
            stop[b, 0, 0], stop[b, 1, 0] = first[b], 1
        else:
            stop[b, 0, :2], stop[b, 1, 0] = [prompt[H - 1, b], first[b]], 2
    c = Case(O.F32, B, V, V, max_input_length=H, gen_len=4, runtime_top_k=[1], prompt=prompt, bad_words=bad,
             stop_words=stop, sequence_limit_length=np.full(B, H + 2, np.uint32))
    p, o = ProductRunner(c), OracleRunner(c)
    for i in range(4):
        p.step(H + i, logits[i], u)
        o.step(H + i, logits[i], u)
        compare(p.snapshot(), o.snapshot(), O.F32, check_logits=False, where="step %d" % i)
        if i == 0:
            assert p.snapshot()["finished"].all()  # every planted stop word fired
    assert bool(p.snapshot()["should_stop"][0])


@pytest.mark.parametrize("dt", [O.F16, O.F32], ids=lambda d: DTYPE_NAMES[d])
def test_config5_full_loop(dt):
    """Benchmark configuration 5 (rows cut to 40, vocab 152064, 12 steps): k=64 then p=0.9, temperature 0.8,
    repetition penalty 1.1, log-probs, finished / sequence_length / length-limit updates."""
    rng = np.random.default_rng(5)
    B, V, H = 40, 152064, 4
    end = 7
    c = Case(dt, B, V, V, max_input_length=H, gen_len=12, runtime_top_k=[64], runtime_top_p=[0.9], temperature=[0.8],
             repetition_penalty=[1.1], end_ids=np.full(B, end, np.int32), prompt=_history(rng, H, B, V),
             with_cum=True, with_out_lp=True, sequence_limit_length=rng.integers(H + 3, H + 12, B))

    def logits_fn(i):
        x = make_logits(rng, dt, B, V, V, 2.5)
        xf = O.to_f32(x, dt)
        xf[rng.random(B) < 0.15, end] = 30.0  # some rows finish early
        return O.to_storage(xf, dt)

    # the fused step with log-probs (two reads of the logits, none mutated), then the reference's kernel sequence,
    # whose in-place results (penalised logits turned into probabilities) must match the oracle's bit for bit
    for sequence in (False, True):
        with kernel_sequence(sequence):
            snap = _run_case(c, rng, 12, logits_fn, check_logits=sequence)
        assert snap["finished"].all() and bool(snap["should_stop"][0])


def test_headline_step_topk_topp_penalty_fused():
    """the benchmark's workload at reduced batch: vocab 128256 fp32, k=64 and p=0.9, temperature,
    repetition penalty, 8 steps, fused path (no log-probs)."""
    rng = np.random.default_rng(6)
    B, V, H = 16, 128256, 32
    c = Case(O.F32, B, V, V, max_input_length=H, gen_len=8, runtime_top_k=[64], runtime_top_p=[0.9],
             temperature=rng.uniform(0.6, 1.2, B), repetition_penalty=[1.1], prompt=_history(rng, H, B, V),
             min_length=[3], input_lengths=rng.integers(8, H + 1, B))
    _run_case(c, rng, 8, lambda i: make_logits(rng, O.F32, B, V, V, 2.5), check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_mixed_batch_with_bias_and_windows(dt):
    """rows split between the two layers (k>0 / k==0,p>0 / greedy), embedding bias, unaligned vocab,
    two micro-batch windows (ite 0 and 1)."""
    rng = np.random.default_rng(7 + dt)
    B, V, Vp, H = 12, 1001, 1003, 5
    ks = np.array([4, 0, 0, 1, 8, 0, 30, 0, 2, 0, 0, 5], np.uint32)
    ps = np.array([0.0, 0.6, 0.0, 0.3, 0.9, 0.8, 1.0, 0.95, 0.5, 0.4, 0.7, 0.0], np.float32)
    bias = O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt)
    for logprobs in (False, True):
        c = Case(dt, B, V, Vp, max_input_length=H, gen_len=4, local_batch=6, runtime_top_k=ks, runtime_top_p=ps,
                 temperature=rng.uniform(0.5, 1.5, B), presence_penalty=rng.uniform(0, 1, B),
                 embedding_bias=bias, prompt=_history(rng, H, B, V), with_cum=logprobs, with_out_lp=logprobs)
        p, o = ProductRunner(c), OracleRunner(c)
        for i in range(4):
            logits = make_logits(rng, dt, B, V, Vp, 2.0)
            u = uniforms(rng, B)
            for ite in (0, 1):
                # each window works on its own copy of the step's logits in both implementations
                p.step(H + i, logits, u, ite=ite)
                o.step(H + i, logits, u, ite=ite)
                compare(p.snapshot(), o.snapshot(), dt, check_logits=False, where="step %d ite %d" % (i, ite))


def test_python_kats_repetition_and_min_length():
    """tests/unittests/th_op/test_th_decode_op.py:233-324: with logits 2 / 1.8 / 1.6 on the last three ids and
    greedy decoding, a repetition penalty of 2 (or presence 0.5 / 1.0) must produce v-1, v-2, v-3, v-1, v-1;
    with the end id made the most probable token, min_length must hold generation open."""
    import torch
    V = 1024
    for B, kwargs in [(4, dict(repetition_penalty=[2.0])), (2048, dict(repetition_penalty=[2.0])),
                      (4, dict(presence_penalty=[0.5])), (4, dict(presence_penalty=[1.0])),
                      (2048, dict(presence_penalty=[0.5]))]:
        H = 4
        x = np.zeros((B, V), np.float32)
        x[:, V - 1], x[:, V - 2], x[:, V - 3] = 2.0, 1.8, 1.6
        c = Case(O.F32, B, V, V, max_input_length=H, gen_len=5, runtime_top_k=[1], runtime_top_p=[0.0],
                 end_ids=np.zeros(B, np.int32), prompt=np.ones((H, B), np.int32),
                 input_lengths=np.full(B, H, np.int32), **kwargs)
        p = ProductRunner(c)
        for i in range(5):
            p.step(H + i, x, None)
        ids = p.snapshot()["output_ids"][H:]
        expect = np.array([V - 1, V - 2, V - 3, V - 1, V - 1], np.int32)
        assert (ids == expect[:, None]).all(), kwargs
    rng = np.random.default_rng(0)
    for method in (dict(runtime_top_k=[1], runtime_top_p=[0.0]), dict(runtime_top_k=[0], runtime_top_p=[0.8])):
        for B, H, min_len, gen in [(4, 4, 2, 4), (4, 4, 32, 40), (2048, 6, 4, 8)]:
            c = Case(O.F32, B, V, V, max_input_length=H, gen_len=gen, min_length=[min_len],
                     end_ids=np.zeros(B, np.int32), prompt=rng.integers(1, V, (H, B)).astype(np.int32), **method)
            p = ProductRunner(c)
            for i in range(gen):
                x = rng.standard_normal((B, V)).astype(np.float32)
                x[:, 0] = x.max(axis=1) + 1  # end id is the most probable token
                p.step(H + i, x, None)
            snap = p.snapshot()
            assert ((snap["sequence_length"] + 1) >= H + min_len).all(), (method, B, min_len)
            if method["runtime_top_k"] == [1]:
                assert snap["finished"].all()  # greedy: it does stop as soon as it is allowed to


def test_seed_reproducibility():
    """tests/unittests/test_sampling_layer.cu:703-785: rows with the same seed sample the same ids; one seed
    for the whole batch or one per row."""
    rng = np.random.default_rng(9)
    B, V = 6, 4000
    for seeds in ([0], [0, 0, 0, 1, 1, 1]):
        for kp in (dict(runtime_top_k=[30], runtime_top_p=[0.0]), dict(runtime_top_k=[0], runtime_top_p=[0.9])):
            c = Case(O.F32, B, V, V, gen_len=4, random_seed=seeds, **kp)
            p = ProductRunner(c)
            for i in range(4):
                row = (rng.uniform(-3, 3, V)).astype(np.float32)
                p.step(i, np.tile(row, (B, 1)), None)
            ids = p.snapshot()["output_ids"]
            assert (ids[:, 0] == ids[:, 1]).all() and (ids[:, 1] == ids[:, 2]).all()
            assert (ids[:, 3] == ids[:, 4]).all() and (ids[:, 4] == ids[:, 5]).all()
            if len(seeds) == 1:
                assert (ids[:, 0] == ids[:, 5]).all()


def test_error_behaviour():
    """argument errors raise like the reference's FT_CHECKs (std::runtime_error)"""
    import torch
    import fastertransformer_amd as fa
    V = 100
    layer = fa.DynamicDecodeLayer(fa.F32, V, V)
    with pytest.raises(fa.FtkError):  # both penalties: BaseSamplingLayer.cc:172-175
        layer.setup(2, 1, {"repetition_penalty": np.array([1.1], np.float32),
                           "presence_penalty": np.array([0.1], np.float32)})
    with pytest.raises(fa.FtkError):  # wrong array size: TopKSamplingLayer.cu:158-160
        layer.setup(4, 1, {"runtime_top_k": np.array([1, 2, 3], np.uint32)})
    with pytest.raises(fa.FtkError):  # wrong seed array size: BaseSamplingLayer.cc:135-139
        layer.setup(4, 1, {"random_seed": np.array([1, 2, 3], np.uint64)})
    layer.setup(4, 2, {})             # beam search: nothing to set up, the step reads its values from its inputs
    with pytest.raises(fa.FtkError):  # per-entry runtime values must be one-dimensional (DynamicDecodeLayer.cc:482)
        layer.setup(4, 2, {"temperature": np.ones((2, 2), np.float32)})
    layer.setup(2, 1, {"runtime_top_k": np.array([2], np.uint32)})
    logits = torch.zeros((2, 1, V), device="cuda")
    out_ids = torch.zeros((3, 2), dtype=torch.int32, device="cuda")
    end = torch.zeros(2, dtype=torch.int32, device="cuda")
    base = {"logits": logits, "step": np.array([0], np.int32), "max_input_length": np.array([0], np.int32),
            "ite": np.array([0], np.uint32), "local_batch_size": np.array([2], np.int32), "end_id": end}
    with pytest.raises(fa.FtkError):  # missing key: Tensor.h:357-362
        layer.forward({"output_ids": out_ids}, {k: v for k, v in base.items() if k != "step"})
    with pytest.raises(fa.FtkError):  # logits must be rank 3: DynamicDecodeLayer.cc:241
        layer.forward({"output_ids": out_ids}, dict(base, logits=logits.reshape(2, V)))
    with pytest.raises(fa.FtkError):  # bad words rank must be 2 or 3: DynamicDecodeLayer.cc:250-251
        layer.forward({"output_ids": out_ids},
                      dict(base, bad_words_list=torch.zeros(4, dtype=torch.int32, device="cuda")))
    layer.forward({"output_ids": out_ids}, base)  # and the well-formed call still works
    torch.cuda.synchronize()
    # all-equal logits: the reference's tie rule picks the highest thread id first, i.e. ids 99 then 98
    assert (to_numpy(out_ids)[0] >= 98).all()
    # top-k beyond 1024 is clipped by the layer, as in the reference (TopKSamplingLayer.cu:56-65)
    layer.setup(2, 1, {"runtime_top_k": np.array([5000], np.uint32)})
    layer.forward({"output_ids": out_ids}, base)
    torch.cuda.synchronize()


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_fused_step_random_scenarios(dt, seed):
    """Seeded random decode scenarios through the fused top-k step (no log-probs): batch sizes that split a row
    over different numbers of workgroups, odd and padded vocabularies, per-row k up to several hundred with
    and without top-p, temperature, repetition or presence penalty over short and long histories with short
    prompts, min length; three steps each, ids / flags / lengths bit-exact against the oracle."""
    rng = np.random.default_rng(900 + 10 * dt + seed)
    for case in range(3):
        B = int(rng.choice([1, 3, 7, 20, 48]))
        V = int(rng.choice([rng.integers(600, 3000), rng.integers(3000, 40000), rng.integers(40000, 131000)]))
        Vp = V + int(rng.choice([0, 0, 3, 61]))
        H = int(rng.choice([4, 40, 300]))
        max_k = int(rng.choice([1, 8, 64, 150, 400]))
        ks = rng.integers(1, max_k + 1, B).astype(np.uint32)
        ks[0] = max_k
        ps = np.where(rng.random(B) < 0.5, 1.0, rng.uniform(0.2, 0.99, B)).astype(np.float32)
        kw = {}
        if rng.random() < 0.7:
            kw["temperature"] = rng.uniform(0.5, 1.6, B)
        pen = int(rng.integers(0, 3))
        if pen == 1:
            kw["repetition_penalty"] = rng.uniform(1.0, 1.6, B)
        elif pen == 2:
            kw["presence_penalty"] = rng.uniform(0.0, 1.5, B)
        if rng.random() < 0.5:
            kw["min_length"] = rng.integers(0, 4, B)
        c = Case(dt, B, V, Vp, max_input_length=H, gen_len=3, runtime_top_k=ks, runtime_top_p=ps,
                 prompt=_history(rng, H, B, V, zipf=1.3 if rng.random() < 0.5 else None),
                 input_lengths=rng.integers(1, H + 1, B), end_ids=rng.integers(0, V, B).astype(np.int32), **kw)
        scale = float(rng.uniform(0.5, 4.0))
        _run_case(c, rng, 3, lambda i: make_logits(rng, dt, B, V, Vp, scale), check_logits=False)


@pytest.mark.gpu
@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("max_k", [200, 700, 1024])
def test_fused_step_large_k_with_bias_and_history(dt, max_k):
    """The large-k variants of the fused step (largest k above 128, above 512): rows with small and large k in one
    launch, an unaligned and padded vocabulary, embedding bias (no tile takes the fast transform), long histories
    with repeated tokens under a repetition penalty, temperature, min length; a second scenario without bias so
    that plain tiles fetch their history flags in one go. Three steps each, bit-exact against the oracle."""
    rng = np.random.default_rng(4100 + 7 * dt + max_k)
    for with_bias in (True, False):
        B = 9
        V = int(rng.integers(36000, 70000)) | 1
        Vp = V + 5
        H = 200
        ks = rng.integers(1, max_k + 1, B).astype(np.uint32)
        ks[0], ks[1] = max_k, 3
        kw = {"temperature": rng.uniform(0.6, 1.4, B), "repetition_penalty": rng.uniform(1.05, 1.5, B),
              "min_length": rng.integers(0, 3, B)}
        if with_bias:
            kw["embedding_bias"] = O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt)
        c = Case(dt, B, V, Vp, max_input_length=H, gen_len=3, runtime_top_k=ks,
                 runtime_top_p=rng.uniform(0.5, 1.0, B).astype(np.float32),
                 prompt=_history(rng, H, B, V, zipf=1.3), input_lengths=rng.integers(H // 2, H + 1, B),
                 end_ids=rng.integers(0, V, B).astype(np.int32), **kw)
        _run_case(c, rng, 3, lambda i: make_logits(rng, dt, B, V, Vp, 2.0), check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("seed", [0, 1])
def test_fused_step_with_log_probs_random_scenarios(dt, seed):
    """The fused step that reads twice (log-probs requested): random batches, vocabularies from 1024 columns up (aligned
    and padded), per-row k up to 128 with and without top-p, temperature, repetition or presence penalty over short
    and long histories, min length, rows that finish; ids / flags / lengths bit-exact, log-probs to tolerance."""
    rng = np.random.default_rng(7000 + 10 * dt + seed)
    for case in range(4):
        B = int(rng.choice([1, 5, 33, 300, 1100]))  # (1024, 512 or 256 threads per row, by rows and vocabulary)
        V = int(rng.choice([1024, int(rng.integers(1025, 9000))] + ([int(rng.integers(30000, 160000))] if B < 1000 else [])))
        Vp = (V + 7) // 8 * 8 + int(rng.choice([0, 8, 64]))
        H = int(rng.choice([3, 40, 300]))
        max_k = int(rng.choice([1, 8, 64, 128]))
        ks = rng.integers(1, max_k + 1, B).astype(np.uint32)
        ks[0] = max_k
        ps = np.where(rng.random(B) < 0.5, 1.0, rng.uniform(0.2, 0.99, B)).astype(np.float32)
        kw = {}
        if rng.random() < 0.7:
            kw["temperature"] = rng.uniform(0.5, 1.6, B)
        pen = int(rng.integers(0, 3))
        if pen == 1:
            kw["repetition_penalty"] = rng.uniform(1.0, 1.6, B)
        elif pen == 2:
            kw["presence_penalty"] = rng.uniform(0.0, 1.5, B)
        if rng.random() < 0.5:
            kw["min_length"] = rng.integers(0, 4, B)
        end = rng.integers(0, V, B).astype(np.int32)
        c = Case(dt, B, V, Vp, max_input_length=H, gen_len=3, runtime_top_k=ks, runtime_top_p=ps,
                 prompt=_history(rng, H, B, V, zipf=1.3 if rng.random() < 0.5 else None),
                 input_lengths=rng.integers(1, H + 1, B), end_ids=end, with_cum=True, with_out_lp=True, **kw)
        scale = float(rng.uniform(0.5, 4.0))

        def logits_fn(i):
            x = O.to_f32(make_logits(rng, dt, B, V, Vp, scale), dt)
            rows = rng.random(B) < 0.2
            x[rows, end[rows]] = 40.0  # these rows finish
            return O.to_storage(x, dt)

        _run_case(c, rng, 3, logits_fn, check_logits=False)


@pytest.mark.parametrize("min_rows", [None, 100])
def test_log_probs_take_the_fused_step_from_the_smallest_window_on(monkeypatch, min_rows):
    """Without the environment's override, log-prob outputs send every window through the fused step (which leaves the
    logits alone); with FT_SAMPLING_FUSED_LOGPROBS_MIN_ROWS=100 windows of fewer than 100 rows take the kernel
    sequence instead (which writes the penalised logits and the probabilities back like the reference); the results
    are the reference's either way."""
    if min_rows is None:
        monkeypatch.delenv("FT_SAMPLING_FUSED_LOGPROBS_MIN_ROWS")
    else:
        monkeypatch.setenv("FT_SAMPLING_FUSED_LOGPROBS_MIN_ROWS", str(min_rows))
    rng = np.random.default_rng(7200)
    V = 2051
    for B in (8, 99, 100, 400):
        mutated = min_rows is not None and B < min_rows
        c = Case(O.F32, B, V, V, max_input_length=4, gen_len=2, runtime_top_k=[8], runtime_top_p=[0.9],
                 temperature=[0.7], repetition_penalty=[1.3], prompt=_history(rng, 4, B, V), with_cum=True,
                 with_out_lp=True)
        fed = []

        def logits_fn(i):
            fed.append(make_logits(rng, O.F32, B, V, V, 2.0))
            return fed[-1]

        snap = _run_case(c, rng, 2, logits_fn, check_logits=mutated)
        assert np.array_equal(np.asarray(snap["logits"]).reshape(B, V), fed[-1].reshape(B, V)) == (not mutated)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_fused_step_with_log_probs_rows_off_vector_boundaries(dt):
    """Log-probs on rows whose pitch is not a multiple of 16 bytes (GPT-2's 50257 columns unpadded, odd paddings): the
    rows of a batch then start at every offset inside a 16-byte vector, the summation chains of the reference's
    softmax are rotated against the loads, and history flags straddle bitmap words. Ids, flags and lengths bit
    for bit, log-probs to tolerance; long histories use the bitmap in memory, short ones the one in LDS."""
    rng = np.random.default_rng(7100 + dt)
    for V, Vp, B, H, max_k in ((50257, 50257, 9, 64, 40), (1024, 1027, 13, 5, 8), (4999, 5001, 6, 700, 64),
                               (33001, 33003, 17, 30, 128), (152063, 152065, 5, 12, 64), (1029, 1029, 3, 0, 1)):
        ks = rng.integers(1, max_k + 1, B).astype(np.uint32)
        ks[0] = max_k
        ps = np.where(rng.random(B) < 0.5, 1.0, rng.uniform(0.2, 0.99, B)).astype(np.float32)
        kw = {"temperature": rng.uniform(0.5, 1.6, B)}
        if H > 0:
            if rng.random() < 0.5:
                kw["repetition_penalty"] = rng.uniform(1.0, 1.6, B)
            else:
                kw["presence_penalty"] = rng.uniform(0.0, 1.5, B)
            kw["prompt"] = _history(rng, H, B, V, zipf=1.3 if rng.random() < 0.5 else None)
            kw["input_lengths"] = rng.integers(1, H + 1, B)
        kw["min_length"] = rng.integers(0, 4, B)
        end = rng.integers(0, V, B).astype(np.int32)
        end[0], end[-1] = 0, V - 1            # the masked end id in the first and in the last chunk of a row
        c = Case(dt, B, V, Vp, max_input_length=H, gen_len=3, runtime_top_k=ks, runtime_top_p=ps, end_ids=end,
                 with_cum=True, with_out_lp=True, **kw)
        scale = float(rng.uniform(0.5, 4.0))

        def logits_fn(i):
            x = O.to_f32(make_logits(rng, dt, B, V, Vp, scale), dt)
            x[:, 0] += 2.0 * scale            # the row's edges matter
            x[:, V - 1] += 2.0 * scale
            return O.to_storage(x, dt)

        _run_case(c, rng, 3, logits_fn, check_logits=False)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_fused_step_with_log_probs_ties_and_flat_rows(dt):
    """Rows where probabilities tie or vanish: logits from a handful of distinct values, a flat row (every
    probability equal; zero after rounding in fp16 at this vocabulary), one dominant column (all other
    probabilities round to zero), and rows where fewer than k columns have a non-zero probability. The picks must
    follow the reference's tie rules on probabilities."""
    rng = np.random.default_rng(7100 + dt)
    B, V, H = 12, 70016, 4
    x = rng.standard_normal((B, V)).astype(np.float32)
    x[0:3] = rng.choice(np.array([-2.0, 0.5, 1.0, 1.5], np.float32), (3, V))   # few distinct values
    x[3] = 0.25                                                                 # flat
    x[4] = -20.0
    x[4, 777] = 30.0                                                            # one column takes everything
    x[5] = -60.0
    x[5, rng.integers(0, V, 20)] = rng.uniform(0, 3, 20)                        # 20 live columns, k = 64
    x[6:9] = np.round(x[6:9] * 4) / 4                                           # quarter steps: many ties
    c = Case(dt, B, V, V, max_input_length=H, gen_len=2, runtime_top_k=[64], runtime_top_p=[0.95],
             temperature=[0.9], repetition_penalty=[1.2], prompt=_history(rng, H, B, V), with_cum=True,
             with_out_lp=True)
    xs = O.to_storage(x, dt)
    _run_case(c, rng, 2, lambda i: xs, check_logits=False)


@pytest.mark.parametrize("seed", range(6))
def test_random_scenarios_over_every_step_variant(seed):
    """Random decode scenarios through the layer against the oracle, ids / flags / lengths bit-exact: all three
    element types, 1 to 70 rows, short to long vocabularies (aligned, padded, odd), per-row k with a largest k from
    1 to 1024 (one read of the logits, two reads, general stream), rows owned by the top-p layer mixed in,
    temperature, repetition / presence / frequency penalties over histories of 1 to 2100 tokens, min length,
    embedding bias, log-prob outputs, windows of the batch, and value patterns that overflow candidate lists
    (few distinct values, constant rows, ramps, all large values in one stage-1 slice)."""
    for case in range(20):
        rng = np.random.default_rng(100000 + 1000 * seed + case)
        dt = int(rng.integers(0, 3))
        long_row = rng.random() < 0.3
        B = int(rng.choice([1, 2, 3, 5])) if long_row else int(rng.choice([1, 2, 7, 33, 70]))
        V = int(rng.integers(70000, 270000)) if long_row else \
            int(rng.choice([int(rng.integers(300, 3000)), int(rng.integers(3000, 20000)), int(rng.integers(20000, 70000))]))
        Vp = (V + 7) // 8 * 8 + int(rng.choice([0, 8, 64])) if rng.random() < 0.7 else V + int(rng.integers(0, 5))
        H = int(rng.choice([1, 3, 40, 300, 2100]))
        max_k = int(rng.choice([1, 8, 64, 128, 150, 192, 193, 300, 700, 1024]))
        ks = rng.integers(1, max_k + 1, B).astype(np.uint32)
        ks[0] = max_k
        ps = np.where(rng.random(B) < 0.5, 1.0, rng.uniform(0.2, 0.99, B)).astype(np.float32)
        if B > 1 and rng.random() < 0.3:  # some rows belong to the top-p layer
            tp = rng.random(B) < 0.4
            tp[0] = False
            ks[tp] = 0
            ps[tp] = rng.uniform(0.3, 0.95, int(tp.sum())).astype(np.float32)
        kw = {}
        if rng.random() < 0.7:
            kw["temperature"] = rng.uniform(0.5, 1.6, B)
        pen = int(rng.integers(0, 4))
        if pen == 1:
            kw["repetition_penalty"] = rng.uniform(0.7, 1.6, B)
        elif pen == 2:
            kw["presence_penalty"] = rng.uniform(-0.5, 1.5, B)
        elif pen == 3:
            kw["presence_penalty"] = rng.uniform(0.0, 1.5, B)
            kw["frequency_penalty"] = rng.uniform(0.0, 0.5, B)
        if rng.random() < 0.5:
            kw["min_length"] = rng.integers(0, 4, B)
        if rng.random() < 0.3:
            kw["embedding_bias"] = O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt)
        lp = rng.random() < 0.3
        local = B // 7 if B % 7 == 0 and rng.random() < 0.4 else None
        end = rng.integers(0, V, B).astype(np.int32)
        c = Case(dt, B, V, Vp, max_input_length=H, gen_len=2, runtime_top_k=ks, runtime_top_p=ps,
                 prompt=_history(rng, H, B, V, zipf=1.3 if rng.random() < 0.5 else None),
                 input_lengths=rng.integers(1, H + 1, B), end_ids=end, with_cum=lp, with_out_lp=lp, local_batch=local,
                 **kw)
        scale = float(rng.uniform(0.5, 4.0))
        kind = rng.choice(["normal", "normal", "rounded", "ramp", "few", "const", "blocks"])

        def logits_fn(i):
            x = O.to_f32(make_logits(rng, dt, B, V, Vp, scale), dt)
            if kind == "rounded":
                x = np.round(x * 2) / 2
            elif kind == "ramp":
                x[:, :V] += np.linspace(-5, 5, V, dtype=np.float32)
            elif kind == "few":
                x = rng.choice(np.array([-1.0, 0.0, 0.5, 2.0, 2.5], np.float32), x.shape)
            elif kind == "const":
                x[:] = 0.75
                x[:, ::997] = 1.0
            elif kind == "blocks":
                x[:, ((np.arange(x.shape[1]) >> 8) & 7) == 5] += 8.0
            rows = rng.random(B) < 0.2
            x[rows, end[rows]] = 40.0  # these rows finish
            return O.to_storage(x, dt)

        p, o = ProductRunner(c), OracleRunner(c)
        for i in range(2):
            step = H + i
            logits, u = logits_fn(i), uniforms(rng, B)
            for ite in range(1 if local is None else B // local):
                p.step(step, logits, u, ite=ite)
                o.step(step, logits, u, ite=ite)
            compare(p.snapshot(), o.snapshot(), dt, False, where="seed %d case %d step %d" % (seed, case, step))
