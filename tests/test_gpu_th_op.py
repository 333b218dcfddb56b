"""torch.classes.FasterTransformer.DynamicDecodeOp: the cases of the reference's own test of this class
(tests/unittests/th_op/test_th_decode_op.py:233-258 min-length at sampling, :292-335 repetition / presence
penalty known answers, batch sizes up to 2048), its argument placement rules
(src/fastertransformer/th_op/common/DynamicDecodeOp.cc:262-276, :355-393) and agreement with the layer
reached through the C handle API."""
import itertools
import os

import numpy as np
import pytest

import ft_oracle as O

LIB = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "fastertransformer_amd", "lib",
                   "libth_transformer.so")
VOCAB = 1024
END_ID = 0


def test_class_is_registered():
    """CPU: the library loads into torch and registers the class under the reference's name."""
    import torch
    assert os.path.exists(LIB), "run python -m fastertransformer_amd.build"
    torch.classes.load_library(LIB)
    cls = torch.classes.FasterTransformer.DynamicDecodeOp
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError):
            cls(VOCAB, VOCAB, 1, 1, torch.float)  # no device: fails loudly, no CPU path behind it
    with pytest.raises(RuntimeError):
        cls(VOCAB, VOCAB, 2, 1, torch.float)      # one GPU only


@pytest.fixture(scope="module")
def th():
    import torch
    assert torch.cuda.is_available()
    torch.classes.load_library(LIB)
    return torch


def _vec(th, batch, value, dtype, cpu):
    if value is None:
        return None
    return value * th.ones(batch, dtype=dtype, device="cpu" if cpu else "cuda")


def _input_tokens(th, batch, max_input_length, random_tokens):
    g = th.Generator(device="cuda")
    g.manual_seed(batch * 131 + max_input_length)
    if random_tokens:
        ids = th.randint(1, VOCAB, (batch, max_input_length), dtype=th.int32, device="cuda", generator=g)
    else:
        ids = th.ones((batch, max_input_length), dtype=th.int32, device="cuda")
    ids = (ids + END_ID).remainder(VOCAB)
    lengths = th.randint(1, max_input_length + 1, (batch,), dtype=th.int32, device="cuda", generator=g)
    lengths[int(th.randint(0, batch, (1,)))] = max_input_length
    steps = th.arange(0, max_input_length, device="cuda").unsqueeze(0).tile(batch, 1)
    ids[lengths.unsqueeze(1) <= steps] = END_ID
    return ids, lengths


def run_decode(th, dtype=None, batch_size=4, max_input_length=4, gen_length=3, top_k=None, top_p=None,
               temperature=None, repetition_penalty=None, presence_penalty=None, min_length=None, random_seed=None,
               logit_fn=None, use_random_input_tokens=True):
    dtype = dtype or th.float
    op = th.classes.FasterTransformer.DynamicDecodeOp(VOCAB, VOCAB, 1, 1, dtype)
    max_seq_length = max_input_length + gen_length
    eos = _vec(th, batch_size, END_ID, th.int32, False)
    top_ks = _vec(th, batch_size, top_k, th.int32, True)
    top_ps = _vec(th, batch_size, top_p, th.float, True)
    temperatures = _vec(th, batch_size, temperature, th.float, True)
    repetition_penalties = _vec(th, batch_size, repetition_penalty, th.float, True)
    presence_penalties = _vec(th, batch_size, presence_penalty, th.float, True)
    min_lengths = _vec(th, batch_size, min_length, th.int32, True)
    seeds = _vec(th, batch_size, random_seed, th.int64, True)
    ids, input_lengths = _input_tokens(th, batch_size, max_input_length, use_random_input_tokens)
    op.setup(batch_size, 1, top_ks, top_ps, temperatures, repetition_penalties, presence_penalties, min_lengths,
             None, None, seeds, None, None, None)
    finished = th.zeros_like(input_lengths).bool()
    sequence_lengths = (max_input_length - 1) * th.ones_like(input_lengths)
    output_token_ids = th.zeros((max_seq_length, batch_size), dtype=th.int32, device="cuda")
    output_token_ids[:max_input_length] = ids.T
    g = th.Generator(device="cuda")
    g.manual_seed(99)
    for step in range(max_input_length, max_seq_length):
        if logit_fn is None:
            logits = th.randn((batch_size, 1, VOCAB), device="cuda", generator=g).to(dtype)
        else:
            logits = logit_fn(batch_size, g).to(dtype)
        should_stop = op.forward(logits, step, max_input_length, 0, batch_size, eos, top_ks, top_ps, temperatures,
                                 repetition_penalties, presence_penalties, min_lengths, None, None, None, None, None,
                                 None, input_lengths, None, None, None, None,
                                 output_token_ids.view(-1, batch_size, 1), finished, sequence_lengths, None, None,
                                 None, None)
        assert should_stop.device.type == "cpu" and should_stop.dtype == th.bool and should_stop.dim() == 0
        if should_stop:
            break
    return dict(output_token_ids=output_token_ids.T, output_sequence_lengths=sequence_lengths + 1)


@pytest.mark.gpu
@pytest.mark.parametrize("method", [dict(top_k=1, top_p=0.0), dict(top_k=0, top_p=0.8)], ids=["topk1", "topp0.8"])
@pytest.mark.parametrize("tc", [dict(batch_size=4, max_input_length=4, min_length=2, gen_length=4),
                                dict(batch_size=4, max_input_length=4, min_length=32, gen_length=64),
                                dict(batch_size=2048, max_input_length=6, min_length=4, gen_length=8)],
                         ids=["b4_min2", "b4_min32", "b2048_min4"])
def test_min_length_correctness_at_sampling(th, tc, method):
    def logit_fn(batch, g):
        logits = th.randn((batch, 1, VOCAB), device="cuda", generator=g)
        logits[..., END_ID] = logits.max(dim=-1)[0] + 1  # the end token is the most probable one
        return logits

    out = run_decode(th, logit_fn=logit_fn, **tc, **method)
    lengths = out["output_sequence_lengths"]
    assert bool((lengths >= tc["max_input_length"] + tc["min_length"]).all()), lengths


@pytest.mark.gpu
@pytest.mark.parametrize("dtype_name", ["float", "half", "bfloat16"])
@pytest.mark.parametrize("tc", [dict(batch_size=4, max_input_length=4, repetition_penalty=2),
                                dict(batch_size=2048, max_input_length=4, repetition_penalty=2),
                                dict(batch_size=4, max_input_length=4, presence_penalty=0.5),
                                dict(batch_size=4, max_input_length=4, presence_penalty=1.0),
                                dict(batch_size=2048, max_input_length=4, presence_penalty=0.5)],
                         ids=["rep2_b4", "rep2_b2048", "pres0.5_b4", "pres1.0_b4", "pres0.5_b2048"])
def test_repetition_penalty_correctness(th, tc, dtype_name):
    """v-1 is the most probable token until penalised: the ids must read v-1, v-2, v-3, v-1, v-1."""
    def logit_fn(batch, g):
        logits = th.zeros((batch, 1, VOCAB), device="cuda")
        logits[..., VOCAB - 1] = 2
        logits[..., VOCAB - 2] = 1.8
        logits[..., VOCAB - 3] = 1.6
        return logits

    gen_length = 5
    expected = (VOCAB - 1) * th.ones((tc["batch_size"], gen_length), dtype=th.int32)
    expected[:, 1] = VOCAB - 2
    expected[:, 2] = VOCAB - 3
    out = run_decode(th, dtype=getattr(th, dtype_name), gen_length=gen_length, use_random_input_tokens=False,
                     logit_fn=logit_fn, top_k=1, top_p=0.0, **tc)
    got = out["output_token_ids"][:, tc["max_input_length"]:].cpu()
    assert bool((expected == got).all())


@pytest.mark.gpu
def test_argument_placement_is_checked(th):
    op = th.classes.FasterTransformer.DynamicDecodeOp(VOCAB, VOCAB, 1, 1, th.float)
    batch = 2
    k_cpu = th.ones(batch, dtype=th.int32)
    with pytest.raises(RuntimeError):   # runtime arguments of setup live on the host
        op.setup(batch, 1, k_cpu.cuda(), None, None, None, None, None, None, None, None, None, None, None)
    with pytest.raises(RuntimeError):   # and have the reference's types
        op.setup(batch, 1, k_cpu.long(), None, None, None, None, None, None, None, None, None, None, None)
    with pytest.raises(RuntimeError):   # the decay tensors live on the device
        op.setup(batch, 1, k_cpu, None, None, None, None, None, None, None, None, th.ones(batch), None, None)
    op.setup(batch, 1, k_cpu, None, None, None, None, None, None, None, None, None, None, None)
    ids = th.zeros((4, batch, 1), dtype=th.int32, device="cuda")
    eos = th.zeros(batch, dtype=th.int32, device="cuda")
    rest = (None,) * 17

    def fwd(logits, end_id=eos, out=ids):
        return op.forward(logits, 1, 1, 0, batch, end_id, *rest, out, None, None, None, None, None, None)

    with pytest.raises(RuntimeError):   # logits of the type the object was built for
        fwd(th.zeros((batch, 1, VOCAB), device="cuda", dtype=th.half))
    with pytest.raises(RuntimeError):   # three dimensions
        fwd(th.zeros((batch, VOCAB), device="cuda"))
    with pytest.raises(RuntimeError):   # padded vocabulary in the last one
        fwd(th.zeros((batch, 1, VOCAB - 8), device="cuda"))
    with pytest.raises(RuntimeError):   # device tensors on the device
        fwd(th.zeros((batch, 1, VOCAB), device="cuda"), end_id=eos.cpu())
    op.setup(batch, 2, k_cpu, None, None, None, None, None, None, None, None, None, None, None)  # beams: no state
    op.setup(batch, 1, k_cpu, None, None, None, None, None, None, None, None, None, None, None)
    assert not bool(fwd(th.zeros((batch, 1, VOCAB), device="cuda")))
    op.broadcast_from_last_pipeline([ids])


@pytest.mark.gpu
def test_matches_the_oracle_layer(th):
    """Same seeded logits through the custom class and through the CPU oracle of the layer (top-k 8 with
    temperature and a repetition penalty, log-probs on): ids, lengths and flags equal, log-probs within 1e-5.
    The class draws from the library's own counter-based generator; the test computes the same draws from the
    seeds (draw number i of a row is Philox-4x32-10 of counter i under the row's seed) and hands them to the
    oracle."""
    import ctypes as C
    from fastertransformer_amd import ops
    host = ops.ftk_hooks()

    def draw(seed, i):
        c = (C.c_uint32 * 4)(i, 0, 0, 0)
        kk = (C.c_uint32 * 2)(seed & 0xFFFFFFFF, seed >> 32)
        out = (C.c_uint32 * 4)()
        host.ftk_host_philox4x32_10(c, kk, out)
        return np.float32(out[0]) * np.float32(2.3283064365386963e-10) + np.float32(1.16415321826934814453125e-10)

    batch, steps, H = 6, 5, 3
    rng = np.random.default_rng(3)
    op = th.classes.FasterTransformer.DynamicDecodeOp(VOCAB, VOCAB, 1, 1, th.float)
    k = th.full((batch,), 8, dtype=th.int32)
    temp = th.full((batch,), 0.7)
    rep = th.full((batch,), 1.3)
    seed = th.arange(batch, dtype=th.int64) + 11
    op.setup(batch, 1, k, None, temp, rep, None, None, None, None, seed, None, None, None)
    out_ids = np.zeros((H + steps, batch), np.int32)
    out_ids[:H] = rng.integers(1, VOCAB, (H, batch))
    d_ids = th.from_numpy(out_ids.copy()).cuda()
    finished = th.zeros(batch, dtype=th.bool, device="cuda")
    seq = th.full((batch,), H - 1, dtype=th.int32, device="cuda")
    cum = th.zeros(batch, device="cuda")
    olp = th.zeros((steps, batch), device="cuda")
    eos = th.full((batch,), END_ID, dtype=th.int32, device="cuda")
    lengths = th.full((batch,), H, dtype=th.int32, device="cuda")

    layer = O.OracleDynamicDecodeLayer(O.F32, VOCAB, VOCAB)
    layer.setup(batch, [8], [0.0], [0.7], [1.3])
    o_fin = np.zeros(batch, np.bool_)
    o_seq = np.full(batch, H - 1, np.int32)
    o_cum = np.zeros(batch, np.float32)
    o_olp = np.zeros((steps, batch), np.float32)
    for i in range(steps):
        x = (rng.standard_normal((batch, VOCAB)) * 2).astype(np.float32)
        x[:, END_ID] = -100.0  # no row finishes: a finished row would stop consuming draws
        u = np.array([draw(11 + b, i) for b in range(batch)], np.float32)
        logits = th.from_numpy(x.copy()).cuda().reshape(batch, 1, VOCAB)
        op.forward(logits, H + i, H, 0, batch, eos, k, None, temp, rep, None, None, None, None, None, None, None,
                   None, lengths, None, None, None, None, d_ids.view(-1, batch, 1), finished, seq, cum, olp, None,
                   None)
        layer.forward(x.copy(), np.full(batch, END_ID, np.int32), out_ids, H + i, H, u, finished=o_fin,
                      sequence_length=o_seq, cum_log_probs=o_cum, output_log_probs=o_olp,
                      input_lengths=np.full(batch, H, np.int32))
    th.cuda.synchronize()
    assert np.array_equal(d_ids.cpu().numpy(), out_ids)
    assert np.array_equal(finished.cpu().numpy(), o_fin)
    assert np.array_equal(seq.cpu().numpy(), o_seq)
    np.testing.assert_allclose(cum.cpu().numpy(), o_cum, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(olp.cpu().numpy(), o_olp, rtol=1e-5, atol=1e-6)
