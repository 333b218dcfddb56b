"""GPU parity of every stand-alone kernel entry point against the CPU oracle, through the C ABI.

Integer / id / flag outputs must be bit-exact; penalised logits must match the oracle's bits
(the contract is 1 ulp in fp32; both sides evaluate the same IEEE operation sequence, so 0 is observed);
probabilities and log-probs: 1e-5 relative in fp32, 2e-3 in fp16/bf16 (observed: bit-exact).
"""
import ctypes as C

import numpy as np
import pytest

import ft_oracle as O
from helpers import DTYPES, DTYPE_NAMES, bits, make_logits, make_word_list, to_numpy, to_torch, ulp_diff_f32, uniforms

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def env():
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    assert torch.cuda.is_available()
    return torch, fa.ftk(), ops


def _sync(torch):
    torch.cuda.synchronize()


def test_device_math_matches_host_bitwise(env):
    torch, _, ops = env
    lib = ops.ftk_hooks()
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.uniform(-104, 89, 400000), rng.uniform(-1, 1, 50000),
                        -np.abs(rng.standard_normal(200000)) * 10, [0.0, -0.0, -103.9, 88.7, -200.0, 100.0]])
    x = x.astype(np.float32)
    d_in = to_torch(x)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(0, d_in.data_ptr(), d_out.data_ptr(), x.size, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), O.expf(x).view(np.uint32))
    xl = np.abs(np.concatenate([rng.uniform(0, 1, 300000), np.exp(rng.uniform(-100, 88, 300000)),
                                [0.0, 1.0, 1e-40, 3e38]])).astype(np.float32)
    d_in = to_torch(xl)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(1, d_in.data_ptr(), d_out.data_ptr(), xl.size, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), O.logf(xl).view(np.uint32))


def test_device_conversions_division_subnormals(env):
    torch, _, ops = env
    lib = ops.ftk_hooks()
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.standard_normal(300000) * 100, rng.uniform(-7e4, 7e4, 100000),
                        rng.standard_normal(100000) * 1e-5, rng.standard_normal(100000) * 1e-7,
                        [65504.0, 65519.9, 65520.0, -65520.0, 6.0e-8, 2.98e-8, 2.9802322e-8]]).astype(np.float32)
    d_in = to_torch(x)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(2, d_in.data_ptr(), d_out.data_ptr(), x.size, ops.current_stream()))
    _sync(torch)
    ref = O.to_f32(O.to_storage(x, O.F16), O.F16)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), ref.view(np.uint32))
    ops.check(lib.ftk_test_device_math(3, d_in.data_ptr(), d_out.data_ptr(), x.size, ops.current_stream()))
    _sync(torch)
    ref = O.to_f32(O.to_storage(x, O.BF16), O.BF16)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), ref.view(np.uint32))
    # correctly rounded division and subnormal arithmetic (the softmax relies on both)
    t = rng.uniform(0.01, 3.0, 200000).astype(np.float32)
    d_in = to_torch(t)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(4, d_in.data_ptr(), d_out.data_ptr(), t.size, ops.current_stream()))
    _sync(torch)
    ref = (np.float32(1.0) / (t + np.float32(1e-6))).astype(np.float32)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), ref.view(np.uint32))
    s = rng.uniform(0.0, 4.0, 100000).astype(np.float32)
    d_in = to_torch(s)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(5, d_in.data_ptr(), d_out.data_ptr(), s.size, ops.current_stream()))
    _sync(torch)
    tiny = np.float32(1.1754944e-38)
    ref = (s * tiny + (s * np.float32(0.5)) * tiny).astype(np.float32)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), ref.view(np.uint32))


def test_device_exp_of_non_positive_arguments(env):
    """The exp without range checks that the log-prob step uses on y - max: bit for bit the oracle's exp on every
    non-positive argument, including the band around the underflow cut-off, -inf, -0 and NaN."""
    torch, _, ops = env
    lib = ops.ftk_hooks()
    rng = np.random.default_rng(77)
    x = np.concatenate([-np.abs(rng.standard_normal(400000) * 30), -rng.uniform(0.0, 110.0, 400000),
                        -rng.uniform(103.0, 105.0, 200000), -np.abs(rng.standard_normal(100000)) * 1e-6,
                        [0.0, -0.0, -103.97283, -103.972832, -103.9728, -104.0, -104.00001, -150.0, -1e30,
                         -np.inf]]).astype(np.float32)
    d_in = to_torch(x)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(6, d_in.data_ptr(), d_out.data_ptr(), x.size, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(to_numpy(d_out).view(np.uint32), O.expf(x).view(np.uint32))
    nan = to_torch(np.array([np.nan], np.float32))
    out = torch.empty_like(nan)
    ops.check(lib.ftk_test_device_math(6, nan.data_ptr(), out.data_ptr(), 1, ops.current_stream()))
    _sync(torch)
    assert np.isnan(to_numpy(out)[0])


def test_device_division_by_a_shared_reciprocal(env):
    """The softmax divides a row by one denominator with the reciprocal's part of the division computed once:
    bit for bit numpy's IEEE quotient, for numerators over the whole range an exponential can take (zero,
    subnormal, the band around the switch to the ordinary division, up to 1) and denominators from 1 to beyond
    the range the short sequence accepts."""
    torch, _, ops = env
    lib = ops.ftk_hooks()
    rng = np.random.default_rng(78)
    n = 1 << 21
    num = np.concatenate([
        np.exp(-rng.uniform(0.0, 104.0, n // 2)), rng.uniform(0.0, 1.0, n // 4),
        np.exp2(-rng.uniform(96.0, 104.0, n // 8)),                         # around 2^-100
        rng.integers(0, 1 << 23, n // 8 - 8).view(np.int64).astype(np.uint32).view(np.float32).astype(np.float64),
        [0.0, 1.0, 2.0 ** -100, np.nextafter(np.float32(2.0 ** -100), np.float32(0)), 2.0 ** -126, 2.0 ** -149,
         np.nextafter(np.float32(1), np.float32(0)), 0.5]]).astype(np.float32)
    den = np.concatenate([
        1.0 + rng.uniform(0.0, 1.0, n // 4), np.exp(rng.uniform(0.0, 20.0, n // 2)),
        rng.integers(1, 200000, n // 8).astype(np.float64) + 1e-6,
        np.exp2(rng.uniform(29.0, 31.0, n // 8 - 4)), [1.0, 2.0 ** 30, np.nextafter(np.float32(2.0 ** 30), np.float32(np.inf)),
                                                      np.nextafter(np.float32(1), np.float32(0))]]).astype(np.float32)
    den = den[rng.permutation(den.size)]
    pairs = np.stack([num, den], axis=1).reshape(-1).copy()
    d_in = to_torch(pairs)
    d_out = torch.empty_like(d_in)
    ops.check(lib.ftk_test_device_math(7, d_in.data_ptr(), d_out.data_ptr(), pairs.size, ops.current_stream()))
    _sync(torch)
    out = to_numpy(d_out).reshape(-1, 2)
    with np.errstate(under="ignore"):
        want = (num / den).astype(np.float32)
    assert np.array_equal(out[:, 0].view(np.uint32), want.view(np.uint32))
    assert np.array_equal(out[:, 1].view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("V,Vp", [(4, 4), (50001, 50001), (50001, 50008), (32000, 32000), (1000, 1024)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_temperature_penalty(env, dt, V, Vp, with_bias):
    torch, lib, ops = env
    rng = np.random.default_rng(V + Vp + dt)
    batch = 6
    logits = make_logits(rng, dt, batch, V, Vp, scale=3.0)
    bias = O.to_storage((rng.standard_normal(Vp) * 2).astype(np.float32), dt) if with_bias else None
    temps = rng.uniform(0.3, 2.0, batch).astype(np.float32)
    # batch variant
    ref = logits.copy()
    O.batch_apply_temperature_penalty(dt, ref, bias, temps, batch, V, Vp)
    d = to_torch(logits, dt)
    d_bias = to_torch(bias, dt)
    d_t = to_torch(temps)
    ops.check(lib.ftk_invoke_batch_apply_temperature_penalty(dt, d.data_ptr(), ops.ptr(d_bias), d_t.data_ptr(), batch,
                                                             V, Vp, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(bits(to_numpy(d, dt), dt), bits(ref, dt))
    # scalar variant
    ref = logits.copy()
    O.apply_temperature_penalty(dt, ref, bias, 0.53, batch, V, Vp)
    d = to_torch(logits, dt)
    ops.check(lib.ftk_invoke_apply_temperature_penalty(dt, d.data_ptr(), ops.ptr(d_bias), 0.53, batch, V, Vp,
                                                       ops.current_stream()))
    _sync(torch)
    got = to_numpy(d, dt)
    if dt == O.F32:
        assert ulp_diff_f32(got, ref).max() <= 1
    assert np.array_equal(bits(got, dt), bits(ref, dt))


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("ptype", [O.PEN_ADDITIVE, O.PEN_MULTIPLICATIVE])
@pytest.mark.parametrize("V,max_input,step", [(4, 5, 8), (50001, 5, 40), (50001, 1003, 1200), (32000, 0, 2048)])
def test_repetition_penalty(env, dt, ptype, V, max_input, step):
    torch, lib, ops = env
    rng = np.random.default_rng(V + step + ptype)
    batch, local = 6, 6
    Vp = V
    logits = make_logits(rng, dt, batch, V, Vp, scale=3.0)
    out_ids = rng.integers(0, V, (step, batch)).astype(np.int32)
    input_lengths = rng.integers(1, max_input + 1, batch).astype(np.int32) if max_input > 0 else np.zeros(batch, np.int32)
    pens = np.array([1.0, 0.53, 2.01, 1.2, 0.0, 3.0], np.float32) if ptype == O.PEN_ADDITIVE else \
        np.array([1.0, 0.53, 2.01, 1.2, 0.7, 3.0], np.float32)
    ref = logits.copy()
    O.batch_apply_repetition_penalty(dt, ref, pens, out_ids, batch, local, Vp, input_lengths, max_input, step, ptype)
    d = to_torch(logits, dt)
    d_ids, d_len, d_pen = to_torch(out_ids), to_torch(input_lengths), to_torch(pens)
    ops.check(lib.ftk_invoke_batch_apply_repetition_penalty(dt, d.data_ptr(), d_pen.data_ptr(), d_ids.data_ptr(), batch,
                                                            local, Vp, d_len.data_ptr(), max_input, step, ptype,
                                                            ops.current_stream()))
    _sync(torch)
    assert np.array_equal(bits(to_numpy(d, dt), dt), bits(ref, dt))
    # scalar variant, without input_lengths
    ref = logits.copy()
    O.apply_repetition_penalty(dt, ref, 1.3, out_ids, batch, local, V, Vp, None, max_input, step, ptype)
    d = to_torch(logits, dt)
    ops.check(lib.ftk_invoke_apply_repetition_penalty(dt, d.data_ptr(), 1.3, None, d_ids.data_ptr(), batch, local, V,
                                                      Vp, None, max_input, step, ptype, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(bits(to_numpy(d, dt), dt), bits(ref, dt))


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("step", [1, 700, 2048, 9000, 16383])
def test_frequency_penalty_extension(env, dt, step):
    """step 700 / 2048: a counting table at most half full; 9000 / 16383: the largest table, nearly full at the end;
    16384 tokens and more are refused."""
    torch, lib, ops = env
    rng = np.random.default_rng(11)
    batch, V, max_input = 4, 32000, min(16, step)
    logits = make_logits(rng, dt, batch, V, V, scale=2.0)
    out_ids = np.minimum(rng.zipf(1.2, (step, batch)), V - 1).astype(np.int32)
    input_lengths = rng.integers(1, max_input + 1, batch).astype(np.int32)
    pres = np.array([0.5, 0.0, 1.0, 0.25], np.float32)
    freq = np.array([0.3, 0.1, 0.0, 0.0], np.float32)
    ref = logits.copy()
    O.batch_apply_frequency_penalty(dt, ref, pres, freq, out_ids, batch, batch, V, input_lengths, max_input, step)
    d = to_torch(logits, dt)
    d_ids, d_len, d_pres, d_freq = to_torch(out_ids), to_torch(input_lengths), to_torch(pres), to_torch(freq)
    ops.check(lib.ftk_invoke_batch_apply_frequency_penalty(dt, d.data_ptr(), d_pres.data_ptr(), d_freq.data_ptr(),
                                                           d_ids.data_ptr(), batch, batch, V, d_len.data_ptr(),
                                                           max_input, step, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(bits(to_numpy(d, dt), dt), bits(ref, dt))
    assert lib.ftk_invoke_batch_apply_frequency_penalty(dt, d.data_ptr(), d_pres.data_ptr(), d_freq.data_ptr(),
                                                        d_ids.data_ptr(), batch, batch, V, d_len.data_ptr(),
                                                        max_input, 16384, ops.current_stream()) == ops.FTK_ERR_ARGUMENT


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_min_length_and_end_mask(env, dt):
    torch, lib, ops = env
    rng = np.random.default_rng(5)
    batch, V, Vp = 70, 1000, 1024
    logits = make_logits(rng, dt, batch, V, Vp)
    min_lengths = rng.integers(0, 8, batch).astype(np.int32)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    seq = rng.integers(3, 12, batch).astype(np.int32)
    ref = logits.copy()
    O.min_length_penalty(dt, ref, min_lengths, end_ids, seq, 4, batch, Vp)
    d = to_torch(logits, dt)
    d_min, d_end, d_seq = to_torch(min_lengths), to_torch(end_ids), to_torch(seq)
    ops.check(lib.ftk_invoke_min_length_penalty(dt, d.data_ptr(), d_min.data_ptr(), d_end.data_ptr(), d_seq.data_ptr(),
                                                4, batch, Vp, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(bits(to_numpy(d, dt), dt), bits(ref, dt))
    finished = (rng.random(batch) < 0.3)
    for bias in (None, O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt)):
        ref = logits.copy()
        O.add_bias_end_mask(dt, ref, bias, end_ids, finished, batch, V, Vp)
        d = to_torch(logits, dt)
        d_bias, d_fin = to_torch(bias, dt), to_torch(finished)
        ops.check(lib.ftk_invoke_add_bias_end_mask(dt, d.data_ptr(), ops.ptr(d_bias), d_end.data_ptr(),
                                                   d_fin.data_ptr(), batch, V, Vp, ops.current_stream()))
        _sync(torch)
        assert np.array_equal(bits(to_numpy(d, dt), dt), bits(ref, dt))


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("V,Vp", [(8, 8), (50, 56), (1000, 1024), (4000, 4000), (50257, 51200)])
def test_softmax(env, dt, V, Vp):
    torch, lib, ops = env
    rng = np.random.default_rng(V * 3 + dt)
    batch = 5
    logits = make_logits(rng, dt, batch, V, Vp, scale=3.0)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    finished = np.array([False, True, False, False, True])
    for bias in (None, O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt)):
        ref = logits.copy()
        O.add_bias_softmax(dt, ref, bias, end_ids, finished, batch, Vp, V)
        d = to_torch(logits, dt)
        d_bias, d_end, d_fin = to_torch(bias, dt), to_torch(end_ids), to_torch(finished)
        ops.check(lib.ftk_invoke_add_bias_softmax(dt, d.data_ptr(), ops.ptr(d_bias), d_end.data_ptr(),
                                                  d_fin.data_ptr(), batch, Vp, V, ops.current_stream()))
        _sync(torch)
        got = to_numpy(d, dt)
        rtol = 1e-5 if dt == O.F32 else 2e-3
        np.testing.assert_allclose(O.to_f32(got, dt), O.to_f32(ref, dt), rtol=rtol, atol=1e-30)
        assert np.array_equal(bits(got, dt), bits(ref, dt))  # same IEEE sequence on both sides


def _run_topk(env, dt, logits, k_arr, p_arr, max_k, end_ids, u, finished=None, seq=None, skip=None, logprobs=False):
    torch, lib, ops = env
    batch, Vp = logits.shape
    d_logits = to_torch(logits, dt)
    d_ids = torch.full((batch,), -7, dtype=torch.int32, device="cuda")
    d_fin = to_torch(finished) if finished is not None else None
    d_seq = to_torch(seq) if seq is not None else None
    d_cum = torch.zeros(batch, dtype=torch.float32, device="cuda") if logprobs else None
    d_out = torch.zeros(batch, dtype=torch.float32, device="cuda") if logprobs else None
    d_k = to_torch(k_arr) if k_arr is not None else None
    d_p = to_torch(p_arr) if p_arr is not None else None
    d_skip = to_torch(skip) if skip is not None else None
    d_end, d_u = to_torch(end_ids), to_torch(u)
    ws_size = C.c_size_t(0)
    ops.check(lib.ftk_invoke_batch_topk_sampling(dt, None, C.addressof(ws_size), None, None, None, None, None, None,
                                                 None, None, max_k, None, 1.0, None, Vp, None, None, batch, None))
    ws = torch.empty(max(ws_size.value, 16), dtype=torch.uint8, device="cuda")
    ops.check(lib.ftk_invoke_batch_topk_sampling(dt, ws.data_ptr(), C.addressof(ws_size), d_logits.data_ptr(),
                                                 d_ids.data_ptr(), ops.ptr(d_seq), ops.ptr(d_fin), ops.ptr(d_cum),
                                                 ops.ptr(d_out), None, d_u.data_ptr(), max_k, ops.ptr(d_k), 1.0,
                                                 ops.ptr(d_p), Vp, d_end.data_ptr(), ops.current_stream(), batch,
                                                 ops.ptr(d_skip)))
    _sync(torch)
    return (to_numpy(d_ids), to_numpy(d_fin) if d_fin is not None else None,
            to_numpy(d_seq) if d_seq is not None else None, to_numpy(d_cum) if logprobs else None,
            to_numpy(d_out) if logprobs else None)


def _oracle_topk(dt, logits, k_arr, p_arr, max_k, end_ids, u, finished=None, seq=None, skip=None, logprobs=False):
    batch, Vp = logits.shape
    ids = np.full(batch, -7, np.int32)
    fin = finished.copy() if finished is not None else None
    sq = seq.copy() if seq is not None else None
    cum = np.zeros(batch, np.float32) if logprobs else None
    out = np.zeros(batch, np.float32) if logprobs else None
    rc = O.batch_topk_sampling(dt, logits, ids, sq, fin, cum, out, u, max_k, k_arr, 1.0, p_arr, Vp, end_ids, batch,
                               skip)
    assert rc == 0
    return ids, fin, sq, cum, out


def _compare_topk(a, b, dt):
    assert np.array_equal(a[0], b[0]), "sampled ids differ"
    for x, y in zip(a[1:3], b[1:3]):
        if x is not None:
            assert np.array_equal(x, y)
    rtol = 1e-5 if dt == O.F32 else 2e-3
    for x, y in zip(a[3:], b[3:]):
        if x is not None:
            np.testing.assert_allclose(x, y, rtol=rtol, atol=1e-6)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("V,batch,ks", [
    (8, 6, [1, 2, 4, 2, 1, 3]), (4000, 8, [1, 4, 63, 16, 17, 33, 64, 5]), (51200, 6, [1, 4, 16, 40, 64, 1024]),
    (50257, 4, [40, 40, 7, 1]), (32000, 5, [50, 50, 200, 300, 1000]),
])
def test_topk_sampling_logits(env, dt, V, batch, ks):
    rng = np.random.default_rng(V + batch)
    logits = make_logits(rng, dt, batch, V, V, scale=3.0, spikes=4 if V > 100 else 0)
    k_arr = np.array(ks, np.int32)
    p_arr = rng.uniform(0.3, 1.0, batch).astype(np.float32)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    finished = np.zeros(batch, bool)
    finished[batch // 2] = True
    seq = rng.integers(1, 9, batch).astype(np.int32)
    skip = np.zeros(batch, bool)
    skip[-1] = V > 8
    for trial in range(3):
        u = uniforms(rng, batch)
        args = (dt, logits, k_arr, p_arr, int(k_arr.max()), end_ids, u, finished, seq, skip)
        _compare_topk(_run_topk(env, *args), _oracle_topk(*args), dt)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_topk_sampling_tie_stress(env, dt):
    """rows with few distinct values: the pick order is decided by the reference's tie rules alone"""
    rng = np.random.default_rng(77)
    for V, ks in [(5000, [8, 40, 64, 100]), (30000, [16, 33, 1, 500]), (1024, [1024, 700, 3, 64])]:
        batch = len(ks)
        levels = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0], np.float32)
        x = levels[rng.integers(0, len(levels), (batch, V))]
        x[0, :] = 1.0  # a completely flat row: takes the literal replay
        logits = O.to_storage(x, dt)
        k_arr = np.array(ks, np.int32)
        p_arr = np.ones(batch, np.float32)
        end_ids = np.zeros(batch, np.int32)
        for trial in range(2):
            u = uniforms(rng, batch)
            args = (dt, logits, k_arr, p_arr, int(k_arr.max()), end_ids, u)
            _compare_topk(_run_topk(env, *args), _oracle_topk(*args), dt)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_topk_sampling_on_probabilities_with_logprobs(env, dt):
    rng = np.random.default_rng(9)
    batch, V = 6, 4000
    logits = make_logits(rng, dt, batch, V, V, scale=3.0)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    probs = logits.copy()
    O.add_bias_softmax(dt, probs, None, end_ids, None, batch, V, V)
    k_arr = np.array([1, 4, 63, 16, 64, 200], np.int32)
    p_arr = rng.uniform(0.2, 1.0, batch).astype(np.float32)
    finished = np.zeros(batch, bool)
    seq = np.ones(batch, np.int32)
    u = uniforms(rng, batch)
    args = (dt, probs, k_arr, p_arr, 200, end_ids, u, finished, seq, None, True)
    _compare_topk(_run_topk(env, *args), _oracle_topk(*args), dt)


def test_topk_domain_error(env):
    torch, lib, ops = env
    ws = C.c_size_t(0)
    rc = lib.ftk_invoke_batch_topk_sampling(O.F32, None, C.addressof(ws), None, None, None, None, None, None, None,
                                            None, 1025, None, 1.0, None, 4000, None, None, 4, None)
    assert rc == -2  # the reference throws std::domain_error for k = 1025


def _run_topp(env, dt, probs, p_arr, end_ids, u, finished=None, seq=None, skip=None, logprobs=False, force_deep=False):
    torch, lib, ops = env
    if force_deep:
        lib = ops.ftk_hooks()  # the switch exists in the test build of the library only
    batch, Vp = probs.shape
    d_probs = to_torch(probs, dt)
    d_ids = torch.full((batch,), -7, dtype=torch.int32, device="cuda")
    d_fin = to_torch(finished) if finished is not None else None
    d_seq = to_torch(seq) if seq is not None else None
    d_cum = torch.zeros(batch, dtype=torch.float32, device="cuda") if logprobs else None
    d_out = torch.zeros(batch, dtype=torch.float32, device="cuda") if logprobs else None
    d_p = to_torch(p_arr)
    d_skip = to_torch(skip) if skip is not None else None
    d_end, d_u = to_torch(end_ids), to_torch(u)
    ws_size, cub = C.c_size_t(0), C.c_size_t(0)
    ops.check(lib.ftk_invoke_batch_topp_sampling(dt, None, C.addressof(ws_size), C.addressof(cub), None, None, None,
                                                 None, None, None, None, None, None, None, None, batch, Vp, None, 1.0,
                                                 None, None, None))
    ws = torch.empty(max(ws_size.value, 16), dtype=torch.uint8, device="cuda")
    if force_deep:
        lib.ftk_test_set_topp_force_deep(1)
    try:
        ops.check(lib.ftk_invoke_batch_topp_sampling(dt, ws.data_ptr(), C.addressof(ws_size), C.addressof(cub),
                                                     d_ids.data_ptr(), ops.ptr(d_seq), ops.ptr(d_fin), ops.ptr(d_cum),
                                                     ops.ptr(d_out), d_probs.data_ptr(), None, None, None, None,
                                                     d_u.data_ptr(), batch, Vp, d_end.data_ptr(),
                                                     float(p_arr.max()), d_p.data_ptr(), ops.current_stream(),
                                                     ops.ptr(d_skip)))
        _sync(torch)
    finally:
        if force_deep:
            lib.ftk_test_set_topp_force_deep(0)
    return (to_numpy(d_ids), to_numpy(d_fin) if d_fin is not None else None,
            to_numpy(d_seq) if d_seq is not None else None, to_numpy(d_cum) if logprobs else None,
            to_numpy(d_out) if logprobs else None)


def _oracle_topp(dt, probs, p_arr, end_ids, u, finished=None, seq=None, skip=None, logprobs=False):
    batch, Vp = probs.shape
    ids = np.full(batch, -7, np.int32)
    fin = finished.copy() if finished is not None else None
    sq = seq.copy() if seq is not None else None
    cum = np.zeros(batch, np.float32) if logprobs else None
    out = np.zeros(batch, np.float32) if logprobs else None
    O.batch_topp_sampling(dt, probs, ids, sq, fin, cum, out, u, batch, Vp, end_ids, 0.0, p_arr, skip)
    return ids, fin, sq, cum, out


def _zipf_probs(rng, dt, batch, V, s=1.1, noise=0.5):
    ranks = np.arange(1, V + 1, dtype=np.float64)
    base = -s * np.log(ranks)
    x = np.empty((batch, V), np.float32)
    for b in range(batch):
        x[b] = (base[rng.permutation(V)] + rng.standard_normal(V) * noise).astype(np.float32)
    logits = O.to_storage(x, dt)
    probs = logits.copy()
    O.add_bias_softmax(dt, probs, None, np.zeros(batch, np.int32), None, batch, V, V)
    return probs


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("V,batch", [(8, 6), (4000, 8), (51200, 6), (128256, 4)])
@pytest.mark.parametrize("force_deep", [False, True])
def test_topp_sampling(env, dt, V, batch, force_deep):
    rng = np.random.default_rng(V + batch + dt)
    probs = _zipf_probs(rng, dt, batch, V) if V > 8 else None
    if probs is None:
        x = np.log(np.array([0.4, 0.3, 0.2, 0.1, 1e-9, 1e-9, 1e-9, 1e-9], np.float32))
        logits = O.to_storage(np.tile(x, (batch, 1)), dt)
        probs = logits.copy()
        O.add_bias_softmax(dt, probs, None, np.zeros(batch, np.int32), None, batch, V, V)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    finished = np.zeros(batch, bool)
    seq = rng.integers(1, 9, batch).astype(np.int32)
    skip = np.zeros(batch, bool)
    skip[1] = True
    for trial in range(3):
        p_arr = rng.uniform(0.2, 1.0, batch).astype(np.float32)
        if trial == 2:
            p_arr[:] = 1.0
        u = uniforms(rng, batch)
        if trial == 2:
            u[0] = 1.0  # draw at the very end of the distribution: may never be crossed
        args = (dt, probs, p_arr, end_ids, u, finished, seq, skip, True)
        got = _run_topp(env, *args, force_deep=force_deep)
        _compare_topk(got, _oracle_topp(*args), dt)


@pytest.mark.parametrize("dt", [O.F32, O.F16], ids=lambda d: DTYPE_NAMES[d])
def test_topp_sampling_flat_and_tied_rows(env, dt):
    """uniform / heavily tied distributions: stable order (ascending id among equals) decides"""
    rng = np.random.default_rng(21)
    batch, V = 4, 20000
    x = np.zeros((batch, V), np.float32)
    x[1] = rng.integers(0, 3, V).astype(np.float32)
    x[2, :100] = 5.0
    x[3] = np.where(rng.random(V) < 0.5, -np.inf, 0.0)
    logits = O.to_storage(x, dt)
    probs = logits.copy()
    O.add_bias_softmax(dt, probs, None, np.zeros(batch, np.int32), None, batch, V, V)
    end_ids = np.zeros(batch, np.int32)
    for trial in range(3):
        p_arr = rng.uniform(0.3, 1.0, batch).astype(np.float32)
        u = uniforms(rng, batch)
        args = (dt, probs, p_arr, end_ids, u)
        _compare_topk(_run_topp(env, *args), _oracle_topp(*args), dt)


@pytest.mark.parametrize("force_deep", [False, True])
def test_topp_pick_follows_the_reference_scan_order(env, force_deep):
    """Draws that lie within a bit of a prefix sum: the position depends on the rounding order of the reference's
    block scan (cub BLOCK_SCAN_RAKING with a running prefix, simulated thread by thread from the vendored sources in
    tests/cub_block_scan.py). Every draw of the set is crossed at another position by a plain running sum, a 64 x 4
    or a 16 x 16 raking of the same terms; the expected ids come from the simulation, not from the oracle."""
    import cub_block_scan as S
    from test_oracle import _topp_rows_for_scan_order
    cases = []
    for probs in _topp_rows_for_scan_order():
        order = np.argsort(-probs, kind="stable")
        for r, pos, alt_pos in S.discriminating_draws(probs[order]):
            cases.append((probs, r, int(order[pos])))
    assert len(cases) >= 60
    V = max(len(c[0]) for c in cases)
    batch = len(cases)
    probs = np.zeros((batch, V), np.float32)          # shorter rows end in zeros: they trail the order
    for b, (row, _, _) in enumerate(cases):
        probs[b, :len(row)] = row
    u = np.array([c[1] for c in cases], np.float32)
    want = np.array([c[2] for c in cases], np.int32)
    p_arr = np.ones(batch, np.float32)                # r = u * 1.0f exactly
    end_ids = np.zeros(batch, np.int32)
    got = _run_topp(env, O.F32, probs, p_arr, end_ids, u, force_deep=force_deep)
    assert np.array_equal(got[0], want), np.nonzero(got[0] != want)[0]
    assert np.array_equal(_oracle_topp(O.F32, probs, p_arr, end_ids, u)[0], want)


def test_topp_decay_and_initialize(env):
    torch, lib, ops = env
    rng = np.random.default_rng(3)
    n = 300
    top_p = rng.uniform(0.1, 1.0, n).astype(np.float32)
    init = rng.uniform(0.1, 1.0, n).astype(np.float32)
    ids = rng.integers(0, 20, n).astype(np.int32)
    reset = rng.integers(0, 20, n).astype(np.int32)
    decay = rng.uniform(0.5, 1.0, n).astype(np.float32)
    pmin = rng.uniform(0.05, 0.6, n).astype(np.float32)
    ref = top_p.copy()
    O.compute_topp_decay(ref, init, ids, decay, pmin, reset, n)
    d = to_torch(top_p)
    d_init, d_ids, d_decay, d_pmin, d_reset = (to_torch(x) for x in (init, ids, decay, pmin, reset))
    ops.check(lib.ftk_invoke_compute_topp_decay(d.data_ptr(), d_init.data_ptr(), d_ids.data_ptr(), d_decay.data_ptr(),
                                                d_pmin.data_ptr(), d_reset.data_ptr(), n, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(to_numpy(d).view(np.uint32), ref.view(np.uint32))
    batch, V = 5, 77
    idv = torch.zeros(batch * V, dtype=torch.int32, device="cuda")
    off = torch.zeros(batch + 1, dtype=torch.int32, device="cuda")
    boff = torch.zeros(batch + 1, dtype=torch.int32, device="cuda")
    ops.check(lib.ftk_invoke_topp_initialize(idv.data_ptr(), off.data_ptr(), boff.data_ptr(), batch, V,
                                             ops.current_stream()))
    _sync(torch)
    assert np.array_equal(to_numpy(idv), np.tile(np.arange(V, dtype=np.int32), batch))
    assert np.array_equal(to_numpy(off), np.arange(batch + 1, dtype=np.int32) * V)
    assert np.array_equal(to_numpy(boff), to_numpy(off))


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("shared", [True, False])
def test_ban_bad_words(env, dt, shared):
    torch, lib, ops = env
    rng = np.random.default_rng(8 + int(shared))
    batch, local, V, step, ite = 8, 4, 500, 9, 1
    logits = make_logits(rng, dt, batch, V, V)
    out_ids = rng.integers(1, V, (step + 1, batch)).astype(np.int32)
    lists = []
    for row in range(batch):
        wl, _ = make_word_list(rng, 12, 4, V, L=48, history=out_ids, step=step, row=row)
        lists.append(wl)
    bad = lists[0] if shared else np.stack(lists)
    ref = logits.copy()
    off = ite * local
    bw = bad if shared else bad[off:]
    O.ban_bad_words(dt, ref[off:], out_ids, batch, local, np.ascontiguousarray(bw), shared, 48, off, V, step)
    d = to_torch(logits, dt)
    d_bad, d_ids = to_torch(np.ascontiguousarray(bw)), to_torch(out_ids)
    elem = 4 if dt == O.F32 else 2
    ops.check(lib.ftk_invoke_ban_bad_words(dt, d.data_ptr() + off * V * elem, d_ids.data_ptr(), None, batch, local, 1,
                                           d_bad.data_ptr(), shared, 48, off, V, step, ops.current_stream()))
    _sync(torch)
    got = to_numpy(d, dt)
    assert np.array_equal(bits(got, dt), bits(ref, dt))
    assert np.isinf(O.to_f32(got, dt)).any()  # the case actually bans something


def test_stop_words_and_length_criterion(env):
    torch, lib, ops = env
    rng = np.random.default_rng(4)
    batch, V, step = 16, 50, 7
    out_ids = rng.integers(1, V, (step + 1, batch)).astype(np.int32)
    lists = []
    for row in range(batch):
        wl, _ = make_word_list(rng, 6, 3, V, L=20)
        if row % 3 == 0:  # plant a stop word that matches the tail including the token at `step`
            n = 1 + row % 3 + (row // 3) % 3
            n = min(n, 3)
            tail = out_ids[step - n + 1:step + 1, row]
            wl[0, :n] = tail
            wl[1, 0] = n
        lists.append(wl)
    stop = np.stack(lists)
    finished = np.zeros(batch, bool)
    ref = finished.copy()
    O.stop_words_criterion(out_ids, stop, ref, 0, 20, batch, batch, step)
    assert ref.any()
    d_fin = to_torch(finished)
    d_ids, d_stop = to_torch(out_ids), to_torch(stop)
    ops.check(lib.ftk_invoke_stop_words_criterion(d_ids.data_ptr(), None, d_stop.data_ptr(), d_fin.data_ptr(), 0, 20,
                                                  batch, 1, step, ops.current_stream()))
    _sync(torch)
    assert np.array_equal(to_numpy(d_fin), ref)
    # length criterion
    limit = rng.integers(3, 12, batch).astype(np.uint32)
    for st, pre in [(5, ref), (20, ref)]:
        fin = pre.copy()
        should = np.zeros(1, bool)
        O.length_criterion(fin, should, limit, batch, st)
        d_fin = to_torch(pre)
        d_limit = to_torch(limit)
        pinned = torch.zeros(1, dtype=torch.int32).pin_memory()
        host_flag = np.zeros(1, bool)
        ops.check(lib.ftk_invoke_length_criterion(d_fin.data_ptr(), host_flag.ctypes.data, pinned.data_ptr(),
                                                  d_limit.data_ptr(), batch, 1, st, ops.current_stream()))
        assert np.array_equal(to_numpy(d_fin), fin)
        assert bool(host_flag[0]) == bool(should[0])
        assert int(pinned[0]) == int(fin.sum())


def test_rng_determinism_and_range(env):
    torch, _, ops = env
    lib = ops.ftk_hooks()
    batch, n = 64, 500
    st = torch.zeros(batch * 2, dtype=torch.int64, device="cuda")
    ops.check(lib.ftk_invoke_curand_initialize(st.data_ptr(), batch, 1234, ops.current_stream()))
    out1 = torch.empty(batch * n, dtype=torch.float32, device="cuda")
    ops.check(lib.ftk_test_rng_uniform(st.data_ptr(), out1.data_ptr(), batch, n, ops.current_stream()))
    _sync(torch)
    a = to_numpy(out1).reshape(batch, n)
    assert (a > 0).all() and (a <= 1).all()
    assert np.array_equal(a[0], a[17])  # same seed, same stream of draws
    assert abs(a.mean() - 0.5) < 0.02
    assert to_numpy(st).reshape(batch, 2)[:, 1].tolist() == [n] * batch  # offsets advanced
    seeds = to_torch(np.arange(batch, dtype=np.uint64) // 3)
    ops.check(lib.ftk_invoke_curand_batch_initialize(st.data_ptr(), batch, seeds.data_ptr(), ops.current_stream()))
    ops.check(lib.ftk_test_rng_uniform(st.data_ptr(), out1.data_ptr(), batch, n, ops.current_stream()))
    _sync(torch)
    b = to_numpy(out1).reshape(batch, n)
    assert np.array_equal(b[0], b[1]) and np.array_equal(b[0], b[2]) and not np.array_equal(b[2], b[3])
    # known answer: first draw of seed 0 is Philox4x32-10(ctr=0,key=0)[0] = 0x6627e8d5
    expect = np.float32(np.float32(0x6627e8d5) * np.float32(2.3283064365386963e-10) + np.float32(1.16415321826934814453125e-10))
    assert b[0, 0] == expect


def _softmax_rows(dt, x):
    logits = O.to_storage(x, dt)
    probs = logits.copy()
    batch, V = x.shape
    O.add_bias_softmax(dt, probs, None, np.zeros(batch, np.int32), None, batch, V, V)
    return probs


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_topp_sampling_sort_paths(env, dt):
    """Rows built to reach every way a segment of the ordered prefix is sorted: a few dozen entries (one
    wave), bins joined into groups, one long group of equal keys (whole workgroup), a bucket longer than the
    in-LDS limit (radix sort in memory), and draws at the far end so that everything is ordered."""
    rng = np.random.default_rng(77 + dt)
    V = 12000
    x = np.full((8, V), -30.0, np.float32)
    x[0, :40] = rng.normal(0, 1, 40)                       # 40 candidates, the rest negligible
    x[1, :3000] = 0.0                                      # 3000 equal keys: one long group
    x[2, :7000] = 0.0                                      # 7000 equal keys: longer than the LDS limit
    x[3] = rng.normal(0, 0.02, V)                          # one or two crowded buckets, distinct keys
    x[4] = rng.normal(0, 3.0, V)                           # wide: many buckets
    x[5, :300] = np.repeat(rng.normal(0, 1, 3), 100)       # three groups of 100 equal keys
    x[6] = np.round(rng.normal(0, 1.0, V) * 4) / 4         # heavy ties over a wide range
    x[7, :5000] = rng.normal(0, 0.001, 5000)               # 5000 nearly equal, distinct keys
    probs = _softmax_rows(dt, x)
    end_ids = np.zeros(8, np.int32)
    for u_val in (0.05, 0.5, 0.93, 0.9999):
        p_arr = np.full(8, 1.0, np.float32)
        u = np.full(8, u_val, np.float32)
        args = (dt, probs, p_arr, end_ids, u, None, None, None, True)
        _compare_topk(_run_topp(env, *args), _oracle_topp(*args), dt)


def test_topp_sampling_unnormalised_input(env):
    """The entry point takes any numbers: values above 1, denormals, zeros, negatives. (NaN is left out: the
    reference's order of a row with NaN is that of cub's radix sort on the bit patterns, which the oracle's
    comparison sort does not define.)"""
    rng = np.random.default_rng(5)
    V = 9000
    probs = rng.random((5, V)).astype(np.float32)
    probs[0] *= 3.0                                         # mass far above 1
    probs[1] *= 1e-12                                       # everything in the lowest bucket
    probs[2, ::2] = 0.0
    probs[3, ::3] = -1.0
    probs[4] = np.float32(1e-40)                            # denormal, all equal
    end_ids = np.zeros(5, np.int32)
    for u_val in (0.2, 0.999):
        p_arr = np.full(5, 0.9, np.float32)
        u = np.full(5, u_val, np.float32)
        args = (O.F32, probs, p_arr, end_ids, u)
        _compare_topk(_run_topp(env, *args), _oracle_topp(*args), O.F32)


def test_topp_sampling_many_rows(env):
    """More rows than one tile of the segment scheduler (1024), a third of them deep."""
    rng = np.random.default_rng(9)
    batch, V = 2500, 700
    x = rng.normal(0, 1.5, (batch, V)).astype(np.float32)
    probs = _softmax_rows(O.F32, x)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    p_arr = rng.uniform(0.3, 1.0, batch).astype(np.float32)
    u = uniforms(rng, batch)
    u[::3] = 0.999
    skip = rng.random(batch) < 0.1
    args = (O.F32, probs, p_arr, end_ids, u, None, None, skip, True)
    _compare_topk(_run_topp(env, *args), _oracle_topp(*args), O.F32)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_softmax_and_topp_random_shapes(env, dt, seed):
    """Seeded random vocabulary sizes (odd ones included: rows that do not start on a 16-byte boundary, heads
    and tails of the vector loops), pad columns, batch sizes, shapes of distribution and draws; the softmax is
    compared bit for bit, top-p by ids, flags, lengths and log-probs."""
    torch, lib, ops = env
    rng = np.random.default_rng(1000 * dt + seed)
    for case in range(4):
        V = int(rng.choice([rng.integers(9, 300), rng.integers(300, 9000), rng.integers(9000, 70000)]))
        Vp = V + int(rng.choice([0, 0, 1, 7, 64]))
        batch = int(rng.integers(1, 10))
        kind = int(rng.integers(0, 4))
        if kind == 0:
            x = rng.standard_normal((batch, Vp)) * rng.uniform(0.1, 4.0)
        elif kind == 1:
            ranks = np.arange(1, Vp + 1, dtype=np.float64)
            x = np.stack([(-rng.uniform(0.8, 1.5) * np.log(ranks))[rng.permutation(Vp)] for _ in range(batch)])
            x = x + rng.standard_normal((batch, Vp)) * 0.3
        elif kind == 2:
            x = rng.integers(0, 4, (batch, Vp)).astype(np.float64) * rng.uniform(0.2, 2.0)   # few distinct values
        else:
            x = np.where(rng.random((batch, Vp)) < 0.7, -np.inf, rng.standard_normal((batch, Vp)))
            x[:, 0] = 0.0
        logits = O.to_storage(x.astype(np.float32), dt)
        end_ids = rng.integers(0, V, batch).astype(np.int32)
        finished = rng.random(batch) < 0.15
        want = logits.copy()
        O.add_bias_softmax(dt, want, None, end_ids, finished, batch, Vp, V)
        d_probs = to_torch(logits, dt)
        d_end, d_fin = to_torch(end_ids), to_torch(finished)
        ops.check(lib.ftk_invoke_add_bias_softmax(dt, d_probs.data_ptr(), None, d_end.data_ptr(), d_fin.data_ptr(),
                                                  batch, Vp, V, ops.current_stream()))
        _sync(torch)
        got = to_numpy(d_probs)
        assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8)), (V, Vp, batch, kind)
        for trial in range(2):
            p_arr = rng.uniform(0.1, 1.0, batch).astype(np.float32)
            u = uniforms(rng, batch)
            if trial == 1:
                u[:] = rng.choice([1e-6, 0.5, 0.999, 1.0], batch).astype(np.float32)
                p_arr[::2] = 1.0
            seq = rng.integers(1, 9, batch).astype(np.int32)
            skip = rng.random(batch) < 0.2
            args = (dt, want, p_arr, end_ids, u, finished.copy(), seq, skip, True)
            _compare_topk(_run_topp(env, *args), _oracle_topp(*args), dt)


@pytest.mark.parametrize("V,Vp", [(1024, 1024), (1025, 1031), (128256, 128256), (152064 - 1, 152064)])
def test_fused_topp_step_full_vocabularies(env, V, Vp):
    """the one-call top-p step at the reference block's width, one column beyond it, and at full vocabulary
    sizes (several chunks per row in the dividing pass)"""
    _fused_topp_cases(env, O.F32, np.random.default_rng(V + Vp), [(V, Vp, 3, 0), (V, Vp, 2, 1), (V, Vp, 3, 2)])


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_fused_topp_step_against_the_three_calls_of_the_oracle(env, dt, seed):
    """ftk_fused_topp_step = softmax, top-p sampler and decay in one call: the probabilities left in the logits
    buffer bit for bit, ids, flags, lengths, log-probs and the decayed top_p, on seeded random shapes with pad
    columns, finished and skipped rows, with and without an embedding bias."""
    rng = np.random.default_rng(7000 + 100 * dt + seed)
    shapes = []
    for case in range(5):
        V = int(rng.choice([rng.integers(9, 300), rng.integers(300, 9000), rng.integers(9000, 70000)]))
        shapes.append((V, V + int(rng.choice([0, 0, 1, 7, 64])), int(rng.integers(1, 12)), int(rng.integers(0, 3))))
    _fused_topp_cases(env, dt, rng, shapes)


@pytest.mark.parametrize("seed", [253, 290, 345, 1628, 2213, 6951, 13587, 22768])
def test_topp_sample_step_equal_probabilities_from_different_numerators(env, seed):
    """Seeded cases (mostly bfloat16, where a probability has one or two numerators) in which entries that share a
    probability come from different buckets of the numerator's histogram: the step that samples straight from the
    logits must keep all of them or none in its ordered prefix and emit the id the reference's stable order of the
    whole row puts at the sampled position."""
    rng = np.random.default_rng(424200 + seed)
    dt = int(rng.integers(0, 3))
    V = int(rng.choice([1024, 1025, rng.integers(1026, 5000), rng.integers(5000, 40000), rng.integers(40000, 160000)]))
    Vp = V + int(rng.choice([0, 0, 1, 7, 64]))
    batch = int(rng.integers(1, 7))
    kind = int(rng.integers(0, 3))
    _fused_topp_cases(env, dt, rng, [(V, Vp, batch, kind)])


def _fused_topp_cases(env, dt, rng, shapes):
    torch, lib, ops = env
    for case, (V, Vp, batch, kind) in enumerate(shapes):
        if kind == 0:
            x = rng.standard_normal((batch, Vp)) * rng.uniform(0.1, 4.0)
        elif kind == 1:
            ranks = np.arange(1, Vp + 1, dtype=np.float64)
            x = np.stack([(-rng.uniform(0.8, 1.5) * np.log(ranks))[rng.permutation(Vp)] for _ in range(batch)])
            x = x + rng.standard_normal((batch, Vp)) * 0.3
        else:
            x = rng.integers(0, 4, (batch, Vp)).astype(np.float64) * rng.uniform(0.2, 2.0)   # few distinct values
        logits = O.to_storage(x.astype(np.float32), dt)
        bias = O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt) if case % 2 else None
        end_ids = rng.integers(0, V, batch).astype(np.int32)
        finished = rng.random(batch) < 0.15
        skip = rng.random(batch) < 0.2
        seq = rng.integers(1, 9, batch).astype(np.int32)
        p_arr = rng.uniform(0.1, 1.0, batch).astype(np.float32)
        init = rng.uniform(0.5, 1.0, batch).astype(np.float32)
        decay = rng.uniform(0.5, 1.0, batch).astype(np.float32)
        pmin = rng.uniform(0.05, 0.4, batch).astype(np.float32)
        u = uniforms(rng, batch)
        with_decay = case != 2
        # the oracle, call by call
        want = logits.copy()
        O.add_bias_softmax(dt, want, bias, end_ids, finished, batch, Vp, V)
        w_ids, w_fin, w_seq, w_cum, w_out = _oracle_topp(dt, want, p_arr, end_ids, u, finished.copy(), seq, skip, True)
        reset = np.where(rng.random(batch) < 0.3, w_ids, -1).astype(np.int32)   # some rows hit their reset id
        w_p = p_arr.copy()
        if with_decay:
            O.compute_topp_decay(w_p, init, w_ids, decay, pmin, reset, batch)
        # the product, one call
        d_x, d_bias = to_torch(logits, dt), to_torch(bias, dt)
        d_ids = torch.full((batch,), -7, dtype=torch.int32, device="cuda")
        d_fin, d_seq, d_skip = to_torch(finished), to_torch(seq), to_torch(skip)
        d_cum = torch.zeros(batch, dtype=torch.float32, device="cuda")
        d_out = torch.zeros(batch, dtype=torch.float32, device="cuda")
        d_p, d_init, d_decay, d_pmin, d_reset = (to_torch(a) for a in (p_arr, init, decay, pmin, reset))
        d_end, d_u = to_torch(end_ids), to_torch(u)
        ws_size = C.c_size_t(0)
        sizes = (dt, None, C.addressof(ws_size), None, None, V, Vp, batch) + (None,) * 8 + (1.0,) + (None,) * 7
        ops.check(lib.ftk_fused_topp_step(*sizes))
        ws = torch.empty(max(ws_size.value, 16), dtype=torch.uint8, device="cuda")
        ops.check(lib.ftk_fused_topp_step(dt, ws.data_ptr(), C.addressof(ws_size), d_x.data_ptr(), ops.ptr(d_bias), V, Vp,
                                          batch, d_end.data_ptr(), d_fin.data_ptr(), d_seq.data_ptr(),
                                          d_ids.data_ptr(), d_cum.data_ptr(), d_out.data_ptr(), None, d_u.data_ptr(),
                                          float(p_arr.max()), d_p.data_ptr(), d_init.data_ptr(),
                                          d_decay.data_ptr() if with_decay else None, d_pmin.data_ptr(),
                                          d_reset.data_ptr(), d_skip.data_ptr(), ops.current_stream()))
        _sync(torch)
        where = (V, Vp, batch, kind, case)
        assert np.array_equal(np.asarray(to_numpy(d_x)).view(np.uint8), np.asarray(want).view(np.uint8)), where
        got = (to_numpy(d_ids), to_numpy(d_fin), to_numpy(d_seq), to_numpy(d_cum), to_numpy(d_out))
        _compare_topk(got, (w_ids, w_fin, w_seq, w_cum, w_out), dt)
        assert np.array_equal(to_numpy(d_p).view(np.uint32), w_p.view(np.uint32)), where
        # the same step straight from the logits, which it leaves alone (no bias, at least a block's width of columns)
        sample_sizes = (dt, None, C.addressof(ws_size), None, V, Vp, batch) + (None,) * 8 + (1.0,) + (None,) * 7
        rc = lib.ftk_fused_topp_sample_step(*sample_sizes)
        if V < 1024:
            assert rc == ops.FTK_ERR_UNSUPPORTED, where
            continue
        ops.check(rc)
        if bias is not None:
            continue
        ws = torch.empty(max(ws_size.value, 16), dtype=torch.uint8, device="cuda")
        d_x = to_torch(logits, dt)
        d_ids = torch.full((batch,), -7, dtype=torch.int32, device="cuda")
        d_fin, d_seq = to_torch(finished), to_torch(seq)
        d_cum = torch.zeros(batch, dtype=torch.float32, device="cuda")
        d_out = torch.zeros(batch, dtype=torch.float32, device="cuda")
        d_p = to_torch(p_arr)
        ops.check(lib.ftk_fused_topp_sample_step(dt, ws.data_ptr(), C.addressof(ws_size), d_x.data_ptr(), V, Vp, batch,
                                                 d_end.data_ptr(), d_fin.data_ptr(), d_seq.data_ptr(), d_ids.data_ptr(),
                                                 d_cum.data_ptr(), d_out.data_ptr(), None, d_u.data_ptr(),
                                                 float(p_arr.max()), d_p.data_ptr(), d_init.data_ptr(),
                                                 d_decay.data_ptr() if with_decay else None, d_pmin.data_ptr(),
                                                 d_reset.data_ptr(), d_skip.data_ptr(), ops.current_stream()))
        _sync(torch)
        assert np.array_equal(np.asarray(to_numpy(d_x)).view(np.uint8), np.asarray(logits).view(np.uint8)), where
        got = (to_numpy(d_ids), to_numpy(d_fin), to_numpy(d_seq), to_numpy(d_cum), to_numpy(d_out))
        _compare_topk(got, (w_ids, w_fin, w_seq, w_cum, w_out), dt)
        assert np.array_equal(to_numpy(d_p).view(np.uint32), w_p.view(np.uint32)), where


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("max_k", [129, 512, 513, 1024])
def test_topk_sampling_large_k_variants(env, dt, max_k):
    """Launches whose largest k exceeds 128 (and 512) take their own streaming variants: rows of several tiles,
    odd vocabulary (rows off the 16-byte grid), small k next to large k in one launch, smooth and heavily tied
    distributions, a row that is constant from some column on (cutting the list back in mid-tile cannot bound
    it: literal replay)."""
    rng = np.random.default_rng(max_k + dt)
    V = 70001
    batch = 6
    x = (rng.standard_normal((batch, V)) * 2.0).astype(np.float32)
    x[1] = rng.integers(0, 6, V).astype(np.float32) * 0.5        # six distinct values
    x[2, 20000:] = 3.0                                           # constant tail above most of the head
    x[3] = np.round(x[3] * 8) / 8                                # many small tie groups
    x[4, ::3] = -np.inf
    logits = O.to_storage(x, dt)
    k_arr = np.array([max_k, max_k, max_k, max(1, max_k // 2), max_k - 1, 5], np.int32)
    end_ids = np.zeros(batch, np.int32)
    for trial in range(2):
        p_arr = np.ones(batch, np.float32) if trial == 0 else rng.uniform(0.3, 1.0, batch).astype(np.float32)
        u = uniforms(rng, batch)
        args = (dt, logits, k_arr, p_arr, max_k, end_ids, u)
        _compare_topk(_run_topk(env, *args), _oracle_topk(*args), dt)


@pytest.mark.parametrize("max_k", [200, 700, 1024])
def test_topk_sampling_large_k_many_tiles_per_workgroup(env, max_k):
    """A vocabulary of more tiles than a row can be split into, so that every workgroup streams two tiles:
    the large-k variants then cut their list back between tiles (and in mid-tile beyond k = 512)."""
    rng = np.random.default_rng(max_k)
    V, batch = 1100003, 2
    x = (rng.standard_normal((batch, V)) * 2.0).astype(np.float32)
    x[1] = np.round(x[1] * 16) / 16   # tie groups of a few thousand columns
    logits = O.to_storage(x, O.F32)
    k_arr = np.array([max_k, max(1, max_k - 3)], np.int32)
    end_ids = np.zeros(batch, np.int32)
    p_arr = np.array([1.0, 0.7], np.float32)
    u = uniforms(rng, batch)
    args = (O.F32, logits, k_arr, p_arr, max_k, end_ids, u)
    _compare_topk(_run_topk(env, *args), _oracle_topk(*args), O.F32)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("seed", [0, 1, 2])
def test_topk_sampling_random_shapes(env, dt, seed):
    """Seeded random vocabulary sizes (odd ones included), batch sizes (hence different numbers of chunk lists
    per row), per-row k from 1 to the launch maximum, per-row top-p, smooth / tied / mostly masked rows,
    finished and skipped rows, log-probs on probabilities for half of the cases."""
    rng = np.random.default_rng(500 * dt + seed)
    for case in range(5):
        V = int(rng.choice([rng.integers(9, 400), rng.integers(400, 20000), rng.integers(20000, 140000)]))
        batch = int(rng.choice([1, 2, 5, 9, 17, 40]))
        max_k = int(rng.choice([1, 7, 64, 100, 200, 600, 1024]))
        max_k = max(1, min(max_k, 1024))
        kind = int(rng.integers(0, 3))
        if kind == 0:
            x = rng.standard_normal((batch, V)) * rng.uniform(0.3, 4.0)
        elif kind == 1:
            x = rng.integers(0, 5, (batch, V)).astype(np.float64) * rng.uniform(0.2, 1.5)
        else:
            x = np.where(rng.random((batch, V)) < 0.9, -np.inf, rng.standard_normal((batch, V)) * 2.0)
            x[:, 0] = 0.5
        logits = O.to_storage(x.astype(np.float32), dt)
        end_ids = rng.integers(0, V, batch).astype(np.int32)
        k_arr = rng.integers(1, max_k + 1, batch).astype(np.int32)
        k_arr[0] = max_k
        p_arr = np.where(rng.random(batch) < 0.5, 1.0, rng.uniform(0.1, 1.0, batch)).astype(np.float32)
        finished = rng.random(batch) < 0.1
        seq = rng.integers(1, 9, batch).astype(np.int32)
        skip = rng.random(batch) < 0.1
        u = uniforms(rng, batch)
        logprobs = bool(case & 1)
        src = logits
        if logprobs:
            src = logits.copy()
            O.add_bias_softmax(dt, src, None, end_ids, None, batch, V, V)
        args = (dt, src, k_arr, p_arr, max_k, end_ids, u, finished.copy(), seq, skip, logprobs)
        _compare_topk(_run_topk(env, *args), _oracle_topk(*args), dt)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_fused_step_lean_gather_equals_general_stream(env, dt):
    """The two streaming kernels of the fused step on the same launch: the lean gather (what a launch with k <= 128
    and no bias takes) and the general stream, forced through the hook of the test build. Sampled ids, lengths
    and flags must be identical, at a batch that splits rows over several workgroups and at one that does not."""
    from helpers import run_fused_step
    torch, _, ops = env
    hooks = ops.ftk_hooks()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(31 + dt)
    V, H, k = 100003, 40, 50
    for B in (24, 1030):
        logits = (torch.randn((B, V), generator=gen, device="cuda") * 2.0).to(ops.torch_dtype(dt))
        history = torch.randint(0, V, (H, B), generator=gen, device="cuda", dtype=torch.int32)
        draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
        finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
        finished0[1] = True
        seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
        lean = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks)
        hooks.ftk_test_set_fused_force_general(1)
        try:
            general = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0,
                                     lib=hooks)
        finally:
            hooks.ftk_test_set_fused_force_general(0)
        assert lean[3] == 0 and general[3] == 0
        for a, b in zip(lean[:3], general[:3]):
            assert np.array_equal(a, b)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_fused_step_one_launch_equals_two_launches(env, dt):
    """Batches that give every row to one workgroup finish the step in the gather's launch (the workgroup goes on to
    order its list and sample). The same launch with the selection kept in a kernel of its own, forced through the
    hook of the test build, must give identical ids, lengths and flags: many short rows, long rows, and a row that
    is finished on entry."""
    from helpers import run_fused_step
    torch, _, ops = env
    hooks = ops.ftk_hooks()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77 + dt)
    for B, V, H, k in ((3000, 9000, 12, 40), (1100, 70001, 30, 64), (5, 3000, 4, 128)):
        logits = (torch.randn((B, V), generator=gen, device="cuda") * 2.0).to(ops.torch_dtype(dt))
        history = torch.randint(0, V, (H, B), generator=gen, device="cuda", dtype=torch.int32)
        draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
        finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
        finished0[1] = True
        seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
        one = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks)
        hooks.ftk_test_set_fused_two_launches(1)
        try:
            two = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks)
        finally:
            hooks.ftk_test_set_fused_two_launches(0)
        assert one[3] == 0 and two[3] == 0
        for a, b in zip(one[:3], two[:3]):
            assert np.array_equal(a, b)
