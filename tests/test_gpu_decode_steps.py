"""GPU parity of the steps either side of the sampling path (through the C ABI) against the oracle:
invokeLogProbFromLogits, invokeDecodingInitialize, invokePlusScalar, invokeTransposeAxis01."""
import ctypes as C

import numpy as np
import pytest

import ft_oracle as O
from helpers import DTYPE_NAMES, DTYPES, to_numpy, to_torch

pytestmark = pytest.mark.gpu


def _lib():
    from fastertransformer_amd import ops
    return ops, ops.ftk()


# the shapes of tests/unittests/test_logprob_kernels.cu:266-303 (max_input_length, batch, vocab)
LOGPROB_SHAPES = [(1, 32, 16), (129, 8, 50211), (1023, 8, 5001), (4096, 8, 5001), (7, 5, 1003)]


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("batch_first", [False, True], ids=["time_major", "batch_first"])
@pytest.mark.parametrize("shape", LOGPROB_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_log_prob_from_logits(dt, batch_first, shape):
    import torch
    ops, lib = _lib()
    max_len, batch, V = shape
    Vp = (V + 7) // 8 * 8 if V != 1003 else V  # 1003: rows that do not start on a 16-byte boundary
    rng = np.random.default_rng(31)
    shp = (batch, max_len, Vp) if batch_first else (max_len, batch, Vp)
    logits = O.to_storage((rng.standard_normal(shp) * 3).astype(np.float32), dt)
    ids = rng.integers(0, V, (batch, max_len) if batch_first else (max_len, batch)).astype(np.int32)
    lengths = rng.integers(1, max_len + 1, batch).astype(np.int32)
    lengths[0] = max_len
    want_cum, want_lp = O.log_prob_from_logits(dt, logits, ids, lengths, max_len, batch, V, Vp, batch_first)

    d_logits, d_ids, d_len = to_torch(logits, dt), to_torch(ids), to_torch(lengths)
    d_cum = torch.full((batch,), 123.0, dtype=torch.float32, device="cuda")
    ws = torch.zeros(max_len * batch, dtype=torch.float32, device="cuda")
    st = ops.current_stream()
    ops.check(lib.ftk_invoke_log_prob_from_logits(dt, d_cum.data_ptr(), d_logits.data_ptr(), d_ids.data_ptr(),
                                                  d_len.data_ptr(), max_len, batch, V, Vp, ws.data_ptr(),
                                                  ws.numel() * 4, st, batch_first))
    torch.cuda.synchronize()
    got_lp = to_numpy(ws)[:max(max_len - 1, 1) * batch]
    # compare the per-step values where the row is inside its sequence
    for b in range(batch):
        for step in range(min(max_len - 1, 64)):
            if step < lengths[b] - 1:
                i = b * (max_len - 1) + step if batch_first else step * batch + b
                assert abs(got_lp[i] - want_lp[i]) <= 2e-5 * max(1.0, abs(want_lp[i])), (b, step)
    np.testing.assert_allclose(to_numpy(d_cum), want_cum, rtol=2e-5, atol=2e-4)
    # a workspace that is too small is refused (the reference asserts)
    assert lib.ftk_invoke_log_prob_from_logits(dt, d_cum.data_ptr(), d_logits.data_ptr(), d_ids.data_ptr(),
                                               d_len.data_ptr(), max_len, batch, V, Vp, ws.data_ptr(), 4, st,
                                               batch_first) == ops.FTK_ERR_WORKSPACE


def test_log_prob_masked_logits():
    """rows holding -inf entries (banned tokens) and one row that is -inf everywhere except the target"""
    import torch
    ops, lib = _lib()
    max_len, batch, V = 3, 4, 300
    rng = np.random.default_rng(32)
    logits = (rng.standard_normal((max_len, batch, V)) * 2).astype(np.float32)
    logits[0, 1, ::3] = -np.inf
    ids = rng.integers(0, V, (max_len, batch)).astype(np.int32)
    logits[1, 2, :] = -np.inf
    logits[1, 2, ids[2, 2]] = 0.5
    ids[1, 1] = 1  # a column that was not banned
    lengths = np.full(batch, max_len, np.int32)
    want_cum, _ = O.log_prob_from_logits(O.F32, logits, ids, lengths, max_len, batch, V, V)
    d = [to_torch(a) for a in (logits, ids, lengths)]
    cum = torch.zeros(batch, dtype=torch.float32, device="cuda")
    ws = torch.zeros(max_len * batch, dtype=torch.float32, device="cuda")
    ops.check(lib.ftk_invoke_log_prob_from_logits(O.F32, cum.data_ptr(), d[0].data_ptr(), d[1].data_ptr(),
                                                  d[2].data_ptr(), max_len, batch, V, V, ws.data_ptr(), ws.numel() * 4,
                                                  ops.current_stream(), False))
    np.testing.assert_allclose(to_numpy(cum), want_cum, rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_decoding_initialize(dt):
    import torch
    ops, lib = _lib()
    rng = np.random.default_rng(33)
    for batch, beam, with_ids in ((5, 1, True), (7, 4, True), (300, 1, False)):
        sent = rng.integers(0, 1000, batch).astype(np.int32)
        n = batch * beam
        fin = torch.ones(n, dtype=torch.bool, device="cuda")
        seq = torch.zeros(n, dtype=torch.int32, device="cuda")
        ids = torch.full((n,), -1, dtype=torch.int32, device="cuda")
        cum = to_torch(O.to_storage(np.full(n, 3.0, np.float32), dt), dt)
        d_sent = to_torch(sent)
        ops.check(lib.ftk_invoke_decoding_initialize(dt, fin.data_ptr(), seq.data_ptr(),
                                                     ids.data_ptr() if with_ids else None, cum.data_ptr(),
                                                     d_sent.data_ptr(), batch, beam, 19, ops.current_stream()))
        w_fin, w_seq, w_ids, w_cum = O.decoding_initialize(dt, sent, batch, beam, 19, with_ids)
        assert np.array_equal(to_numpy(fin), w_fin) and np.array_equal(to_numpy(seq), w_seq)
        if with_ids:
            assert np.array_equal(to_numpy(ids), w_ids)
        else:
            assert (to_numpy(ids) == -1).all()
        assert np.array_equal(O.to_f32(to_numpy(cum, dt), dt), O.to_f32(O.to_storage(w_cum, dt), dt))


def test_plus_scalar_and_transpose():
    import torch
    ops, lib = _lib()
    rng = np.random.default_rng(34)
    for size in (1, 255, 256, 100003):
        buf = rng.integers(-1000, 1000, size).astype(np.int32)
        d = to_torch(buf)
        ops.check(lib.ftk_invoke_plus_scalar(d.data_ptr(), 17, size, ops.current_stream()))
        assert np.array_equal(to_numpy(d), buf + 17)
    for dim0, dim1 in ((1, 1), (37, 53), (64, 32), (1025, 257), (300, 2048)):
        a = rng.integers(0, 1 << 30, (dim0, dim1)).astype(np.int32)
        d_in = to_torch(a)
        d_out = torch.zeros((dim1, dim0), dtype=torch.int32, device="cuda")
        ops.check(lib.ftk_invoke_transpose_axis01(d_out.data_ptr(), d_in.data_ptr(), None, dim0, dim1,
                                                  ops.current_stream()))
        assert np.array_equal(to_numpy(d_out), O.transpose_axis01(a, None, dim0, dim1))
    dim0, dim1 = 41, 70
    big = rng.integers(0, 1 << 30, (dim0 + 6, dim1)).astype(np.int32)
    skip = rng.integers(0, 7, dim1).astype(np.int32)
    d_in, d_skip = to_torch(big), to_torch(skip)
    d_out = torch.zeros((dim1, dim0), dtype=torch.int32, device="cuda")
    ops.check(lib.ftk_invoke_transpose_axis01(d_out.data_ptr(), d_in.data_ptr(), d_skip.data_ptr(), dim0, dim1,
                                              ops.current_stream()))
    assert np.array_equal(to_numpy(d_out), O.transpose_axis01(big, skip, dim0, dim1))
    assert lib.ftk_invoke_transpose_axis01(d_in.data_ptr(), d_in.data_ptr(), None, dim0, dim1,
                                           ops.current_stream()) == ops.FTK_ERR_ARGUMENT


@pytest.mark.parametrize("beam_width,ties", [(1, False), (2, True), (4, False), (16, True), (100, True), (511, False)])
def test_finalize(beam_width, ties):
    """invokeFinalize against the oracle (ranking of the hypotheses of a batch entry by score, smaller index first
    among equal scores; copies without the first position), with and without the optional outputs."""
    import torch
    from test_oracle import _finalize_case
    ops, lib = _lib()
    rng = np.random.default_rng(950 + beam_width)
    batch, max_seq_len = 7, 41
    ids, lens, scores, cum, lps, num = _finalize_case(rng, batch, beam_width, max_seq_len, ties)
    want = O.finalize(ids, lens, scores, cum, lps, num, beam_width, max_seq_len, batch)
    d = [to_torch(a) for a in (ids, lens, scores, cum, lps, num)]
    out_ids = torch.zeros((batch, beam_width, max_seq_len), dtype=torch.int32, device="cuda")
    out_len = torch.zeros((batch, beam_width), dtype=torch.int32, device="cuda")
    out_cum = torch.zeros((batch, beam_width), dtype=torch.float32, device="cuda")
    out_lp = torch.zeros((batch, beam_width, max_seq_len), dtype=torch.float32, device="cuda")
    st = ops.current_stream()
    ops.check(lib.ftk_invoke_finalize(out_ids.data_ptr(), out_len.data_ptr(), out_cum.data_ptr(), out_lp.data_ptr(),
                                      d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                                      d[4].data_ptr(), d[5].data_ptr(), beam_width, max_seq_len, batch, st))
    torch.cuda.synchronize()
    assert np.array_equal(to_numpy(out_ids), want[0]) and np.array_equal(to_numpy(out_len), want[1])
    assert np.array_equal(to_numpy(out_cum), want[2]) and np.array_equal(to_numpy(out_lp), want[3])
    out_ids.zero_()
    ops.check(lib.ftk_invoke_finalize(out_ids.data_ptr(), out_len.data_ptr(), None, None, d[0].data_ptr(),
                                      d[1].data_ptr(), d[2].data_ptr(), None, None, d[5].data_ptr(), beam_width,
                                      max_seq_len, batch, st))
    torch.cuda.synchronize()
    assert np.array_equal(to_numpy(out_ids), want[0])
    assert lib.ftk_invoke_finalize(out_ids.data_ptr(), out_len.data_ptr(), None, None, d[0].data_ptr(),
                                   d[1].data_ptr(), d[2].data_ptr(), None, None, d[5].data_ptr(), 512, max_seq_len,
                                   batch, st) == ops.FTK_ERR_ARGUMENT
