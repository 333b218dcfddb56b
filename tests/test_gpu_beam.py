"""GPU parity of one beam-search step (ftk_invoke_topk_softmax, the reference's invokeTopkSoftMax) against the
oracle through the C ABI: next beams' ids, parents and hypotheses bit for bit, log-probs within tolerance."""
import ctypes as C

import numpy as np
import pytest

import ft_oracle as O
from helpers import DTYPE_NAMES, DTYPES, copy_beam_case, make_beam_case, to_numpy, to_torch

pytestmark = pytest.mark.gpu

HYP_ARRAYS = ("output_ids_tgt", "sequence_lengths_tgt", "cum_log_probs", "normed_scores", "log_probs",
              "min_normed_scores", "num_beams", "is_done", "output_ids_src", "parent_ids_src", "log_probs_src")


def _lib():
    from fastertransformer_amd import ops
    return ops, ops.ftk()


def _run_product(c, dt, batch, K, V, diversity, length_penalty, bias=None, lib=None):
    """the step on the GPU; returns (ids, cum_log_probs, output_log_probs, hypotheses arrays) as numpy"""
    import torch
    ops, product = _lib()
    lib = product if lib is None else lib
    d = {k: to_torch(c[k]) for k in ("finished", "sequence_lengths", "cum_log_probs", "end_ids", "ids",
                                     "output_log_probs")}
    d_x = to_torch(c["log_probs"], dt)
    d_bias = to_torch(bias, dt) if bias is not None else None
    hyps, d_h = None, {}
    if c["hyps"] is not None:
        hyps = ops.BeamHypotheses()
        for name in HYP_ARRAYS:
            d_h[name] = to_torch(c["hyps"][name])
            setattr(hyps, name, d_h[name].data_ptr())
        hyps.end_ids = d["end_ids"].data_ptr()
        for name in ("step", "ite", "batch_size", "local_batch_size", "max_seq_len"):
            setattr(hyps, name, int(c["hyps"][name]))
        hyps.length_penalty = float(length_penalty)
        hyps.early_stopping = bool(c["hyps"]["early_stopping"])
        hyps.is_return_normed_score = True
    size = C.c_size_t(0)
    args = (dt, d_x.data_ptr(), ops.ptr(d_bias), d["finished"].data_ptr(), d["sequence_lengths"].data_ptr(),
            d["cum_log_probs"].data_ptr(), d["output_log_probs"].data_ptr(), d["ids"].data_ptr())
    tail = (C.addressof(hyps) if hyps is not None else None, batch, K, V, d["end_ids"].data_ptr(), float(diversity),
            float(length_penalty), ops.current_stream())
    ops.check(lib.ftk_invoke_topk_softmax(*args, None, C.addressof(size), *tail))
    ws = torch.empty(max(size.value, 16), dtype=torch.uint8, device="cuda")
    ops.check(lib.ftk_invoke_topk_softmax(*args, ws.data_ptr(), C.addressof(size), *tail))
    torch.cuda.synchronize()
    return (to_numpy(d["ids"]), to_numpy(d["cum_log_probs"]), to_numpy(d["output_log_probs"]),
            {k: to_numpy(v) for k, v in d_h.items()})


def _compare(c, want, got, dt):
    ids, cum, out_lp, hyps = got
    rtol = 2e-5 if dt == O.F32 else 4e-3
    where = "ids"
    assert np.array_equal(ids, want["ids"]), where
    np.testing.assert_allclose(cum, want["cum_log_probs"], rtol=rtol, atol=1e-5)
    np.testing.assert_allclose(out_lp, want["output_log_probs"], rtol=rtol, atol=1e-3 if dt != O.F32 else 2e-5)
    if want["hyps"] is not None:
        for name in ("output_ids_tgt", "sequence_lengths_tgt", "num_beams", "is_done"):
            assert np.array_equal(hyps[name], want["hyps"][name]), name
        for name in ("cum_log_probs", "normed_scores", "log_probs", "min_normed_scores"):
            np.testing.assert_allclose(hyps[name], want["hyps"][name], rtol=rtol, atol=1e-3 if dt != O.F32 else 2e-5,
                                       err_msg=name)


def _one_case(rng, dt, batch, K, V, with_hyps, diversity, length_penalty, step=5, max_seq_len=12, **kw):
    c = make_beam_case(rng, dt, batch, K, V, step=step, max_seq_len=max_seq_len, with_hyps=with_hyps, **kw)
    want = copy_beam_case(c)
    rc = O.topk_softmax(dt, want["log_probs"], None, want["finished"], want["sequence_lengths"],
                        want["cum_log_probs"], want["output_log_probs"], want["ids"], want["hyps"], batch, K, V,
                        want["end_ids"], diversity, length_penalty)
    assert rc == 0
    print("beam case", DTYPE_NAMES[dt], batch, K, V, with_hyps, diversity, length_penalty, flush=True)
    _compare(c, want, _run_product(c, dt, batch, K, V, diversity, length_penalty), dt)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("K", [2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64])
def test_beam_step_every_width_class(dt, K):
    """every beam-width class of the reference's dispatch (1-4, 5-8, 9-16, 17-32, 33-64) at its edges, with and
    without hypotheses, penalties on and off"""
    rng = np.random.default_rng(100 * K + dt)
    for V in (2 * K, 2 * K + 1, 1000, 20011):
        for with_hyps in (False, True):
            lp = float(rng.choice([0.0, 0.6, 1.0]))
            dv = float(rng.choice([0.0, 0.0, 0.25]))
            _one_case(rng, dt, int(rng.integers(1, 5)), K, V, with_hyps, dv, lp)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_beam_step_full_vocabularies_and_batches(dt):
    """vocabulary sizes of the headline configurations (several sections per row, merged per row), a batch large
    enough for one section per row, long histories to trace"""
    rng = np.random.default_rng(7 + dt)
    _one_case(rng, dt, 8, 4, 50257, True, 0.0, 0.8, step=30, max_seq_len=40)
    _one_case(rng, dt, 2, 8, 128256, True, 0.1, 0.0)
    _one_case(rng, dt, 300, 4, 3000, True, 0.0, 1.0)
    _one_case(rng, dt, 1, 2, 152064, False, 0.0, 0.0)


@pytest.mark.parametrize("path", [1, 2, 3], ids=["sections_three_launches", "one_workgroup_per_row",
                                                  "one_512_thread_workgroup_per_row"])
def test_beam_step_both_forms_of_the_row_stage(path):
    """The row stage has two forms, chosen by the shape: sections of rows in three launches, and one workgroup per row
    in one launch (1024 threads, or 512 when there are more rows than compute units). The test build of the library forces either on the same cases: every
    beam-width class, tiny and full vocabularies, more rows than compute units, rows of equal values (the bound
    passes more than fits the list), rows masked to -inf, finished beams, NaN columns."""
    from fastertransformer_amd import ops
    hooks = ops.ftk_hooks()
    rng = np.random.default_rng(77)
    hooks.ftk_test_set_beam_path(path)
    try:
        for dt in DTYPES:
            for batch, K, V in ((2, 2, 4), (3, 4, 9), (1, 64, 128), (2, 33, 1000), (4, 8, 50257), (1, 16, 152064),
                                (90, 4, 2500), (2, 3, 20011)):
                c = make_beam_case(rng, dt, batch, K, V, step=5, max_seq_len=12, with_hyps=True)
                want = copy_beam_case(c)
                assert O.topk_softmax(dt, want["log_probs"], None, want["finished"], want["sequence_lengths"],
                                      want["cum_log_probs"], want["output_log_probs"], want["ids"], want["hyps"],
                                      batch, K, V, want["end_ids"], 0.1, 0.7) == 0
                print("beam form", path, DTYPE_NAMES[dt], batch, K, V, flush=True)
                _compare(c, want, _run_product(c, dt, batch, K, V, 0.1, 0.7, lib=hooks), dt)
        batch, K, V = 3, 4, 5000
        for kind in range(4):
            c = make_beam_case(rng, O.F32, batch, K, V, with_hyps=True, finished_frac=0.0)
            if kind == 0:
                c["log_probs"][:] = np.float32(1.5)
                c["cum_log_probs"][:] = np.float32(-1.0)
            elif kind == 1:
                c["log_probs"][:] = -np.inf
                c["log_probs"][:, rng.choice(V, 3 * K, replace=False)] = rng.standard_normal(3 * K).astype(np.float32)
            elif kind == 2:
                c["finished"][:] = True
            else:
                c["log_probs"][:, rng.choice(V, 40, replace=False)] = np.nan
            want = copy_beam_case(c)
            assert O.topk_softmax(O.F32, want["log_probs"], None, want["finished"], want["sequence_lengths"],
                                  want["cum_log_probs"], want["output_log_probs"], want["ids"], want["hyps"], batch,
                                  K, V, want["end_ids"], 0.0, 0.5) == 0
            print("beam form", path, "degenerate kind", kind, flush=True)
            _compare(c, want, _run_product(c, O.F32, batch, K, V, 0.0, 0.5, lib=hooks), O.F32)
    finally:
        hooks.ftk_test_set_beam_path(0)


def test_beam_step_degenerate_rows():
    """rows of equal values (ties settled by the lower id at every stage), rows masked to -inf except a few
    columns, every beam finished, hypotheses already complete for every entry"""
    rng = np.random.default_rng(3)
    batch, K, V = 3, 4, 5000
    for kind in range(4):
        c = make_beam_case(rng, O.F32, batch, K, V, with_hyps=True, finished_frac=0.0)
        if kind == 0:
            c["log_probs"][:] = np.float32(1.5)
            c["cum_log_probs"][:] = np.float32(-1.0)
        elif kind == 1:
            c["log_probs"][:] = -np.inf
            c["log_probs"][:, rng.choice(V, 3 * K, replace=False)] = rng.standard_normal(3 * K).astype(np.float32)
        elif kind == 2:
            c["finished"][:] = True
        else:
            c["hyps"]["num_beams"][:] = K
        want = copy_beam_case(c)
        assert O.topk_softmax(O.F32, want["log_probs"], None, want["finished"], want["sequence_lengths"],
                              want["cum_log_probs"], want["output_log_probs"], want["ids"], want["hyps"], batch, K, V,
                              want["end_ids"], 0.0, 0.5) == 0
        print("degenerate kind", kind, flush=True)
        _compare(c, want, _run_product(c, O.F32, batch, K, V, 0.0, 0.5), O.F32)


def test_beam_step_with_bias_and_refusals():
    import torch
    ops, lib = _lib()
    rng = np.random.default_rng(9)
    batch, K, V = 2, 3, 777
    for dt in DTYPES:
        c = make_beam_case(rng, dt, batch, K, V, with_hyps=True)
        bias = O.to_storage(rng.standard_normal(V).astype(np.float32), dt)
        want = copy_beam_case(c)
        assert O.topk_softmax(dt, want["log_probs"], bias, want["finished"], want["sequence_lengths"],
                              want["cum_log_probs"], want["output_log_probs"], want["ids"], want["hyps"], batch, K, V,
                              want["end_ids"], 0.0, 0.0) == 0
        _compare(c, want, _run_product(c, dt, batch, K, V, 0.0, 0.0, bias=bias), dt)
    size = C.c_size_t(0)
    none = (None,) * 8
    for K_bad in (1, 65):  # the reference's dispatch throws for these
        assert lib.ftk_invoke_topk_softmax(O.F32, *none[:7], None, C.addressof(size), None, 2, K_bad, 1000, None, 0.0,
                                           0.0, None) == ops.FTK_ERR_ARGUMENT
    assert lib.ftk_invoke_topk_softmax(O.F32, *none[:7], None, C.addressof(size), None, 2, 8, 15, None, 0.0, 0.0,
                                       None) == ops.FTK_ERR_ARGUMENT   # fewer columns than 2 * beam_width
    assert lib.ftk_invoke_topk_softmax(7, *none[:7], None, C.addressof(size), None, 2, 8, 100, None, 0.0, 0.0,
                                       None) == ops.FTK_ERR_DTYPE
    ops.check(lib.ftk_invoke_topk_softmax(O.F32, *none[:7], None, C.addressof(size), None, 2, 8, 100, None, 0.0, 0.0,
                                          None))
    ws = torch.empty(16, dtype=torch.uint8, device="cuda")
    small = C.c_size_t(16)
    assert lib.ftk_invoke_topk_softmax(O.F32, *none[:7], ws.data_ptr(), C.addressof(small), None, 2, 8, 100, None,
                                       0.0, 0.0, None) == ops.FTK_ERR_WORKSPACE


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("penalty_type", [0, 1, 2], ids=["presence", "repetition", "none"])
def test_beam_penalties(dt, penalty_type):
    """ftk_invoke_add_bias_apply_penalties against the oracle, bit for bit: even and odd vocabularies (the half2
    form and the generic one), pad columns, with and without bias, windows of a larger batch, long histories"""
    import torch
    from helpers import make_beam_history
    ops, lib = _lib()
    rng = np.random.default_rng(40 + dt + 10 * penalty_type)
    for V, Vp, batch, local, ite, K, step, max_input in ((300, 300, 3, 3, 0, 4, 7, 4), (301, 304, 4, 2, 1, 3, 5, 5),
                                                         (50257, 50264, 2, 2, 0, 2, 1, 1), (32000, 32000, 5, 5, 0, 8, 40, 8),
                                                         (1000, 1024, 2, 1, 1, 64, 12, 3)):
        L = step + 3
        out_ids, parents, input_lengths = make_beam_history(rng, batch, K, V, step, L, max_input)
        rows = local * K
        for with_bias, temperature in ((False, 1.0), (True, 0.7), (False, 1.6)):
            x = O.to_storage((rng.standard_normal((rows, Vp)) * 3).astype(np.float32), dt)
            bias = O.to_storage(rng.standard_normal(Vp).astype(np.float32), dt) if with_bias else None
            seq = rng.integers(max_input, max_input + 6, rows).astype(np.int32)
            end_ids = rng.integers(0, V, local).astype(np.int32)
            current = out_ids[step - 1, ite * rows:(ite + 1) * rows].copy()
            lens = input_lengths[:rows].copy()
            penalty = 1.0 if penalty_type == 2 else float(rng.choice([0.5, 1.3, 2.0]))
            min_length = int(rng.integers(0, 8))
            want = x.copy()
            O.beam_add_bias_apply_penalties(dt, step, want, current, out_ids, parents, lens, seq, bias, ite, max_input,
                                            local, batch, K, V, Vp, end_ids, temperature, penalty, penalty_type,
                                            min_length)
            d = [to_torch(a) for a in (current, out_ids, parents, lens, seq, end_ids)]
            d_x, d_bias = to_torch(x, dt), (to_torch(bias, dt) if with_bias else None)
            print("penalties", DTYPE_NAMES[dt], V, Vp, batch, local, ite, K, step, with_bias, temperature, flush=True)
            ops.check(lib.ftk_invoke_add_bias_apply_penalties(
                dt, step, d_x.data_ptr(), d[0].data_ptr(), d[1].data_ptr(), d[2].data_ptr(), d[3].data_ptr(),
                d[4].data_ptr(), ops.ptr(d_bias), ite, max_input, local, batch, K, V, Vp, d[5].data_ptr(),
                temperature, penalty, penalty_type, min_length, ops.current_stream()))
            torch.cuda.synchronize()
            got = to_numpy(d_x)
            assert np.array_equal(np.asarray(got).view(np.uint8), np.asarray(want).view(np.uint8))


def test_beam_update_and_cache_indirection():
    import torch
    ops, lib = _lib()
    rng = np.random.default_rng(61)
    for batch, K, Vp, L, step in ((4, 3, 500, 9, 5), (70, 64, 32000, 20, 25), (1, 2, 50264, 6, 0), (300, 4, 1000, 64, 63)):
        word = (rng.integers(0, K, (batch, K)) + np.arange(batch)[:, None] * K) * Vp + rng.integers(0, Vp, (batch, K))
        word = word.astype(np.int32).reshape(-1)
        end_ids = rng.integers(0, Vp, batch).astype(np.int32)
        ends = rng.random(batch * K) < 0.2
        word[ends] = word[ends] // Vp * Vp + np.repeat(end_ids, K)[ends]
        word[rng.random(batch * K) < 0.1] = -7   # slots the step never wrote: the caller's old contents
        finished = rng.random(batch * K) < 0.3
        seq = rng.integers(3, 9, batch * K).astype(np.int32)
        num_beams = np.where(rng.random(batch) < 0.3, K, rng.integers(0, K, batch)).astype(np.int32)
        for hyps_on in (True, False):
            f, s_, w = finished.copy(), seq.copy(), word.copy()
            parent, out = np.full(batch * K, -1, np.int32), np.full(batch * K, -1, np.int32)
            O.beam_update(f, parent, s_, w, out, num_beams if hyps_on else None, 0, batch, K, Vp, end_ids)
            d_f, d_s, d_w, d_end, d_num = (to_torch(a) for a in (finished, seq, word, end_ids, num_beams))
            d_parent = torch.full((batch * K,), -1, dtype=torch.int32, device="cuda")
            hyps = ops.BeamHypotheses()
            hyps.num_beams, hyps.ite, hyps.local_batch_size = d_num.data_ptr(), 0, batch
            # output_ids and word_ids are the same array in the layer's call
            ops.check(lib.ftk_invoke_beam_update(d_f.data_ptr(), d_parent.data_ptr(), d_s.data_ptr(), d_w.data_ptr(),
                                                 d_w.data_ptr(), C.addressof(hyps) if hyps_on else None, batch, K, Vp,
                                                 d_end.data_ptr(), ops.current_stream()))
            torch.cuda.synchronize()
            for got, want in ((d_f, f), (d_parent, parent), (d_s, s_), (d_w, w)):
                assert np.array_equal(to_numpy(got), want)
            src = rng.integers(0, K, (batch, K, L)).astype(np.int32)
            tgt = np.full((batch, K, L), -7, np.int32)
            want_tgt = tgt.copy()
            O.update_indir_cache(want_tgt, src, parent, f, batch, K, L, step)
            d_tgt, d_src = to_torch(tgt), to_torch(src)
            ops.check(lib.ftk_invoke_update_indir_cache(d_tgt.data_ptr(), d_src.data_ptr(), d_parent.data_ptr(),
                                                        d_f.data_ptr(), batch, batch, K, L, step,
                                                        ops.current_stream()))
            torch.cuda.synchronize()
            assert np.array_equal(to_numpy(d_tgt), want_tgt)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("penalty", ["repetition_penalty", "presence_penalty", None])
def test_online_beam_search_layer_decode_loop(dt, penalty):
    """OnlineBeamSearchLayer::forward step after step (penalties over beam histories, the step, the update of the
    beams, the cache indirection, hypotheses collected on the way) against the same sequence of oracle calls: ids,
    parents, flags, lengths, hypotheses and cache indirection bit for bit, log-probs within tolerance."""
    rng = np.random.default_rng(200 + dt + (0 if penalty is None else len(penalty)))
    collected = _decode_loop_case(rng, dt, penalty, batch=3, K=4, V=997, Vp=1000, max_input=3, L=12, steps=7,
                                  temperature=0.8, diversity=0.1, len_pen=0.7, min_length=2)
    assert collected > 0   # the loop did collect hypotheses


@pytest.mark.parametrize("shape", [(1, 2, 64, 64, 1, 6, 5), (2, 8, 2051, 2056, 4, 16, 9), (5, 3, 333, 336, 2, 9, 6),
                                   (2, 16, 4099, 4104, 2, 8, 5)], ids=lambda s: "b%d_k%d_v%d" % s[:3])
def test_online_beam_search_layer_decode_loop_shapes(shape):
    """The same loop at other batch sizes, beam widths and vocabularies, with and without length penalty and
    diversity rate."""
    batch, K, V, Vp, max_input, L, steps = shape
    rng = np.random.default_rng(260 + K)
    for dt, penalty, diversity, len_pen in ((O.F32, "repetition_penalty", 0.0, 0.0), (O.F16, None, 0.3, 1.0),
                                            (O.BF16, "presence_penalty", 0.05, 0.4)):
        _decode_loop_case(rng, dt, penalty, batch=batch, K=K, V=V, Vp=Vp, max_input=max_input, L=L, steps=steps,
                          temperature=float(rng.choice([1.0, 0.7, 1.3])), diversity=diversity, len_pen=len_pen,
                          min_length=int(rng.integers(0, 4)))


def _decode_loop_case(rng, dt, penalty, batch, K, V, Vp, max_input, L, steps, temperature, diversity, len_pen,
                      min_length):
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    rows = batch * K
    pen_val = {"repetition_penalty": 1.2, "presence_penalty": 0.4, None: None}[penalty]
    ptype = {"repetition_penalty": 1, "presence_penalty": 0, None: 2}[penalty]
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    # host state of the oracle run
    out_ids = np.zeros((L, rows), np.int32)
    out_ids[:max_input] = rng.integers(0, V, (max_input, rows))
    parents = np.zeros((L, rows), np.int32)
    parents[:max_input] = np.arange(rows) % K
    out_lp = np.zeros((L, rows), np.float32)
    finished = np.zeros(rows, np.bool_)
    seq = np.full(rows, max_input - 1, np.int32)
    cum = np.tile(np.array([0.0] + [-1e20] * (K - 1), np.float32), batch)   # only beam 0 counts at the first step
    input_lengths = rng.integers(1, max_input + 1, rows).astype(np.int32)
    hyps = dict(output_ids_tgt=np.zeros((batch, 2 * K, L), np.int32), sequence_lengths_tgt=np.zeros((batch, 2 * K), np.int32),
                cum_log_probs=np.zeros((batch, 2 * K), np.float32), normed_scores=np.zeros((batch, 2 * K), np.float32),
                log_probs=np.zeros((batch, 2 * K, L), np.float32), min_normed_scores=np.zeros(batch, np.float32),
                num_beams=np.zeros(batch, np.int32), is_done=np.zeros(batch, np.bool_))
    cache = [rng.integers(0, K, (batch, K, L)).astype(np.int32), np.zeros((batch, K, L), np.int32)]
    # the same state on the device
    d = {k: to_torch(v) for k, v in dict(out_ids=out_ids.reshape(L, batch, K), parents=parents, out_lp=out_lp.reshape(L, batch, K),
                                         finished=finished, seq=seq, cum=cum, input_lengths=input_lengths,
                                         end_ids=end_ids).items()}
    d_h = {k: to_torch(v) for k, v in hyps.items()}
    d_cache = [to_torch(c) for c in cache]
    dh = ops.BeamHypotheses()
    for k, v in d_h.items():
        setattr(dh, k, v.data_ptr())
    dh.early_stopping, dh.is_return_normed_score = True, True
    layer = fa.OnlineBeamSearchLayer(dt, V, Vp)
    for i in range(steps):
        step = max_input + i
        x = (rng.standard_normal((rows, Vp)) * 3).astype(np.float32)
        for r in range(rows):       # end tokens show up often enough to fill the hypotheses
            if rng.random() < 0.25:
                x[r, end_ids[r // K]] += 9.0
        logits = O.to_storage(x, dt)
        # ---- oracle
        want = logits.copy()
        O.beam_add_bias_apply_penalties(dt, step, want, out_ids[step - 1], out_ids, parents, input_lengths, seq, None, 0,
                                        max_input, batch, batch, K, V, Vp, end_ids, temperature,
                                        pen_val if pen_val is not None else 1.0, ptype, min_length)
        h = dict(hyps, output_ids_src=out_ids, parent_ids_src=parents, sequence_lengths_src=None, end_ids=end_ids,
                 log_probs_src=out_lp, step=step, ite=0, batch_size=batch, local_batch_size=batch, max_seq_len=L,
                 length_penalty=len_pen, early_stopping=1)
        assert O.topk_softmax(dt, want, None, finished, seq, cum, out_lp[step], out_ids[step], h, batch, K, Vp, end_ids,
                              diversity, len_pen) == 0
        O.beam_update(finished, parents[step], seq, out_ids[step], out_ids[step], hyps["num_beams"], 0, batch, K, Vp,
                      end_ids)
        O.update_indir_cache(cache[1], cache[0], parents[step], finished, batch, K, L, step)
        # ---- the layer
        ins = {"logits": to_torch(logits, dt).reshape(batch, K, Vp), "step": np.array([step], np.int32),
               "ite": np.array([0], np.int32), "max_input_length": np.array([max_input], np.int32),
               "end_id": d["end_ids"], "src_cache_indirection": d_cache[0], "input_lengths": d["input_lengths"],
               "temperature": np.array([temperature], np.float32), "len_penalty": np.array([len_pen], np.float32),
               "beam_search_diversity_rate": np.array([diversity], np.float32),
               "min_length": np.array([min_length], np.int32)}
        if penalty is not None:
            ins[penalty] = np.array([pen_val], np.float32)
        outs = {"output_ids": d["out_ids"], "finished": d["finished"], "cum_log_probs": d["cum"],
                "parent_ids": d["parents"], "sequence_length": d["seq"], "tgt_cache_indirection": d_cache[1],
                "output_log_probs": d["out_lp"], "beam_hyps": dh}
        print("layer step", DTYPE_NAMES[dt], penalty, step, flush=True)
        layer.forward(outs, ins)
        torch.cuda.synchronize()
        rtol, atol = (2e-5, 2e-5) if dt == O.F32 else (4e-3, 1e-3)
        assert np.array_equal(to_numpy(d["out_ids"]).reshape(L, rows)[step], out_ids[step]), step
        assert np.array_equal(to_numpy(d["parents"])[step], parents[step])
        assert np.array_equal(to_numpy(d["finished"]), finished) and np.array_equal(to_numpy(d["seq"]), seq)
        np.testing.assert_allclose(to_numpy(d["cum"]), cum, rtol=rtol, atol=atol)
        np.testing.assert_allclose(to_numpy(d["out_lp"]).reshape(L, rows)[step], out_lp[step], rtol=rtol, atol=atol)
        assert np.array_equal(to_numpy(d_cache[1]), cache[1])
        for name in ("output_ids_tgt", "sequence_lengths_tgt", "num_beams", "is_done"):
            assert np.array_equal(to_numpy(d_h[name]), hyps[name]), name
        for name in ("cum_log_probs", "normed_scores", "log_probs", "min_normed_scores"):
            np.testing.assert_allclose(to_numpy(d_h[name]), hyps[name], rtol=rtol, atol=atol, err_msg=name)
        cache.reverse()
        d_cache.reverse()
    layer.close()
    return int(hyps["num_beams"].sum())


@pytest.mark.parametrize("differing", [False, True], ids=["same_runtime_values", "differing_runtime_values"])
@pytest.mark.parametrize("windows", [1, 2], ids=["one_window", "two_windows"])
def test_dynamic_decode_layer_with_beams(windows, differing):
    """DynamicDecodeLayer::forward on logits [batch, beam_width > 1, vocab]: the beam-search layer per window of the
    batch and the length criterion, against the same oracle calls, with word lists in the one-window variant. When
    setup() saw per-entry runtime values that differ, the entries go to the beam-search layer one by one, each call
    reading the first value of every list (layers/DynamicDecodeLayer.cc:289-294, BaseBeamSearchLayer.cu:220)."""
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    dt = O.F32
    rng = np.random.default_rng(300 + windows)
    batch, K, V, Vp, max_input, L, steps = 4, 3, 500, 504, 2, 10, 5
    local = batch // windows
    rows = batch * K
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    out_ids = np.zeros((L, rows), np.int32)
    out_ids[:max_input] = rng.integers(0, V, (max_input, rows))
    parents = np.zeros((L, rows), np.int32)
    parents[:max_input] = np.arange(rows) % K
    finished = np.zeros(rows, np.bool_)
    seq = np.full(rows, max_input - 1, np.int32)
    cum = np.tile(np.array([0.0] + [-1e20] * (K - 1), np.float32), batch)
    limit = np.full(batch, max_input + 3, np.uint32)     # the length criterion ends every beam at that step
    d = {k: to_torch(v) for k, v in dict(out_ids=out_ids.reshape(L, batch, K), parents=parents, finished=finished,
                                         seq=seq, cum=cum, end_ids=end_ids, limit=limit).items()}
    src = [rng.integers(0, K, (local, K, L)).astype(np.int32), np.zeros((local, K, L), np.int32)]
    d_src = [to_torch(c) for c in src]
    layer = fa.DynamicDecodeLayer(dt, V, Vp)
    temperatures = np.array([0.9, 1.3, 0.9, 0.6] if differing else [0.9], np.float32)
    layer.setup(batch, K, {"temperature": temperatures})
    group = 1 if differing else local     # entries per call of the beam-search layer
    should_stop = np.zeros(1, np.bool_)
    for i in range(steps):
        step = max_input + i
        x = (rng.standard_normal((rows, Vp)) * 3).astype(np.float32)
        d_x = to_torch(x).reshape(batch, K, Vp)
        # Bad-word lists ride along in every variant: each beam is banned from its own entry's list over its own
        # history, whichever window it belongs to (with several windows the reference offsets the launch of a later
        # window by entries instead of by beams, so that the bans land on other beams' rows; that defect is not
        # reproduced). Stop-word lists in the one-window variant.
        bad = stop = None
        if step >= 2:
            bad = _beam_word_lists(rng, batch, K, V, 6, 3, 24, out_ids, parents, step, with_last=False)
            O.ban_bad_words_beams(dt, x, out_ids, parents, batch, batch, K, bad, False, 24, 0, Vp, step)
        for ite in range(windows):
            for sub in range(ite * local // group, (ite + 1) * local // group):
                lo, hi = sub * group * K, (sub + 1) * group * K
                ends = end_ids[sub * group:(sub + 1) * group]
                want = x[lo:hi].copy()
                O.beam_add_bias_apply_penalties(dt, step, want, out_ids[step - 1, lo:hi].copy(), out_ids, parents, None,
                                                seq[lo:hi], None, sub, max_input, group, batch, K, V, Vp, ends, 0.9, 1.0,
                                                2, 0)
                ids_w, cum_w, fin_w, seq_w = (out_ids[step, lo:hi].copy(), cum[lo:hi].copy(), finished[lo:hi].copy(),
                                              seq[lo:hi].copy())
                assert O.topk_softmax(dt, want, None, fin_w, seq_w, cum_w, None, ids_w, None, group, K, Vp, ends, 0.0,
                                      0.0) == 0
                par_w = np.zeros(group * K, np.int32)
                O.beam_update(fin_w, par_w, seq_w, ids_w, ids_w, None, sub, group, K, Vp, ends)
                O.update_indir_cache(src[1], src[0], par_w, fin_w, group, K, L, step)
                out_ids[step, lo:hi], parents[step, lo:hi] = ids_w, par_w
                cum[lo:hi], finished[lo:hi], seq[lo:hi] = cum_w, fin_w, seq_w
            ins = {"logits": d_x, "step": np.array([step], np.int32), "max_input_length": np.array([max_input], np.int32),
                   "ite": np.array([ite], np.uint32), "local_batch_size": np.array([local], np.int32),
                   "end_id": d["end_ids"], "src_cache_indirection": d_src[0],
                   "temperature": temperatures, "sequence_limit_length": d["limit"]}
            outs = {"output_ids": d["out_ids"], "finished": d["finished"], "cum_log_probs": d["cum"],
                    "parent_ids": d["parents"], "sequence_length": d["seq"], "tgt_cache_indirection": d_src[1],
                    "should_stop": should_stop}
            if bad is not None:
                ins["bad_words_list"] = to_torch(bad)
            if bad is not None and windows == 1:
                # stop words: some of them end with what a beam has just chosen (known from the oracle's step)
                stop = _beam_word_lists(rng, batch, K, V, 4, 2, 16, out_ids, parents, step, with_last=True)
                O.stop_words_criterion_beams(out_ids, parents, stop, finished, 0, 16, batch, batch, K, step)
                ins["stop_words_list"] = to_torch(stop)
            print("dynamic decode with beams", windows, step, ite, flush=True)
            layer.forward(outs, ins)
            torch.cuda.synchronize()
            # the length criterion runs over the whole batch after every window
            finished |= step >= np.repeat(limit, K)
            assert np.array_equal(to_numpy(d_src[1]), src[1])
        assert np.array_equal(to_numpy(d["out_ids"]).reshape(L, rows)[step], out_ids[step]), step
        assert np.array_equal(to_numpy(d["parents"])[step], parents[step])
        assert np.array_equal(to_numpy(d["finished"]), finished) and np.array_equal(to_numpy(d["seq"]), seq)
        np.testing.assert_allclose(to_numpy(d["cum"]), cum, rtol=2e-5, atol=2e-5)
        assert bool(should_stop[0]) == bool(finished.all())
        src.reverse()
        d_src.reverse()
    assert finished.all() and should_stop[0]


def _beam_word_lists(rng, batch, K, V, n_words, max_len, L, out_ids, parents, step, with_last):
    """[batch, 2, L] word lists; about half of the words are copied from the history of a beam of their entry,
    followed back through the parent beams (ending at `step` when with_last, one before it otherwise, where a random
    last token is appended), so that they match"""
    lists = np.zeros((batch, 2, L), np.int32)
    lists[:, 1, :] = -1
    for b in range(batch):
        flat, ends = [], []
        for w in range(n_words):
            n = int(rng.integers(1, max_len + 1))
            take = n if with_last else n - 1
            last = step if with_last else step - 1
            if rng.random() < 0.5 and take <= last + 1:
                beam, toks = int(rng.integers(0, K)), []
                for t in range(last, last - take, -1):
                    toks.append(int(out_ids[t, b * K + beam]))
                    beam = int(parents[t, b * K + beam])
                word = toks[::-1] + ([] if with_last else [int(rng.integers(1, V))])
            else:
                word = [int(x) for x in rng.integers(1, V, n)]
            flat += word
            ends.append(len(flat))
        lists[b, 0, :len(flat)] = flat
        lists[b, 1, :len(ends)] = ends
    return lists


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_word_lists_with_beams(dt):
    """ftk_invoke_ban_bad_words and ftk_invoke_stop_words_criterion with beam_width > 1 against the oracle: words
    that match a beam's history through its parent beams, words that do not, shared and per-entry lists, a parent
    outside the beam range (ends the match)"""
    import torch
    ops, lib = _lib()
    rng = np.random.default_rng(77 + dt)
    for batch, K, V, step, L in ((3, 4, 300, 6, 40), (2, 8, 1000, 3, 24), (5, 2, 50, 9, 64)):
        rows = batch * K
        out_ids = rng.integers(1, V, (step + 2, rows)).astype(np.int32)
        parents = rng.integers(0, K, (step + 2, rows)).astype(np.int32)
        parents[step - 1, 0] = K + 3     # a broken chain for whoever walks through it
        for share in (False, True):
            bad = _beam_word_lists(rng, batch, K, V, 8, 4, L, out_ids, parents, step, with_last=False)
            words = bad[0] if share else bad
            x = O.to_storage(rng.standard_normal((rows, V)).astype(np.float32), dt)
            want = x.copy()
            O.ban_bad_words_beams(dt, want, out_ids, parents, batch, batch, K, np.ascontiguousarray(words), share, L, 0, V,
                                  step)
            d_x, d_ids, d_par, d_w = to_torch(x, dt), to_torch(out_ids), to_torch(parents), to_torch(np.ascontiguousarray(words))
            ops.check(lib.ftk_invoke_ban_bad_words(dt, d_x.data_ptr(), d_ids.data_ptr(), d_par.data_ptr(), batch, batch,
                                                   K, d_w.data_ptr(), share, L, 0, V, step, ops.current_stream()))
            torch.cuda.synchronize()
            got = np.asarray(to_numpy(d_x))
            assert np.array_equal(got.view(np.uint8), np.asarray(want).view(np.uint8))
            assert np.isinf(O.to_f32(want, dt)).sum() > 0          # something was banned
        stop = _beam_word_lists(rng, batch, K, V, 6, 3, L, out_ids, parents, step, with_last=True)
        fin = np.zeros(rows, np.bool_)
        O.stop_words_criterion_beams(out_ids, parents, stop, fin, 0, L, batch, batch, K, step)
        d_fin, d_stop = to_torch(np.zeros(rows, np.bool_)), to_torch(stop)
        ops.check(lib.ftk_invoke_stop_words_criterion(d_ids.data_ptr(), d_par.data_ptr(), d_stop.data_ptr(),
                                                      d_fin.data_ptr(), 0, L, batch, K, step, ops.current_stream()))
        torch.cuda.synchronize()
        assert np.array_equal(to_numpy(d_fin), fin) and fin.any()

