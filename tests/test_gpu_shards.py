"""The fused top-k step over vocabulary shards (ftk_fused_topk_shard_gather / ftk_fused_topk_shard_merge, the hand-over
a GEMM epilogue or a tensor-parallel rank would use) on one GPU: the vocabulary of one logits buffer is cut into
n column windows, every window goes through the gather on its own, and the merge must sample exactly what the CPU
oracle samples from the whole rows (ids, lengths and flags bit for bit). The optional (maximum, sum of exponentials)
statistics must give the sampled token's log-probability within 1e-5 relative of a float64 softmax of the oracle's
penalised logits."""
import ctypes as C

import numpy as np
import pytest

import ft_oracle as O
from helpers import DTYPES, DTYPE_NAMES, to_numpy, to_torch, uniforms

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]


def _oracle_step(dt, x, V, Vp, H, history, ks, ps, temps, pens, ptype, min_len, end_ids, u, finished, seq, lengths):
    """the whole-row step on the oracle's layer; returns (ids, seq, finished, penalised logits as the top-k saw them)"""
    B = x.shape[0]
    layer = O.OracleDynamicDecodeLayer(dt, V, Vp)
    layer.setup(B, [int(k) for k in ks], list(ps), list(temps),
                list(pens) if ptype == O.PEN_MULTIPLICATIVE else None,
                list(pens) if ptype == O.PEN_ADDITIVE else None, None, [min_len] if min_len else None)
    out_ids = np.zeros((H + 1, B), np.int32)
    out_ids[:H] = history
    fin, sq = finished.copy(), seq.copy()
    logits = x.copy()
    layer.forward(logits, end_ids, out_ids, H, H, u, finished=fin, sequence_length=sq,
                  input_lengths=lengths)
    return out_ids[H].copy(), sq, fin, logits


def _run_shards(torch, ops, lib, dt, x, V, Vp, H, history, ks, ps, temps, pens, ptype, min_len, end_ids, u, finished,
                seq, lengths, n_shards, with_stats, give_rows=True):
    B = x.shape[0]
    width = -(-V // n_shards)
    if n_shards == 2 or n_shards == 8:
        width = -(-width // 8) * 8   # (the other cuts leave shards that start off 16-byte boundaries)
    d_x = to_torch(x, dt)
    out_ids = torch.zeros((H + 1, B), dtype=torch.int32, device="cuda")
    out_ids[:H] = to_torch(history)
    d_fin, d_seq = to_torch(finished), to_torch(seq)
    keep = [to_torch(np.asarray(a)) for a in (temps.astype(np.float32), pens.astype(np.float32),
                                              np.full(B, min_len, np.int32), end_ids, ks.astype(np.int32),
                                              ps.astype(np.float32), u, lengths)]
    d_temp, d_pen, d_min, d_end, d_k, d_p, d_u, d_len = keep
    partials = torch.zeros((B, n_shards, 2), device="cuda") if with_stats else None
    row_stats = torch.zeros((B, 2), device="cuda") if with_stats else None
    elem = 4 if dt == O.F32 else 2

    def args(logits_ptr, vocab, pitch):
        a = ops.FusedTopkArgs()
        a.dtype, a.logits, a.embedding_bias = dt, logits_ptr, None
        a.vocab_size, a.vocab_size_padded = vocab, pitch
        a.batch_size = a.local_batch_size = B
        a.step, a.max_input_length = H, H
        a.temperatures, a.penalties, a.penalty_type = d_temp.data_ptr(), d_pen.data_ptr(), ptype
        a.min_lengths = d_min.data_ptr() if min_len else None
        a.input_lengths = d_len.data_ptr()
        a.end_ids, a.output_ids = d_end.data_ptr(), out_ids.data_ptr()
        a.top_ks, a.top_ps, a.max_top_k = d_k.data_ptr(), d_p.data_ptr(), int(ks.max())
        a.uniform_draws = d_u.data_ptr()
        a.ids = out_ids.data_ptr() + 4 * H * B
        a.sequence_length, a.finished = d_seq.data_ptr(), d_fin.data_ptr()
        return a

    sh = ops.TopkShards()
    sh.n_shards, sh.shard_width, sh.global_vocab_size_padded = n_shards, width, Vp
    sh.partials = partials.data_ptr() if with_stats else None
    sh.row_stats = row_stats.data_ptr() if with_stats else None
    merged = args(d_x.data_ptr() if give_rows else None, V, Vp)
    merged.workspace = None
    ops.check(lib.ftk_fused_topk_shard_merge(C.addressof(merged), C.addressof(sh), ops.current_stream()), "size")
    ws = torch.empty(merged.workspace_size, dtype=torch.uint8, device="cuda")
    for i in range(n_shards):
        lo = i * width
        cols = max(0, min(V, lo + width) - lo)
        a = args(d_x.data_ptr() + lo * elem, cols, Vp)
        a.workspace, a.workspace_size = ws.data_ptr(), ws.numel()
        sh.shard, sh.col_offset = i, lo
        ops.check(lib.ftk_fused_topk_shard_gather(C.addressof(a), C.addressof(sh), ops.current_stream()), "gather")
    merged.workspace, merged.workspace_size = ws.data_ptr(), ws.numel()
    ops.check(lib.ftk_fused_topk_shard_merge(C.addressof(merged), C.addressof(sh), ops.current_stream()), "merge")
    torch.cuda.synchronize()
    return (to_numpy(out_ids[H]), to_numpy(d_seq), to_numpy(d_fin),
            to_numpy(row_stats) if with_stats else None)


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
@pytest.mark.parametrize("n_shards", [1, 2, 4, 8])
def test_shards_of_one_buffer_sample_what_the_whole_rows_do(dt, n_shards):
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    lib = fa.ftk()
    rng = np.random.default_rng(900 + 10 * dt + n_shards)
    B, V, Vp, H = 40, 50257, 50264, 37
    x = O.to_storage(rng.standard_normal((B, Vp), dtype=np.float32) * np.float32(2.5), dt)
    history = rng.integers(0, V, (H, B)).astype(np.int32)
    lengths = rng.integers(H - 8, H + 1, B).astype(np.int32)
    ks = rng.choice([1, 5, 40, 64, 192], B)
    ps = rng.uniform(0.3, 1.0, B)
    temps = rng.uniform(0.6, 1.4, B)
    end_ids = rng.integers(0, V, B).astype(np.int32)
    finished = rng.random(B) < 0.1
    seq = np.full(B, H - 1, np.int32)
    u = uniforms(rng, B)
    xf = O.to_f32(x, dt)
    for b in range(0, B, 5):
        xf[b, end_ids[b]] = 25.0          # the masked end id would win
    x = O.to_storage(xf, dt)
    for ptype, pens in ((O.PEN_MULTIPLICATIVE, rng.choice([0.8, 1.0, 1.3], B)), (O.PEN_ADDITIVE, rng.uniform(-0.5, 1.0, B))):
        want = _oracle_step(dt, x, V, Vp, H, history, ks, ps, temps, pens, ptype, H + 4, end_ids, u, finished, seq,
                            lengths)
        got = _run_shards(torch, ops, lib, dt, x, V, Vp, H, history, ks, ps, temps, pens, ptype, H + 4, end_ids, u,
                          finished, seq, lengths, n_shards, with_stats=True)
        assert np.array_equal(got[0], want[0]), np.nonzero(got[0] != want[0])[0]
        assert np.array_equal(got[1], want[1]) and np.array_equal(got[2], want[2])
        # log p of the sampled token from the combined statistics against a float64 softmax of the oracle's
        # penalised logits (the layer leaves them in place on its kernel-by-kernel path)
        final = O.to_f32(want[3], dt).astype(np.float64)[:, :V]
        for b in range(B):
            if finished[b]:
                continue
            row = final[b].copy()
            valid = row > -1e30
            m = row[valid].max()
            lse = m + np.log(np.exp(row[valid] - m).sum())
            lp_want = row[want[0][b]] - lse
            lp_got = row[want[0][b]] - got[3][b, 0] - np.log(got[3][b, 1])
            assert abs(lp_got - lp_want) <= 2e-4 + 1e-5 * abs(lp_want), (b, lp_got, lp_want)


def test_shards_full_size_rows_and_rows_not_at_hand():
    """the headline shape in four shards (256 x 128256 fp32, k = 64), merged without the rows at hand (as a rank
    would): nothing overflows on ordinary rows, so every id is there"""
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    lib = fa.ftk()
    rng = np.random.default_rng(77)
    dt, B, V, H = O.F32, 256, 128256, 64
    x = rng.standard_normal((B, V), dtype=np.float32) * np.float32(2.5)
    history = rng.integers(0, V, (H, B)).astype(np.int32)
    lengths = np.full(B, H, np.int32)
    ks, ps, temps, pens = np.full(B, 64), np.full(B, 0.9), np.full(B, 0.8), np.full(B, 1.1)
    end_ids = np.full(B, V - 1, np.int32)
    finished, seq, u = np.zeros(B, bool), np.full(B, H - 1, np.int32), uniforms(rng, B)
    want = _oracle_step(dt, x, V, V, H, history, ks, ps, temps, pens, O.PEN_MULTIPLICATIVE, 0, end_ids, u, finished,
                        seq, lengths)
    got = _run_shards(torch, ops, lib, dt, x, V, V, H, history, ks, ps, temps, pens, O.PEN_MULTIPLICATIVE, 0, end_ids,
                      u, finished, seq, lengths, 4, with_stats=False, give_rows=False)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1]) and np.array_equal(got[2], want[2])


def test_shard_calls_refuse_what_they_do_not_cover():
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    lib = fa.ftk()
    a, sh = ops.FusedTopkArgs(), ops.TopkShards()
    a.dtype, a.vocab_size, a.vocab_size_padded, a.local_batch_size, a.batch_size = O.F32, 1000, 1000, 4, 4
    a.max_top_k = 500
    sh.n_shards, sh.shard_width, sh.global_vocab_size_padded = 2, 500, 1000
    assert lib.ftk_fused_topk_shard_gather(C.addressof(a), C.addressof(sh), None) == ops.FTK_ERR_UNSUPPORTED
    a.max_top_k = 64
    sh.n_shards = 17
    assert lib.ftk_fused_topk_shard_merge(C.addressof(a), C.addressof(sh), None) == ops.FTK_ERR_ARGUMENT
    sh.n_shards = 2
    a.workspace = None
    assert lib.ftk_fused_topk_shard_merge(C.addressof(a), C.addressof(sh), None) == 0 and a.workspace_size > 0
