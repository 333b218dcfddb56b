"""ftk_fused_topk_step_static (the fused step with the library's own fixed workspace, for callers that cannot
allocate) against ftk_fused_topk_step with a caller workspace, through the C ABI: sampled ids, sequence
lengths and finished flags must be identical bit for bit, on two calls in a row, the second one smaller (it
sees what the first left in the array). A step that needs more than the array is refused."""
import ctypes as C

import numpy as np
import pytest

import fastertransformer_amd as fa
from fastertransformer_amd import ops

pytestmark = pytest.mark.gpu


def _step(entry, torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0):
    """one fused step through `entry`; returns (ids, sequence_length, finished, rc, needed bytes)"""
    dev = "cuda"
    out_ids = torch.zeros((H + 1, B), dtype=torch.int32, device=dev)
    out_ids[:H] = history
    finished = finished0.clone()
    seq = seqlen0.clone()
    temps = torch.full((B,), 0.8, device=dev)
    pens = torch.full((B,), 1.1, device=dev)
    end_ids = torch.full((B,), V - 1, dtype=torch.int32, device=dev)
    top_ks = torch.full((B,), k, dtype=torch.int32, device=dev)
    top_ps = torch.full((B,), 0.9, device=dev)
    a = ops.FusedTopkArgs()
    a.dtype, a.logits, a.embedding_bias = dt, logits.data_ptr(), None
    a.vocab_size = a.vocab_size_padded = V
    a.batch_size = a.local_batch_size = B
    a.step, a.max_input_length = H, H
    a.temperatures, a.penalties, a.penalty_type = temps.data_ptr(), pens.data_ptr(), ops.PENALTY_MULTIPLICATIVE
    a.end_ids, a.output_ids = end_ids.data_ptr(), out_ids.data_ptr()
    a.top_ks, a.top_ps, a.max_top_k = top_ks.data_ptr(), top_ps.data_ptr(), k
    a.uniform_draws = draws.data_ptr()
    a.ids = out_ids.data_ptr() + 4 * H * B
    a.sequence_length, a.finished = seq.data_ptr(), finished.data_ptr()
    lib = fa.ftk()
    stream = ops.current_stream()
    ws = None
    if entry == "caller":
        a.workspace = None
        ops.check(lib.ftk_fused_topk_step(C.addressof(a), stream), "size query")
        ws = torch.empty(a.workspace_size, dtype=torch.uint8, device=dev)
        a.workspace = ws.data_ptr()
        rc = lib.ftk_fused_topk_step(C.addressof(a), stream)
    else:
        a.workspace, a.workspace_size = None, 0
        rc = lib.ftk_fused_topk_step_static(C.addressof(a), stream)
    torch.cuda.synchronize()
    return out_ids[H].cpu().numpy(), seq.cpu().numpy(), finished.cpu().numpy(), rc, a.workspace_size


def test_static_workspace_step_matches_caller_workspace_step():
    import torch
    gen = torch.Generator(device="cuda")
    gen.manual_seed(77)
    dt, V, H, k = fa.F32, 128256, 24, 64
    for B in (96, 40):  # the second call is smaller and finds the first call's lists in the array
        logits = torch.randn((B, V), generator=gen, device="cuda") * 2.5
        history = torch.randint(0, V, (H, B), generator=gen, device="cuda", dtype=torch.int32)
        draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
        finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
        finished0[3] = True  # a finished row emits its end id on both paths
        seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
        ref = _step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0)
        got = _step("static", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0)
        assert ref[3] == 0 and got[3] == 0, (ref[3], got[3])
        assert got[4] == ref[4] and got[4] <= ops.FUSED_STATIC_WORKSPACE_BYTES
        assert np.array_equal(got[0], ref[0]), "sampled ids differ at batch %d" % B
        assert np.array_equal(got[1], ref[1]) and np.array_equal(got[2], ref[2])
        assert got[0][3] == V - 1 and (got[0] >= 0).all() and (got[0] < V).all()


def test_static_workspace_step_refuses_what_the_array_cannot_hold():
    import torch
    dt, V, H, k, B = fa.F32, 128256, 4, 64, 2048
    logits = torch.zeros((B, V), device="cuda")  # full size, although the call is refused before any launch
    history = torch.zeros((H, B), dtype=torch.int32, device="cuda")
    draws = torch.ones(B, device="cuda")
    finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
    seqlen0 = torch.zeros(B, dtype=torch.int32, device="cuda")
    ids, _, _, rc, need = _step("static", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0)
    assert rc == ops.FTK_ERR_STATIC_WORKSPACE and need > ops.FUSED_STATIC_WORKSPACE_BYTES
    assert (ids == 0).all()
    assert b"fixed array" in fa.ftk().ftk_error_string(rc)
