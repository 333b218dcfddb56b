"""ftk_fused_topk_step_static (the fused step with the library's own fixed workspace, for callers that cannot
allocate) against ftk_fused_topk_step with a caller workspace, through the C ABI: sampled ids, sequence
lengths and finished flags must be identical bit for bit, on two calls in a row, the second one smaller (it
sees what the first left in the array). A step that needs more than the array is refused. The entry point is
also recorded into a HIP graph and replayed."""
import ctypes as C

import numpy as np
import pytest

import fastertransformer_amd as fa
from fastertransformer_amd import ops
from helpers import run_fused_step as _step

pytestmark = pytest.mark.gpu


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
        if B != 96:  # (the very first call on a device looks up the array's address; nothing is allocated after it)
            assert got[5] == 0, "the static entry point changed the device's free memory by %d bytes" % got[5]
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
    ids, _, _, rc, need, _ = _step("static", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0)
    assert rc == ops.FTK_ERR_STATIC_WORKSPACE and need > ops.FUSED_STATIC_WORKSPACE_BYTES
    assert (ids == 0).all()
    assert b"fixed array" in fa.ftk().ftk_error_string(rc)


def test_static_workspace_step_replayed_from_a_graph():
    """The caller the entry point is for: the step is recorded into a graph once (after a first eager call, which
    looks up the array's address) and replayed on new logits, histories and draws written into the same buffers.
    Every replay must give what an eager step with a caller workspace gives on the same contents; eager work and
    synchronisations of the program's own sit between the replays."""
    import torch
    dev = "cuda"
    lib = fa.ftk()
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    dt, B, V, H, k = fa.F32, 64, 50304, 16, 50
    logits = torch.empty((B, V), device=dev)
    out_ids = torch.zeros((H + 1, B), dtype=torch.int32, device=dev)
    draws = torch.empty(B, device=dev)
    finished = torch.zeros(B, dtype=torch.bool, device=dev)
    seq = torch.zeros(B, dtype=torch.int32, device=dev)
    temps = torch.full((B,), 0.8, device=dev)
    pens = torch.full((B,), 1.1, device=dev)
    end_ids = torch.full((B,), V - 1, dtype=torch.int32, device=dev)
    top_ks = torch.full((B,), k, dtype=torch.int32, device=dev)
    top_ps = torch.full((B,), 0.9, device=dev)

    def args():
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
        return a

    def fill(i):
        logits.copy_(torch.randn((B, V), generator=gen, device=dev) * (1.5 + i))
        out_ids[:H] = torch.randint(0, V, (H, B), generator=gen, device=dev, dtype=torch.int32)
        out_ids[H].zero_()
        draws.copy_(torch.rand(B, generator=gen, device=dev).clamp_(min=1e-6))
        finished.zero_()
        finished[i % B] = True
        seq.fill_(H - 1)

    def results():
        torch.cuda.synchronize()
        return out_ids[H].cpu().numpy().copy(), seq.cpu().numpy().copy(), finished.cpu().numpy().copy()

    a = args()
    a.workspace = None
    ops.check(lib.ftk_fused_topk_step(C.addressof(a), ops.current_stream()), "size query")
    ws = torch.empty(a.workspace_size, dtype=torch.uint8, device=dev)
    fill(0)
    a_static = args()
    a_static.workspace, a_static.workspace_size = None, 0
    ops.check(lib.ftk_fused_topk_step_static(C.addressof(a_static), ops.current_stream()), "first call, eager")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    fill(0)
    with torch.cuda.graph(graph):
        rc = lib.ftk_fused_topk_step_static(C.addressof(a_static), ops.current_stream())
    assert rc == 0
    for i in range(1, 5):
        fill(i)
        state = (out_ids.clone(), seq.clone(), finished.clone())
        a.workspace = ws.data_ptr()
        ops.check(lib.ftk_fused_topk_step(C.addressof(a), ops.current_stream()), "eager step")
        want = results()
        out_ids.copy_(state[0]); seq.copy_(state[1]); finished.copy_(state[2])
        torch.cuda.synchronize()
        graph.replay()
        got = results()
        for w, g, name in zip(want, got, ("ids", "sequence_length", "finished")):
            assert np.array_equal(w, g), "replay %d: %s differ" % (i, name)
        assert (got[0] >= 0).all() and (got[0] < V).all() and got[0][i % B] == V - 1
