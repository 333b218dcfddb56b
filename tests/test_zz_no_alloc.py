"""ftk_fused_topk_step_static (the fused step with the library's own fixed workspace, for callers that cannot
allocate) against ftk_fused_topk_step with a caller workspace, through the C ABI: sampled ids, sequence
lengths and finished flags must be identical bit for bit, on two calls in a row, the second one smaller (it
sees what the first left in the array). A step that needs more than the array is refused."""
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
