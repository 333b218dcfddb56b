"""The one-launch step for batches of about one row per compute unit (a 1024-thread workgroup per row,
csrc/ftk_rowwide.cuh) against the CPU oracle, through DynamicDecodeLayer with injected draws: ids / finished /
sequence_length bit-exact. The shapes are the ones the launcher sends to that kernel (up to 256 rows, or up to 1023
in nearly full rounds of 256 with rows of at least 16384 16-byte vectors; rows on 16-byte boundaries, k <= 192, no
bias, no log-probs);
the last test asks the test build of the library which kernel a launch of such a shape took."""
import numpy as np
import pytest

import ft_oracle as O
from decode_harness import Case, OracleRunner, ProductRunner, compare
from helpers import DTYPES, DTYPE_NAMES, uniforms

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]


def _normal(rng, dt, B, Vp, sigma):
    return O.to_storage(rng.standard_normal((B, Vp), dtype=np.float32) * np.float32(sigma), dt)


def _run(c, rng, steps, logits_fn):
    p, o = ProductRunner(c), OracleRunner(c)
    for i in range(steps):
        step = c.max_input_length + i
        logits = logits_fn(i)
        u = uniforms(rng, c.batch)
        p.step(step, logits, u)
        o.step(step, logits, u)
        compare(p.snapshot(), o.snapshot(), c.dt, False, where="step %d" % step)
    return p.snapshot()


@pytest.mark.parametrize("dt", DTYPES, ids=lambda d: DTYPE_NAMES[d])
def test_rowwide_mixed_rows(dt):
    """Per-row k from 1 to 192, per-row top_p and temperature, a repetition penalty that lowers values in some rows
    and raises them in others (below 1), padded vocabulary, min_length masking the end id, rows that finish on the
    way; two steps."""
    rng = np.random.default_rng(300 + dt)
    B = 256
    V, Vp = (70001, 70004) if dt == O.F32 else (131101, 131104)
    H = 48
    ks = rng.choice([1, 2, 7, 40, 64, 100, 192], B).astype(np.uint32)
    pen = rng.choice([0.7, 1.0, 1.1, 1.5], B).astype(np.float32)
    c = Case(dt, B, V, Vp, max_input_length=H, gen_len=2, runtime_top_k=ks, runtime_top_p=rng.uniform(0.3, 1.0, B),
             temperature=rng.uniform(0.5, 1.5, B), repetition_penalty=pen, min_length=[H + 5],
             end_ids=rng.integers(0, V, B).astype(np.int32), prompt=rng.integers(0, V, (H, B)).astype(np.int32))

    def logits_fn(i):
        x = rng.standard_normal((B, Vp), dtype=np.float32) * np.float32(2.5)
        for b in range(0, B, 9):
            x[b, c.end_ids[b]] = 30.0  # the masked end id would win if it were not masked
        return O.to_storage(x, dt)

    _run(c, rng, 2, logits_fn)


def test_rowwide_ties_flat_and_masked_rows():
    """Rows the bound cannot separate: a handful of distinct values (thousands of ties around the k-th: lists longer
    than 256 after the cut, lists that outgrow LDS and are walked again), constant rows, rows that rise towards
    their end (every late column beats what came before), rows where fewer than k columns are valid; presence
    penalty, no temperature."""
    rng = np.random.default_rng(17)
    dt, B, V = O.F32, 256, 66000
    x = rng.standard_normal((B, V), dtype=np.float32) * np.float32(2.0)
    x[0:40] = rng.integers(0, 4, (40, V)).astype(np.float32)                 # four distinct values
    x[40:60] = 1.5                                                            # constant
    x[60:90] = np.sort(x[60:90], axis=1)                                      # ascending
    x[90:110] = -np.inf
    for b in range(90, 110):
        x[b, rng.integers(0, V, 5 + b % 50)] = rng.standard_normal(5 + b % 50)  # fewer valid columns than k
    x[110:130] = np.round(x[110:130] * 4.0) / 4.0                            # a coarse grid: many ties
    H = 20
    c = Case(dt, B, V, V, max_input_length=H, gen_len=1, runtime_top_k=rng.choice([1, 30, 64, 150], B),
             runtime_top_p=[0.95], presence_penalty=[0.4], prompt=rng.integers(0, V, (H, B)).astype(np.int32))
    _run(c, rng, 1, lambda i: x)


def test_rowwide_long_history_and_second_round():
    """512 rows (two full rounds of workgroups), a
    history of 3000 tokens per row with prompt padding skipped, additive penalty that raises (negative)."""
    rng = np.random.default_rng(23)
    dt, B, V, H = O.F32, 512, 65600, 3000
    prompt = np.minimum(rng.zipf(1.2, (H, B)), V - 1).astype(np.int32)
    lengths = rng.integers(H - 500, H + 1, B).astype(np.int32)
    c = Case(dt, B, V, V, max_input_length=H, gen_len=1, runtime_top_k=[50], runtime_top_p=[0.8],
             temperature=[0.9], presence_penalty=[-0.5], input_lengths=lengths, prompt=prompt)
    _run(c, rng, 1, lambda i: _normal(rng, dt, B, V, 2.0))


def test_rowwide_generated_draws_are_reproducible():
    """Without injected draws the kernel takes them from the layer's generator states: the same seed gives the same
    ids, and the states advance (a second step with the same logits differs from the first somewhere)."""
    import torch
    rng = np.random.default_rng(5)
    dt, B, V = O.F32, 256, 65600
    logits = _normal(rng, dt, B, V, 2.0)
    outs = []
    for rep in range(2):
        c = Case(dt, B, V, V, gen_len=2, runtime_top_k=[64], runtime_top_p=[0.9], temperature=[0.8],
                 random_seed=[1234])
        p = ProductRunner(c)
        p.step(0, logits, None)
        p.step(1, logits, None)
        torch.cuda.synchronize()
        outs.append(p.snapshot()["output_ids"].copy())
    assert np.array_equal(outs[0], outs[1])
    assert (outs[0][0] != outs[0][1]).any()
    assert ((outs[0] >= 0) & (outs[0] < V)).all()


def test_rowwide_kernel_is_what_these_shapes_take():
    """the test build of the library reports the path of its last fused step: 3 = one 1024-thread workgroup per row;
    the same rows in two launches (hook) do not take it, nor does a batch between one round of workgroups and a
    nearly full second one (300 rows); any batch of up to 256 rows does; and all agree on the ids"""
    import torch
    from fastertransformer_amd import ops
    from helpers import run_fused_step
    hooks = ops.ftk_hooks()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(9)
    H, k = 16, 64
    for B, V, want in ((256, 65600, 3), (300, 65600, 1), (100, 128256, 3), (100, 32000, 3)):
        logits = torch.randn((B, V), generator=gen, device="cuda") * 2.0
        history = torch.randint(0, V, (H, B), generator=gen, device="cuda", dtype=torch.int32)
        draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
        finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
        finished0[3] = True
        seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
        one = run_fused_step("caller", torch, O.F32, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks)
        assert one[3] == 0 and hooks.ftk_test_last_fused_path() == want
        hooks.ftk_test_set_fused_two_launches(1)
        try:
            two = run_fused_step("caller", torch, O.F32, B, V, H, k, logits, history, draws, finished0, seqlen0,
                                 lib=hooks)
            assert two[3] == 0 and hooks.ftk_test_last_fused_path() == 1
        finally:
            hooks.ftk_test_set_fused_two_launches(0)
        for a, b in zip(one[:3], two[:3]):
            assert np.array_equal(a, b)


def test_rowwide_rows_walked_again_do_not_depend_on_the_workspace():
    """Rows whose list outgrows LDS are walked again by the four waves that are left of the workgroup, with the
    history bitmap rebuilt in the workspace: constant rows with a few larger columns, some of them in the history
    (so the penalty decides which win), a workspace full of ones. Same ids as the two-launch step."""
    import torch
    from fastertransformer_amd import ops
    from helpers import run_fused_step
    hooks = ops.ftk_hooks()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    B, V, H, k = 32, 149544, 300, 150
    logits = torch.full((B, V), 0.75, device="cuda")
    logits[:, ::997] = 1.0
    history = torch.randint(0, V // 997, (H, B), generator=gen, device="cuda", dtype=torch.int32) * 997
    draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
    finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
    seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
    one = run_fused_step("caller", torch, O.F32, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks,
                         ws_fill=0xFF)
    assert one[3] == 0 and hooks.ftk_test_last_fused_path() == 3
    hooks.ftk_test_set_fused_two_launches(1)
    try:
        two = run_fused_step("caller", torch, O.F32, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks,
                             ws_fill=0xFF)
    finally:
        hooks.ftk_test_set_fused_two_launches(0)
    for a, b in zip(one[:3], two[:3]):
        assert np.array_equal(a, b)
    assert (one[0] % 997 == 0).all()  # only the larger columns can be sampled (k = 150 of them, all tied)


def test_large_k_lists_in_one_launch_agree_with_the_two_launches():
    """With a largest k beyond 192 and at most one row per compute unit, one 1024-thread workgroup per row makes the
    row's candidate list in one launch (csrc/ftk_largek.cuh; path 5) where the lean gather takes two (maxima, then
    gather); the test build can keep the two launches (path 1). Same ids, lengths and flags on rows of three types:
    vocabularies that end inside a 16-byte vector, histories, rows with fewer valid columns than k, constant rows
    (lists that overflow and send the row to the exact replay)."""
    import torch
    from fastertransformer_amd import ops
    from helpers import run_fused_step
    hooks = ops.ftk_hooks()
    gen = torch.Generator(device="cuda")
    gen.manual_seed(21)
    tdt = {O.F32: torch.float32, O.F16: torch.float16, O.BF16: torch.bfloat16}
    for dt, B, V, Vp, H, k, kind in ((O.F16, 256, 50257, 51200, 64, 1024, "normal"), (O.F32, 130, 50261, 50264, 16, 700, "normal"),
                                     (O.BF16, 100, 32000, 32000, 300, 300, "grid"), (O.F32, 24, 20000, 20000, 8, 1024, "sparse"),
                                     (O.F16, 16, 40000, 40000, 8, 512, "flat")):
        x = torch.randn((B, Vp), generator=gen, device="cuda") * 3.0
        if kind == "grid":
            x = torch.round(x * 2.0) / 2.0
        elif kind == "sparse":  # fewer valid columns than k in some rows
            x[::3] = float("-inf")
            for b in range(0, B, 3):
                cols = torch.randint(0, V, (200,), generator=gen, device="cuda")
                x[b, cols] = torch.randn(200, generator=gen, device="cuda")
        elif kind == "flat":
            x[::2] = 0.5
        logits = x.to(tdt[dt])
        history = torch.randint(0, V, (H, B), generator=gen, device="cuda", dtype=torch.int32)
        draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
        finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
        finished0[1] = True
        seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
        one = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks,
                             Vp=Vp, ws_fill=0xFF)
        assert one[3] == 0 and hooks.ftk_test_last_fused_path() == 5, (dt, B, V)
        hooks.ftk_test_set_largek_two_launches(1)
        try:
            two = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=hooks,
                                 Vp=Vp, ws_fill=0xFF)
            assert two[3] == 0 and hooks.ftk_test_last_fused_path() == 1
        finally:
            hooks.ftk_test_set_largek_two_launches(0)
        for name, a, b in zip(("ids", "sequence_length", "finished"), one[:3], two[:3]):
            assert np.array_equal(a, b), (name, DTYPE_NAMES[dt], B, V, kind)
        assert ((one[0] >= 0) & (one[0] < V)).all()
