"""The fused top-k step with log-probs has several launch forms (csrc/ftk_logprob.cuh): row maxima and rows in two
launches, or one launch with 1024, 512 or 256 threads per row. All of them add the row's exponentials in the
reference's order (src/fastertransformer/kernels/sampling_topp_kernels.cu:1308-1344: thread t of 1024 adds columns
t, t + 1024, ... one after the other, then butterflies), so ids, lengths, finished flags and both log-prob outputs
must agree bit for bit between the forms, whatever the batch; parity of the product's own choice with the oracle is
what the layer tests check. The test build of the library selects the form."""
import numpy as np
import pytest

import ft_oracle as O
from helpers import DTYPE_NAMES

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]

FORMS = (1, 1024, 512, 256)  # ftk_test_set_lp_form


def _case(torch, dt, B, V, Vp, H, k, seed, kind):
    gen = torch.Generator(device="cuda")
    gen.manual_seed(seed)
    tdt = {O.F32: torch.float32, O.F16: torch.float16, O.BF16: torch.bfloat16}[dt]
    x = torch.randn((B, Vp), generator=gen, device="cuda") * 2.5
    if kind == "grid":  # a coarse grid: many equal values around the k-th largest
        x = torch.round(x * 2.0) / 2.0
    elif kind == "flat":  # constant rows with a few larger columns, some rows with a NaN or an infinity
        x[:] = 0.25
        x[:, ::211] = 1.5
        x[1, 5] = float("nan")
        x[2, 7] = float("inf")
        x[3, :] = float("-inf")
        x[3, 11] = 0.0
    history = torch.randint(0, V, (H, B), generator=gen, device="cuda", dtype=torch.int32)
    if kind == "edges":  # the largest values in the row's first and last columns, all of them in the history
        x[:, :8] += 20.0
        x[:, V - 8:V] += 20.0
        history[0:8] = torch.arange(8, dtype=torch.int32, device="cuda")[:, None]
        history[8:16] = torch.arange(V - 8, V, dtype=torch.int32, device="cuda")[:, None]
    logits = x.to(tdt)
    draws = torch.rand(B, generator=gen, device="cuda").clamp_(min=1e-6)
    finished0 = torch.zeros(B, dtype=torch.bool, device="cuda")
    finished0[B // 3] = True
    seqlen0 = torch.full((B,), H - 1, dtype=torch.int32, device="cuda")
    return logits, history, draws, finished0, seqlen0


CASES = [
    (O.F32, 40, 50257, 50257, 64, 40, "normal"),    # rows at every 4-byte offset of a 16-byte vector
    (O.F16, 300, 32000, 32004, 300, 50, "normal"),  # padded rows, more rows than compute units
    (O.BF16, 24, 9001, 9001, 16, 128, "grid"),      # one whole batch of columns per thread and a ragged rest
    (O.F32, 9, 1024, 1024, 8, 7, "normal"),         # the shortest row the step takes
    (O.F32, 12, 8192, 8192, 8, 33, "grid"),         # exactly one batch, nothing behind it
    (O.F16, 16, 16500, 16504, 2000, 64, "normal"),  # a long history
    (O.F32, 8, 30011, 30011, 32, 20, "flat"),       # rows the candidates' bound cannot separate, NaN, infinities
    (O.F16, 520, 152064, 152064, 64, 64, "normal"),  # two rounds of 512-thread workgroups
    (O.BF16, 13, 1024, 1027, 16, 8, "edges"),       # rows off 16-byte boundaries whose maxima lie in the columns in
    (O.F32, 11, 4999, 5001, 16, 30, "edges"),       # front of the first whole vector and behind the last
    (O.F16, 19, 33001, 33003, 16, 64, "edges"),
]


@pytest.mark.parametrize("dt,B,V,Vp,H,k,kind", CASES,
                         ids=["%s-%dx%d-%s" % (DTYPE_NAMES[c[0]], c[1], c[2], c[6]) for c in CASES])
def test_forms_of_the_log_prob_step_agree_bit_for_bit(dt, B, V, Vp, H, k, kind):
    import torch
    from fastertransformer_amd import ops
    from helpers import run_fused_step
    hooks = ops.ftk_hooks()
    logits, history, draws, finished0, seqlen0 = _case(torch, dt, B, V, Vp, H, k, 1000 + B + V, kind)
    cum0 = np.linspace(-3.0, 0.0, B).astype(np.float32)
    results = {}
    try:
        for form in FORMS:
            hooks.ftk_test_set_lp_form(form)
            lp = {"cum": cum0.copy()}
            out = run_fused_step("caller", torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0,
                                 lib=hooks, log_probs=lp, Vp=Vp)
            assert out[3] == 0 and hooks.ftk_test_last_fused_path() == 4
            results[form] = (out[0], out[1], out[2], lp["cum"].view(np.uint32), lp["out"].view(np.uint32))
    finally:
        hooks.ftk_test_set_lp_form(0)
    ref = results[FORMS[0]]
    assert ((ref[0] >= 0) & (ref[0] < V)).all()
    live = ~finished0.cpu().numpy()
    assert (ref[3][live] != cum0.view(np.uint32)[live]).any()  # log-probs were written
    for form in FORMS[1:]:
        for name, a, b in zip(("ids", "sequence_length", "finished", "cum_log_probs", "output_log_probs"), ref,
                              results[form]):
            assert np.array_equal(a, b), "%s differ between the two-launch form and %d threads per row" % (name, form)
