#!/usr/bin/env python3
"""Headline benchmark: one DynamicDecodeLayer step (top-k + top-p + temperature + repetition penalty)
over a [256, 128256] fp32 logits batch on one MI355X.

A "step" is one DynamicDecodeLayer::forward over one batch of seeded synthetic logits already resident in
HBM. The logits cycle through several buffers whose total size exceeds the 256 MB last-level cache, so
every step streams its logits from HBM. Prints one JSON line (see the keys below).

    python bench.py --gpus 1 --steps 50 --warmup 5
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0
PLAIN_READ = "plain_read_b256_v128256_f32"
# HBM bytes per launch of the dominant kernel on the headline workload, from rocprofv3 --pmc FETCH_SIZE and
# WRITE_SIZE runs of this script scaled by a copy kernel of known size (summary under profiles/)
TRAFFIC_BYTES_PER_LAUNCH = 132478941

WORKLOADS = {
    # the configuration the headline metric is quoted on
    "decode_step_b256_v128256_f32_topk64_topp0.9_temp0.8_rep1.1": dict(
        dtype="f32", batch=256, vocab=128256, vocab_padded=128256, top_k=64, top_p=0.9, temperature=0.8,
        repetition_penalty=1.1, prompt=64, sigma=2.5),
    # secondary line (only with --workload): the top-p layer on Zipf-distributed rows, per-row top_p in
    # [0.5, 0.99] with decay; the logits buffer is restored outside the timed events (with
    # FT_SAMPLING_DISABLE_FUSED=1 the layer turns it into probabilities in place, like the reference)
    "topp_step_b256_v128256_f32_zipf1.1_p0.5-0.99_decay0.9": dict(
        dtype="f32", batch=256, vocab=128256, vocab_padded=128256, top_k=0, top_p=(0.5, 0.99), top_p_decay=0.9,
        top_p_min=0.3, top_p_reset_id=13, zipf_s=1.1, noise=0.5, prompt=0),
    # secondary line (only with --workload): the fused step with a per-row k drawn from {1, 4, 16, 40, 64, 1024}
    # (fp16, vocabulary 51200): the rows with k = 1024 set the pace of the launch, which reads the logits twice
    "decode_step_b256_v51200_f16_topk1-1024_topp0.9_temp0.8_rep1.1": dict(
        dtype="f16", batch=256, vocab=51200, vocab_padded=51200, top_k=(1, 4, 16, 40, 64, 1024), top_p=0.9,
        temperature=0.8, repetition_penalty=1.1, prompt=64, sigma=2.5),
    # secondary line (only with --workload): the fused step at batch 1024 (fp16, vocabulary 152064), no log-probs
    "decode_step_b1024_v152064_f16_topk64_topp0.9_temp0.8_rep1.1": dict(
        dtype="f16", batch=1024, vocab=152064, vocab_padded=152064, top_k=64, top_p=0.9, temperature=0.8,
        repetition_penalty=1.1, prompt=64, sigma=2.5),
    # secondary line (only with --workload): the full decode loop at batch 1024 (fp16, vocabulary 152064), per-step
    # latency with cum_log_probs / output_log_probs and the length criterion on (the fused step with log-probs:
    # row maximum, then one kernel per row that sums, gathers and samples)
    "decode_loop_b1024_v152064_f16_topk64_topp0.9_logprobs": dict(
        dtype="f16", batch=1024, vocab=152064, vocab_padded=152064, top_k=64, top_p=0.9, temperature=0.8,
        repetition_penalty=1.1, prompt=8, sigma=2.5),
    # secondary line (only with --workload): the reference's own CPU-runnable case, batch 8 with log-probs
    "decode_loop_b8_v50257_f32_topk40_rep1.2_logprobs": dict(
        dtype="f32", batch=8, vocab=50257, vocab_padded=50257, top_k=40, top_p=0.0, temperature=1.0,
        repetition_penalty=1.2, prompt=64, sigma=2.0, end_id=50256),
    # secondary line (only with --workload): the penalty- and mask-heavy step: 2048-token Zipf(1.2) history per
    # row, presence and frequency penalties, min_length beyond the steps taken, 64 bad-word and 16 stop-word
    # sequences per row, no log-probs
    "decode_loop_b128_v32000_bf16_hist2048_presence0.5_freq0.3_minlen_badwords_stopwords_topk50": dict(
        dtype="bf16", batch=128, vocab=32000, vocab_padded=32000, top_k=50, top_p=0.0, temperature=1.0,
        presence_penalty=0.5, frequency_penalty=0.3, prompt=2048, zipf_history=1.2, min_length_beyond=52,
        bad_words=(64, 4), stop_words=(16, 3), end_id=2, sigma=2.0, logprobs=False),
    # secondary line (only with --workload): one beam-search step (invokeTopkSoftMax), 32 entries x 4 beams,
    # hypotheses kept, a few beams ending per step; the beams' state is restored outside the timed events
    "beam_step_b32_k4_v50257_f16": dict(dtype="f16", batch=32, beam_width=4, vocab=50257, sigma=3.0),
    "beam_step_b64_k8_v152064_f16": dict(dtype="f16", batch=64, beam_width=8, vocab=152064, sigma=3.0),
}


def algorithmic_bytes(w, step):
    elem = 4 if w["dtype"] == "f32" else 2
    history = step if w.get("repetition_penalty") else 0
    return w["batch"] * w["vocab_padded"] * elem + w["batch"] * history * 4 + w["batch"] * 32


def run_gpu(name, w, steps, warmup, nbuf=4, check_oracle=False):
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops

    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    dt = {"f32": fa.F32, "f16": fa.F16, "bf16": fa.BF16}[w["dtype"]]
    B, V, Vp, H = w["batch"], w["vocab"], w["vocab_padded"], w["prompt"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(1234)
    bufs = [(torch.randn((B, 1, Vp), generator=gen, device=dev, dtype=torch.float32) * w["sigma"]).to(fa.torch_dtype(dt))
            for _ in range(nbuf)]
    total = steps + warmup
    max_seq = H + total + 1
    output_ids = torch.zeros((max_seq, B), dtype=torch.int32, device=dev)
    output_ids[:H] = torch.randint(0, V, (H, B), generator=gen, device=dev, dtype=torch.int32)
    finished = torch.zeros(B, dtype=torch.bool, device=dev)
    seq_len = torch.full((B,), H - 1, dtype=torch.int32, device=dev)
    end_id = torch.full((B,), V - 1, dtype=torch.int32, device=dev)
    draws = [torch.rand(B, generator=gen, device=dev).clamp_(min=1e-7) for _ in range(nbuf)]

    layer = fa.DynamicDecodeLayer(dt, V, Vp)
    if isinstance(w["top_k"], tuple):  # one k per row, drawn from the choices
        top_ks = np.random.default_rng(0).choice(np.array(w["top_k"], np.uint32), B).astype(np.uint32)
    else:
        top_ks = np.array([w["top_k"]], np.uint32)
    args = {"runtime_top_k": top_ks, "runtime_top_p": np.array([w["top_p"]], np.float32),
            "temperature": np.array([w["temperature"]], np.float32),
            "repetition_penalty": np.array([w["repetition_penalty"]], np.float32),
            "random_seed": np.array([7], np.uint64)}
    layer.setup(B, 1, args)
    outs = {"output_ids": output_ids, "finished": finished, "sequence_length": seq_len}
    step_arr = np.zeros(1, np.int32)
    base = {"step": step_arr, "max_input_length": np.array([H], np.int32), "ite": np.array([0], np.uint32),
            "local_batch_size": np.array([B], np.int32), "end_id": end_id}

    def one_step(i):
        step_arr[0] = H + i
        ins = dict(base, logits=bufs[i % nbuf], uniform_draws=draws[i % nbuf])
        layer.forward(outs, ins)

    lib = fa.ftk()
    for i in range(warmup):
        one_step(i)
    torch.cuda.synchronize()
    state0 = (finished.clone(), seq_len.clone())
    # timed region: exactly `steps` steps, no per-kernel instrumentation
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for i in range(warmup, total):
        one_step(i)
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = ev0.elapsed_time(ev1)
    checksum = int(output_ids[H + warmup:H + total].to(torch.int64).sum().item())
    # the same steps once more (same logits, draws and history positions) with a HIP event pair carried by
    # every kernel launch of the library, on the stream the kernels run on: per-kernel durations
    finished.copy_(state0[0])
    seq_len.copy_(state0[1])
    ops.check(lib.ftk_profile_enable(steps))
    torch.cuda.synchronize()
    for i in range(warmup, total):
        one_step(i)
    torch.cuda.synchronize()
    kernel_ms = []
    for k in range(4):
        tot, n = C.c_double(0.0), C.c_int(0)
        ops.check(lib.ftk_profile_read(k, C.addressof(tot), C.addressof(n)))
        kernel_ms.append((tot.value / n.value) if n.value else 0.0)
    ops.check(lib.ftk_profile_enable(0))
    assert checksum == int(output_ids[H + warmup:H + total].to(torch.int64).sum().item()), "the two passes differ"
    oracle = None
    if check_oracle:
        # one more step, outside every timed region, repeated on the CPU oracle from the same state
        from helpers import to_numpy
        state = (to_numpy(finished), to_numpy(seq_len))
        one_step(total)
        torch.cuda.synchronize()
        oracle = check_step_against_oracle(w, bufs[total % nbuf], draws[total % nbuf], output_ids, H + total, H,
                                           top_ks, state)

    ms_per_step = wall * 1e3 / steps
    mid_step = H + warmup + steps // 2
    alg = algorithmic_bytes(w, mid_step)
    gather_ms = kernel_ms[1]
    achieved = alg / (gather_ms * 1e-3) / 1e9 if gather_ms > 0 else 0.0
    # Which kernel streams the logits: one 1024-thread workgroup per row does the whole step in one launch where the
    # batch fills the chip in nearly full rounds of 256 rows (rowwide_step_kernel); otherwise the lean gather
    # (largest k beyond 192 on more than 256 rows: twice, maxima first) followed by a selection launch. Timer 1
    # carries either.
    rounds = (B + 255) // 256
    rowwide = (not isinstance(w["top_k"], tuple) and w["top_k"] <= 192 and B < 1024 and B * 5 >= rounds * 256 * 4
               and V // (16 // (4 if w["dtype"] == "f32" else 2)) >= 4 * 4096)
    # (a largest k beyond 192 on up to 256 rows: one 1024-thread workgroup per row makes the lists, in one launch)
    largek = (isinstance(w["top_k"], tuple) and max(w["top_k"]) > 192 and B <= 256
              and (B >= 128 or V * (4 if w["dtype"] == "f32" else 2) <= (128 << 10)))
    dominant = "rowwide_step_kernel" if rowwide else ("largek_gather_kernel" if largek else "lean_gather_kernel")
    return dict(
        tokens_per_s=B * steps / wall, ms_per_step=ms_per_step, gpu_ms_per_step=gpu_ms / steps,
        kernel_ms=dict(history_bitmap=kernel_ms[0], gather=kernel_ms[1], select=kernel_ms[2], maxima=kernel_ms[3]),
        roofline=dict(bound="hbm", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS,
                      traffic=TRAFFIC_BYTES_PER_LAUNCH if name == next(iter(WORKLOADS)) else None, kernel=dominant, algorithmic_bytes_per_launch=alg),
        step_gbs=alg / (gpu_ms / steps * 1e-3) / 1e9,
        sampled_ids_checksum=checksum, oracle_check=oracle,
    )


def check_step_against_oracle(w, logits, draws, output_ids, step, H, top_ks, state):
    """One decode step of the benchmark repeated on the CPU oracle (same logits, draws, token history, finished
    flags and lengths): the sampled ids of every row must be identical. Returns what was compared."""
    import ft_oracle as O
    from helpers import to_numpy
    odt = {"f32": O.F32, "f16": O.F16, "bf16": O.BF16}[w["dtype"]]
    B, V, Vp = w["batch"], w["vocab"], w["vocab_padded"]
    ids = to_numpy(output_ids)
    got = ids[step].copy()
    history = ids.copy()
    history[step:] = 0
    layer = O.OracleDynamicDecodeLayer(odt, V, Vp)
    layer.setup(B, [int(k) for k in top_ks], [w["top_p"]], [w["temperature"]], [w["repetition_penalty"]])
    finished, seq = state[0].copy(), state[1].copy()
    end = np.full(B, V - 1, np.int32)
    x = to_numpy(logits.reshape(B, Vp), odt)
    layer.forward(x, end, history, step, H, to_numpy(draws), finished=finished, sequence_length=seq)
    want = history[step]
    assert np.array_equal(got, want), "sampled ids differ from the oracle in %d of %d rows" % (
        int((got != want).sum()), B)
    return dict(rows=B, step=int(step), ids_checksum=int(want.astype(np.int64).sum()), identical=True)


def run_plain_read(steps, warmup, nbuf=4):
    """The yardstick: a kernel that only fetches 256 x 128256 fp32 with the streaming kernel's launch shape
    (ftk_measure_plain_read), buffers in rotation like the decode step's logits."""
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
    torch.cuda.set_device(0)
    B, V = 256, 128256
    bufs = [torch.randn((B, V), device="cuda:0") for _ in range(nbuf)]
    sink = torch.zeros(8192, device="cuda:0")
    lib = fa.ftk()
    nbytes = B * V * 4
    ms = C.c_float(0.0)
    times = []
    for i in range(warmup + steps):
        ops.check(lib.ftk_measure_plain_read(bufs[i % nbuf].data_ptr(), nbytes, sink.data_ptr(), sink.numel(),
                                             ops.current_stream(), C.addressof(ms)))
        if i >= warmup:
            times.append(ms.value)
    avg = sum(times) / len(times)
    return dict(bytes=nbytes, ms=avg, best_ms=min(times), gbs=nbytes / (avg * 1e-3) / 1e9)


def run_gpu_topp(name, w, steps, warmup, nbuf=3):
    """Top-p layer steps; every step is bracketed by its own pair of events so that restoring the logits (which the
    layer turns into probabilities in place when it is asked for the reference's side effects) stays outside the
    measured time."""
    import torch
    import fastertransformer_amd as fa

    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    B, V = w["batch"], w["vocab"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(4321)
    base = -w["zipf_s"] * torch.log(torch.arange(1, V + 1, device=dev, dtype=torch.float64))
    base = base - torch.logsumexp(base, 0)
    bufs = []
    for _ in range(nbuf):
        x = torch.empty((B, V), device=dev, dtype=torch.float32)
        for b in range(B):
            perm = torch.randperm(V, device=dev, generator=gen)
            x[b] = (base[perm] + torch.randn(V, device=dev, generator=gen, dtype=torch.float64) * w["noise"]).float()
        bufs.append(x.reshape(B, 1, V))
    work = torch.empty_like(bufs[0])
    total = steps + warmup
    lo, hi = w["top_p"]
    top_ps = (torch.rand(B, generator=gen, device=dev) * (hi - lo) + lo).cpu().numpy().astype(np.float32)
    layer = fa.DynamicDecodeLayer(fa.F32, V, V)
    layer.setup(B, 1, {"runtime_top_k": np.array([0], np.uint32), "runtime_top_p": top_ps,
                       "top_p_decay": torch.full((B,), w["top_p_decay"], device=dev),
                       "top_p_min": torch.full((B,), w["top_p_min"], device=dev),
                       "top_p_reset_ids": torch.full((B,), w["top_p_reset_id"], dtype=torch.int32, device=dev),
                       "random_seed": np.array([1], np.uint64)})
    output_ids = torch.zeros((total + 1, B), dtype=torch.int32, device=dev)
    finished = torch.zeros(B, dtype=torch.bool, device=dev)
    seq_len = torch.zeros(B, dtype=torch.int32, device=dev)
    end_id = torch.full((B,), V - 1, dtype=torch.int32, device=dev)
    outs = {"output_ids": output_ids, "finished": finished, "sequence_length": seq_len}
    step_arr = np.zeros(1, np.int32)
    fixed = {"step": step_arr, "max_input_length": np.array([0], np.int32), "ite": np.array([0], np.uint32),
             "local_batch_size": np.array([B], np.int32), "end_id": end_id}
    events = []
    for i in range(total):
        step_arr[0] = i
        finished.zero_()
        work.copy_(bufs[i % nbuf])
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        layer.forward(outs, dict(fixed, logits=work))
        e1.record()
        if i >= warmup:
            events.append((e0, e1))
    torch.cuda.synchronize()
    ms = [a.elapsed_time(b) for a, b in events]
    gpu_ms = sum(ms) / len(ms)
    return dict(tokens_per_s=B / (gpu_ms * 1e-3), ms_per_step=gpu_ms, p50_ms=float(np.median(ms)), max_ms=max(ms),
                sampled_ids_checksum=int(output_ids[warmup:total].to(torch.int64).sum().item()))


def run_gpu_loop(name, w, steps, warmup, nbuf=2):
    """Decode loop with stop criteria and, per workload, log-probs, additive penalties, a minimum length and
    bad / stop word lists; per-step events, logits restored outside them (this path works in place, like the
    reference)."""
    import torch
    import fastertransformer_amd as fa

    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    dt = {"f32": fa.F32, "f16": fa.F16, "bf16": fa.BF16}[w["dtype"]]
    B, V, Vp, H = w["batch"], w["vocab"], w["vocab_padded"], w["prompt"]
    gen = torch.Generator(device=dev)
    gen.manual_seed(55)
    bufs = [(torch.randn((B, 1, Vp), generator=gen, device=dev, dtype=torch.float32) * w["sigma"]).to(fa.torch_dtype(dt))
            for _ in range(nbuf)]
    work = torch.empty_like(bufs[0])
    total = steps + warmup
    layer = fa.DynamicDecodeLayer(dt, V, Vp)
    args = {"runtime_top_k": np.array([w["top_k"]], np.uint32), "runtime_top_p": np.array([w["top_p"]], np.float32),
            "temperature": np.array([w["temperature"]], np.float32), "random_seed": np.array([1], np.uint64)}
    for key in ("repetition_penalty", "presence_penalty", "frequency_penalty"):
        if w.get(key) is not None:
            args[key] = np.array([w[key]], np.float32)
    if "min_length_beyond" in w:  # the end id stays masked during every measured step
        args["min_length"] = np.array([H + total + w["min_length_beyond"]], np.int32)
    layer.setup(B, 1, args)
    rng = np.random.default_rng(104)
    output_ids = torch.zeros((H + total + 1, B), dtype=torch.int32, device=dev)
    if "zipf_history" in w:
        history = np.minimum(rng.zipf(w["zipf_history"], (H, B)), V - 1).astype(np.int32)
        output_ids[:H] = torch.from_numpy(history).to(dev)
    else:
        output_ids[:H] = torch.randint(0, V, (H, B), generator=gen, device=dev, dtype=torch.int32)
    finished = torch.zeros(B, dtype=torch.bool, device=dev)
    seq_len = torch.full((B,), H - 1, dtype=torch.int32, device=dev)
    end_id = torch.full((B,), w.get("end_id", V - 1), dtype=torch.int32, device=dev)
    limit = torch.full((B,), H + total + 8, dtype=torch.int32, device=dev)
    outs = {"output_ids": output_ids, "finished": finished, "sequence_length": seq_len,
            "should_stop": np.zeros(1, np.bool_)}
    if w.get("logprobs", True):
        outs["cum_log_probs"] = torch.zeros(B, device=dev)
        outs["output_log_probs"] = torch.zeros((total + 1, B), device=dev)
    step_arr = np.zeros(1, np.int32)
    fixed = {"step": step_arr, "max_input_length": np.array([H], np.int32), "ite": np.array([0], np.uint32),
             "local_batch_size": np.array([B], np.int32), "end_id": end_id, "sequence_limit_length": limit}
    def word_list(n, longest):
        # [2, L] in the reference's format: ids back to back (0 padded), then inclusive end offsets (-1 padded)
        words = [rng.integers(1, V, int(rng.integers(1, longest + 1))) for _ in range(n)]
        out = np.zeros((2, n * longest), np.int32)
        out[1, :] = -1
        flat = np.concatenate(words)
        out[0, :flat.size] = flat
        out[1, :n] = np.cumsum([len(x) for x in words])
        return out

    for key, spec in (("bad_words_list", w.get("bad_words")), ("stop_words_list", w.get("stop_words"))):
        if spec:  # [B, 2, L] word lists, random ids
            lists = np.stack([word_list(*spec) for _ in range(B)])
            fixed[key] = torch.from_numpy(lists).to(dev)
    if "stop_words_list" in fixed:
        outs["parent_ids"] = torch.zeros(1, dtype=torch.int32, device=dev)
    ms = []
    for i in range(total):
        step_arr[0] = H + i
        work.copy_(bufs[i % nbuf])
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        layer.forward(outs, dict(fixed, logits=work))   # returns with should_stop valid
        e1.record()
        torch.cuda.synchronize()
        if i >= warmup:
            ms.append(e0.elapsed_time(e1))
    ms = np.array(ms)
    return dict(tokens_per_s=B / (ms.mean() * 1e-3), ms_per_step=float(ms.mean()), p50_ms=float(np.percentile(ms, 50)),
                p99_ms=float(np.percentile(ms, 99)), max_ms=float(ms.max()),
                sampled_ids_checksum=int(output_ids[H + warmup:H + total].to(torch.int64).sum().item()))


def run_gpu_beam(name, w, steps, warmup):
    """Beam-search steps over one synthetic state: logits [batch * beam_width, vocab] in rotation, cumulative
    log-probs and hypothesis counts restored before every step outside its pair of events."""
    import ctypes as C
    import torch
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops

    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    dt = {"f32": fa.F32, "f16": fa.F16, "bf16": fa.BF16}[w["dtype"]]
    batch, K, V = w["batch"], w["beam_width"], w["vocab"]
    rows, step, max_seq_len = batch * K, 5, 12
    gen = torch.Generator(device=dev)
    gen.manual_seed(1)
    rnd = lambda *shape: torch.rand(*shape, generator=gen, device=dev)
    end_ids = torch.randint(0, V, (batch,), generator=gen, device=dev, dtype=torch.int32)
    row_end = end_ids.repeat_interleave(K).long()
    logits = []
    for _ in range(3):
        x = torch.randn((rows, V), generator=gen, device=dev, dtype=torch.float32) * w["sigma"]
        ending = rnd(rows) < 0.05                      # a few beams are about to end
        x[torch.arange(rows, device=dev)[ending], row_end[ending]] += 4.0 * w["sigma"]
        logits.append(x.to(fa.torch_dtype(dt)))
    d = {"finished": rnd(rows) < 0.05,
         "sequence_lengths": torch.randint(1, step + 2, (rows,), generator=gen, device=dev, dtype=torch.int32),
         "cum_log_probs": -torch.randn(rows, generator=gen, device=dev).abs() * 4, "end_ids": end_ids,
         "ids": torch.full((batch, K), -1, dtype=torch.int32, device=dev),
         "output_log_probs": torch.zeros((batch, K), device=dev)}
    normed = -torch.randn((batch, 2 * K), generator=gen, device=dev).abs() * 3
    num = torch.randint(0, K, (batch,), generator=gen, device=dev, dtype=torch.int32)
    mins = torch.stack([normed[b, :int(num[b])].min() if int(num[b]) else normed.new_zeros(()) for b in range(batch)])
    keep = {"output_ids_tgt": torch.zeros((batch, 2 * K, max_seq_len), dtype=torch.int32, device=dev),
            "sequence_lengths_tgt": torch.zeros((batch, 2 * K), dtype=torch.int32, device=dev),
            "cum_log_probs": torch.zeros((batch, 2 * K), device=dev), "normed_scores": normed,
            "log_probs": torch.zeros((batch, 2 * K, max_seq_len), device=dev), "min_normed_scores": mins,
            "num_beams": num, "is_done": torch.zeros(batch, dtype=torch.bool, device=dev),
            "output_ids_src": torch.randint(0, V, (max_seq_len, batch, K), generator=gen, device=dev,
                                            dtype=torch.int32),
            "parent_ids_src": torch.randint(0, K, (max_seq_len, batch, K), generator=gen, device=dev,
                                            dtype=torch.int32),
            "log_probs_src": -torch.randn((max_seq_len, batch, K), generator=gen, device=dev).abs()}
    hyps = ops.BeamHypotheses()
    for key, val in keep.items():
        setattr(hyps, key, val.data_ptr())
    hyps.end_ids = end_ids.data_ptr()
    hyps.step, hyps.ite, hyps.batch_size, hyps.local_batch_size, hyps.max_seq_len = step, 0, batch, batch, max_seq_len
    hyps.early_stopping = True
    lib = fa.ftk()
    size = C.c_size_t(0)

    def call(x, ws):
        ops.check(lib.ftk_invoke_topk_softmax(
            dt, x.data_ptr(), None, d["finished"].data_ptr(), d["sequence_lengths"].data_ptr(),
            d["cum_log_probs"].data_ptr(), d["output_log_probs"].data_ptr(), d["ids"].data_ptr(),
            ws.data_ptr() if ws is not None else None, C.addressof(size), C.addressof(hyps), batch, K, V,
            d["end_ids"].data_ptr(), 0.0, 0.0, ops.current_stream()))

    call(logits[0], None)
    ws = torch.empty(size.value, dtype=torch.uint8, device=dev)
    num0, cum0 = keep["num_beams"].clone(), d["cum_log_probs"].clone()
    ms, checksum = [], 0
    for i in range(steps + warmup):
        keep["num_beams"].copy_(num0)
        d["cum_log_probs"].copy_(cum0)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        call(logits[i % len(logits)], ws)
        e1.record()
        torch.cuda.synchronize()
        if i >= warmup:
            ms.append(e0.elapsed_time(e1))
            checksum += int(d["ids"].to(torch.int64).sum().item())
    ms = np.array(ms)
    alg = batch * K * V * (4 if w["dtype"] == "f32" else 2)
    return dict(ms_per_step=float(ms.mean()), p50_ms=float(np.percentile(ms, 50)), max_ms=float(ms.max()),
                beams_per_s=batch * K / (ms.mean() * 1e-3), gbs=alg / (ms.mean() * 1e-3) / 1e9, bytes=alg,
                ids_checksum=checksum)


# ---- the other benchmark configurations: short timed runs and a one-step oracle check each -------------------------

SECONDARY = [
    "topp_step_b256_v128256_f32_zipf1.1_p0.5-0.99_decay0.9",
    "decode_step_b256_v51200_f16_topk1-1024_topp0.9_temp0.8_rep1.1",
    "decode_loop_b1024_v152064_f16_topk64_topp0.9_logprobs",
    "decode_loop_b128_v32000_bf16_hist2048_presence0.5_freq0.3_minlen_badwords_stopwords_topk50",
]


def _secondary_case(name, w, rng):
    """the workload as one decode step of the test harness: (Case arguments, logits [B, Vp] as numpy storage, step)"""
    import ft_oracle as O
    from helpers import make_word_list
    dt = {"f32": O.F32, "f16": O.F16, "bf16": O.BF16}[w["dtype"]]
    B, V, Vp, H = w["batch"], w["vocab"], w["vocab_padded"], w["prompt"]
    kw = dict(max_input_length=H, gen_len=1)
    if name.startswith("topp_step"):
        base = -w["zipf_s"] * np.log(np.arange(1, V + 1, dtype=np.float64))
        base = (base - np.log(np.exp(base).sum())).astype(np.float32)
        x = rng.standard_normal((B, V), dtype=np.float32) * np.float32(w["noise"])
        for b in range(B):
            x[b] += base[rng.permutation(V)]
        lo, hi = w["top_p"]
        kw.update(runtime_top_k=[0], runtime_top_p=rng.uniform(lo, hi, B), top_p_decay=np.full(B, w["top_p_decay"]),
                  top_p_min=np.full(B, w["top_p_min"]), top_p_reset_ids=np.full(B, w["top_p_reset_id"]))
        return dt, kw, x, 0
    x = O.to_storage(rng.standard_normal((B, Vp), dtype=np.float32) * np.float32(w["sigma"]), dt)
    if "zipf_history" in w:
        prompt = np.minimum(rng.zipf(w["zipf_history"], (H, B)), V - 1).astype(np.int32)
    else:
        prompt = rng.integers(0, V, (H, B)).astype(np.int32)
    if isinstance(w["top_k"], tuple):
        top_ks = np.random.default_rng(0).choice(np.array(w["top_k"], np.uint32), B).astype(np.uint32)
    else:
        top_ks = [w["top_k"]]
    kw.update(runtime_top_k=top_ks, runtime_top_p=[w["top_p"]], temperature=[w["temperature"]], prompt=prompt,
              end_ids=np.full(B, w.get("end_id", V - 1), np.int32))
    for key in ("repetition_penalty", "presence_penalty", "frequency_penalty"):
        if w.get(key) is not None:
            kw[key] = [w[key]]
    if "min_length_beyond" in w:
        kw["min_length"] = [H + w["min_length_beyond"]]
    if name.startswith("decode_loop"):
        kw["sequence_limit_length"] = np.full(B, H + 8, np.uint32)
        if w.get("logprobs", True):
            kw.update(with_cum=True, with_out_lp=True)
    if w.get("bad_words"):
        n, longest = w["bad_words"]
        kw["bad_words"] = np.stack([make_word_list(rng, n, longest, V, L=n * longest)[0] for _ in range(B)])
    if w.get("stop_words"):
        n, longest = w["stop_words"]
        kw["stop_words"] = np.stack([make_word_list(rng, n, longest, V, L=n * longest)[0] for _ in range(B)])
    return dt, kw, x, H


def secondary_oracle_check(name, w, rows_checked=None):
    """One step of the workload at its full batch through the product's DynamicDecodeLayer, and the same step on the
    CPU oracle for the first `rows_checked` rows (rows are independent): ids, flags and lengths must be identical,
    log-probs within the tolerance of the type. Outside every timed region."""
    import ft_oracle as O
    from decode_harness import Case, OracleRunner, ProductRunner
    from helpers import uniforms
    rng = np.random.default_rng(2025)
    dt, kw, x, step = _secondary_case(name, w, rng)
    B, V, Vp = w["batch"], w["vocab"], w["vocab_padded"]
    n = B if rows_checked is None else min(B, rows_checked)
    u = uniforms(rng, B)
    full = Case(dt, B, V, Vp, **kw)
    product = ProductRunner(full)
    product.step(step, x, u)
    got = product.snapshot()

    def cut(key, v):
        if v is None or np.ndim(v) == 0 or key in ("max_input_length", "gen_len"):
            return v
        v = np.asarray(v)
        if key == "prompt":
            return v[:, :n]
        return v[:n] if v.shape[0] == B else v
    sub = Case(dt, n, V, Vp, **{k: cut(k, v) for k, v in kw.items()})
    oracle = OracleRunner(sub)
    oracle.step(step, x[:n].copy(), u[:n])
    ref = oracle.snapshot()
    ok = np.array_equal(got["output_ids"][:, :n], ref["output_ids"])
    for key in ("finished", "sequence_length"):
        if ref[key] is not None:
            ok = ok and np.array_equal(got[key][:n], ref[key])
    rtol = 1e-5 if dt == O.F32 else 2e-3
    for key in ("cum_log_probs", "output_log_probs"):
        if ref[key] is not None:
            a = got[key][..., :n] if key == "output_log_probs" else got[key][:n]
            ok = ok and bool(np.allclose(a, ref[key], rtol=rtol, atol=1e-6))
    return dict(rows=n, of=B, step=int(step), ids_checksum=int(ref["output_ids"][step].astype(np.int64).sum()),
                identical=bool(ok))


def run_secondary(steps, warmup):
    """the other configurations of the benchmark set, a few steps each: per-step time, algorithmic bytes per step,
    their share of the HBM peak, and the one-step oracle check"""
    out = []
    for name in SECONDARY:
        w = WORKLOADS[name]
        elem = 4 if w["dtype"] == "f32" else 2
        if name.startswith("topp_step"):
            r = run_gpu_topp(name, w, steps, warmup)
            ms, extra, hist = r["ms_per_step"], dict(p50_ms=r["p50_ms"], max_ms=r["max_ms"]), 0
        elif name.startswith("decode_loop"):
            r = run_gpu_loop(name, w, steps, warmup)
            ms, extra = r["ms_per_step"], dict(p50_ms=r["p50_ms"], p99_ms=r["p99_ms"], max_ms=r["max_ms"])
            hist = w["prompt"] + warmup + steps // 2
        else:
            r = run_gpu(name, w, steps, warmup)
            ms, extra, hist = r["gpu_ms_per_step"], dict(kernel_ms=r["kernel_ms"]), w["prompt"] + warmup + steps // 2
        alg = w["batch"] * w["vocab_padded"] * elem + w["batch"] * hist * 4 + w["batch"] * 32
        check = secondary_oracle_check(name, w, rows_checked=64 if w["batch"] > 256 else None)
        out.append(dict(workload=name, dtype=w["dtype"], batch=w["batch"], vocab=w["vocab"], steps=steps, warmup=warmup,
                        ms_per_step=ms, tokens_per_s=w["batch"] / (ms * 1e-3), algorithmic_bytes_per_step=alg,
                        hbm_gbs=alg / (ms * 1e-3) / 1e9, frac=alg / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                        oracle_check=check, **extra))
    return out


def _oracle_rows_per_second(w, rows, budget_s, seed):
    """the oracle's DynamicDecodeLayer on `rows`-row batches of the workload for about `budget_s` seconds of this
    thread's time; returns (rows done, seconds)"""
    import ft_oracle as O
    dt = {"f32": O.F32, "f16": O.F16, "bf16": O.BF16}[w["dtype"]]
    V, Vp, H = w["vocab"], w["vocab_padded"], w["prompt"]
    rng = np.random.default_rng(seed)
    layer = O.OracleDynamicDecodeLayer(dt, V, Vp)
    layer.setup(rows, [w["top_k"]], [w["top_p"]], [w["temperature"]], [w["repetition_penalty"]])
    max_steps = 4096
    out_ids = np.zeros((H + max_steps + 1, rows), np.int32)
    out_ids[:H] = rng.integers(0, V, (H, rows))
    finished = np.zeros(rows, np.bool_)
    seq = np.full(rows, H - 1, np.int32)
    end = np.full(rows, V - 1, np.int32)
    # a few logits batches generated up front and reused, so that the loop times the oracle and nothing else
    batches = [O.to_storage((rng.standard_normal((rows, Vp)) * w["sigma"]).astype(np.float32), dt) for _ in range(2)]
    done, spent, step = 0, 0.0, H
    while spent < budget_s and step < H + max_steps:
        logits = batches[(step - H) % len(batches)].copy()
        u = rng.random(rows).astype(np.float32) * 0.999 + 0.001
        finished[:] = False
        t0 = time.perf_counter()
        layer.forward(logits, end, out_ids, step, H, u, finished=finished, sequence_length=seq)
        spent += time.perf_counter() - t0
        done += rows
        step += 1
    return done, spent


def run_cpu_baseline(w, budget_s=8.0):
    """The CPU baseline beside the GPU number: the oracle (a scalar restatement of the reference algorithm; the
    reference's own host functions live inside CUDA unit tests and cannot be built here) on rows of the same
    workload, first on one core, then with one thread per core, every thread on rows of its own (rows are
    independent; the oracle's C code runs outside the interpreter lock). Bounded: about `budget_s` seconds each."""
    from concurrent.futures import ThreadPoolExecutor
    cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1))
    try:
        cores = min(cores, len(os.sched_getaffinity(0)))
    except AttributeError:
        pass
    rows = 8
    done1, spent1 = _oracle_rows_per_second(w, rows, budget_s, 99)
    t0 = time.perf_counter()
    with ThreadPoolExecutor(max_workers=cores) as pool:
        parts = list(pool.map(lambda i: _oracle_rows_per_second(w, rows, budget_s, 100 + i), range(cores)))
    wall = time.perf_counter() - t0
    done_all = sum(p[0] for p in parts)
    busy = max(p[1] for p in parts)  # the threads run side by side: the slowest one bounds the rate
    return dict(value=done_all / busy, unit="tokens/s", cores=cores, kind="port",
                single_core_value=done1 / spent1,
                sample="%d-row batches of the same workload (V=%d): %d rows in %.1f s on one core, then %d rows in "
                       "%.1f s with one thread on each of %d cores (%.1f s wall including input generation)"
                       % (rows, w["vocab"], done1, spent1, done_all, busy, cores, wall))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true",
                    help="skip the short runs of the other configurations that the default line carries under `configs`")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run five plain device copies of 128 MiB, the known-size kernel that FETCH_SIZE / "
                         "WRITE_SIZE counter readings are scaled by")
    ap.add_argument("--workload", default=next(iter(WORKLOADS)), choices=list(WORKLOADS) + [PLAIN_READ],
                    help="default: the headline decode step; the others print a secondary line of their own")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU leg (rows shard across GPUs with no "
              "exchange); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    name = a.workload
    if name == PLAIN_READ:
        r = run_plain_read(a.steps, a.warmup)
        print(json.dumps({
            "metric": "HBM GB/s of a kernel that only reads 256 x 128256 fp32 (the streaming kernel's launch shape)",
            "value": r["gbs"], "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "ms_per_step": r["ms"], "best_ms": r["best_ms"], "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "f32", "data": "synthetic", "config": {"workload": name},
            "roofline": {"bound": "hbm", "achieved": r["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": r["gbs"] / HBM_PEAK_GBS, "traffic": None, "kernel": "read_yardstick_kernel",
                         "algorithmic_bytes_per_launch": r["bytes"]}}))
        return
    w = WORKLOADS[name]
    if name.startswith("topp_step"):
        r = run_gpu_topp(name, w, a.steps, a.warmup)
        print(json.dumps({
            "metric": "sampled tokens/s, top-p decode step B=256 V=128256 (softmax + nucleus sampling + decay)",
            "value": r["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "ms_per_step": r["ms_per_step"], "p50_ms": r["p50_ms"], "max_ms": r["max_ms"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": name, "batch": w["batch"], "vocab": w["vocab"]},
            "sampled_ids_checksum": r["sampled_ids_checksum"]}))
        return
    if name.startswith("beam_step"):
        r = run_gpu_beam(name, w, a.steps, a.warmup)
        print(json.dumps({
            "metric": "beams extended per second, beam-search step B=%d K=%d V=%d (log-softmax, 2K best per beam, "
                      "K best per entry, hypotheses)" % (w["batch"], w["beam_width"], w["vocab"]),
            "value": r["beams_per_s"], "unit": "beams/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "ms_per_step": r["ms_per_step"], "p50_ms": r["p50_ms"], "max_ms": r["max_ms"], "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic",
            "config": {"workload": name, "batch": w["batch"], "beam_width": w["beam_width"], "vocab": w["vocab"]},
            "roofline": {"bound": "hbm", "achieved": r["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": r["gbs"] / HBM_PEAK_GBS, "traffic": None, "kernel": "whole step (four kernels)",
                         "algorithmic_bytes_per_launch": r["bytes"]},
            "ids_checksum": r["ids_checksum"]}))
        return
    if name.startswith("decode_loop"):
        r = run_gpu_loop(name, w, a.steps, a.warmup)
        print(json.dumps({
            "metric": "per-step latency, decode loop B=%d V=%d %s (top-k%s + penalties%s, stop criteria)"
                      % (w["batch"], w["vocab"], w["dtype"], " + top-p" if w["top_p"] else "",
                         ", log-probs" if w.get("logprobs", True) else ", bad and stop words, minimum length"),
            "value": r["p50_ms"], "unit": "ms (p50)", "p99_ms": r["p99_ms"], "max_ms": r["max_ms"], "n_gpus": 1,
            "steps": a.steps, "warmup": a.warmup, "ms_per_step": r["ms_per_step"], "tokens_per_s": r["tokens_per_s"],
            "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": w["dtype"],
            "data": "synthetic",
            "config": {"workload": name, "batch": w["batch"], "vocab": w["vocab"], "top_k": w["top_k"],
                       "top_p": w["top_p"], "history": w["prompt"]},
            "sampled_ids_checksum": r["sampled_ids_checksum"]}))
        return
    r = run_gpu(name, w, a.steps, a.warmup, check_oracle=(name == next(iter(WORKLOADS))))
    if name != next(iter(WORKLOADS)):
        r["roofline"]["traffic"] = None  # the counter runs cover the headline workload only
        print(json.dumps({
            "metric": "sampled tokens/s, decode step B=%d V=%d (full top-k+top-p+penalty DynamicDecodeLayer step)"
                      % (w["batch"], w["vocab"]),
            "value": r["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
            "dtype": w["dtype"], "data": "synthetic",
            "config": {"workload": name, "batch": w["batch"], "vocab": w["vocab"],
                       "top_k": list(w["top_k"]) if isinstance(w["top_k"], tuple) else w["top_k"],
                       "top_p": w["top_p"], "temperature": w["temperature"],
                       "repetition_penalty": w["repetition_penalty"], "history": w["prompt"]},
            "roofline": r["roofline"], "gpu_ms_per_step": r["gpu_ms_per_step"], "kernel_ms": r["kernel_ms"],
            "sampled_ids_checksum": r["sampled_ids_checksum"]}))
        return
    if a.copy_calibration:
        import torch
        src = torch.empty(128 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
    line = {
        "metric": "sampled tokens/s, decode step B=256 V=128256 (full top-k+top-p+penalty DynamicDecodeLayer step)",
        "value": r["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": r["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": name, "batch": w["batch"], "vocab": w["vocab"], "top_k": w["top_k"],
                   "top_p": w["top_p"], "temperature": w["temperature"],
                   "repetition_penalty": w["repetition_penalty"], "history": w["prompt"]},
        "roofline": r["roofline"],
        "gpu_ms_per_step": r["gpu_ms_per_step"], "kernel_ms": r["kernel_ms"], "step_hbm_gbs": r["step_gbs"],
        "step_hbm_frac": r["step_gbs"] / HBM_PEAK_GBS, "sampled_ids_checksum": r["sampled_ids_checksum"],
        "oracle_check": r["oracle_check"],
    }
    if not a.no_secondary:
        line["configs"] = run_secondary(min(a.steps, 20), min(a.warmup, 3))
    if not a.no_cpu_baseline:
        line["cpu_baseline"] = run_cpu_baseline(w)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
