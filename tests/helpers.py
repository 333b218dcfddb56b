"""Shared helpers of the test-suite: seeded input generators and numpy <-> torch storage conversions."""
import numpy as np

import ft_oracle as O

DTYPES = [O.F32, O.F16, O.BF16]
DTYPE_NAMES = {O.F32: "f32", O.F16: "f16", O.BF16: "bf16"}


def to_torch(arr, dt=None, device="cuda"):
    """numpy storage array -> torch tensor on `device` (bf16 travels as uint16 bits)"""
    import torch
    if arr is None:
        return None
    if dt == O.BF16 and arr.dtype == np.uint16:
        return torch.from_numpy(arr.view(np.int16).copy()).view(torch.bfloat16).to(device)
    if arr.dtype == np.uint32:
        return torch.from_numpy(arr.view(np.int32).copy()).to(device)
    if arr.dtype == np.uint64:
        return torch.from_numpy(arr.view(np.int64).copy()).to(device)
    return torch.from_numpy(arr.copy()).to(device)


def to_numpy(t, dt=None):
    """torch tensor -> numpy storage array"""
    import torch
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def bits(arr, dt):
    """storage array -> integer bit patterns (for exact comparison)"""
    if dt == O.F32:
        return np.asarray(arr, np.float32).view(np.uint32)
    return np.asarray(arr).view(np.uint16)


def ulp_diff_f32(a, b):
    """distance in units of the last place between two float32 arrays (sign-magnitude aware)"""
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7FFFFFFF), a)
    b = np.where(b < 0, -(b & 0x7FFFFFFF), b)
    return np.abs(a - b)


def make_logits(rng, dt, batch, V, Vp, scale=2.0, spikes=0):
    x = (rng.standard_normal((batch, Vp)) * scale).astype(np.float32)
    for b in range(batch):
        if spikes:
            x[b, rng.integers(0, V, spikes)] += 12.0
    return O.to_storage(x, dt)


def make_word_list(rng, n_words, max_len, vocab, L=None, history=None, step=None, row=None, batch=None):
    """[2, L] int32 word list in the reference's format (row 0: ids back to back, 0 padded;
    row 1: inclusive end offsets, -1 padded). Some words are copied from the history tail so they match."""
    words = []
    for w in range(n_words):
        n = int(rng.integers(1, max_len + 1))
        if history is not None and step is not None and step >= n and rng.random() < 0.5:
            # tail of the history followed by a random last token (bad words) or the tail itself
            tail = [int(history[step - n + 1 + t, row]) for t in range(n - 1)] if n > 1 else []
            words.append(tail + [int(rng.integers(1, vocab))])
        else:
            words.append([int(x) for x in rng.integers(1, vocab, n)])
    flat = [t for w in words for t in w]
    offs = np.cumsum([len(w) for w in words]).tolist()
    if L is None:
        L = max(len(flat), len(offs))
    out = np.zeros((2, L), np.int32)
    out[1, :] = -1
    out[0, :len(flat)] = flat
    out[1, :len(offs)] = offs
    return out, words


def uniforms(rng, n):
    """draws in (0, 1] like curand_uniform"""
    u = rng.random(n).astype(np.float32)
    u = np.where(u == 0.0, np.float32(1.0), u)
    return u.astype(np.float32)


def run_fused_step(entry, torch, dt, B, V, H, k, logits, history, draws, finished0, seqlen0, lib=None, ws_fill=None,
                   log_probs=None, Vp=None):
    """One fused decode step straight through the C ABI (temperature 0.8, repetition penalty 1.1 over `history`,
    top-k `k`, top-p 0.9, injected draws). entry: "caller" = ftk_fused_topk_step with a workspace of the queried
    size, "static" = ftk_fused_topk_step_static. Returns (ids, sequence_length, finished, rc, needed bytes, change of
    the device's free memory across the static call). With a dict as `log_probs` the step also keeps log-probs:
    cum_log_probs start at the dict's "cum" (zeros without it) and come back there, output_log_probs under "out".
    `Vp` is the pitch of the logits' rows in elements when they are padded."""
    import ctypes as C
    import fastertransformer_amd as fa
    from fastertransformer_amd import ops
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
    a.vocab_size = V
    a.vocab_size_padded = V if Vp is None else Vp
    a.batch_size = a.local_batch_size = B
    a.step, a.max_input_length = H, H
    a.temperatures, a.penalties, a.penalty_type = temps.data_ptr(), pens.data_ptr(), ops.PENALTY_MULTIPLICATIVE
    a.end_ids, a.output_ids = end_ids.data_ptr(), out_ids.data_ptr()
    a.top_ks, a.top_ps, a.max_top_k = top_ks.data_ptr(), top_ps.data_ptr(), k
    a.uniform_draws = draws.data_ptr()
    a.ids = out_ids.data_ptr() + 4 * H * B
    a.sequence_length, a.finished = seq.data_ptr(), finished.data_ptr()
    if log_probs is not None:
        cum = torch.zeros(B, device=dev) if "cum" not in log_probs else torch.as_tensor(log_probs["cum"]).to(dev)
        olp = torch.zeros(B, device=dev)
        a.cum_log_probs, a.output_log_probs = cum.data_ptr(), olp.data_ptr()
    lib = fa.ftk() if lib is None else lib
    stream = ops.current_stream()
    ws = None
    if entry == "caller":
        a.workspace = None
        ops.check(lib.ftk_fused_topk_step(C.addressof(a), stream), "size query")
        ws = torch.empty(a.workspace_size, dtype=torch.uint8, device=dev)
        if ws_fill is not None:
            ws.fill_(ws_fill)  # (nothing in the workspace has to start at zero)
        a.workspace = ws.data_ptr()
        rc = lib.ftk_fused_topk_step(C.addressof(a), stream)
        torch.cuda.synchronize()
        freed = 0
    else:
        a.workspace, a.workspace_size = None, 0
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]  # (the driver's figure: torch's own pool does not hide anything)
        rc = lib.ftk_fused_topk_step_static(C.addressof(a), stream)
        torch.cuda.synchronize()
        freed = torch.cuda.mem_get_info()[0] - free_before
    if log_probs is not None:
        log_probs["cum"], log_probs["out"] = cum.cpu().numpy(), olp.cpu().numpy()
    return out_ids[H].cpu().numpy(), seq.cpu().numpy(), finished.cpu().numpy(), rc, a.workspace_size, freed


def make_beam_case(rng, dt, batch, K, V, step=5, max_seq_len=12, with_hyps=True, finished_frac=0.2, full_frac=0.2,
                   scale=3.0, end_spike=0.5):
    """Seeded inputs of one beam-search step (invokeTopkSoftMax): logits [batch * K, V] in storage type `dt`, the
    running beams' state and, optionally, the arrays of a BeamHypotheses with some entries already collected.
    Returns a dict of numpy arrays and ints (the names of the reference's arguments and struct fields)."""
    import ft_oracle as O
    rows = batch * K
    x = rng.standard_normal((rows, V)).astype(np.float32) * np.float32(scale)
    end_ids = rng.integers(0, V, batch).astype(np.int32)
    for r in range(rows):  # some beams are about to end: their end token is among their best
        if rng.random() < end_spike:
            x[r, end_ids[r // K]] += np.float32(rng.uniform(2.0, 5.0) * scale)
    c = dict(log_probs=O.to_storage(x, dt), finished=rng.random(rows) < finished_frac,
             sequence_lengths=rng.integers(1, step + 2, rows).astype(np.int32),
             cum_log_probs=(-np.abs(rng.standard_normal(rows)) * 4).astype(np.float32), end_ids=end_ids,
             ids=np.full((batch, K), -1, np.int32), output_log_probs=np.zeros((batch, K), np.float32))
    if with_hyps:
        num = np.where(rng.random(batch) < full_frac, K, rng.integers(0, K, batch)).astype(np.int32)
        normed = (-np.abs(rng.standard_normal((batch, 2 * K))) * 3).astype(np.float32)
        mins = np.array([normed[b, :num[b]].min() if num[b] else 0.0 for b in range(batch)], np.float32)
        c["hyps"] = dict(
            output_ids_tgt=np.zeros((batch, 2 * K, max_seq_len), np.int32),
            sequence_lengths_tgt=np.zeros((batch, 2 * K), np.int32),
            cum_log_probs=np.zeros((batch, 2 * K), np.float32), normed_scores=normed,
            log_probs=np.zeros((batch, 2 * K, max_seq_len), np.float32), min_normed_scores=mins, num_beams=num,
            is_done=np.zeros(batch, np.bool_),
            output_ids_src=rng.integers(0, V, (max_seq_len, batch, K)).astype(np.int32),
            parent_ids_src=rng.integers(0, K, (max_seq_len, batch, K)).astype(np.int32),
            sequence_lengths_src=None, end_ids=end_ids,
            log_probs_src=(-np.abs(rng.standard_normal((max_seq_len, batch, K)))).astype(np.float32),
            step=step, ite=0, batch_size=batch, local_batch_size=batch, max_seq_len=max_seq_len, length_penalty=0.0,
            early_stopping=1)
    else:
        c["hyps"] = None
    return c


def copy_beam_case(c):
    """deep copy (the step updates its arguments in place)"""
    out = {k: (v.copy() if isinstance(v, np.ndarray) else v) for k, v in c.items() if k != "hyps"}
    out["hyps"] = None if c["hyps"] is None else {k: (v.copy() if isinstance(v, np.ndarray) else v)
                                                  for k, v in c["hyps"].items()}
    if out["hyps"] is not None:
        out["hyps"]["end_ids"] = out["end_ids"]
    return out


def make_beam_history(rng, batch, K, V, step, max_seq_len, max_input_length):
    """ids and parent beams of `step` earlier steps ([max_seq_len, batch * K]) and per-beam input lengths"""
    out_ids = np.zeros((max_seq_len, batch * K), np.int32)
    parents = np.zeros((max_seq_len, batch * K), np.int32)
    out_ids[:step] = rng.integers(0, V, (step, batch * K))
    parents[:step] = rng.integers(0, K, (step, batch * K))
    input_lengths = rng.integers(1, max_input_length + 1, batch * K).astype(np.int32)
    return out_ids, parents, input_lengths
