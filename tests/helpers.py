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
