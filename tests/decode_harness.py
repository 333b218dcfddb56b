"""Drives the product's DynamicDecodeLayer (GPU, through the C handle API) and the oracle's layer
restatement (CPU) with the same named tensors, step by step, and compares every output."""
import contextlib
import os

import numpy as np

import ft_oracle as O
from helpers import bits, to_numpy, to_torch


@contextlib.contextmanager
def kernel_sequence(enabled=True):
    """Inside: the product's top-k layer runs the reference's kernel-by-kernel sequence (which mutates the caller's
    logits like the reference) instead of its fused step (which leaves them alone)."""
    key, old = "FT_SAMPLING_DISABLE_FUSED", os.environ.get("FT_SAMPLING_DISABLE_FUSED")
    if enabled:
        os.environ[key] = "1"
    else:
        os.environ.pop(key, None)
    try:
        yield
    finally:
        if old is None:
            os.environ.pop(key, None)
        else:
            os.environ[key] = old


class Case:
    """One decode scenario: static arguments + per-step logits generator."""

    def __init__(self, dt, batch, V, Vp, max_input_length=0, gen_len=3, local_batch=None,
                 runtime_top_k=None, runtime_top_p=None, temperature=None, repetition_penalty=None,
                 presence_penalty=None, frequency_penalty=None, min_length=None, top_p_decay=None, top_p_min=None,
                 top_p_reset_ids=None, end_ids=None, embedding_bias=None, input_lengths=None, prompt=None,
                 sequence_limit_length=None, stop_words=None, bad_words=None, with_finished=True, with_seq_len=True,
                 with_cum=False, with_out_lp=False, random_seed=None):
        self.__dict__.update(locals())
        del self.__dict__["self"]
        self.local_batch = batch if local_batch is None else local_batch
        self.max_seq_len = max_input_length + gen_len
        self.end_ids = np.full(batch, V - 1, np.int32) if end_ids is None else np.asarray(end_ids, np.int32)


def _runtime_arg_tensors(c):
    """runtime arguments as the CPU tensors setup() expects (top_p_* as GPU tensors, like the reference)"""
    args = {}

    def put(key, val, dtype):
        if val is not None:
            args[key] = np.ascontiguousarray(np.atleast_1d(np.asarray(val)).astype(dtype))

    put("runtime_top_k", c.runtime_top_k, np.uint32)
    put("runtime_top_p", c.runtime_top_p, np.float32)
    put("temperature", c.temperature, np.float32)
    put("repetition_penalty", c.repetition_penalty, np.float32)
    put("presence_penalty", c.presence_penalty, np.float32)
    put("frequency_penalty", c.frequency_penalty, np.float32)
    put("min_length", c.min_length, np.int32)
    put("random_seed", c.random_seed, np.uint64)
    return args


class ProductRunner:
    def __init__(self, c):
        import torch
        import fastertransformer_amd as fa
        self.torch, self.fa, self.c = torch, fa, c
        self.layer = fa.DynamicDecodeLayer(c.dt, c.V, c.Vp)
        args = _runtime_arg_tensors(c)
        self._keep = [args]
        for key, val, dtype in (("top_p_decay", c.top_p_decay, np.float32), ("top_p_min", c.top_p_min, np.float32),
                                ("top_p_reset_ids", c.top_p_reset_ids, np.uint32)):
            if val is not None:
                args[key] = to_torch(np.ascontiguousarray(np.asarray(val, dtype)))
        self.layer.setup(c.batch, 1, args)
        B = c.batch
        self.output_ids = torch.zeros((c.max_seq_len, B), dtype=torch.int32, device="cuda")
        if c.prompt is not None:
            self.output_ids[:c.max_input_length] = to_torch(np.asarray(c.prompt, np.int32))
        self.finished = torch.zeros(B, dtype=torch.bool, device="cuda") if c.with_finished else None
        self.sequence_length = torch.full((B,), max(c.max_input_length - 1, 0) if c.prompt is not None else 0,
                                          dtype=torch.int32, device="cuda") if c.with_seq_len else None
        self.cum = torch.zeros(B, dtype=torch.float32, device="cuda") if c.with_cum else None
        self.out_lp = torch.zeros((c.gen_len, B), dtype=torch.float32, device="cuda") if c.with_out_lp else None
        self.end_ids = to_torch(c.end_ids)
        self.bias = to_torch(c.embedding_bias, c.dt) if c.embedding_bias is not None else None
        self.input_lengths = to_torch(np.asarray(c.input_lengths, np.int32)) if c.input_lengths is not None else None
        self.limit = to_torch(np.asarray(c.sequence_limit_length, np.uint32)) \
            if c.sequence_limit_length is not None else None
        self.stop = to_torch(np.asarray(c.stop_words, np.int32)) if c.stop_words is not None else None
        self.bad = to_torch(np.asarray(c.bad_words, np.int32)) if c.bad_words is not None else None
        self.should_stop = np.zeros(1, np.bool_)
        self.logits = None

    def step(self, step, logits_np, draws, ite=0):
        torch, c = self.torch, self.c
        from fastertransformer_amd.ops import NullTensor
        self.logits = to_torch(logits_np, c.dt).reshape(c.batch, 1, c.Vp)
        ins = {
            "logits": self.logits,
            "step": np.array([step], np.int32),
            "max_input_length": np.array([c.max_input_length], np.int32),
            "ite": np.array([ite], np.uint32),
            "local_batch_size": np.array([c.local_batch], np.int32),
            "end_id": self.end_ids,
        }
        if draws is not None:
            self.draws = to_torch(draws)
            ins["uniform_draws"] = self.draws
        if self.bias is not None:
            ins["embedding_bias"] = self.bias
        else:
            ins["embedding_bias"] = NullTensor(11, (c.Vp,))  # present with a null pointer, as in the reference tests
        if self.input_lengths is not None:
            ins["input_lengths"] = self.input_lengths.reshape(c.batch, 1)
        if self.limit is not None:
            ins["sequence_limit_length"] = self.limit
        if self.stop is not None:
            ins["stop_words_list"] = self.stop
        if self.bad is not None:
            ins["bad_words_list"] = self.bad
        outs = {"output_ids": self.output_ids}
        outs["finished"] = self.finished if self.finished is not None else NullTensor(1, (c.batch,))
        outs["sequence_length"] = self.sequence_length if self.sequence_length is not None \
            else NullTensor(8, (c.batch,))
        if self.cum is not None:
            outs["cum_log_probs"] = self.cum
        if self.out_lp is not None:
            outs["output_log_probs"] = self.out_lp
        if self.limit is not None:
            outs["should_stop"] = self.should_stop
        if self.stop is not None:
            outs["parent_ids"] = torch.zeros(1, dtype=torch.int32, device="cuda")
        self.layer.forward(outs, ins)
        torch.cuda.synchronize()

    def snapshot(self):
        g = lambda t: None if t is None else to_numpy(t)
        return dict(output_ids=g(self.output_ids), finished=g(self.finished), sequence_length=g(self.sequence_length),
                    cum_log_probs=g(self.cum), output_log_probs=g(self.out_lp), should_stop=self.should_stop.copy(),
                    logits=to_numpy(self.logits, self.c.dt).reshape(self.c.batch, self.c.Vp))


class OracleRunner:
    def __init__(self, c):
        self.c = c
        self.layer = O.OracleDynamicDecodeLayer(c.dt, c.V, c.Vp)
        self.layer.setup(c.batch, c.runtime_top_k, c.runtime_top_p, c.temperature, c.repetition_penalty,
                         c.presence_penalty, c.frequency_penalty, c.min_length, c.top_p_decay, c.top_p_min,
                         c.top_p_reset_ids)
        B = c.batch
        self.output_ids = np.zeros((c.max_seq_len, B), np.int32)
        if c.prompt is not None:
            self.output_ids[:c.max_input_length] = np.asarray(c.prompt, np.int32)
        self.finished = np.zeros(B, np.bool_) if c.with_finished else None
        self.sequence_length = np.full(B, max(c.max_input_length - 1, 0) if c.prompt is not None else 0, np.int32) \
            if c.with_seq_len else None
        self.cum = np.zeros(B, np.float32) if c.with_cum else None
        self.out_lp = np.zeros((c.gen_len, B), np.float32) if c.with_out_lp else None
        self.should_stop = np.zeros(1, np.bool_)
        self.logits = None

    def step(self, step, logits_np, draws, ite=0):
        c = self.c
        self.logits = logits_np.copy()
        self.layer.forward(
            self.logits, c.end_ids, self.output_ids, step, c.max_input_length, draws, ite=ite,
            local_batch_size=c.local_batch,
            embedding_bias=c.embedding_bias,
            input_lengths=None if c.input_lengths is None else np.asarray(c.input_lengths, np.int32),
            sequence_limit_length=None if c.sequence_limit_length is None
            else np.asarray(c.sequence_limit_length, np.uint32),
            stop_words=None if c.stop_words is None else np.ascontiguousarray(c.stop_words, np.int32),
            bad_words=None if c.bad_words is None else np.ascontiguousarray(c.bad_words, np.int32),
            finished=self.finished, sequence_length=self.sequence_length, cum_log_probs=self.cum,
            output_log_probs=self.out_lp, should_stop=self.should_stop)

    def snapshot(self):
        g = lambda a: None if a is None else a.copy()
        return dict(output_ids=g(self.output_ids), finished=g(self.finished), sequence_length=g(self.sequence_length),
                    cum_log_probs=g(self.cum), output_log_probs=g(self.out_lp), should_stop=self.should_stop.copy(),
                    logits=self.logits.copy())


def compare(got, ref, dt, check_logits, where=""):
    assert np.array_equal(got["output_ids"], ref["output_ids"]), "output_ids differ " + where
    for key in ("finished", "sequence_length", "should_stop"):
        if ref[key] is not None:
            assert np.array_equal(got[key], ref[key]), key + " differs " + where
    rtol = 1e-5 if dt == O.F32 else 2e-3
    for key in ("cum_log_probs", "output_log_probs"):
        if ref[key] is not None:
            np.testing.assert_allclose(got[key], ref[key], rtol=rtol, atol=1e-6, err_msg=key + " " + where)
    if check_logits:
        # the unfused path mutates the caller's logits exactly as the reference does
        assert np.array_equal(bits(got["logits"], dt), bits(ref["logits"], dt)), "mutated logits differ " + where
