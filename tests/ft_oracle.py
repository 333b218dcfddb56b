"""ctypes front-end of the CPU oracle (oracle/libft_oracle.so).

Test infrastructure only: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg, never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_SO = os.path.join(_ROOT, "oracle", "libft_oracle.so")

F32, F16, BF16 = 0, 1, 2
PEN_ADDITIVE, PEN_MULTIPLICATIVE, PEN_NONE = 0, 1, 2

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            subprocess.check_call(["make", "-C", os.path.join(_ROOT, "oracle")])
        _lib = C.CDLL(_SO)
        _lib.oracle_expf.restype = C.c_float
        _lib.oracle_expf.argtypes = [C.c_float]
        _lib.oracle_logf.restype = C.c_float
        _lib.oracle_logf.argtypes = [C.c_float]
        _lib.oracle_layer_create.restype = C.c_void_p
        _lib.oracle_layer_create.argtypes = [C.c_int, C.c_int, C.c_int]
        _lib.oracle_layer_destroy.argtypes = [C.c_void_p]
    return _lib


def _p(a):
    """numpy array (or None) -> void pointer"""
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


def np_dtype(dt):
    return {F32: np.float32, F16: np.float16, BF16: np.uint16}[dt]


def max_t(dt):
    if dt == F32:
        return np.float32(np.finfo(np.float32).max)
    if dt == F16:
        return np.float32(65504.0)
    return bf16_to_f32(np.array([0x7F7F], np.uint16))[0]


# ---- storage conversions ---------------------------------------------------------------------
def f32_to_bf16(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().oracle_float_to_bf16(_p(x), _p(y), C.c_long(x.size))
    return y


def bf16_to_f32(x):
    x = np.ascontiguousarray(x, np.uint16)
    return (x.astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty(x.shape, np.uint16)
    lib().oracle_float_to_half(_p(x), _p(y), C.c_long(x.size))
    return y


def to_storage(x, dt):
    """float32 values -> storage array of dtype `dt` (round-to-nearest-even)"""
    x = np.ascontiguousarray(x, np.float32)
    if dt == F32:
        return x.copy()
    if dt == F16:
        return f32_to_f16_bits(x).view(np.float16)
    return f32_to_bf16(x)


def to_f32(x, dt):
    if dt == F32:
        return np.asarray(x, np.float32)
    if dt == F16:
        return np.asarray(x).view(np.float16).astype(np.float32)
    return bf16_to_f32(x)


def expf(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    lib().oracle_expf_array(_p(x), _p(y), C.c_long(x.size))
    return y


def logf(x):
    x = np.ascontiguousarray(x, np.float32)
    y = np.empty_like(x)
    lib().oracle_logf_array(_p(x), _p(y), C.c_long(x.size))
    return y


# ---- kernels (all in place on numpy arrays, like the reference kernels on device buffers) -----
def ban_bad_words(dt, logits, output_ids, batch_size, local_batch_size, bad_words, share_words, bad_words_len,
                  id_offset, vocab_size_padded, step):
    return lib().oracle_ban_bad_words(dt, _p(logits), _p(output_ids), batch_size, local_batch_size, _p(bad_words),
                                      int(share_words), bad_words_len, id_offset, vocab_size_padded, step)


def apply_temperature_penalty(dt, logits, bias, temperature, batch, V, Vp):
    return lib().oracle_apply_temperature_penalty(dt, _p(logits), _p(bias), C.c_float(temperature), batch, V, Vp)


def batch_apply_temperature_penalty(dt, logits, bias, temperatures, batch, V, Vp):
    return lib().oracle_batch_apply_temperature_penalty(dt, _p(logits), _p(bias), _p(temperatures), batch, V, Vp)


def batch_apply_repetition_penalty(dt, logits, penalties, output_ids, batch_size, local_batch_size, vocab_stride,
                                   input_lengths, max_input_length, step, ptype):
    return lib().oracle_batch_apply_repetition_penalty(dt, _p(logits), _p(penalties), _p(output_ids), batch_size,
                                                       local_batch_size, vocab_stride, _p(input_lengths),
                                                       max_input_length, step, ptype)


def apply_repetition_penalty(dt, logits, penalty, output_ids, batch_size, local_batch_size, vocab_size,
                             vocab_size_padded, input_lengths, max_input_length, step, ptype):
    return lib().oracle_apply_repetition_penalty(dt, _p(logits), C.c_float(penalty), _p(output_ids), batch_size,
                                                 local_batch_size, vocab_size, vocab_size_padded, _p(input_lengths),
                                                 max_input_length, step, ptype)


def batch_apply_frequency_penalty(dt, logits, presence, frequency, output_ids, batch_size, local_batch_size,
                                  vocab_stride, input_lengths, max_input_length, step):
    return lib().oracle_batch_apply_frequency_penalty(dt, _p(logits), _p(presence), _p(frequency), _p(output_ids),
                                                      batch_size, local_batch_size, vocab_stride, _p(input_lengths),
                                                      max_input_length, step)


def min_length_penalty(dt, logits, min_lengths, end_ids, sequence_lengths, max_input_length, batch, Vp):
    return lib().oracle_min_length_penalty(dt, _p(logits), _p(min_lengths), _p(end_ids), _p(sequence_lengths),
                                           max_input_length, batch, Vp)


def add_bias_end_mask(dt, logits, bias, end_ids, finished, batch, V, Vp):
    return lib().oracle_add_bias_end_mask(dt, _p(logits), _p(bias), _p(end_ids), _p(finished), batch, V, Vp)


def add_bias_softmax(dt, logits, bias, end_ids, finished, m, n_padded, n):
    return lib().oracle_add_bias_softmax(dt, _p(logits), _p(bias), _p(end_ids), _p(finished), m, n_padded, n)


def batch_topk_sampling(dt, log_probs, ids, sequence_length, finished, cum_log_probs, output_log_probs, uniforms,
                        max_top_k, top_ks, top_p, top_ps, vocab_size_padded, end_ids, batch, skip_decode):
    return lib().oracle_batch_topk_sampling(dt, _p(log_probs), _p(ids), _p(sequence_length), _p(finished),
                                            _p(cum_log_probs), _p(output_log_probs), _p(uniforms), max_top_k,
                                            _p(top_ks), C.c_float(top_p), _p(top_ps), vocab_size_padded, _p(end_ids),
                                            batch, _p(skip_decode))


def batch_topp_sampling(dt, probs, ids, sequence_length, finished, cum_log_probs, output_log_probs, uniforms, batch,
                        vocab_size_padded, end_ids, top_p, top_ps, skip_decode):
    return lib().oracle_batch_topp_sampling(dt, _p(probs), _p(ids), _p(sequence_length), _p(finished),
                                            _p(cum_log_probs), _p(output_log_probs), _p(uniforms), batch,
                                            vocab_size_padded, _p(end_ids), C.c_float(top_p), _p(top_ps),
                                            _p(skip_decode))


def compute_topp_decay(runtime_top_p, initial_top_p, output_ids, decay, top_p_min, reset_ids, n):
    lib().oracle_compute_topp_decay(_p(runtime_top_p), _p(initial_top_p), _p(output_ids), _p(decay), _p(top_p_min),
                                    _p(reset_ids), n)


def stop_words_criterion(output_ids, stop_words, finished, id_offset, stop_words_len, batch_size, local_batch_size,
                         step):
    lib().oracle_stop_words_criterion(_p(output_ids), _p(stop_words), _p(finished), id_offset, stop_words_len, batch_size, local_batch_size, step)


def length_criterion(finished, should_stop, sequence_limit_length, batch_size, step):
    lib().oracle_length_criterion(_p(finished), _p(should_stop), _p(sequence_limit_length), batch_size, step)


# ---- layer -----------------------------------------------------------------------------------
class ForwardArgs(C.Structure):
    _fields_ = [
        ("logits", C.c_void_p), ("embedding_bias", C.c_void_p), ("end_ids", C.c_void_p),
        ("input_lengths", C.c_void_p), ("sequence_limit_length", C.c_void_p), ("stop_words", C.c_void_p),
        ("bad_words", C.c_void_p), ("uniform_draws", C.c_void_p), ("output_ids", C.c_void_p),
        ("finished", C.c_void_p), ("sequence_length", C.c_void_p), ("cum_log_probs", C.c_void_p),
        ("output_log_probs", C.c_void_p), ("should_stop", C.c_void_p),
        ("step", C.c_int), ("max_input_length", C.c_int), ("ite", C.c_int), ("local_batch_size", C.c_int),
        ("batch_size", C.c_int), ("stop_words_len", C.c_int), ("bad_words_len", C.c_int),
        ("bad_words_shared", C.c_int),
    ]


def _arr(x, dtype):
    """scalar / sequence / None -> (contiguous numpy array or None, element count)"""
    if x is None:
        return None, 0
    a = np.ascontiguousarray(np.atleast_1d(np.asarray(x)).astype(dtype))
    return a, a.size


class OracleDynamicDecodeLayer:
    """Restates DynamicDecodeLayer<T> for beam_width == 1 on host arrays."""

    def __init__(self, dt, vocab_size, vocab_size_padded):
        self.dt, self.V, self.Vp = dt, vocab_size, vocab_size_padded
        self.h = C.c_void_p(lib().oracle_layer_create(dt, vocab_size, vocab_size_padded))
        self.batch = 0

    def __del__(self):
        if getattr(self, "h", None):
            lib().oracle_layer_destroy(self.h)
            self.h = None

    def setup(self, batch, runtime_top_k=None, runtime_top_p=None, temperature=None, repetition_penalty=None,
              presence_penalty=None, frequency_penalty=None, min_length=None, top_p_decay=None, top_p_min=None,
              top_p_reset_ids=None):
        self.batch = batch
        k, nk = _arr(runtime_top_k, np.uint32)
        p, npp = _arr(runtime_top_p, np.float32)
        t, nt = _arr(temperature, np.float32)
        r, nr = _arr(repetition_penalty, np.float32)
        pr, npr = _arr(presence_penalty, np.float32)
        fr, nfr = _arr(frequency_penalty, np.float32)
        m, nm = _arr(min_length, np.int32)
        d, _ = _arr(top_p_decay, np.float32)
        mn, _ = _arr(top_p_min, np.float32)
        rs, _ = _arr(top_p_reset_ids, np.uint32)
        rc = lib().oracle_layer_setup(self.h, batch, _p(k), nk, _p(p), npp, _p(t), nt, _p(r), nr, _p(pr), npr,
                                      _p(fr), nfr, _p(m), nm, _p(d), _p(mn), _p(rs))
        if rc != 0:
            raise RuntimeError("oracle_layer_setup rc=%d" % rc)

    def state(self, which):
        k = np.zeros(self.batch, np.uint32)
        p = np.zeros(self.batch, np.float32)
        s = np.zeros(self.batch, np.uint8)
        lib().oracle_layer_get_state(self.h, which, _p(k), _p(p), _p(s))
        return k, p, s

    def forward(self, logits, end_ids, output_ids, step, max_input_length, uniform_draws, ite=0,
                local_batch_size=None, embedding_bias=None, input_lengths=None, sequence_limit_length=None,
                stop_words=None, bad_words=None, finished=None, sequence_length=None, cum_log_probs=None,
                output_log_probs=None, should_stop=None):
        a = ForwardArgs()
        batch = logits.shape[0]
        a.logits, a.embedding_bias, a.end_ids = _p(logits), _p(embedding_bias), _p(end_ids)
        a.input_lengths, a.sequence_limit_length = _p(input_lengths), _p(sequence_limit_length)
        a.stop_words, a.bad_words, a.uniform_draws = _p(stop_words), _p(bad_words), _p(uniform_draws)
        a.output_ids, a.finished, a.sequence_length = _p(output_ids), _p(finished), _p(sequence_length)
        a.cum_log_probs, a.output_log_probs, a.should_stop = _p(cum_log_probs), _p(output_log_probs), _p(should_stop)
        a.step, a.max_input_length, a.ite = step, max_input_length, ite
        a.local_batch_size = batch if local_batch_size is None else local_batch_size
        a.batch_size = batch
        a.stop_words_len = 0 if stop_words is None else stop_words.shape[-1]
        a.bad_words_len = 0 if bad_words is None else bad_words.shape[-1]
        a.bad_words_shared = int(bad_words is not None and (bad_words.ndim == 2 or bad_words.shape[0] == 1))
        rc = lib().oracle_layer_forward(self.h, C.byref(a))
        if rc != 0:
            raise RuntimeError("oracle_layer_forward rc=%d" % rc)

# ---- the steps either side of the path --------------------------------------------------------------
def log_prob_from_logits(dt, logits, ids, lengths, max_len, batch, V, Vp, batch_first=False):
    """returns (cum_log_probs[batch], log_probs[(max_len-1) * batch])"""
    cum = np.zeros(batch, np.float32)
    lp = np.zeros(max(max_len - 1, 1) * batch, np.float32)
    f = lib().oracle_log_prob_from_logits
    f.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                  C.c_size_t, C.c_size_t, C.c_int]
    f(dt, _p(cum), _p(lp), _p(logits), _p(ids), _p(lengths), max_len, batch, V, Vp, int(batch_first))
    return cum, lp


def decoding_initialize(dt, sentence_ids, batch, beam, max_input_length, with_word_ids=True):
    n = batch * beam
    finished = np.ones(n, np.bool_)
    seq = np.zeros(n, np.int32)
    word_ids = np.zeros(n, np.int32) if with_word_ids else None
    cum = np.zeros(n, np.float32)
    lib().oracle_decoding_initialize(dt, _p(finished), _p(seq), _p(word_ids), _p(cum), _p(sentence_ids), batch, beam,
                                     max_input_length)
    return finished, seq, word_ids, cum


def plus_scalar(buf, val):
    lib().oracle_plus_scalar(_p(buf), int(val), buf.size)


def transpose_axis01(inp, skipping, dim0, dim1):
    out = np.zeros(dim0 * dim1, np.int32)
    lib().oracle_transpose_axis01(_p(out), _p(inp), _p(skipping), dim0, dim1)
    return out.reshape(dim1, dim0)


def finalize(topk_output_ids, topk_sequence_lengths, scores, topk_cum_log_probs, topk_log_probs, num_beams, beam_width,
             max_seq_len, batch):
    """invokeFinalize: returns (output_ids [batch, beam, max_seq_len], sequence_lengths, cum_log_probs,
    output_log_probs); positions past a sequence's length stay zero"""
    out_ids = np.zeros((batch, beam_width, max_seq_len), np.int32)
    seq = np.zeros((batch, beam_width), np.int32)
    cum = np.zeros((batch, beam_width), np.float32) if topk_cum_log_probs is not None else None
    lp = np.zeros((batch, beam_width, max_seq_len), np.float32) if topk_log_probs is not None else None
    lib().oracle_finalize(_p(out_ids), _p(seq), _p(cum), _p(lp), _p(topk_output_ids), _p(topk_sequence_lengths),
                          _p(scores), _p(topk_cum_log_probs), _p(topk_log_probs), _p(num_beams), beam_width,
                          max_seq_len, batch)
    return out_ids, seq, cum, lp


class BeamHyps(C.Structure):
    """BeamHyps of oracle/ft_oracle.cc"""
    _fields_ = [("output_ids_tgt", C.c_void_p), ("sequence_lengths_tgt", C.c_void_p), ("cum_log_probs", C.c_void_p),
                ("normed_scores", C.c_void_p), ("log_probs", C.c_void_p), ("min_normed_scores", C.c_void_p),
                ("num_beams", C.c_void_p), ("is_done", C.c_void_p), ("output_ids_src", C.c_void_p),
                ("parent_ids_src", C.c_void_p), ("sequence_lengths_src", C.c_void_p), ("end_ids", C.c_void_p),
                ("log_probs_src", C.c_void_p), ("step", C.c_int), ("ite", C.c_int), ("batch_size", C.c_int),
                ("local_batch_size", C.c_int), ("max_seq_len", C.c_int), ("length_penalty", C.c_float),
                ("early_stopping", C.c_int)]


def topk_softmax(dt, log_probs, bias, finished, sequence_lengths, cum_log_probs, output_log_probs, ids, hyps,
                 batch, beam_width, vocab, end_ids, diversity_rate, length_penalty):
    """invokeTopkSoftMax: cum_log_probs, output_log_probs, ids and the arrays `hyps` (a dict of numpy arrays and
    ints, or None) points to are updated in place; returns the oracle's status (0 = done)"""
    h = None
    if hyps is not None:
        h = BeamHyps()
        for name, _ in BeamHyps._fields_:
            val = hyps.get(name)
            if isinstance(val, np.ndarray):
                setattr(h, name, val.ctypes.data)
            elif val is None:
                setattr(h, name, None if name not in ("step", "ite", "batch_size", "local_batch_size", "max_seq_len",
                                                        "length_penalty", "early_stopping") else 0)
            else:
                setattr(h, name, val)
    fn = lib().oracle_topk_softmax
    fn.restype = C.c_int
    fn.argtypes = [C.c_int] + [C.c_void_p] * 8 + [C.c_int] * 3 + [C.c_void_p, C.c_float, C.c_float]
    return fn(dt, _p(log_probs), _p(bias), _p(finished), _p(sequence_lengths), _p(cum_log_probs), _p(output_log_probs),
              _p(ids), C.addressof(h) if h is not None else None, batch, beam_width, vocab, _p(end_ids),
              float(diversity_rate), float(length_penalty))


def beam_add_bias_apply_penalties(dt, step, logits, current_ids, previous_ids, parent_ids, input_lengths,
                                  sequence_lengths, bias, ite, max_input_length, local_batch, batch, beam_width, V, Vp,
                                  end_ids, temperature, repetition_penalty, penalty_type, min_length):
    """invokeAddBiasApplyPenalties: logits [local_batch * beam_width, Vp] are updated in place"""
    fn = lib().oracle_beam_add_bias_apply_penalties
    fn.restype = C.c_int
    fn.argtypes = [C.c_int, C.c_int] + [C.c_void_p] * 7 + [C.c_int] * 7 + [C.c_void_p, C.c_float, C.c_float, C.c_int,
                                                                          C.c_int]
    return fn(dt, step, _p(logits), _p(current_ids), _p(previous_ids), _p(parent_ids), _p(input_lengths),
              _p(sequence_lengths), _p(bias), ite, max_input_length, local_batch, batch, beam_width, V, Vp,
              _p(end_ids), float(temperature), float(repetition_penalty), penalty_type, min_length)


def beam_update(finished, parent_ids, sequence_length, word_ids, output_ids, num_beams, ite, local_batch, beam_width,
                Vp, end_ids):
    """invokeUpdate; num_beams (or None) stands for the BeamHypotheses argument"""
    h = None
    if num_beams is not None:
        h = BeamHyps()
        h.num_beams, h.ite, h.local_batch_size = num_beams.ctypes.data, ite, local_batch
    fn = lib().oracle_beam_update
    fn.restype = None
    fn.argtypes = [C.c_void_p] * 6 + [C.c_int] * 3 + [C.c_void_p]
    fn(_p(finished), _p(parent_ids), _p(sequence_length), _p(word_ids), _p(output_ids),
       C.addressof(h) if h is not None else None, local_batch, beam_width, Vp, _p(end_ids))


def update_indir_cache(tgt, src, beam_ids, finished, local_batch, beam_width, max_seq_len, step):
    fn = lib().oracle_update_indir_cache
    fn.restype = None
    fn.argtypes = [C.c_void_p] * 4 + [C.c_int] * 4
    fn(_p(tgt), _p(src), _p(beam_ids), _p(finished), local_batch, beam_width, max_seq_len, step)


def ban_bad_words_beams(dt, logits, output_ids, parent_ids, batch, local_batch, beam_width, bad_words, share_words,
                        bad_words_len, id_offset, Vp, step):
    fn = lib().oracle_ban_bad_words_beams
    fn.restype = C.c_int
    fn.argtypes = [C.c_int] + [C.c_void_p] * 3 + [C.c_int] * 3 + [C.c_void_p] + [C.c_int] * 5
    return fn(dt, _p(logits), _p(output_ids), _p(parent_ids), batch, local_batch, beam_width, _p(bad_words),
              int(share_words), bad_words_len, id_offset, Vp, step)


def stop_words_criterion_beams(output_ids, parent_ids, stop_words, finished, id_offset, stop_words_len, batch, rows,
                               beam_width, step):
    fn = lib().oracle_stop_words_criterion_beams
    fn.restype = None
    fn.argtypes = [C.c_void_p] * 4 + [C.c_int] * 6
    fn(_p(output_ids), _p(parent_ids), _p(stop_words), _p(finished), id_offset, stop_words_len, batch, rows,
       beam_width, step)

