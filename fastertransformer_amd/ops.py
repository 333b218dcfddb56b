"""ctypes bindings of the two native libraries. Pointers come from torch tensors (device memory and
pinned host memory are torch's job here; nothing is computed in Python)."""
import ctypes as C
import os

import numpy as np
import torch

F32, F16, BF16 = 0, 1, 2
PENALTY_ADDITIVE, PENALTY_MULTIPLICATIVE, PENALTY_NONE = 0, 1, 2

_PKG = os.path.dirname(os.path.abspath(__file__))


def lib_dir():
    return os.path.join(_PKG, "lib")


class FtkError(RuntimeError):
    pass


_ftk = None
_dec = None

_vp, _i, _f, _sz, _ull, _b = C.c_void_p, C.c_int, C.c_float, C.c_size_t, C.c_ulonglong, C.c_bool

class BeamHypotheses(C.Structure):
    """ftk_beam_hypotheses of include/ftk_sampling.h (BeamHypotheses of the reference, field for field)"""
    _fields_ = [("output_ids_tgt", C.c_void_p), ("sequence_lengths_tgt", C.c_void_p), ("cum_log_probs", C.c_void_p),
                ("normed_scores", C.c_void_p), ("log_probs", C.c_void_p), ("min_normed_scores", C.c_void_p),
                ("num_beams", C.c_void_p), ("is_done", C.c_void_p), ("output_ids_src", C.c_void_p),
                ("parent_ids_src", C.c_void_p), ("sequence_lengths_src", C.c_void_p), ("end_ids", C.c_void_p),
                ("log_probs_src", C.c_void_p), ("step", C.c_int), ("ite", C.c_int), ("batch_size", C.c_int),
                ("local_batch_size", C.c_int), ("max_seq_len", C.c_int), ("length_penalty", C.c_float),
                ("early_stopping", C.c_bool), ("is_return_normed_score", C.c_bool)]


# name -> argtypes (restype int unless listed in _RESTYPES)
_SIGNATURES = {
    "ftk_invoke_curand_initialize": [_vp, _sz, _ull, _vp],
    "ftk_invoke_curand_batch_initialize": [_vp, _sz, _vp, _vp],
    "ftk_invoke_add_bias_end_mask": [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_invoke_batch_topk_sampling": [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _vp, _f, _vp, _i, _vp,
                                       _vp, _i, _vp],
    "ftk_invoke_topp_initialize": [_vp, _vp, _vp, _sz, _i, _vp],
    "ftk_invoke_add_bias_softmax": [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_invoke_batch_topp_sampling": [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i,
                                       _sz, _vp, _f, _vp, _vp, _vp],
    "ftk_invoke_compute_topp_decay": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _vp],
    "ftk_fused_topp_step": [_i, _vp, _vp, _vp, _vp, _i, _sz, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp, _vp,
                            _vp, _vp, _vp, _vp, _vp],
    "ftk_fused_topp_sample_step": [_i, _vp, _vp, _vp, _i, _sz, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _f, _vp, _vp,
                                   _vp, _vp, _vp, _vp, _vp],
    "ftk_invoke_apply_temperature_penalty": [_i, _vp, _vp, _f, _i, _i, _i, _vp],
    "ftk_invoke_batch_apply_temperature_penalty": [_i, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_invoke_apply_repetition_penalty": [_i, _vp, _f, _vp, _vp, _i, _i, _i, _i, _vp, _i, _i, _i, _vp],
    "ftk_invoke_batch_apply_repetition_penalty": [_i, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _i, _i, _vp],
    "ftk_invoke_batch_apply_frequency_penalty": [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _i, _i, _vp],
    "ftk_invoke_min_length_penalty": [_i, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_invoke_ban_bad_words": [_i, _vp, _vp, _vp, _i, _i, _i, _vp, _b, _sz, _i, _i, _sz, _vp],
    "ftk_invoke_stop_words_criterion": [_vp, _vp, _vp, _vp, _sz, _sz, _i, _i, _i, _vp],
    "ftk_invoke_stop_words_criterion_rows": [_vp, _vp, _vp, _vp, _sz, _sz, _i, _i, _i, _i, _vp],
    "ftk_invoke_length_criterion": [_vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_fused_topk_step": [_vp, _vp],
    "ftk_fused_topk_step_static": [_vp, _vp],
    "ftk_measure_plain_read": [_vp, _sz, _vp, _sz, _vp, _vp],
    "ftk_invoke_log_prob_from_logits": [_i, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _vp, _sz, _vp, _b],
    "ftk_invoke_decoding_initialize": [_i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_invoke_plus_scalar": [_vp, _i, _i, _vp],
    "ftk_invoke_transpose_axis01": [_vp, _vp, _vp, _i, _i, _vp],
    "ftk_invoke_finalize": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp],
    "ftk_invoke_topk_softmax": [_i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _f, _f, _vp],
    "ftk_invoke_add_bias_apply_penalties": [_i, _i, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp,
                                            _f, _f, _i, _i, _vp],
    "ftk_invoke_beam_update": [_vp, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp],
    "ftk_invoke_update_indir_cache": [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp],
    "ftk_fused_topk_shard_gather": [_vp, _vp, _vp],
    "ftk_fused_topk_shard_merge": [_vp, _vp, _vp],
    "ftk_error_string": [_i],
    "ftk_profile_enable": [_i],
    "ftk_profile_read": [_i, _vp, _vp],
}
# include/ftk_test_hooks.h: only libftk_sampling_hooks.so (the test build) exports these
_HOOK_SIGNATURES = {
    "ftk_host_expf": [_f],
    "ftk_host_logf": [_f],
    "ftk_test_device_math": [_i, _vp, _vp, _sz, _vp],
    "ftk_test_rng_uniform": [_vp, _vp, _i, _i, _vp],
    "ftk_test_set_topp_force_deep": [_i],
    "ftk_test_set_fused_force_general": [_i],
    "ftk_test_set_fused_two_launches": [_i],
    "ftk_test_last_fused_path": [],
    "ftk_test_set_beam_path": [_i],
    "ftk_test_set_lp_form": [_i],
    "ftk_test_set_largek_two_launches": [_i],
    "ftk_host_philox4x32_10": [_vp, _vp, _vp],
}
_RESTYPES = {"ftk_host_expf": _f, "ftk_host_logf": _f, "ftk_error_string": C.c_char_p,
             "ftk_test_set_topp_force_deep": None, "ftk_test_set_fused_force_general": None,
             "ftk_test_set_fused_two_launches": None, "ftk_test_set_beam_path": None,
             "ftk_test_set_lp_form": None, "ftk_test_set_largek_two_launches": None,
             "ftk_host_philox4x32_10": None}


# error codes of include/ftk_sampling.h (positive values are hipError_t)
FTK_ERR_DTYPE, FTK_ERR_TOPK_DOMAIN, FTK_ERR_ARGUMENT, FTK_ERR_WORKSPACE, FTK_ERR_STATIC_WORKSPACE = -1, -2, -3, -4, -5
FTK_ERR_UNSUPPORTED = -6
FUSED_STATIC_WORKSPACE_BYTES = 32 << 20


def exported_symbols():
    """names every entry point include/ftk_sampling.h declares"""
    return sorted(_SIGNATURES)


def hook_symbols():
    """names every entry point include/ftk_test_hooks.h declares"""
    return sorted(_HOOK_SIGNATURES)


def ftk():
    """libftk_sampling.so; raises when it has not been built"""
    global _ftk
    if _ftk is None:
        path = os.path.join(lib_dir(), "libftk_sampling.so")
        if not os.path.exists(path):
            raise FtkError("%s is missing: run `python -m fastertransformer_amd.build` "
                           "(there is no fallback path)" % path)
        lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = _RESTYPES.get(name, _i)
        _ftk = lib
    return _ftk


_hooks = None


def ftk_hooks():
    """libftk_sampling_hooks.so: the test build of the kernel library (every product entry point plus the hooks
    of include/ftk_test_hooks.h). Its symbols stay local, so it does not get in the way of the product library."""
    global _hooks
    if _hooks is None:
        path = os.path.join(lib_dir(), "libftk_sampling_hooks.so")
        if not os.path.exists(path):
            raise FtkError("%s is missing: run `python -m fastertransformer_amd.build`" % path)
        lib = C.CDLL(path, mode=C.RTLD_LOCAL)
        for table in (_SIGNATURES, _HOOK_SIGNATURES):
            for name, argtypes in table.items():
                fn = getattr(lib, name)
                fn.argtypes = argtypes
                fn.restype = _RESTYPES.get(name, _i)
        _hooks = lib
    return _hooks


class FtTensor(C.Structure):
    _fields_ = [("where", _i), ("type", _i), ("ndim", _i), ("shape", _sz * 4), ("data", _vp)]


def decode_lib():
    """libft_decode.so (host C++ layers)"""
    global _dec
    if _dec is None:
        ftk()
        path = os.path.join(lib_dir(), "libft_decode.so")
        if not os.path.exists(path):
            raise FtkError("%s is missing: run `python -m fastertransformer_amd.build`" % path)
        lib = C.CDLL(path)
        lib.ft_decode_last_error.restype = C.c_char_p
        lib.ft_dynamic_decode_create.restype = _vp
        lib.ft_dynamic_decode_create.argtypes = [_i, _sz, _sz, _i, _vp, _i]
        lib.ft_dynamic_decode_destroy.argtypes = [_vp]
        lib.ft_dynamic_decode_destroy.restype = None
        lib.ft_dynamic_decode_set_stream.argtypes = [_vp, _vp]
        lib.ft_dynamic_decode_setup.argtypes = [_vp, _sz, _sz, _i, C.POINTER(C.c_char_p), C.POINTER(FtTensor)]
        lib.ft_dynamic_decode_forward.argtypes = [_vp, _i, C.POINTER(C.c_char_p), C.POINTER(FtTensor), _i,
                                                  C.POINTER(C.c_char_p), C.POINTER(FtTensor)]
        lib.ft_online_beam_search_create.restype = _vp
        lib.ft_online_beam_search_create.argtypes = [_i, _sz, _sz, _vp]
        lib.ft_online_beam_search_destroy.argtypes = [_vp]
        lib.ft_online_beam_search_destroy.restype = None
        lib.ft_online_beam_search_forward.argtypes = [_vp, _i, C.POINTER(C.c_char_p), C.POINTER(FtTensor), _i,
                                                      C.POINTER(C.c_char_p), C.POINTER(FtTensor)]
        _dec = lib
    return _dec


def check(rc, what=""):
    if rc != 0:
        raise FtkError("%s failed: %s (code %d)" % (what, ftk().ftk_error_string(rc).decode(), rc))


def ptr(t):
    """torch tensor / numpy array / None -> address"""
    if t is None:
        return None
    if isinstance(t, torch.Tensor):
        return t.data_ptr()
    if isinstance(t, np.ndarray):
        return t.ctypes.data
    return t


def current_stream():
    return torch.cuda.current_stream().cuda_stream


def torch_dtype(dt):
    return {F32: torch.float32, F16: torch.float16, BF16: torch.bfloat16}[dt]


def dtype_of(t):
    return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[t.dtype]


class FusedTopkArgs(C.Structure):
    """struct ftk_fused_topk_args"""
    _fields_ = [
        ("dtype", _i), ("logits", _vp), ("embedding_bias", _vp), ("vocab_size", _i), ("vocab_size_padded", _i),
        ("batch_size", _i), ("local_batch_size", _i), ("step", _i), ("max_input_length", _i),
        ("temperatures", _vp), ("penalties", _vp), ("penalty_type", _i), ("min_lengths", _vp), ("end_ids", _vp),
        ("input_lengths", _vp), ("output_ids", _vp), ("top_ks", _vp), ("top_ps", _vp), ("max_top_k", _i),
        ("skip_decode", _vp), ("rng_state", _vp), ("uniform_draws", _vp), ("ids", _vp), ("sequence_length", _vp),
        ("finished", _vp), ("cum_log_probs", _vp), ("output_log_probs", _vp), ("workspace", _vp),
        ("workspace_size", _sz), ("frequency_penalties", _vp),
    ]


class TopkShards(C.Structure):
    """struct ftk_topk_shards"""
    _fields_ = [("n_shards", _i), ("shard_width", _i), ("global_vocab_size_padded", _i), ("shard", _i),
                ("col_offset", _i), ("partials", _vp), ("row_stats", _vp)]


# ---- DynamicDecodeLayer over the C handle API ------------------------------------------------------
_TYPE_CODES = {
    torch.bool: 1, torch.uint8: 2, torch.int8: 6, torch.int16: 7, torch.int32: 8, torch.int64: 9,
    torch.float16: 10, torch.float32: 11, torch.float64: 12, torch.bfloat16: 14,
}
_NP_TYPE_CODES = {
    np.dtype(np.bool_): 1, np.dtype(np.uint8): 2, np.dtype(np.uint32): 4, np.dtype(np.uint64): 5,
    np.dtype(np.int32): 8, np.dtype(np.int64): 9, np.dtype(np.float32): 11,
}
MEMORY_CPU, MEMORY_CPU_PINNED, MEMORY_GPU = 0, 1, 2


class NullTensor:
    """a key that exists with a null data pointer (the reference tests register such outputs)"""

    def __init__(self, type_code, shape, where=MEMORY_GPU):
        self.type_code, self.shape, self.where = type_code, tuple(shape), where


def _describe(value, type_override=None):
    t = FtTensor()
    if isinstance(value, NullTensor):
        t.where, t.type, t.data = value.where, value.type_code, None
        shape = value.shape
    elif isinstance(value, torch.Tensor):
        if not value.is_contiguous():
            raise FtkError("tensors must be contiguous")
        t.where = MEMORY_GPU if value.is_cuda else (MEMORY_CPU_PINNED if value.is_pinned() else MEMORY_CPU)
        t.type = _TYPE_CODES[value.dtype]
        t.data = value.data_ptr()
        shape = tuple(value.shape)
    elif isinstance(value, np.ndarray):
        if not value.flags["C_CONTIGUOUS"]:
            raise FtkError("arrays must be contiguous")
        t.where, t.type, t.data = MEMORY_CPU, _NP_TYPE_CODES[value.dtype], value.ctypes.data
        shape = tuple(value.shape)
    else:
        raise FtkError("unsupported tensor value %r" % (type(value),))
    if type_override is not None:
        t.type = type_override
    if len(shape) > 4:
        raise FtkError("at most 4 dimensions")
    t.ndim = len(shape)
    for i, d in enumerate(shape):
        t.shape[i] = d
    return t


def _pack(tensors):
    names = (C.c_char_p * len(tensors))()
    descs = (FtTensor * len(tensors))()
    keep = []
    for i, (k, v) in enumerate(tensors.items()):
        names[i] = k.encode()
        descs[i] = _describe(v)
        keep.append(v)
    return names, descs, keep


class _PackedMap:
    """Named tensors marshalled for the handle API, reused from call to call: a decode loop passes the same
    objects every step (only the logits buffer or a draw array may differ), so only entries whose object
    changed are described again. Objects are compared by identity; a torch tensor that was resized in place
    must be passed as a new object."""

    def __init__(self):
        self.keys = None

    def update(self, tensors):
        keys = tuple(tensors)
        if keys != self.keys:
            self.names, self.descs, self.objs = _pack(tensors)
            self.keys = keys
            return
        objs, descs = self.objs, self.descs
        for i, v in enumerate(tensors.values()):
            if v is not objs[i]:
                descs[i] = _describe(v)
                objs[i] = v


class DynamicDecodeLayer:
    """fastertransformer::DynamicDecodeLayer<T>: setup(batch, beam, named tensors), forward(outputs, inputs).

    Values are torch tensors (GPU or CPU), numpy arrays (CPU) or NullTensor. Tensor names and shapes are
    those of the reference layer; see include/ft_decode_c.h.
    """

    def __init__(self, dtype, vocab_size, vocab_size_padded, end_id=0, stream=None, is_free_buffer_after_forward=False):
        self._lib = decode_lib()
        self.dtype = dtype
        self.vocab_size, self.vocab_size_padded = vocab_size, vocab_size_padded
        s = current_stream() if stream is None else stream
        self._h = self._lib.ft_dynamic_decode_create(dtype, vocab_size, vocab_size_padded, end_id, s,
                                                     int(is_free_buffer_after_forward))
        if not self._h:
            raise FtkError("ft_dynamic_decode_create: " + self._lib.ft_decode_last_error().decode())
        self._packed_in, self._packed_out = _PackedMap(), _PackedMap()

    def close(self):
        if getattr(self, "_h", None):
            self._lib.ft_dynamic_decode_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def _raise(self, rc, what):
        msg = self._lib.ft_decode_last_error().decode()
        if rc == 2:
            raise ValueError("%s: %s" % (what, msg))  # std::domain_error
        raise FtkError("%s: %s" % (what, msg))

    def setup(self, batch_size, beam_width, runtime_args):
        names, descs, keep = _pack(runtime_args)
        rc = self._lib.ft_dynamic_decode_setup(self._h, batch_size, beam_width, len(keep), names, descs)
        if rc != 0:
            self._raise(rc, "setup")

    def forward(self, output_tensors, input_tensors):
        pin, pout = self._packed_in, self._packed_out
        pin.update(input_tensors)
        pout.update(output_tensors)
        rc = self._lib.ft_dynamic_decode_forward(self._h, len(pin.objs), pin.names, pin.descs, len(pout.objs),
                                                 pout.names, pout.descs)
        if rc != 0:
            self._raise(rc, "forward")


class OnlineBeamSearchLayer:
    """fastertransformer::OnlineBeamSearchLayer<T>: forward(outputs, inputs) is one beam-search step over a window
    of the batch. Tensor names and shapes are those of the reference layer (include/ft_decode_c.h); the optional
    output "beam_hyps" is a BeamHypotheses structure of this module."""

    def __init__(self, dtype, vocab_size, vocab_size_padded, stream=None):
        self._lib = decode_lib()
        s = current_stream() if stream is None else stream
        self._h = self._lib.ft_online_beam_search_create(dtype, vocab_size, vocab_size_padded, s)
        if not self._h:
            raise FtkError("ft_online_beam_search_create: " + self._lib.ft_decode_last_error().decode())

    def close(self):
        if getattr(self, "_h", None):
            self._lib.ft_online_beam_search_destroy(self._h)
            self._h = None

    def __del__(self):
        self.close()

    def forward(self, output_tensors, input_tensors):
        outs = dict(output_tensors)
        if isinstance(outs.get("beam_hyps"), BeamHypotheses):
            # the layer reads the structure through a host pointer, as the reference's does
            outs["beam_hyps"] = np.frombuffer(outs["beam_hyps"], dtype=np.uint8)
        n_in, d_in, keep_in = _pack(input_tensors)
        n_out, d_out, keep_out = _pack(outs)
        rc = self._lib.ft_online_beam_search_forward(self._h, len(keep_in), n_in, d_in, len(keep_out), n_out, d_out)
        if rc != 0:
            raise FtkError("forward: " + self._lib.ft_decode_last_error().decode())

