"""MI355X-native decode-step sampling engine (drop-in for FasterTransformer's DynamicDecodeLayer path).

The product is native: fastertransformer_amd/lib/libftk_sampling.so (HIP kernels, C ABI declared in
include/ftk_sampling.h) and fastertransformer_amd/lib/libft_decode.so (host C++ layers, C handle API in
include/ft_decode_c.h). This package only loads them and passes device pointers of torch tensors
through; there is no Python or CPU fallback, and loading fails loudly when the libraries are missing.
"""
from .ops import (F32, F16, BF16, PENALTY_ADDITIVE, PENALTY_MULTIPLICATIVE, PENALTY_NONE, BeamHypotheses,
                  DynamicDecodeLayer, FtkError, OnlineBeamSearchLayer, decode_lib, ftk, lib_dir, torch_dtype)

__all__ = ["F32", "F16", "BF16", "PENALTY_ADDITIVE", "PENALTY_MULTIPLICATIVE", "PENALTY_NONE", "BeamHypotheses",
           "DynamicDecodeLayer", "FtkError", "OnlineBeamSearchLayer", "decode_lib", "ftk", "lib_dir", "torch_dtype"]
