"""What can be checked of the product without a GPU: the C-ABI libraries load and export every function
their headers declare, the host-side argument logic of the entry points (workspace queries, domain and
argument errors), the shared deterministic arithmetic, the generator's known answers, the host classes'
TensorMap semantics, and that nothing falls back to a CPU path when no GPU is present."""
import ctypes as C
import os
import re
import subprocess

import numpy as np
import pytest

import ft_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")
PKG = os.path.join(ROOT, "fastertransformer_amd")


def _ensure_built():
    lib = os.path.join(PKG, "lib")
    if not (os.path.exists(os.path.join(lib, "libftk_sampling.so")) and os.path.exists(os.path.join(lib, "libft_decode.so"))):
        from fastertransformer_amd import build
        build.build()


def _declared_functions(header):
    text = open(os.path.join(INCLUDE, header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"//[^\n]*", "", text)
    names = re.findall(r"\b((?:ftk|ft)_[a-z0-9_]+)\s*\(", text)
    return sorted(set(names))


def test_kernel_library_exports_every_declared_function():
    _ensure_built()
    from fastertransformer_amd import ops
    lib = ops.ftk()
    declared = _declared_functions("ftk_sampling.h")
    assert len(declared) >= 25
    for name in declared:
        assert hasattr(lib, name), name
    # the Python binding table covers the same set
    assert sorted(ops.exported_symbols()) == declared


def test_test_hooks_live_in_their_own_library_only():
    """include/ftk_test_hooks.h is served by libftk_sampling_hooks.so (the test build); the product library has
    neither the hooks nor the process-wide switches behind them"""
    _ensure_built()
    from fastertransformer_amd import ops
    declared = [n for n in _declared_functions("ftk_test_hooks.h")]
    assert sorted(ops.hook_symbols()) == declared and len(declared) >= 7
    hooks, product = ops.ftk_hooks(), ops.ftk()
    for name in declared:
        assert hasattr(hooks, name), name
        assert not hasattr(product, name), name
    for name in ops.exported_symbols():  # the hooks build is a complete library
        assert hasattr(hooks, name), name


def test_decode_library_exports_every_declared_function():
    _ensure_built()
    from fastertransformer_amd import ops
    lib = ops.decode_lib()
    declared = _declared_functions("ft_decode_c.h")
    assert len(declared) >= 5
    for name in declared:
        assert hasattr(lib, name), name


def test_workspace_queries_and_argument_errors():
    """the reference's size-query convention (sampling_topk_kernels.cu:378-382, sampling_topp_kernels.cu:1076-1094):
    a null workspace returns the size and launches nothing; k outside [1, 1024] is a domain error (:393-394)"""
    _ensure_built()
    from fastertransformer_amd import ops
    import fastertransformer_amd as fa
    lib = ops.ftk()
    size = C.c_size_t(0)

    def topk_query(dtype, max_k, vocab, batch):
        return lib.ftk_invoke_batch_topk_sampling(dtype, None, C.addressof(size), None, None, None, None, None, None,
                                                  None, None, max_k, None, 1.0, None, vocab, None, None, batch, None)

    assert topk_query(fa.F32, 64, 128256, 256) == 0 and size.value > 0
    small = size.value
    assert topk_query(fa.F32, 1024, 128256, 256) == 0 and size.value >= small
    assert topk_query(fa.F32, 64, 128256, 8) == 0 and size.value > 0
    assert topk_query(fa.F32, 0, 1000, 4) == fa.ops.FTK_ERR_TOPK_DOMAIN
    assert topk_query(fa.F32, 1025, 1000, 4) == fa.ops.FTK_ERR_TOPK_DOMAIN
    assert topk_query(7, 4, 1000, 4) == fa.ops.FTK_ERR_DTYPE
    # a too small workspace is refused before anything is launched
    size.value = 16
    dummy = C.create_string_buffer(64)
    rc = lib.ftk_invoke_batch_topk_sampling(fa.F32, C.addressof(dummy), C.addressof(size), None, None, None, None,
                                            None, None, None, None, 4, None, 1.0, None, 1000, None, None, 4, None)
    assert rc == fa.ops.FTK_ERR_WORKSPACE
    # fused step: size query through the argument block
    a = ops.FusedTopkArgs()
    a.dtype, a.vocab_size, a.vocab_size_padded, a.batch_size, a.local_batch_size, a.max_top_k = fa.F16, 50257, 51200, 256, 256, 64
    a.workspace = None
    assert lib.ftk_fused_topk_step(C.addressof(a), None) == 0 and a.workspace_size > 0
    # with log-prob outputs the fused step takes rows of any pitch and start (GPT-2's 50257 fp32 columns unpadded,
    # a buffer that starts on an odd element), but no vocabulary under 1024 columns
    keep = C.create_string_buffer(64)
    a.cum_log_probs = C.addressof(keep)
    a.dtype, a.vocab_size, a.vocab_size_padded, a.logits = fa.F32, 50257, 50257, 0x1000 + 4
    assert lib.ftk_fused_topk_step(C.addressof(a), None) == 0 and a.workspace_size > 0
    a.dtype, a.logits = fa.F16, 0x1000 + 6
    assert lib.ftk_fused_topk_step(C.addressof(a), None) == 0
    a.logits = 0x1000 + 1      # not even an element boundary
    assert lib.ftk_fused_topk_step(C.addressof(a), None) == fa.ops.FTK_ERR_UNSUPPORTED
    a.logits, a.vocab_size, a.vocab_size_padded = 0x1000, 1000, 1000
    assert lib.ftk_fused_topk_step(C.addressof(a), None) == fa.ops.FTK_ERR_UNSUPPORTED
    a.cum_log_probs, a.logits, a.vocab_size, a.vocab_size_padded = None, None, 50257, 51200
    a.max_top_k = 2000
    assert lib.ftk_fused_topk_step(C.addressof(a), None) == fa.ops.FTK_ERR_TOPK_DOMAIN
    assert lib.ftk_fused_topk_step(None, None) == fa.ops.FTK_ERR_ARGUMENT
    for code, text in ((0, "success"), (fa.ops.FTK_ERR_TOPK_DOMAIN, "1<=k<=1024"), (fa.ops.FTK_ERR_WORKSPACE, "workspace")):
        assert text in lib.ftk_error_string(code).decode()


def test_shared_arithmetic_matches_the_oracle_bit_for_bit():
    _ensure_built()
    from fastertransformer_amd import ops
    lib = ops.ftk_hooks()
    rng = np.random.default_rng(2)
    x = np.concatenate([rng.uniform(-90, 90, 5000), [0.0, -0.0, -np.inf, 88.7, -103.9]]).astype(np.float32)
    got = np.array([lib.ftk_host_expf(C.c_float(float(v))) for v in x], np.float32)
    assert np.array_equal(got.view(np.uint32), O.expf(x).view(np.uint32))
    y = np.concatenate([np.exp(rng.uniform(-80, 80, 5000)), [1.0, 0.0, np.inf]]).astype(np.float32)
    got = np.array([lib.ftk_host_logf(C.c_float(float(v))) for v in y], np.float32)
    assert np.array_equal(got.view(np.uint32), O.logf(y).view(np.uint32))


def test_philox_known_answers():
    """Random123 known-answer vectors for Philox-4x32-10"""
    _ensure_built()
    from fastertransformer_amd import ops
    lib = ops.ftk_hooks()
    vectors = [
        ((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
        ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
        ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
         (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
    ]
    for ctr, key, want in vectors:
        c = (C.c_uint32 * 4)(*ctr)
        k = (C.c_uint32 * 2)(*key)
        out = (C.c_uint32 * 4)()
        lib.ftk_host_philox4x32_10(c, k, out)
        assert tuple(out) == want


def test_no_cpu_fallback_without_a_gpu():
    """the product must fail loudly, not compute on the host, when no GPU is there"""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    _ensure_built()
    import fastertransformer_amd as fa
    with pytest.raises(RuntimeError):
        layer = fa.DynamicDecodeLayer(fa.F32, 8, 8)
        layer.setup(2, 1, {"runtime_top_k": np.array([2], np.uint32)})


def test_product_does_not_reference_the_oracle():
    """the oracle is test infrastructure: nothing under the package or include/ may name it"""
    hits = []
    for base in (PKG, INCLUDE):
        for d, _, files in os.walk(base):
            for f in files:
                if f.endswith((".py", ".h", ".cc", ".hip", ".cuh")):
                    text = open(os.path.join(d, f), errors="ignore").read()
                    if re.search(r"ft_oracle|libft_oracle|oracle/", text):
                        hits.append(os.path.join(d, f))
    assert hits == []


def test_tensor_map_semantics(tmp_path):
    _ensure_built()
    exe = str(tmp_path / "test_tensor_map")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I", PKG, "-I", INCLUDE,
                           "-I", "/opt/rocm/include", os.path.join(ROOT, "tests", "cpp", "test_tensor_map.cc"),
                           "-L", os.path.join(PKG, "lib"), "-lft_decode", "-lftk_sampling",
                           "-L", "/opt/rocm/lib", "-lamdhip64",
                           "-Wl,-rpath," + os.path.join(PKG, "lib"), "-Wl,-rpath,/opt/rocm/lib", "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr


def test_kernel_wrappers_instantiate_and_answer_host_queries(tmp_path):
    """the launcher templates under the reference's header names compile for float, half and bfloat16 and their
    host-only calls (size queries, refused arguments) answer without a device"""
    _ensure_built()
    exe = str(tmp_path / "test_kernel_wrappers")
    subprocess.check_call(["g++", "-O1", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I", PKG, "-I", INCLUDE,
                           "-I", "/opt/rocm/include", os.path.join(ROOT, "tests", "cpp", "test_kernel_wrappers.cc"),
                           "-L", os.path.join(PKG, "lib"), "-lft_decode", "-lftk_sampling",
                           "-L", "/opt/rocm/lib", "-lamdhip64",
                           "-Wl,-rpath," + os.path.join(PKG, "lib"), "-Wl,-rpath,/opt/rocm/lib", "-o", exe])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
