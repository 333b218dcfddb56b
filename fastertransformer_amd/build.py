"""Builds the native libraries of the sampling engine in-tree.

  fastertransformer_amd/lib/libftk_sampling.so  HIP kernels + C ABI (include/ftk_sampling.h), gfx950
  fastertransformer_amd/lib/libftk_sampling_hooks.so  the same with the test hooks of include/ftk_test_hooks.h
                                                (loaded by the test-suite only)
  fastertransformer_amd/lib/libft_decode.so     host C++ layers (DynamicDecodeLayer, TopK/TopPSamplingLayer)
                                                + the handle API used by bindings
  fastertransformer_amd/lib/libth_transformer.so  torch.classes.FasterTransformer.DynamicDecodeOp (PyTorch-ROCm
                                                custom class over libft_decode.so; skipped with --no-torch)

Run `python -m fastertransformer_amd.build`. hipcc cross-compiles for gfx950 without a GPU.
"""
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
SRC = os.path.join(PKG, "src")
LIB = os.path.join(PKG, "lib")
INCLUDE = os.path.join(ROOT, "include")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# (source, object, extra flags): lean_kernels.hip is built once per element type so the three sets of kernels
# compile side by side
KERNEL_UNITS = [
    ("fused_dtype_kernels.hip", "fused_kernels_f16.o", ["-DFTK_FUSED_DT=1"]),
    ("fused_dtype_kernels.hip", "fused_kernels_bf16.o", ["-DFTK_FUSED_DT=2"]),
    ("fused_dtype_kernels.hip", "fused_kernels_f32.o", ["-DFTK_FUSED_DT=0"]),
    ("fused_kernels.hip", "fused_kernels.o", []),
    ("topp_kernels.hip", "topp_kernels.o", []),
    ("topk_kernels.hip", "topk_kernels.o", []),
    ("logprob_kernels.hip", "logprob_kernels_f32.o", ["-DFTK_LP_DT=0"]),
    ("logprob_kernels.hip", "logprob_kernels_f16.o", ["-DFTK_LP_DT=1"]),
    ("logprob_kernels.hip", "logprob_kernels_bf16.o", ["-DFTK_LP_DT=2"]),
    ("lean_kernels.hip", "lean_kernels_f32.o", ["-DFTK_LEAN_DT=0"]),
    ("lean_kernels.hip", "lean_kernels_f16.o", ["-DFTK_LEAN_DT=1"]),
    ("lean_kernels.hip", "lean_kernels_bf16.o", ["-DFTK_LEAN_DT=2"]),
    ("penalty_kernels.hip", "penalty_kernels.o", []),
    ("criteria_kernels.hip", "criteria_kernels.o", []),
    ("decode_step_kernels.hip", "decode_step_kernels.o", []),
    ("beam_kernels.hip", "beam_kernels.o", []),
]

# -ffp-contract=off: results must match a plain IEEE evaluation operation by operation.
# Packed fp32 instructions are disabled on purpose: the compiler forms them from ordinary float code, and some of
# their forms have produced wrong results without an error on this hardware.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # private arrays stay out of LDS: the kernels' LDS budgets (workgroups per compute unit) are planned by hand
    "-mllvm", "-disable-promote-alloca-to-lds=1",
    "-Wno-unused-result", "-I", CSRC, "-I", INCLUDE,
]


HOOK_UNITS = [("fused_kernels.hip", "fused_kernels.o"), ("topp_kernels.hip", "topp_kernels.o"),
              ("criteria_kernels.hip", "criteria_kernels.o"), ("beam_kernels.hip", "beam_kernels.o")]


def _run(cmd):
    print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def _newer(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _includes(path, seen=None):
    """the files a source includes with #include "..." (searched in csrc/ and include/), transitively"""
    seen = set() if seen is None else seen
    for line in open(path):
        line = line.strip()
        if line.startswith('#include "'):
            name = line.split('"')[1]
            for d in (CSRC, INCLUDE):
                dep = os.path.join(d, name)
                if os.path.exists(dep) and dep not in seen:
                    seen.add(dep)
                    _includes(dep, seen)
    return seen


def build(force=True, verbose=True, with_torch=True):
    os.makedirs(LIB, exist_ok=True)
    objs, jobs = [], []
    for src, obj_name, extra in KERNEL_UNITS:
        path = os.path.join(CSRC, src)
        obj = os.path.join(LIB, obj_name)
        if force or _newer(obj, [path] + sorted(_includes(path))):
            jobs.append([HIPCC] + HIP_FLAGS + extra + ["-c", path, "-o", obj])
        objs.append(obj)
    # the translation units are independent: compile them side by side (at most 8 at a time)
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        list(pool.map(_run, jobs))
    kernels_so = os.path.join(LIB, "libftk_sampling.so")
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", kernels_so] + objs)
    # The hooks build for the test-suite (include/ftk_test_hooks.h): the translation units that carry
    # hooks are compiled again with -DFTK_TEST_HOOKS, everything else is shared with the product library.
    hook_objs = list(objs)
    hook_jobs = []
    for src, obj_name in HOOK_UNITS:
        path = os.path.join(CSRC, src)
        obj = os.path.join(LIB, obj_name.replace(".o", "_hooks.o"))
        if force or _newer(obj, [path] + sorted(_includes(path))):
            hook_jobs.append([HIPCC] + HIP_FLAGS + ["-DFTK_TEST_HOOKS", "-c", path, "-o", obj])
        hook_objs[hook_objs.index(os.path.join(LIB, obj_name))] = obj
    with ThreadPoolExecutor(max_workers=4) as pool:
        list(pool.map(_run, hook_jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", os.path.join(LIB, "libftk_sampling_hooks.so")]
         + hook_objs)

    host_sources, th_sources = [], []
    for d, _, files in os.walk(SRC):
        into = th_sources if os.sep + "th_op" in d else host_sources
        into += [os.path.join(d, f) for f in files if f.endswith(".cc")]
    if host_sources:
        decode_so = os.path.join(LIB, "libft_decode.so")
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-Wall", "-Wno-unused-function",
              "-D__HIP_PLATFORM_AMD__", "-I", PKG, "-I", INCLUDE, "-I", "/opt/rocm/include", "-o", decode_so]
             + sorted(host_sources)
             + ["-L", LIB, "-lftk_sampling", "-L", "/opt/rocm/lib", "-lamdhip64",
                "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"])
    if th_sources and with_torch:
        build_th_op(sorted(th_sources))
    return LIB


def build_th_op(sources):
    """The PyTorch custom class: plain g++ against the headers and libraries of the installed torch."""
    import torch
    from torch.utils import cpp_extension as ce
    th_so = os.path.join(LIB, "libth_transformer.so")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function", "-Wno-sign-compare",
           "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I", PKG, "-I", INCLUDE, "-I", "/opt/rocm/include"]
    for inc in ce.include_paths():
        cmd += ["-isystem", inc]
    cmd += ["-o", th_so] + sources + ["-L", LIB, "-lft_decode", "-lftk_sampling"]
    for lp in ce.library_paths():
        cmd += ["-L", lp, "-Wl,-rpath," + lp]
    cmd += ["-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip", "-L", "/opt/rocm/lib", "-lamdhip64",
            "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"]
    _run(cmd)
    return th_so


if __name__ == "__main__":
    build(force="--incremental" not in sys.argv, with_torch="--no-torch" not in sys.argv)
