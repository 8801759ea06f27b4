"""Build recipe for libaicomp_kv.so (hipcc, gfx950 only).

``python -m aicomp_amd.build`` compiles every HIP source under ``csrc/`` and
links the C-ABI shared library next to this file.  hipcc cross-compiles for
gfx950 without a GPU present.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libaicomp_kv.so")
SOURCES = ["capi.hip", "kv_append.hip", "decode_generic.hip", "decode_mfma.hip", "prefill_mfma.hip",
           "prefill_mfma_f32.hip", "prefill_tiled.hip", "rope_append.hip", "sample.hip"]
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
# Per-source extras.  The prefill kernel's row maxima read MFMA results directly; without this
# flag every fmaxf operand is first canonicalised by a self-max (one extra VALU op per score).
EXTRA_FLAGS = {"prefill_mfma.hip": ["-fno-honor-nans"]}


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, src.replace(".hip", ".o"))
    cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    return obj


def build(verbose: bool = True, jobs: int = 8) -> str:
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {LIB}")
    return LIB


TORCH_LIB = os.path.join(HERE, "libaicomp_kv_torch.so")


def build_torch_ops(verbose: bool = True) -> str:
    """Compile csrc/torch_ops.cpp: the TORCH_LIBRARY(mi355_kv) registration of the C ABI (host code
    only: it links libaicomp_kv.so and libtorch, and holds no device code)."""
    import torch
    from torch.utils import cpp_extension as ce
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    abi = int(torch.compiled_with_cxx11_abi())
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1",
           "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={abi}", *[f"-I{d}" for d in ce.include_paths()],
           "-I/opt/rocm/include", os.path.join(CSRC, "torch_ops.cpp"), "-o", TORCH_LIB, f"-L{tlib}", "-ltorch",
           "-ltorch_cpu", "-lc10", "-ltorch_hip", "-lc10_hip", f"-L{HERE}", "-laicomp_kv", "-Wl,-rpath,$ORIGIN",
           f"-Wl,-rpath,{tlib}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"compiling torch_ops.cpp failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {TORCH_LIB}")
    return TORCH_LIB


def build_fast_call(verbose: bool = True) -> str:
    """Compile csrc/fast_call.cpp into the CPython module aicomp_amd._aicomp_fast: the operator's
    decode call as one METH_FASTCALL function over the same library (host code only)."""
    import sysconfig
    import torch
    from torch.utils import cpp_extension as ce
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = os.path.join(HERE, "_aicomp_fast" + sysconfig.get_config_var("EXT_SUFFIX"))
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1",
           "-DUSE_ROCM=1", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch.compiled_with_cxx11_abi())}",
           f"-I{sysconfig.get_paths()['include']}", *[f"-I{d}" for d in ce.include_paths()], "-I/opt/rocm/include",
           os.path.join(CSRC, "fast_call.cpp"), "-o", out, f"-L{tlib}", "-ltorch", "-ltorch_cpu", "-lc10",
           "-ltorch_hip", "-lc10_hip", "-ltorch_python", f"-L{HERE}", "-laicomp_kv", "-Wl,-rpath,$ORIGIN",
           f"-Wl,-rpath,{tlib}"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"compiling fast_call.cpp failed:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {out}")
    return out


def build_host_example(verbose: bool = True) -> str:
    """Compile tests/cabi_host.cpp, a C++ program that links the library directly (no Python, no
    torch): the boundary as a C or C++ host sees it."""
    root = os.path.dirname(HERE)
    src, exe = os.path.join(root, "tests", "cabi_host.cpp"), os.path.join(root, "tests", "cabi_host")
    cmd = [HIPCC, "--offload-arch=gfx950", "-O2", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-I" + os.path.join(root, "include"), src,
           "-L" + HERE, "-laicomp_kv", "-Wl,-rpath,$ORIGIN/../aicomp_amd", "-o", exe]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    if verbose:
        print(f"built {exe}")
    return exe


if __name__ == "__main__":
    build()
    build_torch_ops()
    build_fast_call()
    build_host_example()
    sys.exit(0)
