"""Build libranncgrad.so (the HIP kernel library) in-tree for gfx950.

Run as ``python rannc_amd/build.py`` (by path, so that the package - which loads the library on
import - is not imported first); ``__graft_entry__.build()`` calls :func:`build` the same way.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_NAME = "libranncgrad.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ["rg_kernels.hip", "rg_api.hip", "rg_optim.hip", "rg_ceilings.hip"]

# -ffp-contract=off: the unscale and clip multiplies must stay two roundings.
# The packed-fp32 feature is switched off for every HIP translation unit of this project.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
    "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
]


def build_pybind(verbose: bool = True) -> str:
    """Compile rannc_amd/_ranncgrad: pybind11 entry points over the C ABI plus the native registry.  Host code only;
    it sees tensors through PyTorch's C++ headers (as the reference's extension does) and is linked against the
    libraries of the PyTorch it was built with."""
    import sysconfig
    from concurrent.futures import ThreadPoolExecutor

    import torch
    from torch.utils import cpp_extension

    out = os.path.join(HERE, "_ranncgrad" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))
    cxx = os.environ.get("CXX", "g++")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    flags = ["-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-DTORCH_EXTENSION_NAME=_ranncgrad",
             "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM", "-isystem", os.path.join(rocm, "include"),      # c10/hip/HIPStream.h
             "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)]
    for inc in cpp_extension.include_paths():
        flags += ["-isystem", inc]
    flags += ["-I", sysconfig.get_paths()["include"], "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc")]
    build_dir = os.path.join(HERE, "build")
    os.makedirs(build_dir, exist_ok=True)
    units = ["rg_pybind.cpp", "rg_registry.cpp"]

    def compile_unit(name: str) -> str:
        obj = os.path.join(build_dir, name + ".o")
        cmd = [cxx, *flags, "-c", os.path.join(HERE, "csrc", name), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if proc.returncode != 0:
            raise RuntimeError(f"pybind11 build failed ({proc.returncode}):\n{proc.stdout}")
        return obj

    with ThreadPoolExecutor(max_workers=len(units)) as pool:
        objs = list(pool.map(compile_unit, units))
    torch_lib = cpp_extension.library_paths()[0]
    cmd = [cxx, "-shared", *objs, "-o", out + ".tmp", "-L", HERE, "-l:" + LIB_NAME, "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch",
           "-ltorch_cpu", "-ltorch_python", "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"pybind11 link failed ({proc.returncode}):\n{proc.stdout}")
    os.replace(out + ".tmp", out)
    return out


def build_abi_driver(verbose: bool = True) -> str:
    """Compile tests/abi_driver.c - the C ABI driven from plain C99 with only the HIP runtime beside it - into
    tests/abi_driver (run by tests/test_gpu_c_abi.py on the GPU)."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    out = os.path.join(ROOT, "tests", "abi_driver")
    cmd = [os.environ.get("CC", "gcc"), "-std=c99", "-O1", "-Wall", "-Wextra", "-Werror", "-ffp-contract=off",
           "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(rocm, "include"), "-I", os.path.join(ROOT, "include"),
           os.path.join(ROOT, "tests", "abi_driver.c"), "-o", out + ".tmp",
           "-L", HERE, "-l:" + LIB_NAME, "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../rannc_amd", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"C driver build failed ({proc.returncode}):\n{proc.stdout}")
    os.replace(out + ".tmp", out)
    return out


def build(verbose: bool = True) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(HERE, "csrc", s) for s in SOURCES]
    cmd = [hipcc, *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-I", os.path.join(HERE, "csrc"),
           "-o", LIB_PATH + ".tmp", *srcs]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if verbose and out.strip():
        print(out, flush=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{proc.stdout}")
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    build()
    build_pybind()
    build_abi_driver()
    sys.exit(0)
