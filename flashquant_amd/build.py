"""Builds the in-tree native libraries of flashquant_amd for gfx950.

  libfq_hip.so   HIP kernels + C ABI (include/fq_hip.h); hipcc only, no torch
  _C.*.so        pybind11 module over the C ABI (torch tensors in and out)

Run ``python -m flashquant_amd.build`` from the repository root.  hipcc
cross-compiles for gfx950 without a GPU.
"""
from __future__ import annotations

import glob
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB = os.path.join(PKG, "libfq_hip.so")

HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    f"-I{os.path.join(ROOT, 'include')}",
]


# Per-file additions.  The compress and decompress-with-rotation kernels consume their MFMA results in
# the vector ALU right away: with the accumulators in ordinary vector registers (instead of the
# accumulation registers the compiler picks under register pressure) there is no copy between the two.
FILE_FLAGS = {
    "fq_compress.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
    "fq_decompress_rotate.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"],
}


def _run(cmd):
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    lines = [ln for ln in r.stdout.splitlines() if "is not a recognized feature for this target" not in ln]
    if r.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + "\n".join(lines))
    return "\n".join(lines)


def build_hip(verbose: bool = True) -> str:
    os.makedirs(OBJ, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        out = _run(["hipcc", *HIP_FLAGS, *FILE_FLAGS.get(os.path.basename(src), []), "-c", src, "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(one, zip(srcs, objs)))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs])
    return LIB


def build_bindings(verbose: bool = True) -> str:
    import pybind11
    import torch
    from torch.utils import cpp_extension

    ext = sysconfig.get_config_var("EXT_SUFFIX")
    target = os.path.join(PKG, "_C" + ext)
    srcs = sorted(glob.glob(os.path.join(CSRC, "bindings", "*.cpp")))
    inc = [f"-I{p}" for p in cpp_extension.include_paths()] + [
        f"-I{pybind11.get_include()}", f"-I{sysconfig.get_paths()['include']}",
        f"-I{os.path.join(ROOT, 'include')}", "-I/opt/rocm/include",
    ]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    os.makedirs(OBJ, exist_ok=True)
    objs = []

    def one(src):
        obj = os.path.join(OBJ, "bind_" + os.path.basename(src)[:-4] + ".o")
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden",
              "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
              f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
              "-DTORCH_EXTENSION_NAME=_C", *inc, "-c", src, "-o", obj])
        return obj

    with ThreadPoolExecutor(max_workers=min(8, max(1, len(srcs)))) as ex:
        objs = list(ex.map(one, srcs))
    _run(["g++", "-shared", "-o", target, *objs, f"-L{PKG}", "-lfq_hip",
          f"-L{tlib}", "-ltorch_python", "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip",
          "-L/opt/rocm/lib", "-lamdhip64",
          "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}", "-Wl,-rpath,/opt/rocm/lib"])
    return target


def build_all(verbose: bool = True) -> None:
    lib = build_hip(verbose)
    if verbose:
        print("built", lib)
    mod = build_bindings(verbose)
    if verbose:
        print("built", mod)


if __name__ == "__main__":
    build_all()
    sys.exit(0)
