"""Builds the two in-tree binaries of the package for gfx950:

  f2cgt_amd/lib/libf2cgt_hip.so   HIP kernels + C ABI (include/f2cgt.h), hipcc only
  f2cgt_amd/lib/F2CGTLib.<ext>    pybind11/libtorch shim over the C ABI, host compiler only

Run `python -m f2cgt_amd.build` (cross-compiles without a GPU).
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB = os.path.join(PKG, "lib")
OBJ = os.path.join(PKG, "build")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")

HIP_SOURCES = ["runtime.hip", "packbits.hip", "sq.hip", "vq.hip", "spmm.hip", "spmm_fast.hip",
               "vq_fast.hip", "encode.hip", "fetch.hip", "kmeans.hip"]
EXPERIMENT_SOURCES = ["overlap_probe.hip", "lds_rate_probe.hip"]   # compiled into the --experiments build only
HIP_FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "--offload-arch=gfx950", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-pragmas",
]
# MFMA results go to ordinary VGPRs: the arg-min update of the encode kernel then reads the scores
# directly instead of copying every accumulator out of the AGPR file first.  An internal LLVM switch:
# a compiler that no longer knows it must not break the build (the kernels are correct either way,
# the encode step is slower without it), so it is probed before use.
OPTIONAL_LLVM_FLAGS = ["-amdgpu-mfma-vgpr-form"]

CAPI_LIB = os.path.join(LIB, "libf2cgt_hip.so")
EXT_LIB = os.path.join(LIB, "F2CGTLib" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), proc.stdout))
    return proc.stdout


def _optional_flags(hipcc, verbose=True):
    """The OPTIONAL_LLVM_FLAGS this compiler accepts, as `-mllvm <flag>` pairs."""
    import tempfile

    accepted = []
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "probe.hip")
        with open(src, "w") as fh:
            fh.write("#include <hip/hip_runtime.h>\n__global__ void probe(float* p) { p[0] = 1.f; }\n")
        for flag in OPTIONAL_LLVM_FLAGS:
            proc = subprocess.run([hipcc, "--offload-arch=gfx950", "-c", src, "-o", os.path.join(tmp, "probe.o"),
                                   "-mllvm", flag], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
            if proc.returncode == 0:
                accepted += ["-mllvm", flag]
            elif verbose:
                print("build: this hipcc does not accept -mllvm %s; building without it" % flag)
    return accepted


def build_capi(verbose=True, experiments=False):
    """experiments=True also compiles the kernels that were measured and not adopted (they are
    selected at run time by the environment variables their sources name); the shipped library
    is built without them."""
    os.makedirs(LIB, exist_ok=True)
    os.makedirs(OBJ, exist_ok=True)
    hipcc = shutil.which("hipcc") or os.path.join(ROCM, "bin", "hipcc")
    sources = [s for s in HIP_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    if experiments:
        sources += [s for s in EXPERIMENT_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    optional = _optional_flags(hipcc, verbose)

    def compile_one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        extra = optional + (["-DF2CGT_EXPERIMENTS=1"] if experiments else [])
        out = _run([hipcc, *HIP_FLAGS, *extra, "-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out.strip():
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=min(6, len(sources))) as pool:
        objs = list(pool.map(compile_one, sources))
    _run([hipcc, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", CAPI_LIB, *objs,
          "-Wl,-rpath," + os.path.join(ROCM, "lib")])
    if verbose:
        print("built", CAPI_LIB)
    return CAPI_LIB


def build_extension(verbose=True):
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(LIB, exist_ok=True)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    includes = ce.include_paths() + [pybind11.get_include(), sysconfig.get_paths()["include"],
                                     os.path.join(ROCM, "include")]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           "-DTORCH_EXTENSION_NAME=F2CGTLib", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-Wno-deprecated-declarations"]
    cmd += ["-I" + p for p in includes]
    cmd += [os.path.join(CSRC, "f2cgtlib_pybind.cpp"), "-o", EXT_LIB,
            "-L" + LIB, "-lf2cgt_hip", "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-L" + torch_lib,
            "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
            "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + torch_lib]
    out = _run(cmd)
    if verbose and out.strip():
        print(out)
    if verbose:
        print("built", EXT_LIB)
    return EXT_LIB


def build_all(verbose=True, experiments=False):
    build_capi(verbose, experiments)
    build_extension(verbose)


if __name__ == "__main__":
    build_all(experiments="--experiments" in sys.argv[1:])
    sys.exit(0)
