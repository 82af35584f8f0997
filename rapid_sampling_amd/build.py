"""In-tree build of the two shared objects of the package.

  librapid_sampling_hip.so   hand-written gfx950 kernels + the C ABI (hipcc)
  _sample.<abi>.so           the PyTorch-ROCm extension module (g++), linked
                             against the first through include/rapid_sampling.h

Plain compiler command lines on purpose: the kernel source never goes through
torch's extension builder (which rewrites sources), and the built files stay
next to the package so that they travel with the tree.
"""
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(ROOT, "include")
KERNEL_LIB = os.path.join(HERE, "librapid_sampling_hip.so")
EXT_SUFFIX = sysconfig.get_config_var("EXT_SUFFIX")
EXT_LIB = os.path.join(HERE, "_sample" + EXT_SUFFIX)

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-ffp-contract=off", "-fno-fast-math",
    # packed fp32 instructions are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)


KERNEL_SOURCES = ["rs_api.hip", "rs_cluster.hip", "rs_stream.hip", "rs_wide.hip", "rs_row.hip"]


def build_kernels(verbose=False):
    """One object per translation unit, compiled side by side (each instantiates its own kernels;
    no device code is linked across objects), then one shared library."""
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    flags = [f for f in HIP_FLAGS if f != "-shared"]
    procs = []
    for src in KERNEL_SOURCES:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [HIPCC] + flags + ["-c", "-I" + INCLUDE, "-I" + CSRC, "-o", obj, os.path.join(CSRC, src)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((cmd, obj, subprocess.Popen(cmd)))
    objs = []
    for cmd, obj, proc in procs:
        if proc.wait() != 0:
            raise subprocess.CalledProcessError(proc.returncode, cmd)
        objs.append(obj)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", KERNEL_LIB] + objs, verbose)
    return KERNEL_LIB


def build_extension(verbose=False):
    import torch
    from torch.utils import cpp_extension as ce

    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for p in ce.include_paths() + [sysconfig.get_paths()["include"], INCLUDE, "/opt/rocm/include"]:
        inc += ["-isystem" if "torch" in p or "rocm" in p else "-I", p]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall",
           "-DTORCH_EXTENSION_NAME=_sample", "-DTORCH_API_INCLUDE_EXTENSION_H",
           "-DUSE_ROCM", "-D__HIP_PLATFORM_AMD__",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)] + inc + [
        "-o", EXT_LIB, os.path.join(CSRC, "sampling.cpp"),
        "-L" + tlib, "-Wl,-rpath," + tlib,
        "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-ltorch_python",
        "-L" + HERE, "-lrapid_sampling_hip", "-Wl,-rpath,$ORIGIN",
        "-L/opt/rocm/lib", "-Wl,-rpath,/opt/rocm/lib", "-lamdhip64",
    ]
    _run(cmd, verbose)
    return EXT_LIB


def build_all(verbose=False):
    build_kernels(verbose)
    build_extension(verbose)
    return KERNEL_LIB, EXT_LIB


if __name__ == "__main__":
    build_all(verbose="-q" not in sys.argv)
