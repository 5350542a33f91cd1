"""Builds the two shared libraries of this package with hipcc / g++ (no cmake, no JIT cache).

  lib/libmi355x_rownorm.so       HIP kernels + the extern "C" launcher ABI (include/mi355x_rownorm.h)
  lib/libmi355x_rownorm_aten.so  C++ host layer with the ATen operator signatures, registered
                                 as torch.ops.mi355x.*; links libtorch and the library above
  lib/cabi_check                 torch-free test program that calls the C ABI on hipMalloc memory
                                 (tests/native/cabi_check.cpp; needs only libdl + the HIP runtime)

Run `python build.py` (or call build_all()).  Objects go to build/ (git-ignored); the .so files
stay in-tree under lib/ so they travel with the source tree to the GPU machine.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
KERNEL_DIR = os.path.join(HERE, "csrc", "kernels")
HOST_DIR = os.path.join(HERE, "csrc", "host")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
KERNEL_LIB = os.path.join(LIB_DIR, "libmi355x_rownorm.so")
HOST_LIB = os.path.join(LIB_DIR, "libmi355x_rownorm_aten.so")
CABI_CHECK = os.path.join(LIB_DIR, "cabi_check")
CABI_CHECK_SRC = os.path.join(ROOT, "tests", "native", "cabi_check.cpp")

# Device numerics mirror the reference's flags (cmake/BuildFlags.cmake:111-160 there): no
# fast-math, FMA contraction on, correctly rounded fp32 division and square root (hipcc's
# default).  Packed fp32 VALU instructions are switched off for the device pass.  The device
# code of each object is stored compressed (the HIP runtime expands it when the library is
# loaded): about 1000 kernel instances, a fifth of the size on disk.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=fast", "--offload-compress",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wall",
]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines()
                    if "is not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(extra_flags=(), out=KERNEL_LIB, jobs=8, verbose=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    tag = "" if not extra_flags else "_" + str(abs(hash(tuple(extra_flags))) % 100000)
    obj_dir = OBJ_DIR + tag
    os.makedirs(obj_dir, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(KERNEL_DIR, "*.hip")))
    objs = [os.path.join(obj_dir, os.path.basename(s)[:-4] + ".o") for s in srcs]

    def one(pair):
        src, obj = pair
        return _run(["hipcc"] + HIPCC_FLAGS + list(extra_flags) + ["-c", src, "-o", obj])

    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for msg in ex.map(one, zip(srcs, objs)):
            if verbose and msg.strip():
                print(msg)
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", out])
    return out


def build_host(out=HOST_LIB, verbose=False):
    import torch  # only for the include / library paths
    tdir = os.path.dirname(torch.__file__)
    srcs = sorted(glob.glob(os.path.join(HOST_DIR, "*.cpp")))
    cmd = ["g++", "-std=c++17", "-O2", "-fPIC", "-shared", "-Wall", "-Wno-unknown-pragmas",
           "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM", "-D_GLIBCXX_USE_CXX11_ABI=1",
           "-I" + os.path.join(tdir, "include"),
           "-I" + os.path.join(tdir, "include", "torch", "csrc", "api", "include"),
           "-I/opt/rocm/include", "-I" + os.path.join(ROOT, "include")] + srcs + [
           "-L" + os.path.join(tdir, "lib"), "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip",
           "-L" + LIB_DIR, "-lmi355x_rownorm",
           "-Wl,-rpath," + os.path.join(tdir, "lib"), "-Wl,-rpath,$ORIGIN", "-o", out]
    msg = _run(cmd)
    if verbose and msg.strip():
        print(msg)
    return out


def build_cabi_check(out=CABI_CHECK, verbose=False):
    """The torch-free caller of the C ABI (host code only: hipcc is used as the C++ compiler that
    knows where the HIP runtime headers and library are)."""
    msg = _run(["hipcc", "-O2", "-std=c++17", "-Wall", "-Wno-unused-command-line-argument",
                "-D__HIP_PLATFORM_AMD__", "-x", "c++", CABI_CHECK_SRC, "-I/opt/rocm/include",
                "-L/opt/rocm/lib", "-lamdhip64", "-ldl", "-Wl,-rpath,/opt/rocm/lib", "-o", out])
    if verbose and msg.strip():
        print(msg)
    return out


def build_all(verbose=False):
    build_kernels(verbose=verbose)
    build_host(verbose=verbose)
    build_cabi_check(verbose=verbose)
    return KERNEL_LIB, HOST_LIB, CABI_CHECK


if __name__ == "__main__":
    libs = build_all(verbose=True)
    for l in libs:
        print("built", l, os.path.getsize(l), "bytes")
    sys.exit(0)
