"""Builds the gfx950 library and the host-side driver in-tree with hipcc.

    python -m catccos_amd.build            # everything
    python -m catccos_amd.build --only lib
    python -m catccos_amd.build --only lib --define CCH_V_NOLOAD --out /tmp/noload   # a measurement build of the GEMM kernels

Outputs (git-ignored, shipped as built files):
    catccos_amd/libcatccos_hip.so      C ABI + HIP kernels   (include/catccos_hip.h)
    catccos_amd/libcatccos_host.so     C++ operator surface  (catccos_amd/csrc/host/)
    catccos_amd/catccos_run            command-line driver over the operator surface
    catccos_amd/libcatccos_torch.so    torch.ops.catccos.* (C++ TORCH_LIBRARY, catccos_amd/csrc/torch/)
"""
import argparse
import concurrent.futures
import glob
import os
import subprocess
import sys

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "build")
LIB = os.path.join(PKG, "libcatccos_hip.so")
HOST_LIB = os.path.join(PKG, "libcatccos_host.so")
DRIVER = os.path.join(PKG, "catccos_run")
TORCH_LIB = os.path.join(PKG, "libcatccos_torch.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
    # packed fp32 VALU forms are kept out of all device code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
    # the direct-to-LDS loads are inline assembly that writes M0 and names it as clobbered
    "-Wno-inline-asm",
]


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out, file=sys.stderr)


def _compile(src, defines=(), obj_dir=None):
    obj_dir = obj_dir or OBJ
    os.makedirs(obj_dir, exist_ok=True)
    obj = os.path.join(obj_dir, os.path.basename(src) + ".o")
    _run([HIPCC] + HIP_FLAGS + ["-D" + d for d in defines] + ["-c", src, "-o", obj])
    return obj


def build_lib(jobs=8, defines=(), out_dir=None):
    """The shipped library, or (with `defines` and `out_dir`) a measurement build of it in a directory of its own."""
    if defines and not out_dir:
        raise ValueError("a build with extra defines needs --out: it must not replace the shipped library")
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    obj_dir = os.path.join(out_dir, "obj") if out_dir else None
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda src: _compile(src, defines, obj_dir), srcs))
    lib = os.path.join(out_dir, "libcatccos_hip.so") if out_dir else LIB
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs)
    return lib


def build_host():
    host_dir = os.path.join(CSRC, "host")
    srcs = sorted(glob.glob(os.path.join(host_dir, "*.cpp")))
    if not srcs:
        return None
    lib_srcs = [s for s in srcs if os.path.basename(s) != "catccos_run.cpp"]
    common = ["g++", "-O2", "-std=c++17", "-fPIC", "-Wall", "-I" + os.path.join(ROOT, "include"), "-I" + host_dir]
    rpath = ["-L" + PKG, "-Wl,-rpath,$ORIGIN"]
    _run(common + ["-shared", "-o", HOST_LIB] + lib_srcs + rpath + ["-lcatccos_hip"])
    # the operators and launchers register themselves from static initialisers of the host library,
    # so the driver must keep the dependency although it names none of its symbols
    _run(common + ["-o", DRIVER, os.path.join(host_dir, "catccos_run.cpp")] + rpath +
         ["-Wl,--no-as-needed", "-lcatccos_host", "-lcatccos_hip"])
    return HOST_LIB


def build_torch():
    """torch.ops.catccos.* as a C++ TORCH_LIBRARY (catccos_amd/csrc/torch/torch_bindings.cpp): host code only, against
    this interpreter's PyTorch and the HIP library above."""
    import torch
    from torch.utils import cpp_extension as ce
    src = os.path.join(CSRC, "torch", "torch_bindings.cpp")
    tlib = ce.library_paths()[0]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           # the platform macro the HIP runtime headers ask for, and PyTorch's switch for its ROCm headers
           "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-I" + os.path.join(ROOT, "include"), "-I/opt/rocm/include"] + ["-isystem" + d for d in ce.include_paths()] + [
           src, "-o", TORCH_LIB, "-L" + tlib, "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip", "-L" + PKG, "-lcatccos_hip",
           "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    _run(cmd)
    return TORCH_LIB


def build_all(jobs=8):
    build_lib(jobs)
    build_host()
    build_torch()


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", choices=["lib", "host", "torch"])
    ap.add_argument("-j", type=int, default=8)
    ap.add_argument("--define", action="append", default=[], metavar="NAME", help="extra -D for the HIP sources (needs --out)")
    ap.add_argument("--out", metavar="DIR", help="directory for a library built with --define")
    a = ap.parse_args()
    if a.only in (None, "lib"):
        print(build_lib(a.j, a.define, a.out))
    if a.only in (None, "host"):
        print(build_host())
    if a.only in (None, "torch"):
        print(build_torch())
