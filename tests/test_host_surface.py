"""Host operator surface (registry, dispatch keys, error convention) without a GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DRIVER = os.path.join(ROOT, "catccos_amd", "catccos_run")

# registry names and CocCommType values of the reference (utils/info.h:46-83, :242-275)
EXPECT = {
    "mxqtag": ("MxQuantAllGather", 24, 36),
    "agmmdq": ("AllGatherMatmulDequant", 13, 2),
    "a5mxfp8mmrs": ("Ascend950MxFp8MatmulReduceScatter", 18, 36),
    "dgds": ("DispatchGmmDequantSwiglu", 21, 2),
    "a5fp4mxatavgmm": ("Ascend950Fp4MxAllToAllVGroupedMatmul", 28, 27),
    "a5fp8mxatavgmm": ("Ascend950Fp8MxAllToAllVGroupedMatmul", 27, 27),
    # down projection: the reference registers these two for fp16 output (launch_map.h:98-99);
    # this build has those launchers (keys (25 << 8) | 1, (26 << 8) | 1) and bf16 twins, which --list shows
    "a5fp8gmmata": ("Ascend950Fp8MxGroupedMatmulAllToAllV", 25, 27),
    "a5fp4gmmata": ("Ascend950Fp4MxGroupedMatmulAllToAllV", 26, 27),
    # the MXFP8 FFN from routing to combine on one rank (bf16 in and out, as the reference's run.sh runs it)
    "a5moe": ("Ascend950DispatchFFNCombine", 32, 27),
}


def run(*args):
    return subprocess.run([DRIVER, *args], capture_output=True, text=True, timeout=120)


def test_driver_is_built():
    assert os.path.exists(DRIVER), "build with python -m catccos_amd.build"


def test_registry_and_dispatch_keys_match_reference():
    out = run("--list")
    assert out.returncode == 0
    ops = {l.split()[1] for l in out.stdout.splitlines() if l.startswith("operator ")}
    assert ops == {v[0] for v in EXPECT.values()}
    seen = {}
    for l in out.stdout.splitlines():
        if l.startswith("launcher "):
            f = l.split()
            kv = dict(x.split("=") for x in f[2:6])
            seen.setdefault(f[1], []).append((kv["name"], int(kv["type"]), int(kv["dtype"]), int(kv["key"])))
    for short, (name, ctype, dtype) in EXPECT.items():
        assert (name, ctype, dtype, (ctype << 8) | dtype) in seen[short]
    # the four MX grouped operators also have the half-precision launchers the reference registers
    # (dtype FP16 = 1, launch_map.h:98-101)
    for short, ctype in (("a5fp8gmmata", 25), ("a5fp4gmmata", 26), ("a5fp8mxatavgmm", 27), ("a5fp4mxatavgmm", 28)):
        assert any(e[1:] == (ctype, 1, (ctype << 8) | 1) for e in seen[short])
    assert sum(len(v) for v in seen.values()) == 13


def test_unknown_kernel_and_bad_shape_fail_like_the_reference_main():
    r = run("nosuchkernel", "128", "128", "128", "-")
    assert r.returncode != 0 and "[ERROR]" in r.stdout
    r = run("mxqtag", "128", "0", "100", "-")   # n not a multiple of 32
    assert r.returncode != 0 and "[ERROR]" in r.stdout
    r = run("mxqtag")
    assert r.returncode != 0 and "usage" in r.stdout


def test_no_device_is_an_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    r = run("agmmdq", "128", "128", "128", "-")
    assert r.returncode != 0 and "cch_init failed" in r.stdout


FACADE_PROGRAM = r"""
#include <cstdio>
#include "device_dgemm.h"
using namespace Catccos;
using Op = DGemm::Device::DeviceDGemm<DGemm::Kernel::AllGatherMatmulDequant>;
using Mx = DGemm::Device::DeviceDGemm<DGemm::Kernel::MxAllToAllVGroupMatmul>;
int main()
{
    Op op;
    if (op.Run(nullptr, 20, 0) != Status::kErrorInvalidProblem) return 1;          // not initialised
    Op::Arguments args{};
    args.problemShape = GemmCoord{128, 256, 512};
    args.rankSize = 1;
    args.transB = 7;                                                               // not a layout
    if (Op::GetWorkspaceSize(args) != 0) return 2;
    if (op.Initialize(args) != Status::kSuccess) return 3;
    if (op.params().problemShape.m() != 128 || op.params().problemShape.n() != 256 || op.params().problemShape.k() != 512) return 4;
    if (op(nullptr, 20, 0) != Status::kErrorInvalidProblem) return 5;              // refused by the C ABI's argument checks
    Mx::Arguments g{};
    g.gemmShape = GemmCoord{64, 128, 256};
    g.expertNum = 32;
    g.epSize = 4;
    Mx mx;
    mx.Initialize(g);
    if (mx.params().localExperts != 8) return 6;
    puts("facade ok");
    return 0;
}
"""


def test_device_operator_facade(tmp_path):
    """DeviceDGemm<Kernel>: GetWorkspaceSize / Initialize / Run as the reference's launcher bodies call
    them (include/catccos/dgemm/device/device_dgemm.hpp:50-126), without a GPU: state and error paths."""
    src = tmp_path / "facade.cpp"
    src.write_text(FACADE_PROGRAM)
    exe = tmp_path / "facade"
    pkg = os.path.join(ROOT, "catccos_amd")
    subprocess.run(["g++", "-std=c++17", "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(pkg, "csrc", "host"),
                    str(src), "-o", str(exe), "-L" + pkg, "-Wl,-rpath," + pkg, "-lcatccos_hip"], check=True, timeout=120)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and "facade ok" in r.stdout, (r.returncode, r.stdout, r.stderr)
