"""Builds libnzhip.so (HIP kernels + C-ABI) for gfx950 with hipcc, in-tree."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libnzhip.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

SOURCES = ["nzhip_gemm.hip", "nzhip_gemm_h16.hip", "nzhip_skinny.hip", "nzhip_conv.hip", "nzhip_ops.hip", "nzhip_fp32.hip",
           "nzhip_nn.hip", "nzhip_probe.hip",
           "nzhip_runtime.cpp"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=default",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def build_library(verbose: bool = False) -> str:
    objs = []
    procs = []
    os.makedirs(os.path.join(HERE, "build"), exist_ok=True)
    for src in SOURCES:
        obj = os.path.join(HERE, "build", src.rsplit(".", 1)[0] + ".o")
        cmd = [HIPCC, *FLAGS, "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    failed = False
    for src, p in procs:
        out, _ = p.communicate()
        out = "\n".join(l for l in out.splitlines() if "packed-fp32-ops" not in l)
        if p.returncode != 0:
            failed = True
            print(f"--- {src} failed ---\n{out}", file=sys.stderr)
        elif verbose and out.strip():
            print(f"--- {src} ---\n{out}")
    if failed:
        raise RuntimeError("hipcc failed")
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs]
    subprocess.check_call(cmd)
    return LIB


NZ = os.path.join(HERE, "nz")
NZ_LIB = os.path.join(HERE, "libnz_amd.so")
CXX = os.environ.get("CXX", "g++")


def build_host_layer(verbose: bool = False) -> str:
    """libnz_amd.so: the C++ nz:: API (plain host C++; talks to libnzhip.so through the C-ABI),
    plus its two test executables."""
    inc = ["-I" + os.path.join(NZ, "include"), "-I" + os.path.join(os.path.dirname(HERE), "include")]
    srcs = sorted(os.path.join(NZ, "src", f) for f in os.listdir(os.path.join(NZ, "src")) if f.endswith(".cpp"))
    link = ["-L" + HERE, "-lnzhip"]

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.check_call(cmd)

    run([CXX, "-std=c++17", "-O2", "-Wall", "-Wextra", "-fPIC", "-shared", "-fvisibility=hidden", *inc, *srcs,
         "-o", NZ_LIB, *link, "-Wl,-rpath,$ORIGIN"])
    tests = os.path.join(NZ, "tests")
    common = ["-std=c++17", "-Wall", "-Wno-unused-result", *inc, "-L" + HERE, "-lnz_amd", "-lnzhip",
              "-Wl,-rpath,$ORIGIN/../..", "-pthread"]
    # host-only tests run under AddressSanitizer + UBSan (host code only; no GPU code is involved)
    run([CXX, "-O1", "-g", "-fsanitize=address,undefined", os.path.join(tests, "test_host.cpp"),
         "-o", os.path.join(tests, "test_host"), *common])
    run([CXX, "-O2", "-mf16c", os.path.join(tests, "test_gpu.cpp"), "-o", os.path.join(tests, "test_gpu"), *common])
    examples = os.path.join(NZ, "examples")
    run([CXX, "-O2", os.path.join(examples, "readme_example.cpp"), "-o", os.path.join(examples, "readme_example"), *common])
    run([CXX, "-O2", os.path.join(examples, "layer_bench.cpp"), "-o", os.path.join(examples, "layer_bench"), *common])
    return NZ_LIB


def build_all(verbose: bool = False) -> None:
    build_library(verbose=verbose)
    build_host_layer(verbose=verbose)


if __name__ == "__main__":
    build_all(verbose="-v" in sys.argv)
    print(LIB)
