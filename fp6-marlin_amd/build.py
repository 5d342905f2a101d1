"""Build the native parts of fp6_marlin for gfx950, in-tree.

    python fp6-marlin_amd/build.py            # C-ABI library + torch extension
    python fp6-marlin_amd/build.py --no-torch # C-ABI library only
    python fp6-marlin_amd/build.py --timeline # also the instrumented library that `bench.py --timeline` loads

Outputs (next to the Python package, so they travel with the source tree):
    fp6_marlin/libfp6m.so        C ABI of include/fp6m.h: host packers + HIP kernels (hipcc)
    fp6_marlin/_fp6m_torch.so    thin torch extension that unwraps tensors and calls the C ABI (g++)
    fp6_marlin/libfp6m_timeline.so   (--timeline) the same library with -DFP6M_TIMELINE: every workgroup of the GEMM
                                 kernels writes eight clock stamps; a measuring tool, never loaded by the package
"""
import argparse
import os
import subprocess
import sys
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
PKG = os.path.join(HERE, "fp6_marlin")
INCLUDE = os.path.join(ROOT, "include")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
ARCH = "gfx950"

# Packed-FP32 VALU forms are switched off for every device compile.
HIP_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
             "-packed-fp32-ops", "-Wall", "-Wno-unused-function", f"-I{INCLUDE}", f"-I{CSRC}"]


def run(cmd):
    print("+", " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_lib(timeline=False):
    hipcc = os.path.join(ROCM, "bin", "hipcc")
    out = os.path.join(PKG, "libfp6m_timeline.so" if timeline else "libfp6m.so")
    srcs = [os.path.join(CSRC, f) for f in ("fp6m_cpu.cpp", "fp6m_gemm.hip", "fp6m_pack.hip")]
    run([hipcc, *HIP_FLAGS, *(["-DFP6M_TIMELINE"] if timeline else []), "-shared", "-pthread", "-o", out, *srcs])
    return out


def build_torch_ext():
    import torch
    from torch.utils import cpp_extension

    out = os.path.join(PKG, "_fp6m_torch.so")
    inc = [f"-I{p}" for p in cpp_extension.include_paths()] + [f"-I{sysconfig.get_paths()['include']}",
                                                               f"-I{INCLUDE}", f"-I{ROCM}/include"]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cxx11 = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={cxx11}", "-DTORCH_EXTENSION_NAME=_fp6m_torch",
           "-DTORCH_API_INCLUDE_EXTENSION_H", *inc, os.path.join(CSRC, "fp6m_torch.cpp"), "-o", out,
           f"-L{PKG}", "-lfp6m", f"-L{tlib}", "-ltorch", "-ltorch_cpu", "-ltorch_python", "-lc10", "-lc10_hip",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"]
    run(cmd)
    return out


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-torch", action="store_true")
    ap.add_argument("--timeline", action="store_true", help="also build the instrumented library for bench.py --timeline")
    args = ap.parse_args(argv)
    build_lib()
    if args.timeline:
        build_lib(timeline=True)
    if not args.no_torch:
        build_torch_ext()


if __name__ == "__main__":
    sys.exit(main())
