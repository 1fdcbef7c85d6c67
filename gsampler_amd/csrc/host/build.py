#!/usr/bin/env python3
"""Builds gsampler_amd/lib/libgs.so: the C++ operator library that registers
gs_classes.Graph and gs_ops with PyTorch-ROCm and calls the C ABI of
libgsampler_hip.so (built first by ../Makefile).  Host code only: compiled with
g++ against the torch headers, no device code in this library."""
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.normpath(os.path.join(HERE, "..", "..", "lib"))
BUILD = os.path.join(HERE, "build")


def main() -> None:
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(BUILD, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    abi = int(torch._C._GLIBCXX_USE_CXX11_ABI)
    inc = [f"-I{p}" for p in ce.include_paths()] + ["-I/opt/rocm/include"]
    flags = ["-O2", "-std=c++17", "-fPIC", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
             f"-D_GLIBCXX_USE_CXX11_ABI={abi}", "-Wall", "-Wno-unused-parameter",
             "-Wno-sign-compare", "-Wno-deprecated-declarations"]
    srcs = sorted(glob.glob(os.path.join(HERE, "*.cc")))
    hdrs = glob.glob(os.path.join(HERE, "*.h")) + [
        os.path.normpath(os.path.join(HERE, "..", "..", "..", "include", "gsampler_hip.h"))]
    newest_hdr = max(os.path.getmtime(h) for h in hdrs)
    force = "--force" in sys.argv

    def compile_one(src):
        obj = os.path.join(BUILD, os.path.basename(src)[:-3] + ".o")
        if (not force and os.path.exists(obj)
                and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_hdr)):
            return obj
        cmd = ["g++", *flags, *inc, "-c", src, "-o", obj]
        print("+", " ".join(cmd[:3]), "...", os.path.basename(src), flush=True)
        subprocess.check_call(cmd)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as pool:
        objs = list(pool.map(compile_one, srcs))
    torch_lib = ce.library_paths()[0]
    out = os.path.join(LIB_DIR, "libgs.so")
    cmd = ["g++", "-shared", "-o", out, *objs, f"-L{torch_lib}", "-ltorch", "-ltorch_cpu",
           "-lc10", "-lc10_hip", "-ltorch_hip", f"-L{LIB_DIR}", "-lgsampler_hip",
           "-L/opt/rocm/lib", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    print("+ link", out, flush=True)
    subprocess.check_call(cmd)


if __name__ == "__main__":
    main()
