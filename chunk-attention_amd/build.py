"""Builds the native parts in-tree for gfx950 (MI355X).

  python build.py            # libchunkattn_hip.so (HIP kernels + C-ABI) and chunk_attn_c (pybind11/libtorch module)
  python build.py --no-pybind
  python build.py --host-sanitize   # host-only half (tables, prefix tree) under ASan + UBSan, for the CPU tests

Outputs go to chunk_attn/lib/.  hipcc cross-compiles, so this runs without a GPU.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import sysconfig
import time

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "chunk_attn", "lib")
HIP_LIB = os.path.join(LIBDIR, "libchunkattn_hip.so")

# -packed-fp32-ops off: hipcc otherwise forms v_pk_*_f32 from scalar float code
# kernarg preload: the first kernel-argument dwords arrive in scalar registers with the wave
# instead of through a load every workgroup starts with (0.2-0.3 us per forward, measured)
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
             "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
             "-mllvm", "-amdgpu-kernarg-preload-count=16"]


def _run(cmd):
    print("+ " + " ".join(cmd), flush=True)
    subprocess.check_call(cmd)


def build_hip_lib() -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    srcs = [os.path.join(CSRC, f) for f in ("kernels.hip", "rotary.hip", "norm.hip", "c_api.cpp", "c_api_host.cpp", "tables.cpp", "prefix_tree.cpp")]
    cmd = [hipcc] + HIP_FLAGS + ["-shared", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
                                  "-o", HIP_LIB] + srcs
    _run(cmd)
    return HIP_LIB


HOST_SAN_LIB = os.path.join(LIBDIR, "libchunkattn_host_san.so")


def build_host_sanitized() -> str:
    """The host-only half of the C-ABI (table builder and prefix-tree manager: c_api_host.cpp,
    tables.cpp, prefix_tree.cpp -- no HIP header, no device code) compiled by g++ with
    AddressSanitizer and UndefinedBehaviorSanitizer.  A checking build for the CPU tests
    (tests/test_host_sanitized.py), never loaded by the product."""
    os.makedirs(LIBDIR, exist_ok=True)
    srcs = [os.path.join(CSRC, f) for f in ("c_api_host.cpp", "tables.cpp", "prefix_tree.cpp")]
    cmd = [os.environ.get("CXX", "g++"), "-O1", "-g", "-std=c++17", "-fPIC", "-shared", "-fno-omit-frame-pointer",
           "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
           "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, "-o", HOST_SAN_LIB] + srcs
    _run(cmd)
    return HOST_SAN_LIB


def pybind_target() -> str:
    return os.path.join(LIBDIR, "chunk_attn_c" + sysconfig.get_config_var("EXT_SUFFIX"))


def build_pybind() -> str:
    """chunk_attn_c: the libtorch/pybind11 `Attention` class on top of the C-ABI library."""
    import pybind11
    import torch
    from torch.utils import cpp_extension as ce

    os.makedirs(LIBDIR, exist_ok=True)
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    out = pybind_target()
    incs = ["-I" + p for p in ce.include_paths()] + ["-I" + pybind11.get_include(),
                                                     "-I" + sysconfig.get_paths()["include"],
                                                     "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
                                                     "-I/opt/rocm/include"]
    srcs = [os.path.join(CSRC, f) for f in ("attention.cpp", "python_exports.cpp")]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=chunk_attn_c",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI)] + incs + srcs + [
        "-o", out, "-L" + LIBDIR, "-lchunkattn_hip", "-L" + tlib, "-ltorch", "-ltorch_cpu",
        "-ltorch_python", "-lc10", "-lc10_hip", "-ltorch_hip",
        "-Wl,-rpath,$ORIGIN", "-Wl,-rpath," + tlib]
    _run(cmd)
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-pybind", action="store_true")
    ap.add_argument("--host-sanitize", action="store_true",
                    help="only build the host-only half of the C-ABI with ASan + UBSan (for tests/test_host_sanitized.py)")
    args = ap.parse_args()
    t0 = time.time()
    if args.host_sanitize:
        build_host_sanitized()
        print("built in %.1f s" % (time.time() - t0))
        return 0
    build_hip_lib()
    if not args.no_pybind:
        build_pybind()
    print("built in %.1f s" % (time.time() - t0))
    return 0


if __name__ == "__main__":
    sys.exit(main())
